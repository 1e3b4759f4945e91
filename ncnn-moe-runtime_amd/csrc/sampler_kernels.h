// Kernels of the gfx950 generation sampler.
//
//   scan_select_kernel     (sampler_select.h) the one HBM pass over the [rows, vocab] logits for greedy
//                          rows and rows with a Top-K window: streaming, bound, candidate list, exact
//                          best K, the CPU sampler's epilogue.
//   general_sort_kernel    (sampler_full_order.h) full stable order of a row that has no Top-K window
//   general_replay_kernel  and the sampler's walk over it with exactly reproduced sequential sums
//                          (sampler_exact_sum.h).
#ifndef NCNN_MOE_HIP_SAMPLER_KERNELS_H
#define NCNN_MOE_HIP_SAMPLER_KERNELS_H

#include "sampler_full_order.h"
#include "sampler_select.h"
#include "sampler_split.h"

namespace ncnn_moe_hip {

#ifdef NCNN_MOE_TESTING
// Evaluates expf_libm on n values (test hook; in the testing build of the library only).
__global__ void expf_probe_kernel(const float* in, float* out, size_t n)
{
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n)
        out[i] = expf_libm(in[i]);
}
#endif

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_SAMPLER_KERNELS_H
