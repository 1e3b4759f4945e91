"""ncnn_moe_hip_sampler_sample_device through the C ABI with every operand in device memory (torch only
allocates the buffers and owns the stream): the entry the decode step calls.  Checks the three
passes (batch-shaped select, wide select, full order), the may_need_full_order contract and that the
call does not need the handle's own logits buffer."""
import numpy as np
import pytest

import parity_util
from ncnn_moe_runtime_amd import hip_sampler

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _device(array):
    return torch.from_numpy(np.ascontiguousarray(array).view(np.uint8).reshape(-1)).to("cuda:0")


def _run(sampler, logits, params, uniforms, may_need_full_order, stream):
    rows, vocab = logits.shape
    dtype = hip_sampler.LOGITS_F32 if logits.dtype == np.float32 else hip_sampler.LOGITS_BF16
    d_logits, d_params, d_uniforms = _device(logits), _device(params), _device(uniforms)
    d_results = torch.zeros(rows * 16, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    sampler.sample_device(d_logits.data_ptr(), dtype, rows, vocab, vocab, d_params.data_ptr(), d_uniforms.data_ptr(),
                          None, d_results.data_ptr(), may_need_full_order, stream.cuda_stream)
    stream.synchronize()
    return d_results.cpu().numpy().view(hip_sampler.RESULT_DTYPE).reshape(rows)


@pytest.mark.parametrize("rows", [24, 300])
def test_three_passes_on_a_caller_stream(rows):
    print("[case] sample_device, %d rows, mixed windows" % rows, flush=True)
    rng = np.random.default_rng(rows)
    vocab = 50021
    logits = (rng.standard_normal((rows, vocab)) * 2.5).astype(np.float32)
    params = hip_sampler.make_params(rows, 0.8, 0, 0.92, 0.0)
    params["top_k"] = np.array([(1, 20, 64, 65, 700, 1024, 1025, 0)[i % 8] for i in range(rows)], dtype=np.uint32)
    params["temperature"][::11] = 0.0
    uniforms = rng.random(rows).astype(np.float32)
    cpu = parity_util.run_oracle(logits, params, uniforms)
    stream = torch.cuda.Stream(device="cuda:0")
    with hip_sampler.HipSampler(rows, vocab) as sampler:
        full = _run(sampler, logits, params, uniforms, True, stream)
        parity_util.assert_results_match(full, cpu, "f32", "sample_device, all passes")
        served_by_select = (params["temperature"] == 0.0) | ((params["top_k"] >= 1) & (params["top_k"] <= 1024))
        assert ((full["flags"][served_by_select] & hip_sampler.FLAG_GENERAL_PATH) == 0).all()
        # one kernel only: rows that need a later pass say so, the others are final
        first = _run(sampler, logits, params, uniforms, False, stream)
        narrow = (params["temperature"] == 0.0) | ((params["top_k"] >= 1) & (params["top_k"] <= 64))
        assert (first["status"][~narrow] == hip_sampler.ROW_NEEDS_FULL_ORDER).all()
        assert (first["token_id"][~narrow] == -1).all()
        parity_util.assert_results_match(first[narrow], cpu[narrow], "f32", "sample_device, select pass only")
        # and a second call with every pass finishes them
        again = _run(sampler, logits, params, uniforms, True, stream)
        parity_util.assert_results_match(again, cpu, "f32", "sample_device, repeated")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_later_passes_side_by_side(dtype):
    """Rows with wide windows and rows without a window in one batch: the wide select on the handle's
    second stream beside the full-order kernels (flag NCNN_MOE_PASSES_SIDE_BY_SIDE, and sample() by
    itself from 32 rows of each kind), with tie-heavy rows that the wide select, and the first select for a
    window of 20, hand on to the full-order kernels behind the join.  Same results as one pass after the
    other, and as the oracle."""
    print("[case] later passes side by side, %s" % dtype, flush=True)
    from ncnn_moe_runtime_amd import workloads
    rng = np.random.default_rng(77)
    rows, vocab = 120, 30011
    logits = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    logits[5::12] = np.round(logits[5::12])  # a few thousand equal logits around every cut
    logits[2::12] = np.round(logits[2::12] / 2.0) * 2.0  # (top_k 20: hundreds of equal logits at the cut)
    params = hip_sampler.make_params(rows, 0.9, 0, 0.9, 0.0)
    params["top_k"] = np.array([(700, 0, 20, 300, 2000, 1024)[i % 6] for i in range(rows)], dtype=np.uint32)
    params["temperature"][::17] = 0.0
    uniforms = rng.random(rows).astype(np.float32)
    data = workloads.float32_to_bf16_bits(logits) if dtype == "bf16" else logits
    cpu = parity_util.run_oracle(data, params, uniforms)
    stream = torch.cuda.Stream(device="cuda:0")
    with hip_sampler.HipSampler(rows, vocab) as sampler:
        in_turn = _run(sampler, data, params, uniforms, hip_sampler.PASSES_FULL_ORDER, stream)
        beside = _run(sampler, data, params, uniforms, hip_sampler.PASSES_FULL_ORDER | hip_sampler.PASSES_SIDE_BY_SIDE, stream)
        # (a row that the first select hands on is served by the wide select when the passes run in turn and by
        # the full-order kernels behind the join when they run side by side: the same result, and the flag
        # that names the path differs)
        handed_on = np.zeros(rows, dtype=bool)
        handed_on[2::12] = params["temperature"][2::12] != 0.0
        assert in_turn[~handed_on].tobytes() == beside[~handed_on].tobytes()
        assert ((beside["flags"] ^ in_turn["flags"])[handed_on] == hip_sampler.FLAG_GENERAL_PATH).all()
        for field in beside.dtype.names:
            if field != "flags":
                assert in_turn[field].tobytes() == beside[field].tobytes(), field
        parity_util.assert_results_match(beside, cpu, dtype, "side by side, device entry")
        for _ in range(3):  # the second stream forks and joins again on every call
            again = _run(sampler, data, params, uniforms, hip_sampler.PASSES_FULL_ORDER | hip_sampler.PASSES_SIDE_BY_SIDE, stream)
            assert again.tobytes() == beside.tobytes()
        sampler.upload_logits(data)
        host = sampler.sample(params, uniforms)
        parity_util.assert_results_match(host, cpu, dtype, "side by side, host entry")


def test_bf16_strided_rows_on_the_default_stream():
    print("[case] sample_device, bf16, stride wider than the vocabulary", flush=True)
    from ncnn_moe_runtime_amd import workloads
    rng = np.random.default_rng(5)
    rows, vocab, stride = 70, 40001, 40008
    values = (rng.standard_normal((rows, stride)) * 2).astype(np.float32)
    bits = workloads.float32_to_bf16_bits(values)
    bits[:, vocab:] = workloads.float32_to_bf16_bits(np.full((rows, stride - vocab), 60.0, dtype=np.float32))  # never read
    params = hip_sampler.make_params(rows, 0.7, 40, 0.9, 0.01)
    uniforms = rng.random(rows).astype(np.float32)
    cpu = parity_util.run_oracle(np.ascontiguousarray(bits[:, :vocab]), params, uniforms)
    d_logits, d_params, d_uniforms = _device(bits), _device(params), _device(uniforms)
    d_results = torch.zeros(rows * 16, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    with hip_sampler.HipSampler(rows, vocab) as sampler:
        sampler.sample_device(d_logits.data_ptr(), hip_sampler.LOGITS_BF16, rows, vocab, stride, d_params.data_ptr(),
                              d_uniforms.data_ptr(), None, d_results.data_ptr(), False, None)
        torch.cuda.synchronize()
    gpu = d_results.cpu().numpy().view(hip_sampler.RESULT_DTYPE).reshape(rows)
    parity_util.assert_results_match(gpu, cpu, "bf16", "sample_device, bf16 strided")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_no_wide_windows_flag(dtype):
    """NCNN_MOE_PASSES_NO_WIDE_WINDOWS leaves out the select kernel for 64 < top_k <= 1024.  With no such row
    the results are those of the full set of passes; a row that has such a window after all (the caller's
    promise broken) is served by the full-order kernels, with the same result."""
    print("[case] sample_device without the wide select, %s" % dtype, flush=True)
    from ncnn_moe_runtime_amd import workloads
    rng = np.random.default_rng(404)
    rows, vocab = 96, 40013
    logits = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    data = workloads.float32_to_bf16_bits(logits) if dtype == "bf16" else logits
    params = hip_sampler.make_params(rows, 0.9, 0, 0.9, 0.0)
    params["top_k"] = np.array([(0, 20, 5000, 1, 64, 0)[i % 6] for i in range(rows)], dtype=np.uint32)
    uniforms = rng.random(rows).astype(np.float32)
    stream = torch.cuda.Stream(device="cuda:0")
    flags = hip_sampler.PASSES_FULL_ORDER | hip_sampler.PASSES_NO_WIDE_WINDOWS
    with hip_sampler.HipSampler(rows, vocab) as sampler:
        cpu = parity_util.run_oracle(data, params, uniforms)
        every_pass = _run(sampler, data, params, uniforms, hip_sampler.PASSES_FULL_ORDER, stream)
        without = _run(sampler, data, params, uniforms, flags, stream)
        assert every_pass.tobytes() == without.tobytes()
        parity_util.assert_results_match(without, cpu, dtype, "no wide windows")
        params["top_k"][3::6] = 700   # wide windows after all
        cpu = parity_util.run_oracle(data, params, uniforms)
        broken_promise = _run(sampler, data, params, uniforms, flags | hip_sampler.PASSES_SIDE_BY_SIDE, stream)
        parity_util.assert_results_match(broken_promise, cpu, dtype, "wide windows without the wide select")
        assert (broken_promise["flags"][3::6] & hip_sampler.FLAG_GENERAL_PATH != 0).all()
