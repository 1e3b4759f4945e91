"""ncnn_moe_hip_sampler_sample_device_static through the C ABI: the select pass with no handle and no
allocation (its scratch is a static device array).  Its output is compared byte for byte with
ncnn_moe_hip_sampler_sample_device (may_need_full_order = 0) on the same operands, on calls in a row of
which the later ones are smaller, and with the CPU oracle for the rows the pass finishes."""
import ctypes

import numpy as np
import pytest

import parity_util
from ncnn_moe_runtime_amd import hip_sampler, workloads

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _device(array):
    return torch.from_numpy(np.ascontiguousarray(array).view(np.uint8).reshape(-1)).to("cuda:0")


def _free_device_memory():
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def _case(seed, rows, vocab, dtype, stride=None, turn=0):
    """`turn` rotates the per-row option pattern: a row that one call leaves to the full-order pass, or
    rejects, is a narrow or a greedy row in the next."""
    rng = np.random.default_rng(seed)
    stride = vocab if stride is None else stride
    logits = (rng.standard_normal((rows, stride)) * 2.5).astype(np.float32)
    params = hip_sampler.make_params(rows, 0.8, 0, 0.9, 0.01)
    params["top_k"] = np.array([(20, 1, 64, 65, 50, 0, 3)[(i + turn) % 7] for i in range(rows)], dtype=np.uint32)
    params["temperature"][(turn * 4) % 9::9] = 0.0
    params["top_p"][(turn * 5) % 13::13] = 1.5  # an invalid row
    uniforms = rng.random(rows).astype(np.float32)
    data = workloads.float32_to_bf16_bits(logits) if dtype == "bf16" else logits
    return data, params, uniforms


def _both_entries(sampler, data, params, uniforms, vocab, stream, check_memory=False):
    rows, stride = data.shape
    dtype = hip_sampler.LOGITS_F32 if data.dtype == np.float32 else hip_sampler.LOGITS_BF16
    d_logits, d_params, d_uniforms = _device(data), _device(params), _device(uniforms)
    with_handle = torch.zeros(rows * 16, dtype=torch.uint8, device="cuda:0")
    without = torch.full((rows * 16,), 0xEE, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    sampler.sample_device(d_logits.data_ptr(), dtype, rows, vocab, stride, d_params.data_ptr(), d_uniforms.data_ptr(),
                          None, with_handle.data_ptr(), 0, stream.cuda_stream)
    stream.synchronize()
    free_before = _free_device_memory() if check_memory else 0
    rc = hip_sampler.sample_device_static(0, d_logits.data_ptr(), dtype, rows, vocab, stride, d_params.data_ptr(),
                                          d_uniforms.data_ptr(), None, without.data_ptr(), stream.cuda_stream)
    assert rc == hip_sampler.RC_SUCCESS, hip_sampler.last_static_error()
    stream.synchronize()
    if check_memory:
        assert _free_device_memory() == free_before, "the call changed the amount of free device memory"
    expected = with_handle.cpu().numpy().view(hip_sampler.RESULT_DTYPE).reshape(rows)
    got = without.cpu().numpy().view(hip_sampler.RESULT_DTYPE).reshape(rows)
    return got, expected


def test_static_entry_matches_the_handle_entry_on_calls_in_a_row():
    print("[case] sample_device_static: 48 x 50021 fp32, then 7 x 20011 bf16, then 300 x 12000 fp32, then 5 x 151936", flush=True)
    stream = torch.cuda.Stream(device="cuda:0")
    shapes = [(1, 48, 50021, "f32", None), (2, 7, 20011, "bf16", 20016), (3, 300, 12000, "f32", None), (4, 5, 151936, "f32", None),
              (5, 3, 9000, "f32", None)]
    with hip_sampler.HipSampler(300, 151936) as sampler:
        for call, (seed, rows, vocab, dtype, stride) in enumerate(shapes):
            print("[call %d] rows %d vocab %d %s" % (call, rows, vocab, dtype), flush=True)
            data, params, uniforms = _case(seed, rows, vocab, dtype, stride, turn=call)
            got, expected = _both_entries(sampler, data, params, uniforms, vocab, stream, check_memory=call > 0)
            assert got.tobytes() == expected.tobytes(), "call %d differs from sample_device" % call
            final = got["status"] != hip_sampler.ROW_NEEDS_FULL_ORDER
            narrow = (params["temperature"] == 0.0) | ((params["top_k"] >= 1) & (params["top_k"] <= 64)) | (params["top_p"] > 1.0)
            assert np.array_equal(final, narrow)
            cpu = parity_util.run_oracle(np.ascontiguousarray(data[:, :vocab]), params, uniforms)
            parity_util.assert_results_match(got[final], cpu[final], dtype, "static entry, call %d" % call)


def _static_only(data, params, uniforms, vocab, stream, testing=False):
    rows, stride = data.shape
    dtype = hip_sampler.LOGITS_F32 if data.dtype == np.float32 else hip_sampler.LOGITS_BF16
    d_logits, d_params, d_uniforms = _device(data), _device(params), _device(uniforms)
    out = torch.full((rows * 16,), 0xEE, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    rc = hip_sampler.sample_device_static(0, d_logits.data_ptr(), dtype, rows, vocab, stride, d_params.data_ptr(),
                                          d_uniforms.data_ptr(), None, out.data_ptr(), stream.cuda_stream, testing=testing)
    assert rc == hip_sampler.RC_SUCCESS, hip_sampler.last_static_error(testing)
    stream.synchronize()
    return out.cpu().numpy().view(hip_sampler.RESULT_DTYPE).reshape(rows)


def test_static_entry_reuses_its_records_from_one_static_call_to_the_next():
    """Static calls back to back, no handle call in between, every one through the one-chunk split kernel with
    another number of workgroups per row and another window: the records and per-row words that one call
    leaves in the static array are what the next one finds.  Checked against the CPU oracle.  Then the same
    across the point where the launch numbers of the records start over (in the testing build of the library,
    which has the hook that sets them and, like every build, a static array of its own)."""
    stream = torch.cuda.Stream(device="cuda:0")
    shapes = [(31, 48, 50021, 20), (32, 48, 151936, 64), (33, 9, 20481, 1), (34, 48, 30000, 33), (35, 64, 151936, 20), (36, 5, 41000, 50)]
    for repeat in range(2):
        for call, (seed, rows, vocab, window) in enumerate(shapes):
            print("[case] static call %d (%s): %d x %d, Top-K %d" % (call, "after the restart set-up" if repeat else "first round", rows, vocab, window), flush=True)
            segments, chunks, variant = hip_sampler.select_geometry(hip_sampler.LOGITS_F32, rows, vocab)
            assert variant == hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK and segments > 1
            data, params, uniforms = _case(seed + 10 * repeat, rows, vocab, "f32", turn=call)
            params["top_k"] = window
            got = _static_only(data, params, uniforms, vocab, stream, testing=repeat == 1)
            cpu = parity_util.run_oracle(data, params, uniforms)
            parity_util.assert_results_match(got, cpu, "f32", "static call %d, round %d" % (call, repeat))
        if repeat == 0:
            # (the hook needs a static array that has served a call: one call of the testing build, then the set-up)
            data, params, uniforms = _case(77, 48, 50021, "f32")
            params["top_k"] = 64
            _static_only(data, params, uniforms, 50021, stream, testing=True)
            assert hip_sampler.set_static_row_epochs(0, hip_sampler.LAST_EPOCH - 2) == hip_sampler.RC_SUCCESS


def test_static_entry_rejects_what_its_scratch_cannot_hold():
    print("[case] sample_device_static: argument errors", flush=True)
    rows = hip_sampler.STATIC_MAX_ROWS + 1
    buffer = torch.zeros(rows * 16, dtype=torch.uint8, device="cuda:0")
    pointer = buffer.data_ptr()
    rc = hip_sampler.sample_device_static(0, pointer, hip_sampler.LOGITS_F32, rows, 4, 4, pointer, pointer, None, pointer, None)
    assert rc == hip_sampler.RC_INVALID_ARGUMENT
    assert "NCNN_MOE_STATIC_MAX_ROWS" in hip_sampler.last_static_error()
    rc = hip_sampler.sample_device_static(0, pointer, hip_sampler.LOGITS_F32, 2, 8, 4, pointer, pointer, None, pointer, None)
    assert rc == hip_sampler.RC_INVALID_ARGUMENT and "row_stride" in hip_sampler.last_static_error()
    rc = hip_sampler.sample_device_static(0, None, hip_sampler.LOGITS_F32, 2, 8, 8, pointer, pointer, None, pointer, None)
    assert rc == hip_sampler.RC_INVALID_ARGUMENT and "null" in hip_sampler.last_static_error()
    torch.cuda.synchronize()
