"""The HIP sampler (through its C ABI) against the golden vectors recorded from the reference library."""
import numpy as np
import pytest

import golden_util
from ncnn_moe_runtime_amd import hip_sampler

pytestmark = pytest.mark.gpu

STATUS_OF_ANY_ERROR = {hip_sampler.ROW_NO_FINITE_LOGIT, hip_sampler.ROW_INVALID_DISTRIBUTION,
                       hip_sampler.ROW_BAD_TEMPERATURE, hip_sampler.ROW_BAD_TOP_P, hip_sampler.ROW_BAD_MIN_P}


@pytest.mark.parametrize("general", [False, True])
def test_small_rows(general):
    g = golden_util.load()
    print("[case] golden small rows general=%s" % general, flush=True)
    with hip_sampler.HipSampler(1, 64, testing=general) as sampler:
        sampler.force_general(general)
        for case in range(g["small_vocab"].size):
            vocab = int(g["small_vocab"][case])
            sampler.upload_logits(g["small_logits"][case:case + 1, :vocab])
            options = golden_util.options_of(g["small_options"][case])
            status, ids, probabilities, count = sampler.distribution(0, **options)
            if g["small_rc"][case] != 0:
                assert status in STATUS_OF_ANY_ERROR, case
                continue
            expected = int(g["small_count"][case])
            assert status == 0 and count == expected, (case, options)
            assert np.array_equal(ids, g["small_ids"][case, :expected]), case
            assert np.array_equal(probabilities.view(np.uint32),
                                  g["small_probabilities"][case, :expected].view(np.uint32)), case


def test_session_steps():
    """Every recorded Session::sample call with the uniform the Session drew for it."""
    g = golden_util.load()
    steps = g["session_token"].size
    print("[case] golden session steps", flush=True)
    params = np.zeros(steps, dtype=hip_sampler.PARAMS_DTYPE)
    for step in range(steps):
        options = golden_util.options_of(g["session_options"][step])
        params[step] = (options["temperature"], options["top_k"], options["top_p"], options["min_p"], 0, 0)
    with hip_sampler.HipSampler(steps, 48) as sampler:
        sampler.upload_logits(g["session_logits"])
        got = sampler.sample(params, g["session_uniform"])
    ok = g["session_rc"] == 0
    assert np.array_equal(got["status"] == 0, ok)
    assert np.array_equal(got["token_id"][ok], g["session_token"][ok])
    assert np.array_equal(got["probability"][ok].view(np.uint32), g["session_probability"][ok].view(np.uint32))
    assert np.array_equal(got["draw_consumed"][ok], g["session_drew"][ok])


def test_benchmark_sized_rows():
    g = golden_util.load()
    for case in range(g["large_kept"].size):
        seed, vocab, scale, bf16, temperature, top_k, top_p, min_p = g["large_spec"][case]
        print("[case] golden large row %d vocab %d bf16 %d" % (case, vocab, bf16), flush=True)
        logits = golden_util.large_row(seed, vocab, scale, bool(bf16))
        assert np.array_equal(golden_util.sha256(logits), g["large_logits_sha"][case]), "row generator drifted"
        device_rows = np.tile(logits, (8, 1))
        if bf16:
            device_rows = golden_util.float32_to_bf16_bits(device_rows)
        options = golden_util.options_of((temperature, top_k, top_p, min_p))
        with hip_sampler.HipSampler(8, int(vocab)) as sampler:
            sampler.upload_logits(device_rows)
            status, ids, probabilities, count = sampler.distribution(3, **options)
            assert status == 0 and count == int(g["large_kept"][case])
            head = min(64, count)
            assert np.array_equal(ids[:head], g["large_head_ids"][case, :head])
            assert np.array_equal(probabilities[:head].view(np.uint32),
                                  g["large_head_probabilities"][case, :head].view(np.uint32))
            assert np.array_equal(golden_util.sha256(ids), g["large_ids_sha"][case])
            assert np.array_equal(golden_util.sha256(probabilities), g["large_probabilities_sha"][case])
            params = hip_sampler.make_params(8, **options)
            got = sampler.sample(params, g["large_uniform"][case])
        assert np.array_equal(got["token_id"], g["large_token"][case])
        assert np.array_equal(got["probability"].view(np.uint32), g["large_probability"][case].view(np.uint32))
