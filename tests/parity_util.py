"""Shared helpers of the GPU parity tests: run a workload through the HIP sampler (C ABI) and the
CPU oracle, and compare them to the bar the sampler is held to."""
import numpy as np

import oracle_lib
from ncnn_moe_runtime_amd import hip_sampler

# Filtered probabilities: relative tolerance 1e-5 for fp32 logits, 1e-3 for bf16 logits.
PROBABILITY_RTOL = {"f32": 1e-5, "bf16": 1e-3}


def run_oracle(logits, params, uniforms, stop_ids=None, threads=16, vocab=None):
    return oracle_lib.oracle_sample_batch(logits, params, uniforms, stop_ids, threads=threads, vocab=vocab)


def assert_results_match(gpu, cpu, dtype="f32", context=""):
    """Token ids, statuses, kept counts, stop and draw flags bit-exact; probabilities within tolerance."""
    assert gpu.shape == cpu.shape
    bad_status = np.nonzero(gpu["status"] != cpu["status"])[0]
    assert bad_status.size == 0, "%s status mismatch rows %s: gpu %s cpu %s" % (
        context, bad_status[:8], gpu["status"][bad_status[:8]], cpu["status"][bad_status[:8]])
    bad_token = np.nonzero(gpu["token_id"] != cpu["token_id"])[0]
    assert bad_token.size == 0, "%s token mismatch rows %s: gpu %s cpu %s (cdf_gap %s top_p_gap %s)" % (
        context, bad_token[:8], gpu["token_id"][bad_token[:8]], cpu["token_id"][bad_token[:8]],
        cpu["cdf_gap"][bad_token[:8]], cpu["top_p_gap"][bad_token[:8]])
    bad_kept = np.nonzero(gpu["kept_count"] != cpu["kept_count"])[0]
    assert bad_kept.size == 0, "%s kept_count mismatch rows %s: gpu %s cpu %s" % (
        context, bad_kept[:8], gpu["kept_count"][bad_kept[:8]], cpu["kept_count"][bad_kept[:8]])
    assert np.array_equal(gpu["is_stop"], cpu["is_stop"]), context + " is_stop mismatch"
    assert np.array_equal(gpu["draw_consumed"], cpu["draw_consumed"]), context + " draw_consumed mismatch"
    has_nan = (gpu["flags"] & hip_sampler.FLAG_HAS_NAN) != 0
    ok = gpu["status"] == 0
    assert np.array_equal(has_nan[ok], cpu["has_nan"][ok] != 0), context + " has_nan mismatch"
    np.testing.assert_allclose(gpu["probability"], cpu["probability"], rtol=PROBABILITY_RTOL[dtype], atol=0,
                               err_msg=context + " probability mismatch")


def parity_counters(gpu, cpu):
    """The counters reported beside a parity run."""
    ok = cpu["status"] == 0
    return {
        "rows": int(gpu.shape[0]),
        "token_mismatches": int(np.count_nonzero(gpu["token_id"] != cpu["token_id"])),
        "probability_bit_mismatches": int(np.count_nonzero(
            gpu["probability"].view(np.uint32) != cpu["probability"].view(np.uint32))),
        "draws_within_1e-6_of_cdf_boundary": int(np.count_nonzero(ok & (cpu["cdf_gap"] < 1e-6))),
        "top_p_cumulative_within_1e-6": int(np.count_nonzero(ok & (cpu["top_p_gap"] < 1e-6))),
    }


def run_workload_on_gpu(workload, sampler=None, force_general=False):
    own = sampler is None
    if own:
        sampler = hip_sampler.HipSampler(workload["rows"], workload["vocab"], testing=force_general)
    try:
        sampler.force_general(force_general)
        sampler.upload_logits(workload["logits"])
        return sampler.sample(workload["params"], workload["uniforms"], workload["stop_ids"])
    finally:
        sampler.force_general(False)
        if own:
            sampler.close()
