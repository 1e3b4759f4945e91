"""Seeded random batches through the C ABI against the CPU oracle: random shapes (row counts on both
sides of every geometry switch, vocabularies that are not multiples of anything), dtypes, row kinds
(ties, -inf tails, spikes, sorted rows, NaN) and per-row options (every window size class, greedy,
Min-P, Top-P).  Token ids, statuses, kept counts and flags bit-exact."""
import numpy as np
import pytest

import parity_util
from ncnn_moe_runtime_amd import hip_sampler, workloads

pytestmark = pytest.mark.gpu

MAX_ROWS, MAX_VOCAB = 300, 70000


@pytest.fixture(scope="module")
def sampler():
    handle = hip_sampler.HipSampler(MAX_ROWS, MAX_VOCAB, testing=True)
    yield handle
    handle.close()


def _random_row(rng, vocab):
    kind = int(rng.integers(0, 9))
    row = (rng.standard_normal(vocab) * rng.uniform(0.2, 6.0)).astype(np.float32)
    if kind == 1:
        row = np.round(row * 2) / 2
    elif kind == 2:
        row[rng.integers(0, vocab, max(1, vocab // 7))] = -np.inf
    elif kind == 3:
        row[rng.integers(0, vocab, 4)] += np.float32(20.0)
    elif kind == 4:
        row = np.sort(row)[::-1] if rng.random() < 0.5 else np.sort(row)
    elif kind == 5:
        row[rng.integers(0, vocab, 3)] = np.nan
    elif kind == 6:
        row[:] = np.float32(rng.standard_normal())
    elif kind == 7:
        row[int(rng.integers(0, vocab)):] = -np.inf
    return np.ascontiguousarray(row, dtype=np.float32)


@pytest.mark.parametrize("seed", range(24))
def test_random_batches(sampler, seed):
    rng = np.random.default_rng(9000 + seed)
    rows = int(rng.choice([1, 2, 7, 31, 64, 65, 100, 129, 255, 256, 257, 300]))
    vocab = int(rng.choice([1, 5, 63, 64, 65, 513, 4099, 10240, 10241, 20481, 33333, 69999]))
    bf16 = bool(rng.random() < 0.4)
    print("[case] fuzz seed %d: %d x %d %s" % (seed, rows, vocab, "bf16" if bf16 else "f32"), flush=True)
    logits = np.stack([_random_row(rng, vocab) for _ in range(rows)])
    params = hip_sampler.make_params(rows)
    params["temperature"] = rng.choice(np.array([0.0, 0.05, 0.5, 0.8, 1.0, 1.7, 5.0], dtype=np.float32), size=rows)
    params["top_k"] = rng.choice(np.array([0, 1, 2, 19, 63, 64, 65, 200, 511, 512, 513, 1024, 1025, 5000], dtype=np.uint32), size=rows)
    params["top_p"] = rng.choice(np.array([1.0, 0.999, 0.95, 0.8, 0.3, 0.01], dtype=np.float32), size=rows)
    params["min_p"] = rng.choice(np.array([0.0, 0.0, 0.01, 0.1, 0.7, 1.0], dtype=np.float32), size=rows)
    stop_ids = rng.integers(0, vocab, size=rows * 2).astype(np.int32)
    params["stop_begin"] = np.arange(rows, dtype=np.uint32) * 2
    params["stop_count"] = rng.integers(0, 3, size=rows).astype(np.uint32)
    uniforms = rng.random(rows).astype(np.float32)
    if bf16:
        logits = workloads.float32_to_bf16_bits(logits)
    sampler.upload_logits(logits)
    # every other seed without the XCD-aware numbering of the workgroups: the segments of a row then run
    # on several XCDs and the merge reads their records around the L2
    sampler.scatter_segments(seed % 2 == 1)
    try:
        gpu = sampler.sample(params, uniforms, stop_ids)
    finally:
        sampler.scatter_segments(False)
    cpu = parity_util.run_oracle(logits, params, uniforms, stop_ids)
    parity_util.assert_results_match(gpu, cpu, "bf16" if bf16 else "f32", "fuzz seed %d" % seed)
