"""GPU parity of the wide select where it takes its bound from a sample of the row: Top-K windows wider than 512
over rows of four chunks or more (a chunk: 10,240 fp32 or 12,288 bf16 logits).  The sample is one chunk's worth
of 16-byte vectors in runs of four, the runs spaced evenly over the row; a row whose list ends short of the window
under that bound is handed to the full-order kernels.  Results are the oracle's either way, bit for bit."""
import numpy as np
import pytest

import oracle_lib
import parity_util
from ncnn_moe_runtime_amd import hip_sampler, workloads

pytestmark = pytest.mark.gpu

VOCAB_F32 = 129280
VOCAB_BF16 = 201088


def _announce(text):
    print("[case] " + text, flush=True)


@pytest.fixture(scope="module")
def sampler():
    handle = hip_sampler.HipSampler(64, VOCAB_BF16 + 8, testing=True)
    yield handle
    handle.close()


def _sampled_positions(vocab, dtype):
    """Elements of an aligned row that the kernel's sample reads."""
    width, vectors_per_lane = (4, 5) if dtype == "f32" else (8, 3)
    vectors = 512 * vectors_per_lane
    runs = vectors // 4
    spacing = (vocab // width) // runs
    g = np.arange(vectors)
    vector = (g // 4) * spacing + g % 4
    return (vector[:, None] * width + np.arange(width)[None, :]).reshape(-1)


def _both_ways(sampler, logits, params, uniforms, dtype, context, vocab=None):
    """Parity with the oracle with the sampled bound and without it; returns the results with it."""
    results = {}
    cpu = parity_util.run_oracle(logits, params, uniforms, None, vocab=vocab)
    for sampled in (True, False):
        _announce("%s, %s, bound from %s" % (context, dtype, "a sample" if sampled else "the first chunk"))
        sampler.wide_sampled_bound(sampled)
        try:
            sampler.upload_logits(logits, vocab=vocab)
            results[sampled] = sampler.sample(params, uniforms)
        finally:
            sampler.wide_sampled_bound(True)
        parity_util.assert_results_match(results[sampled], cpu, dtype, context)
    return results[True], results[False]


def _rows_of_many_shapes(rng, rows, vocab):
    """Rows whose large values lie where a bound from one place of the row would go wrong."""
    logits = (rng.standard_normal((rows, vocab)) * 2.5).astype(np.float32)
    for row in range(rows):
        shape = row % 8
        if shape == 1:
            logits[row] = -np.sort(-logits[row])                      # descending: the window is the row's head
        elif shape == 2:
            logits[row] = np.sort(logits[row])                        # ascending: the window is the row's tail
        elif shape == 3:
            logits[row, :9000] += 9.0                                 # the first chunk holds nearly all of the window
        elif shape == 4:
            logits[row, -7000:] += 9.0                                # the last chunk does
        elif shape == 5:
            logits[row] = np.round(logits[row] * 4.0) / 4.0           # a few dozen distinct values: ties everywhere
        elif shape == 6:
            logits[row] += np.linspace(-6.0, 6.0, vocab, dtype=np.float32)   # a trend along the row
        elif shape == 7:
            logits[row] += (4.0 * np.sin(np.arange(vocab) * (2.0 * np.pi / 50.0))).astype(np.float32)  # a period near the runs' spacing
    return logits


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_rows_of_many_shapes(sampler, dtype):
    rng = np.random.default_rng(20251 + len(dtype))
    rows = 48
    vocab = VOCAB_F32 if dtype == "f32" else VOCAB_BF16
    logits = _rows_of_many_shapes(rng, rows, vocab)
    data = workloads.float32_to_bf16_bits(logits) if dtype == "bf16" else logits
    params = hip_sampler.make_params(rows, 0.9, 1000, 0.98, 0.0)
    params["top_k"] = np.array([(513, 700, 1000, 1024, 900)[i % 5] for i in range(rows)], dtype=np.uint32)
    params["temperature"][::3] = 1.4
    params["top_p"][::4] = 1.0
    uniforms = rng.random(rows, dtype=np.float32)
    with_sample, without = _both_ways(sampler, data, params, uniforms, dtype, "rows of many shapes")
    assert with_sample["token_id"].tobytes() == without["token_id"].tobytes()
    # Under the sampled bound the select serves every row itself but those with ties everywhere and those whose values
    # follow the runs' spacing.  (Under the first chunk's bound it hands on the rows whose values grow along the row:
    # every chunk then pours a good part of its values into the list.)
    untied = np.array([row % 8 not in (5, 7) for row in range(rows)])
    if dtype == "f32":
        assert ((with_sample["flags"][untied] & hip_sampler.FLAG_GENERAL_PATH) == 0).all()
        ascending = np.array([row % 8 == 2 for row in range(rows)])
        assert ((without["flags"][ascending] & hip_sampler.FLAG_GENERAL_PATH) != 0).all()


def test_row_lengths_and_misaligned_rows(sampler):
    """Row lengths around four chunks (where the sample starts to be used) and rows that start off a 16-byte
    boundary (a stride that is no multiple of four)."""
    rng = np.random.default_rng(977)
    rows = 12
    for vocab in (40959, 40960, 40961, 40963, 51200, 129277, 129283):
        stride = vocab + 3
        logits = np.full((rows, stride), 60.0, dtype=np.float32)     # what lies beyond a row would win every window
        logits[:, :vocab] = (rng.standard_normal((rows, vocab)) * 3.0).astype(np.float32)
        params = hip_sampler.make_params(rows, 1.1, 1000, 1.0, 0.0)
        params["top_k"][1::2] = 640
        uniforms = rng.random(rows, dtype=np.float32)
        _both_ways(sampler, logits, params, uniforms, "f32", "vocab %d, stride %d" % (vocab, stride), vocab=vocab)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_masked_rows(sampler, dtype):
    """Rows that are -inf but for a few elements: fewer finite logits than the window is wide (the window is all
    of them), as many, a few more, and several times as many; the finite ones at the row's end, its start, or spread."""
    rng = np.random.default_rng(5150)
    vocab = VOCAB_F32 if dtype == "f32" else VOCAB_BF16
    finite_counts = [1, 300, 999, 1000, 1001, 1100, 2500, 20000]
    rows = 3 * len(finite_counts)
    logits = np.full((rows, vocab), -np.inf, dtype=np.float32)
    for row in range(rows):
        count = finite_counts[row // 3]
        where = (np.arange(vocab - count, vocab), np.arange(count), rng.choice(vocab, size=count, replace=False))[row % 3]
        logits[row, where] = (rng.standard_normal(count) * 2.0).astype(np.float32)
    data = workloads.float32_to_bf16_bits(logits) if dtype == "bf16" else logits
    params = hip_sampler.make_params(rows, 1.0, 1000, 1.0, 0.0)
    uniforms = (0.05 + 0.9 * rng.random(rows)).astype(np.float32)
    _both_ways(sampler, data, params, uniforms, dtype, "masked rows")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_a_sample_that_misleads(sampler, dtype):
    """Large values exactly where the sample looks and nowhere else: the sample's bound is reached by a few hundred
    values of the row, fewer than the window holds, and the full-order kernels take the row (the flag says so);
    from the first chunk's bound the select serves it itself.  Same tokens and counts."""
    rng = np.random.default_rng(1812)
    rows = 6
    vocab = VOCAB_F32 if dtype == "f32" else VOCAB_BF16
    logits = rng.standard_normal((rows, vocab)).astype(np.float32)
    positions = _sampled_positions(vocab, dtype)
    assert positions.max() < vocab and np.unique(positions).size == positions.size
    misled = np.array([True, True, False, True, False, True])
    for row in np.nonzero(misled)[0]:
        logits[row, positions] += 12.0
    data = workloads.float32_to_bf16_bits(logits) if dtype == "bf16" else logits
    params = hip_sampler.make_params(rows, 8.0, 1000, 1.0, 0.0)    # a flat distribution: draws land all over the window
    uniforms = np.array([0.11, 0.93, 0.5, 0.62, 0.97, 0.31], dtype=np.float32)
    with_sample, without = _both_ways(sampler, data, params, uniforms, dtype, "a sample that misleads")
    assert (with_sample["kept_count"] == 1000).all()
    assert np.array_equal((with_sample["flags"] & hip_sampler.FLAG_GENERAL_PATH) != 0, misled)
    assert ((without["flags"] & hip_sampler.FLAG_GENERAL_PATH) == 0).all()


def test_distribution_under_a_sampled_bound(sampler):
    """The exported distribution of windows of a thousand over a long row: ids and probabilities bit for bit."""
    rng = np.random.default_rng(31)
    logits = (rng.standard_normal((3, VOCAB_F32)) * 2.0).astype(np.float32)
    sampler.upload_logits(logits)
    for row, options in enumerate([dict(temperature=1.0, top_k=1000, top_p=1.0, min_p=0.0),
                                   dict(temperature=1.2, top_k=1024, top_p=0.99, min_p=0.0),
                                   dict(temperature=0.8, top_k=513, top_p=0.9, min_p=0.0005)]):
        _announce("distribution under a sampled bound, row %d" % row)
        status, ids, probabilities, count = sampler.distribution(row, **options)
        oracle_status, oracle_ids, oracle_probabilities = oracle_lib.oracle_distribution(logits[row], **options)
        assert status == oracle_status
        assert count == len(oracle_ids) and count > 64
        assert np.array_equal(ids[:count], oracle_ids)
        assert np.array_equal(probabilities[:count].view(np.uint32),
                              np.asarray(oracle_probabilities, dtype=np.float32).view(np.uint32))


def test_random_rows_under_a_sampled_bound(sampler):
    """Thirty random batches (row length, type, spread, quantisation, masked parts, infinities, NaN, sorted rows, options
    and windows drawn at random; windows from 400, below where the sample is used, to 1100, beyond the wide select):
    against the oracle under both bounds, and the two results byte for byte."""
    rng = np.random.default_rng(6006)
    for case in range(30):
        dtype = "bf16" if case % 3 == 2 else "f32"
        rows = int(rng.integers(1, 13))
        vocab = int(rng.integers(30000, VOCAB_BF16))
        spread = float(rng.choice([0.05, 0.5, 2.0, 6.0]))
        logits = (rng.standard_normal((rows, vocab)) * spread + float(rng.choice([0.0, -30.0, 100.0]))).astype(np.float32)
        kind = case % 6
        if kind == 1:
            logits = np.round(logits * 8) / 8                              # few distinct values
        elif kind == 2:
            logits[:, rng.integers(0, vocab, vocab // 3)] = -np.inf
            logits[0, rng.integers(0, vocab, 3)] = np.nan
        elif kind == 3:
            logits[:, vocab // 2:] = logits[:, :1]                         # half of every row one value
        elif kind == 4:
            logits = np.sort(logits, axis=1)                               # the window at the row's end
            logits[rows // 2:] = logits[rows // 2:, ::-1]                  # ... or at its start
        elif kind == 5:
            logits[:, :int(rng.integers(1, vocab))] = -np.inf              # a masked head of any length
            logits[-1, rng.integers(0, vocab)] = np.inf
        data = workloads.float32_to_bf16_bits(logits) if dtype == "bf16" else logits
        params = hip_sampler.make_params(rows, 1.0, 0, 1.0, 0.0)
        params["temperature"] = rng.choice(np.array([0.1, 0.5, 0.9, 1.3, 2.0], dtype=np.float32), size=rows)
        params["top_p"] = rng.choice(np.array([0.3, 0.9, 0.99, 1.0], dtype=np.float32), size=rows)
        params["min_p"] = rng.choice(np.array([0.0, 0.0, 0.01], dtype=np.float32), size=rows)
        params["top_k"] = rng.choice(np.array([400, 513, 600, 777, 1000, 1024, 1100], dtype=np.uint32), size=rows)
        uniforms = rng.random(rows, dtype=np.float32)
        context = "random case %d: %d x %d, spread %.2f, kind %d" % (case, rows, vocab, spread, kind)
        with_sample, without = _both_ways(sampler, data, params, uniforms, dtype, context)
        # (the flags differ where one bound lets the select serve a row that the other hands on)
        for field in ("token_id", "probability", "kept_count", "status", "is_stop", "draw_consumed"):
            assert with_sample[field].tobytes() == without[field].tobytes(), "%s: %s" % (context, field)
