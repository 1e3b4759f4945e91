"""Rows split over several workgroups (batches of fewer than 256 rows), through the C ABI against the CPU
oracle: both split kernels (one chunk per workgroup with the epoch-tagged records; several chunks per
workgroup), the shapes at which two or three segments of several rows share cache lines of the hand-over
words, with the XCD-aware numbering of the workgroups and without it, and many launches in a row on one
handle (the per-row epochs move on, nothing is cleared in between)."""
import numpy as np
import pytest

import parity_util
from ncnn_moe_runtime_amd import hip_sampler, workloads

pytestmark = pytest.mark.gpu


def _batch(seed, rows, vocab, window=64):
    rng = np.random.default_rng(seed)
    logits = (rng.standard_normal((rows, vocab)) * 2.5).astype(np.float32)
    logits[1::7] = np.round(logits[1::7] * 4) / 4            # ties at the cut
    logits[2::11, : vocab // 3] = -np.inf                     # a third of the row carries nothing
    logits[3::13, rng.integers(0, vocab, 5)] += np.float32(15.0)
    params = hip_sampler.make_params(rows, 0.8, 0, 0.9, 0.0)
    params["top_k"] = rng.choice(np.array([1, 2, 20, 33, 50, window], dtype=np.uint32), size=rows)
    params["temperature"] = rng.choice(np.array([0.0, 0.6, 1.0, 1.4], dtype=np.float32), size=rows)
    params["top_p"] = rng.choice(np.array([1.0, 0.95, 0.8, 0.4], dtype=np.float32), size=rows)
    params["min_p"] = rng.choice(np.array([0.0, 0.0, 0.02], dtype=np.float32), size=rows)
    uniforms = rng.random(rows).astype(np.float32)
    return logits, params, uniforms


def _check(sampler, logits, params, uniforms, context, dtype="f32", scattered=False, must_select=None):
    print("[case] " + context, flush=True)
    sampler.scatter_segments(scattered)
    try:
        sampler.upload_logits(logits)
        gpu = sampler.sample(params, uniforms)
    finally:
        sampler.scatter_segments(False)
    cpu = parity_util.run_oracle(logits, params, uniforms)
    parity_util.assert_results_match(gpu, cpu, dtype, context)
    if must_select is not None:
        sorted_rows = np.nonzero(must_select & ((gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH) != 0))[0]
        assert sorted_rows.size == 0, "%s: rows %s took the full-order path" % (context, sorted_rows[:8])
    return gpu


@pytest.fixture(scope="module")
def long_sampler():
    sampler = hip_sampler.HipSampler(255, 262144, testing=True)
    yield sampler
    sampler.close()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("vocab", [163841, 201088, 262144])
@pytest.mark.parametrize("rows", [1, 8, 64, 130, 255])
def test_rows_of_seventeen_to_thirty_two_one_chunk_workgroups(long_sampler, rows, vocab, dtype):
    """Rows longer than 16 chunks in batches below 256 rows (fp32 from 163,841 logits on, bf16 from 196,609):
    the one-chunk kernel in its shape for up to 32 segments, whose merge reads a segment's record with 16 lanes."""
    code = hip_sampler.LOGITS_F32 if dtype == "f32" else hip_sampler.LOGITS_BF16
    segments, chunks, variant = hip_sampler.select_geometry(code, rows, vocab)
    if dtype == "bf16" and vocab <= 196608:
        assert variant == hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK and segments <= 16
        pytest.skip("a bf16 row of %d logits is 16 chunks or fewer" % vocab)
    if dtype == "bf16" and rows * ((vocab + 12287) // 12288) > 2304:
        # (large batches of long bf16 rows keep the looped kernel, which is as fast there)
        assert variant == hip_sampler.GEOMETRY_SPLIT_LOOPED and segments > 1 and chunks > 1
    else:
        assert variant == hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK and 16 < segments <= 32 and chunks == 1
    logits, params, uniforms = _batch(rows * 1000 + vocab, rows, vocab)
    data = workloads.float32_to_bf16_bits(logits) if dtype == "bf16" else logits
    plain = np.ones(rows, dtype=bool)
    plain[1::7] = False  # heavy ties may overflow the lists and take the full-order kernels
    plain[2::11] = False  # ... and so may a row whose first third is -inf (a segment that starts without a bound)
    for repeat in range(2):  # the same handle again: stale records and counts of the launch before are in place
        _check(long_sampler, data, params, uniforms, "%d segments, %d x %d %s, launch %d" % (segments, rows, vocab, dtype, repeat),
               dtype=dtype, scattered=repeat == 1 and rows == 64, must_select=plain)


@pytest.fixture(scope="module")
def longest_sampler():
    sampler = hip_sampler.HipSampler(130, 340000, testing=True)
    yield sampler
    sampler.close()


@pytest.mark.parametrize("rows", [8, 64, 130])
def test_fp32_workgroups_that_stream_several_chunks(longest_sampler, rows):
    """fp32 rows longer than 32 chunks in batches below 256 rows: several workgroups per row, several
    chunks per workgroup, hand-over through the segments' records."""
    vocab = 340000
    segments, chunks, variant = hip_sampler.select_geometry(hip_sampler.LOGITS_F32, rows, vocab)
    assert variant == hip_sampler.GEOMETRY_SPLIT_LOOPED and segments > 1 and chunks > 1
    logits, params, uniforms = _batch(rows * 1000 + vocab, rows, vocab)
    plain = np.ones(rows, dtype=bool)
    plain[1::7] = False  # heavy ties may overflow the lists and take the full-order kernels
    plain[2::11] = False  # ... and so may a row whose first third is -inf (a segment that starts without a bound)
    _check(longest_sampler, logits, params, uniforms, "looped split, %d x %d fp32 (%d segments x %d chunks)" % (rows, vocab, segments, chunks),
           must_select=plain)


@pytest.mark.parametrize("scattered", [False, True])
@pytest.mark.parametrize("vocab", [10241, 20481, 30000])
@pytest.mark.parametrize("rows", [129, 200, 255])
def test_two_or_three_segments_per_row(long_sampler, rows, vocab, scattered):
    """Two or three segments per row in batches of 129 to 255 rows: the hand-over words of rows eight
    apart (which run on one XCD) lie in one cache line."""
    segments, chunks, variant = hip_sampler.select_geometry(hip_sampler.LOGITS_F32, rows, vocab)
    assert variant == hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK and segments in (2, 3) and chunks == 1
    logits, params, uniforms = _batch(rows * 77 + vocab, rows, vocab)
    plain = np.ones(rows, dtype=bool)
    plain[1::7] = False
    for repeat in range(3):  # the same handle again: stale records and counts of the launch before are in place
        _check(long_sampler, logits, params, uniforms,
               "%d segments, %d x %d fp32%s, launch %d" % (segments, rows, vocab, ", scattered" if scattered else "", repeat),
               scattered=scattered, must_select=plain)


def test_many_launches_on_one_handle():
    """300 launches of the one-chunk split kernel on one handle, shapes and data changing: the epochs of
    the rows move on independently (a row that is not in a launch keeps its epoch), records are never
    cleared, and every launch must match the oracle."""
    rng = np.random.default_rng(5150)
    with hip_sampler.HipSampler(96, 60000, testing=True) as sampler:
        for launch in range(300):
            rows = int(rng.choice([1, 3, 17, 64, 96]))
            vocab = int(rng.choice([10241, 25000, 41000, 60000]))
            dtype = "bf16" if launch % 5 == 4 else "f32"
            logits, params, uniforms = _batch(launch, rows, vocab)
            data = workloads.float32_to_bf16_bits(logits) if dtype == "bf16" else logits
            sampler.scatter_segments(launch % 7 == 3)
            sampler.upload_logits(data)
            gpu = sampler.sample(params, uniforms)
            if launch % 10 == 0 or launch < 20:
                print("[case] launch %d: %d x %d %s" % (launch, rows, vocab, dtype), flush=True)
                cpu = parity_util.run_oracle(data, params, uniforms)
                parity_util.assert_results_match(gpu, cpu, dtype, "launch %d" % launch)
        sampler.scatter_segments(False)


def test_launch_numbers_start_over():
    """The per-row launch numbers (epochs) that tag the hand-over records run 1 .. 8191 and start over; a
    serving loop gets there within minutes.  A handle that has records of its first launches in place is
    set three launches in front of that point and runs eight launches of changing shape, data and window
    across it: the launch at the last number clears the rows' records, so that what the first launches
    tagged 1, 2, 3 cannot pass for an entry of the launches that get those numbers again."""
    rng = np.random.default_rng(909)
    shapes = [(64, 41000), (17, 60000), (96, 25000), (64, 41000), (3, 60000), (96, 10241), (64, 25000), (17, 41000)]
    with hip_sampler.HipSampler(96, 60000, testing=True) as sampler:
        for launch in range(4):  # numbers 1 .. 4: wide windows, so that the records are long
            logits, params, uniforms = _batch(7000 + launch, 96, 60000)
            params["top_k"] = 64
            _check(sampler, logits, params, uniforms, "launch number %d, 96 x 60000" % (launch + 1))
        sampler.set_row_epochs(hip_sampler.LAST_EPOCH - 2)
        for launch, (rows, vocab) in enumerate(shapes):
            logits, params, uniforms = _batch(7100 + launch, rows, vocab)
            params["top_k"] = rng.choice(np.array([1, 5, 20, 64], dtype=np.uint32), size=rows)
            _check(sampler, logits, params, uniforms, "launch %d across the restart, %d x %d" % (launch, rows, vocab),
                   scattered=launch % 3 == 2)
