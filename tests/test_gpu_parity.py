"""GPU parity: the HIP sampler, called through its C ABI, against the CPU oracle on identical seeded
inputs.  Token ids, statuses, kept counts and flags must match bit for bit."""
import numpy as np
import pytest

import oracle_lib
import parity_util
from ncnn_moe_runtime_amd import hip_sampler, workloads

pytestmark = pytest.mark.gpu


def _announce(text):
    print("[case] " + text, flush=True)


@pytest.fixture(scope="module")
def small_sampler():
    sampler = hip_sampler.HipSampler(64, 40000, testing=True)
    yield sampler
    sampler.close()


def _check_rows(sampler, logits, params, uniforms, stop_ids=None, dtype="f32", context="", general=False, vocab=None,
                select_rows=None):
    """select_rows: rows that the select kernels must serve themselves (no sort)."""
    _announce(context + (" [general]" if general else ""))
    sampler.force_general(general)
    try:
        sampler.upload_logits(logits, vocab=vocab)
        gpu = sampler.sample(params, uniforms, stop_ids)
    finally:
        sampler.force_general(False)
    cpu = parity_util.run_oracle(logits, params, uniforms, stop_ids, vocab=vocab)
    parity_util.assert_results_match(gpu, cpu, dtype, context)
    if select_rows is not None:
        sorted_rows = np.nonzero(select_rows & ((gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH) != 0))[0]
        assert sorted_rows.size == 0, "%s: rows %s took the full-order path" % (context, sorted_rows[:8])
    return gpu, cpu


def test_device_expf_matches_libm(small_sampler):
    _announce("device expf vs libm expf")
    # every 53rd float in [-110, -0.0], every 997th positive float up to 90, and special values
    negative = np.arange(0x80000000, 0xC2DC0000, 53, dtype=np.uint64).astype(np.uint32).view(np.float32)
    positive = np.arange(0, 0x42B40000, 997, dtype=np.uint64).astype(np.uint32).view(np.float32)
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, -88.0, -87.5, -103.0, -103.9, -104.0, -150.0,
                        88.7, 88.8, 1e-30, -1e-30], dtype=np.float32)
    values = np.concatenate([negative, positive, special])
    device = small_sampler.expf(values)
    host = oracle_lib.expf_libm(values)
    both_nan = np.isnan(device) & np.isnan(host)
    mismatch = (device.view(np.uint32) != host.view(np.uint32)) & ~both_nan
    assert not mismatch.any(), "first mismatch at x=%r" % values[np.nonzero(mismatch)[0][:4]]


# logf of {0.4, 0.3, 0.2, 0.1} in fp32, as bit patterns (the inputs of the recorded reference answers)
LN_4321 = np.array([3211432455, 3214547912, 3217949200, 3222494606], dtype=np.uint32).view(np.float32).tolist()

KNOWN = [
    # logits, options, expected kept ids, expected probabilities (recorded from the reference)
    (LN_4321, dict(min_p=0.45, top_p=0.75), [0, 1, 2], [0.444444478, 0.333333313, 0.222222209]),
    (LN_4321, dict(min_p=0.5, top_p=0.75), [0, 1], [0.571428597, 0.428571403]),
    (LN_4321, dict(top_p=0.5), [0, 1], [0.571428597, 0.428571403]),
    ([1, 2, 3], dict(top_k=7), [2, 1, 0], [0.665240943, 0.244728476, 0.0900305733]),
    ([1, 2, 3, 4, 5], dict(temperature=0.5, top_k=3, top_p=0.9, min_p=0.05), [4, 3], [0.880797088, 0.119202919]),
    ([2, 2, 1], dict(min_p=1.0), [0, 1], [0.5, 0.5]),
    ([5, 7, 7, 7], dict(top_k=2), [1, 2], [0.5, 0.5]),
    ([1, 1], dict(top_p=0.5), [0], [1.0]),
    ([3, -np.inf, -np.inf], dict(top_k=2), [0], [1.0]),
]


@pytest.mark.parametrize("general", [False, True])
def test_known_answers_distribution(small_sampler, general):
    small_sampler.force_general(general)
    try:
        for logits, options, ids, probabilities in KNOWN:
            _announce("known answer %s %s general=%s" % (logits, options, general))
            row = np.array([logits], dtype=np.float32)
            small_sampler.upload_logits(row)
            status, got_ids, got_probabilities, count = small_sampler.distribution(0, **options)
            assert status == 0
            assert count == len(ids)
            assert got_ids.tolist() == ids
            np.testing.assert_allclose(got_probabilities, np.array(probabilities, dtype=np.float32), rtol=2e-7)
            oracle_status, oracle_ids, oracle_probabilities = oracle_lib.oracle_distribution(row[0], **options)
            assert oracle_status == 0 and oracle_ids.tolist() == ids
            assert np.array_equal(got_probabilities.view(np.uint32), oracle_probabilities.view(np.uint32))
    finally:
        small_sampler.force_general(False)


@pytest.mark.parametrize("general", [False, True])
def test_reference_test_vectors_and_errors(small_sampler, general):
    """The reference's own sampler checks (tests/test_runtime.cpp:4332-4362) and its error cases."""
    nan, inf = np.nan, np.inf
    cases = [
        ([1, 2, 3], dict(temperature=0.0), 0, 2, 1.0),
        ([3, nan, 3], dict(temperature=0.0), 0, 0, 1.0),
        ([nan, inf], dict(temperature=0.0), hip_sampler.ROW_NO_FINITE_LOGIT, -1, 0.0),
        ([1, 2, 3], dict(top_k=1), 0, 2, 1.0),
        ([1, 2, 3], dict(top_p=0.0), hip_sampler.ROW_BAD_TOP_P, -1, 0.0),
        ([1, 2, 3], dict(top_p=1.5), hip_sampler.ROW_BAD_TOP_P, -1, 0.0),
        ([1, 2, 3], dict(temperature=-1.0), hip_sampler.ROW_BAD_TEMPERATURE, -1, 0.0),
        ([1, 2, 3], dict(temperature=inf), hip_sampler.ROW_BAD_TEMPERATURE, -1, 0.0),
        ([1, 2, 3], dict(temperature=nan), hip_sampler.ROW_BAD_TEMPERATURE, -1, 0.0),
        ([1, 2, 3], dict(min_p=-0.1), hip_sampler.ROW_BAD_MIN_P, -1, 0.0),
        ([1, 2, 3], dict(min_p=1.1), hip_sampler.ROW_BAD_MIN_P, -1, 0.0),
        ([0.0, -0.0], dict(top_k=1), 0, 0, 1.0),
        ([-0.0, 0.0], dict(top_k=1), 0, 0, 1.0),
        ([-inf, -inf], dict(temperature=0.0), hip_sampler.ROW_NO_FINITE_LOGIT, -1, 0.0),
        ([-inf, -inf], dict(temperature=1.0), hip_sampler.ROW_NO_FINITE_LOGIT, -1, 0.0),
        ([1, inf, 2], dict(temperature=0.7, top_k=20, top_p=0.8), hip_sampler.ROW_NO_FINITE_LOGIT, -1, 0.0),
        ([1, inf, 2], dict(temperature=0.0), 0, 2, 1.0),
        ([1, 2], dict(temperature=1e-39), hip_sampler.ROW_INVALID_DISTRIBUTION, -1, 0.0),
        ([1, 2], dict(temperature=1e-30), 0, 1, 1.0),
        ([1, 3, 2], dict(temperature=-0.0), 0, 1, 1.0),
    ]
    small_sampler.force_general(general)
    try:
        for logits, options, status, token, probability in cases:
            _announce("reference vector %s %s general=%s" % (logits, options, general))
            row = np.array([logits], dtype=np.float32)
            params = hip_sampler.make_params(1, **options)
            small_sampler.upload_logits(row)
            got = small_sampler.sample(params, np.array([0.25], dtype=np.float32))[0]
            assert got["status"] == status, (logits, options, got)
            assert got["token_id"] == token, (logits, options, got)
            assert got["probability"] == np.float32(probability)
            cpu = oracle_lib.oracle_sample(row[0], 0.25, **options)
            assert cpu["status"] == status and cpu["token_id"] == token
            if status != 0:
                assert hip_sampler.status_message(status) == oracle_lib.STATUS_MESSAGES[status]
    finally:
        small_sampler.force_general(False)


def test_empty_logits(small_sampler):
    _announce("empty logits")
    small_sampler.upload_logits(np.zeros((2, 0), dtype=np.float32))
    got = small_sampler.sample(hip_sampler.make_params(2), np.zeros(2, dtype=np.float32))
    assert (got["status"] == hip_sampler.ROW_EMPTY_LOGITS).all() and (got["token_id"] == -1).all()
    assert hip_sampler.status_message(hip_sampler.ROW_EMPTY_LOGITS) == "cannot sample empty logits"


def test_rng_lockstep_draws(small_sampler):
    """{0,5,5,-1}, Top-K 2, uniforms from mt19937_64(1234): token = u < 0.5 ? 1 : 2 (reference probe)."""
    _announce("rng lock-step")
    rng = oracle_lib.OracleRng(1234)
    uniforms = np.array([rng.uniform() for _ in range(64)], dtype=np.float32)
    logits = np.tile(np.array([0, 5, 5, -1], dtype=np.float32), (64, 1))
    small_sampler.upload_logits(logits)
    got = small_sampler.sample(hip_sampler.make_params(64, top_k=2), uniforms)
    assert np.array_equal(got["token_id"], np.where(uniforms < 0.5, 1, 2))
    assert (got["probability"] == 0.5).all() and (got["draw_consumed"] == 1).all() and (got["kept_count"] == 2).all()


@pytest.mark.parametrize("general", [False, True])
def test_cfg1_plumbing(small_sampler, general):
    w = workloads.make_workload("cfg1_plumbing", rows=8)
    greedy = w["params"].copy()
    greedy["temperature"] = 0.0
    select_rows = None if general else np.ones(8, dtype=bool)
    _check_rows(small_sampler, w["logits"], greedy, w["uniforms"], context="cfg1 greedy", general=general,
                select_rows=select_rows)
    _check_rows(small_sampler, w["logits"], w["params"], w["uniforms"], context="cfg1 T.8 K50 P.9", general=general,
                select_rows=select_rows)
    if not general:
        _check_rows(small_sampler, w["logits"][:1], w["params"][:1], w["uniforms"][:1], context="cfg1, one row",
                    select_rows=select_rows[:1])
    status, ids, probabilities, count = small_sampler.distribution(0, 0.8, 50, 0.9, 0.0)
    oracle_status, oracle_ids, oracle_probabilities = oracle_lib.oracle_distribution(w["logits"][0], 0.8, 50, 0.9, 0.0)
    assert status == oracle_status == 0 and count == oracle_ids.size
    assert np.array_equal(ids, oracle_ids)
    np.testing.assert_allclose(probabilities, oracle_probabilities, rtol=1e-5)


def test_uniform_sweep_hits_every_cdf_boundary(small_sampler):
    """One row, 64 uniforms spread over [0, 1): the draw must agree with the oracle everywhere."""
    w = workloads.make_workload("cfg1_plumbing", rows=1, seed=5)
    logits = np.tile(w["logits"], (64, 1))
    uniforms = ((np.arange(64, dtype=np.float32) + 0.5) / 64).astype(np.float32)
    uniforms[-1] = np.float32(1.0) - np.float32(2.0 ** -24)
    uniforms[0] = 0.0
    _check_rows(small_sampler, logits, hip_sampler.make_params(64, 0.8, 50, 0.9), uniforms, context="uniform sweep")


def test_edge_rows(small_sampler):
    """Ties across the Top-K boundary, NaN / inf rows, one-token vocabularies, misaligned strides."""
    rng = np.random.default_rng(11)
    vocab = 12345
    rows = 16
    logits = rng.standard_normal((rows, vocab)).astype(np.float32)
    logits[0, :] = 1.0                       # every logit tied
    logits[1, ::3] = 2.5                     # a third of the row tied at the top
    logits[2, 100:200] = np.nan
    logits[3, 5] = np.nan
    logits[3, 0] = 9.0
    logits[4, :] = -np.inf
    logits[4, 777] = -3.0
    logits[5, :] = np.nan
    logits[6, 10] = np.inf
    logits[7, :] = np.round(logits[7, :] * 2) / 2   # heavy ties
    logits[8, :] = -0.0
    logits[8, ::2] = 0.0
    logits[9, 4000:] = -np.inf
    params = hip_sampler.make_params(rows, 0.9, 20, 0.95, 0.0)
    params["top_k"][10] = 1
    params["top_k"][11] = 64
    params["top_k"][12] = 0
    params["top_k"][13] = 65
    params["temperature"][14] = 0.0
    params["min_p"][15] = 0.3
    uniforms = rng.random(rows).astype(np.float32)
    _check_rows(small_sampler, logits, params, uniforms, context="edge rows")
    greedy = params.copy()
    greedy["temperature"] = 0.0
    _check_rows(small_sampler, logits, greedy, uniforms, context="edge rows greedy")
    # stride wider than the vocabulary and not a multiple of four: rows start misaligned
    wide = np.full((rows, vocab + 3), 50.0, dtype=np.float32)
    wide[:, :vocab] = logits
    _check_rows(small_sampler, wide, params, uniforms, context="edge rows, misaligned stride", vocab=vocab)
    for tiny in (1, 2, 3, 63, 64, 65):
        small = rng.standard_normal((4, tiny)).astype(np.float32)
        _check_rows(small_sampler, small, hip_sampler.make_params(4, 1.1, 0, 0.9, 0.01), uniforms[:4],
                    context="vocab %d" % tiny)


def test_bf16_rows(small_sampler):
    rng = np.random.default_rng(3)
    logits = workloads.float32_to_bf16_bits(rng.standard_normal((8, 30011)).astype(np.float32) * 2)
    params = hip_sampler.make_params(8, 0.6, 64, 0.9, 0.02)
    uniforms = rng.random(8).astype(np.float32)
    _check_rows(small_sampler, logits, params, uniforms, dtype="bf16", context="bf16 rows K64")
    _check_rows(small_sampler, logits, params, uniforms, dtype="bf16", context="bf16 rows K64", general=True)
    params["top_k"] = 0
    _check_rows(small_sampler, logits, params, uniforms, dtype="bf16", context="bf16 rows no Top-K")


def test_stop_tokens(small_sampler):
    w = workloads.make_workload("cfg4_service_mix", rows=32, vocab=20000)
    _check_rows(small_sampler, w["logits"], w["params"], w["uniforms"], w["stop_ids"], context="service mix, small")


def _full_config(name, dtype):
    w = workloads.make_workload(name)
    _announce("%s full size: %s" % (name, w["description"]))
    gpu = parity_util.run_workload_on_gpu(w)
    cpu = parity_util.run_oracle(w["logits"], w["params"], w["uniforms"], w["stop_ids"])
    counters = parity_util.parity_counters(gpu, cpu)
    print("[parity] %s %s" % (name, counters), flush=True)
    parity_util.assert_results_match(gpu, cpu, dtype, name)
    return gpu, cpu


def test_cfg2_full():
    gpu, _ = _full_config("cfg2_topk_topp", "f32")
    assert (gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH == 0).all()


def test_cfg2_with_scattered_segments():
    """The same batch launched without the XCD-aware numbering of the workgroups (the merge then takes the
    records of segments that ran on other XCDs around the L2): identical results."""
    w = workloads.make_workload("cfg2_topk_topp")
    _announce("cfg2 with scattered segments")
    with hip_sampler.HipSampler(w["rows"], w["vocab"], testing=True) as sampler:
        grouped = parity_util.run_workload_on_gpu(w, sampler)
        sampler.scatter_segments(True)
        scattered = parity_util.run_workload_on_gpu(w, sampler)
        sampler.scatter_segments(False)
    assert grouped.tobytes() == scattered.tobytes()
    cpu = parity_util.run_oracle(w["logits"], w["params"], w["uniforms"], w["stop_ids"])
    parity_util.assert_results_match(scattered, cpu, "f32", "cfg2 scattered")


def test_cfg3_full():
    _full_config("cfg3_full_nucleus", "bf16")


def test_cfg4_full():
    _full_config("cfg4_service_mix", "f32")


def test_cfg5_full():
    gpu, _ = _full_config("cfg5_tie_stress", "bf16")
    assert (gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH == 0).all()


WINDOW_SIZES = [1, 2, 20, 64, 65, 100, 257, 512, 513, 1000, 1024, 1025, 0]


def _mixed_params(rows, rng):
    params = hip_sampler.make_params(rows, 1.0, 0, 1.0, 0.0)
    params["top_k"] = np.array([WINDOW_SIZES[i % len(WINDOW_SIZES)] for i in range(rows)], dtype=np.uint32)
    params["temperature"] = rng.uniform(0.3, 1.6, size=rows).astype(np.float32)
    params["temperature"][rng.random(rows) < 0.08] = 0.0
    params["top_p"] = np.where(rng.random(rows) < 0.3, 1.0, rng.uniform(0.4, 1.0, size=rows)).astype(np.float32)
    params["min_p"] = np.where(rng.random(rows) < 0.5, 0.0, rng.uniform(0.0, 0.05, size=rows)).astype(np.float32)
    return params


def _plant_edge_rows(logits, first):
    """Tie-heavy, NaN, infinite and nearly empty rows starting at row `first`; returns the rows used."""
    vocab = logits.shape[1]
    logits[first + 0, :] = 1.0                         # every logit tied: candidate lists overflow
    logits[first + 1, ::3] = 2.5                       # a third of the row tied at the top
    logits[first + 2, 100:200] = np.nan
    logits[first + 3, :] = -np.inf
    logits[first + 3, vocab // 2] = -3.0               # one finite logit
    logits[first + 4, :] = np.nan
    logits[first + 5, 10] = np.inf
    logits[first + 6, :] = np.round(logits[first + 6, :] * 4) / 4   # heavy ties at every level
    logits[first + 7, vocab // 3:] = -np.inf           # the tail of the row carries nothing
    logits[first + 8, :] = -np.inf
    logits[first + 8, :700] = np.linspace(0, -5, 700, dtype=np.float32)   # fewer finite logits than most windows
    return 9


def _select_rows(params, edge_blocks):
    """Rows the select kernels must serve without the sort: greedy or 1 <= Top-K <= 1024, outside the edge rows."""
    mask = (params["temperature"] == 0.0) | ((params["top_k"] >= 1) & (params["top_k"] <= 1024))
    for first in edge_blocks:
        mask[first:first + 9] = False
    return mask


@pytest.fixture(scope="module")
def batch_sampler():
    sampler = hip_sampler.HipSampler(320, 110000, testing=True)
    yield sampler
    sampler.close()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_whole_row_workgroups(batch_sampler, dtype):
    """From 256 rows on one workgroup streams a whole row and serves Top-K windows up to 1024."""
    rng = np.random.default_rng(71)
    rows, vocab = 300, 33333
    logits = (rng.standard_normal((rows, vocab)) * 2.5).astype(np.float32)
    for block in range(0, rows, 13 * 9):
        _plant_edge_rows(logits, block)
    _plant_edge_rows(logits, 150)
    params = _mixed_params(rows, rng)
    uniforms = rng.random(rows).astype(np.float32)
    if dtype == "bf16":
        logits = workloads.float32_to_bf16_bits(logits)
    _check_rows(batch_sampler, logits, params, uniforms, dtype=dtype, context="whole-row workgroups " + dtype,
                select_rows=_select_rows(params, list(range(0, rows, 13 * 9)) + [150]))


def test_whole_row_long_rows(batch_sampler):
    """Eleven chunks per workgroup: the running bound and the list tightening see many chunks."""
    rng = np.random.default_rng(72)
    rows, vocab = 256, 109999
    logits = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    logits.sort(axis=1)                                 # ascending: every chunk beats the bound so far
    logits[1::2] = logits[1::2, ::-1]                   # and descending rows
    _plant_edge_rows(logits, 40)
    params = _mixed_params(rows, rng)
    uniforms = rng.random(rows).astype(np.float32)
    _check_rows(batch_sampler, logits, params, uniforms, context="whole-row workgroups, long sorted rows")


def test_whole_row_long_final_lists(batch_sampler):
    """Eleven chunks under the first chunk's bound leave a few hundred candidates for windows up to 64:
    the workgroup cuts the final list with all its waves (loosely, then exactly where ties or a wide
    window leave more than 128) before it ranks it."""
    rng = np.random.default_rng(73)
    rows, vocab = 256, 109999
    logits = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    logits[64:128] = np.round(logits[64:128] * 8) / 8    # ties at every level, the cut included
    logits[128:160] = np.round(logits[128:160])          # hundreds of candidates tie with the cut
    params = hip_sampler.make_params(rows, 1.0, 0, 1.0, 0.0)
    params["top_k"] = np.array([(2, 20, 33, 48, 63, 64)[i % 6] for i in range(rows)], dtype=np.uint32)
    params["temperature"] = rng.uniform(0.4, 1.3, size=rows).astype(np.float32)
    params["top_p"] = rng.uniform(0.5, 1.0, size=rows).astype(np.float32)
    uniforms = rng.random(rows).astype(np.float32)
    select_rows = np.ones(rows, dtype=bool)
    select_rows[128:160] = False                         # these may go on to the full-order kernels
    _check_rows(batch_sampler, logits, params, uniforms, context="whole-row workgroups, long final lists",
                select_rows=select_rows)
    _check_rows(batch_sampler, workloads.float32_to_bf16_bits(logits), params, uniforms, dtype="bf16",
                context="whole-row workgroups, long final lists, bf16", select_rows=None)


@pytest.mark.parametrize("rows", [200, 130, 90])
def test_many_segments_per_row(batch_sampler, rows):
    """Between 65 and 255 rows of a long vocabulary: eleven (fp32) or nine (bf16) one-chunk workgroups per
    row, with sorted rows whose chunks defeat each other's bounds.  (Workgroups that stream several chunks
    before the hand-over: tests/test_gpu_split_rows.py.)"""
    rng = np.random.default_rng(73 + rows)
    vocab = 109000
    assert hip_sampler.select_geometry(hip_sampler.LOGITS_F32, rows, vocab) == (11, 1, hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK)
    assert hip_sampler.select_geometry(hip_sampler.LOGITS_BF16, rows, vocab) == (9, 1, hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK)
    logits = (rng.standard_normal((rows, vocab)) * 2).astype(np.float32)
    logits[::4] = np.sort(logits[::4], axis=1)
    _plant_edge_rows(logits, 20)
    params = _mixed_params(rows, rng)
    uniforms = rng.random(rows).astype(np.float32)
    select_rows = _select_rows(params, [20])
    select_rows[::4] = False   # ascending rows may overflow the candidate list: every chunk beats the bound
    _check_rows(batch_sampler, logits, params, uniforms, context="many segments per row, %d rows" % rows,
                select_rows=select_rows)
    bf16 = workloads.float32_to_bf16_bits(logits)
    _check_rows(batch_sampler, bf16, params, uniforms, dtype="bf16", context="many segments per row, bf16, %d rows" % rows)


def test_wide_windows_small_batch(small_sampler):
    """A small batch is split over segments (windows up to 64); wider windows take the second select launch."""
    rng = np.random.default_rng(74)
    rows, vocab = 26, 39999
    logits = (rng.standard_normal((rows, vocab)) * 2).astype(np.float32)
    _plant_edge_rows(logits, 13)
    params = _mixed_params(rows, rng)
    uniforms = rng.random(rows).astype(np.float32)
    gpu, _ = _check_rows(small_sampler, logits, params, uniforms, context="wide windows, small batch")
    served_by_select = (gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH) == 0
    plain = np.ones(rows, dtype=bool)
    plain[13:22] = False
    wide = plain & (params["top_k"] >= 1) & (params["top_k"] <= 1024)
    assert served_by_select[wide].all(), "rows with Top-K <= 1024 must not need the sort"


def test_bf16_rows_of_few_distinct_values(batch_sampler):
    """bf16 rows reach the full-order path as runs of equal keys; here the runs are enormous (one value
    for the whole row, two or three values, a few hundred), so binade crossings and the Top-P / draw
    stops fall deep inside a run, and Top-K windows end inside one."""
    rng = np.random.default_rng(91)
    rows, vocab = 48, 109000
    logits = np.empty((rows, vocab), dtype=np.float32)
    for row in range(rows):
        distinct = int((1, 2, 3, 7, 40, 300)[row % 6])
        values = (rng.standard_normal(distinct) * 3).astype(np.float32)
        weights = rng.random(distinct) ** 3 + 1e-3
        logits[row] = values[rng.choice(distinct, size=vocab, p=weights / weights.sum())]
    logits[5, ::1000] = -np.inf
    logits[11, 7] = np.nan
    params = hip_sampler.make_params(rows, 1.0, 0, 1.0, 0.0)
    params["temperature"] = rng.choice(np.array([0.3, 1.0, 2.5], dtype=np.float32), size=rows)
    params["top_k"] = rng.choice(np.array([0, 0, 1025, 5000, 60000], dtype=np.uint32), size=rows)
    params["top_p"] = rng.choice(np.array([1.0, 0.999, 0.9, 0.5, 0.05], dtype=np.float32), size=rows)
    params["min_p"] = rng.choice(np.array([0.0, 0.0, 0.5, 1.0], dtype=np.float32), size=rows)
    uniforms = rng.random(rows).astype(np.float32)
    uniforms[::5] = np.float32(1.0) - np.float32(2.0 ** -24)
    bits = workloads.float32_to_bf16_bits(logits)
    gpu, _ = _check_rows(batch_sampler, bits, params, uniforms, dtype="bf16", context="bf16 rows of few distinct values")
    assert ((gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH) != 0).all()
    _check_rows(batch_sampler, logits, params, uniforms, context="the same rows as fp32 (radix sort)")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_windows_around_the_quad_maxima_bound(batch_sampler, dtype):
    """Windows up to 64 take their first bound from the 128 quad maxima of a chunk; a chunk with values in
    fewer than 4 K / 3 quads of lanes (a short row, a short last segment) falls back to the exact selection
    over the lane maxima.  Window sizes across the range, on row lengths that fill a few lanes, one chunk,
    and several segments; the select path must serve all."""
    rng = np.random.default_rng(88)
    windows = np.array([1, 2, 15, 16, 17, 23, 24, 25, 31, 32, 33, 63, 64], dtype=np.uint32)
    for vocab in (40, 64, 700, 2049, 10240, 10300, 40000, 100003):
        rows = len(windows) * 3
        logits = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
        logits[1::3] = np.round(logits[1::3] * 8) / 8          # ties inside the window
        logits[2::3, vocab // 2:] = -np.inf                      # half of the row carries nothing
        params = hip_sampler.make_params(rows, 0.8, 0, 0.9, 0.0)
        params["top_k"] = np.repeat(windows, 3)
        params["top_p"][::2] = 1.0
        uniforms = rng.random(rows).astype(np.float32)
        data = workloads.float32_to_bf16_bits(logits) if dtype == "bf16" else logits
        select_rows = np.ones(rows, dtype=bool)
        select_rows[1::3] = vocab < 5000  # heavy ties on long rows may overflow the lists: allowed to take the sort
        if dtype == "bf16":
            select_rows[:] = vocab < 5000   # bf16 rounding makes every row tie-heavy
        _check_rows(batch_sampler, data, params, uniforms, dtype=dtype,
                    context="bound switch, V=%d %s" % (vocab, dtype), select_rows=select_rows)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("vocab", [16384, 16385, 24577, 65536, 109999])
def test_full_order_rows_sorted_by_several_workgroups(batch_sampler, dtype, vocab):
    """Full-order rows (no Top-K, nucleus over the whole row) whose radix sort is spread over two to seven
    workgroups, part boundaries on and off a tile edge, heavy ties and edge rows included: the oracle's
    results, and byte for byte those of the one-workgroup sort.  The exported distribution takes the sort
    that carries the token indices."""
    rng = np.random.default_rng(9100 + vocab)
    rows = 48
    logits = (rng.standard_normal((rows, vocab)) * 3.0).astype(np.float32)
    used = _plant_edge_rows(logits, 8)
    logits[20, :] = np.round(logits[20, :])            # a few dozen distinct values
    logits[21, :] = np.float32(0.5)
    logits[21, vocab - 1] = 4.0                        # the winner is the row's last logit
    if dtype == "bf16":
        logits = workloads.float32_to_bf16_bits(logits)
    params = hip_sampler.make_params(rows, 1.0, 0, 1.0, 0.0)
    params["temperature"] = rng.uniform(0.4, 1.5, size=rows).astype(np.float32)
    params["top_p"] = np.where(np.arange(rows) % 3 == 0, 1.0, rng.uniform(0.5, 0.999, size=rows)).astype(np.float32)
    params["min_p"] = np.where(np.arange(rows) % 4 == 1, rng.uniform(0.0, 0.02, size=rows), 0.0).astype(np.float32)
    params["top_k"][5::7] = 5000                       # wider than the select kernels take
    uniforms = rng.random(rows, dtype=np.float32)
    assert used <= 12
    spread, _ = _check_rows(batch_sampler, logits, params, uniforms, dtype=dtype, vocab=vocab,
                            context="full order, %s, V=%d, spread sort" % (dtype, vocab))
    assert (spread["flags"] & hip_sampler.FLAG_GENERAL_PATH != 0).sum() >= rows - 12
    batch_sampler.spread_sort(False)
    try:
        single = batch_sampler.sample(params, uniforms, None)
    finally:
        batch_sampler.spread_sort(True)
    assert spread.tobytes() == single.tobytes()
    # ... and with every chunk of the normaliser summed round by round instead of in its precomputed step
    batch_sampler.chunk_steps(False)
    try:
        by_rounds = batch_sampler.sample(params, uniforms, None)
    finally:
        batch_sampler.chunk_steps(True)
    assert spread.tobytes() == by_rounds.tobytes()
    for row in (0, 20):
        options = dict(temperature=float(params["temperature"][row]), top_k=0, top_p=0.9, min_p=0.0)
        status, ids, probabilities, count = batch_sampler.distribution(row, **options)
        oracle_status, oracle_ids, oracle_probabilities = oracle_lib.oracle_distribution(
            oracle_lib.widen_bf16(logits[row]) if dtype == "bf16" else logits[row], **options)
        assert status == oracle_status
        assert count == len(oracle_ids)
        assert np.array_equal(ids[:count], oracle_ids)
        assert np.array_equal(probabilities[:count].view(np.uint32), np.asarray(oracle_probabilities, dtype=np.float32).view(np.uint32))


def test_full_order_rows_listed_in_a_batch_of_many_rows():
    """The kernels of the spread sort find their rows in a list that one workgroup writes 1,024 rows at a time:
    a batch of 1,300 rows, greedy but for a few dozen full-order rows at both ends of the batch, around row
    1,024 and scattered in between (fp32 rows of four tiles each)."""
    _announce("row list of the full-order kernels, 1300 rows")
    rng = np.random.default_rng(1300)
    rows, vocab = 1300, 32768
    logits = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    params = hip_sampler.make_params(rows, 0.0, 0, 1.0, 0.0)
    full_order = np.unique(np.concatenate([[0, 1, 63, 64, 1022, 1023, 1024, 1025, 1298, 1299], rng.choice(rows, size=30, replace=False)]))
    params["temperature"][full_order] = rng.uniform(0.5, 1.3, size=full_order.size).astype(np.float32)
    params["top_p"][full_order] = rng.uniform(0.6, 1.0, size=full_order.size).astype(np.float32)
    uniforms = rng.random(rows, dtype=np.float32)
    with hip_sampler.HipSampler(rows, vocab) as sampler:
        sampler.upload_logits(logits)
        gpu = sampler.sample(params, uniforms, None)
    cpu = parity_util.run_oracle(logits, params, uniforms)
    parity_util.assert_results_match(gpu, cpu, "f32", "row list, 1300 rows")
    served_in_full_order = (gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH) != 0
    assert np.array_equal(np.nonzero(served_in_full_order)[0], full_order)


@pytest.mark.parametrize("fused", [True, False])
def test_bf16_counters_that_overflow_sixteen_bits(batch_sampler, fused):
    """(fused: the count and the walk in one kernel, the shipped path, or in the two kernels it replaces.)
    bf16 full-order rows are counted in 16-bit counters, two to a word; a row in which one value occurs
    65536 times or more is counted again in 32-bit counters.  Rows just below and at the limit, in the lower
    and in the upper half of a word (neighbouring bf16 values), in both, a constant row, and rows whose NaN
    or zeros add up to the limit."""
    rng = np.random.default_rng(77)
    vocab = 109999
    rows = 12
    logits = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    low, high = np.float32(1.5), np.float32(1.5078125)   # neighbouring bf16 values: keys 2w and 2w + 1 or the reverse
    for row, (count_low, count_high) in enumerate([(65535, 0), (65536, 0), (0, 65535), (0, 65536), (65536, 40000),
                                                    (30000, 65537), (65535, 44464), (109999, 0), (0, 109999)]):
        order = rng.permutation(vocab)
        logits[row, order[:count_low]] = low
        logits[row, order[count_low:count_low + count_high]] = high
    logits[9, :] = -np.inf
    logits[9, :70000] = 0.25
    bits = workloads.float32_to_bf16_bits(logits)
    # NaN of many payloads and both signs, and zeros of both signs, are counted under keys of their own first and
    # then added up under one key each: sums that just fit a 16-bit counter and sums that do not
    nan_payloads = np.concatenate([np.arange(0x7F81, 0x8000), np.arange(0xFF81, 0x10000)]).astype(np.uint16)
    for row, (nans, positive_zeros, negative_zeros) in zip((10, 11), ((65535, 30000, 35535), (65536, 30000, 35536))):
        order = rng.permutation(vocab)
        bits[row, order[:nans]] = nan_payloads[rng.integers(0, nan_payloads.size, size=nans)]
        bits[row, order[nans:nans + positive_zeros]] = 0x0000
        bits[row, order[nans + positive_zeros:nans + positive_zeros + negative_zeros]] = 0x8000
    params = hip_sampler.make_params(rows, 1.0, 0, 0.95, 0.0)
    params["temperature"] = rng.uniform(0.5, 1.4, size=rows).astype(np.float32)
    params["top_p"][::2] = 1.0
    batch_sampler.fused_bf16(fused)
    try:
        for trial in range(3):
            uniforms = rng.random(rows, dtype=np.float32)
            gpu, _ = _check_rows(batch_sampler, bits, params, uniforms, dtype="bf16", vocab=vocab,
                                 context="bf16 counters at the 16-bit limit, draw %d, fused %s" % (trial, fused))
            assert (gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH != 0).all()
    finally:
        batch_sampler.fused_bf16(True)


@pytest.mark.parametrize("fused", [True, False])
def test_bf16_rows_of_many_runs(batch_sampler, fused):
    """bf16 full-order rows with more distinct values than the walk keeps in LDS (10,920 runs in the one kernel
    that counts and walks, 6,144 in the replay kernel of the two-kernel path): the runs and their exp terms are then
    walked from device memory.  Logits spread over sixty binades."""
    rng = np.random.default_rng(515)
    rows, vocab = 40, 109999
    magnitude = np.exp2(rng.uniform(-40.0, 4.0, size=(rows, vocab)))
    logits = (rng.standard_normal((rows, vocab)) * magnitude).astype(np.float32)
    bits = workloads.float32_to_bf16_bits(logits)
    distinct = [np.unique(bits[row]).size for row in range(rows)]
    assert min(distinct) > 10920, distinct
    params = hip_sampler.make_params(rows, 1.0, 0, 1.0, 0.0)
    params["temperature"] = rng.uniform(0.5, 3.0, size=rows).astype(np.float32)
    params["top_p"] = np.where(np.arange(rows) % 3 == 0, 1.0, rng.uniform(0.6, 0.999, size=rows)).astype(np.float32)
    params["min_p"][1::5] = 0.001
    batch_sampler.fused_bf16(fused)
    try:
        for trial in range(2):
            uniforms = rng.random(rows, dtype=np.float32)
            gpu, _ = _check_rows(batch_sampler, bits, params, uniforms, dtype="bf16", vocab=vocab,
                                 context="bf16 rows of more than 10920 runs, draw %d, fused %s" % (trial, fused))
            assert (gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH != 0).all()
    finally:
        batch_sampler.fused_bf16(True)


def test_bf16_rows_counted_and_walked_by_one_kernel_or_two(batch_sampler):
    """Full-nucleus bf16 rows (the shape of configuration 3, and rows of 6,145 to 10,920 runs, which only the one
    kernel keeps in LDS): byte-identical results from the fused kernel and from the two it replaces, and the oracle's."""
    rng = np.random.default_rng(616)
    rows, vocab = 48, 109999
    mix = (rng.gumbel(0.0, 1.0, size=(rows, vocab)) + rng.standard_normal((rows, vocab))).astype(np.float32)
    magnitude = np.exp2(rng.uniform(-18.0, 3.0, size=(rows // 2, vocab)))
    mix[rows // 2:] = (rng.standard_normal((rows // 2, vocab)) * magnitude).astype(np.float32)
    bits = workloads.float32_to_bf16_bits(mix)
    distinct = [np.unique(bits[row]).size for row in range(rows // 2, rows)]
    assert 6144 < min(distinct) and max(distinct) <= 10920, distinct
    params = hip_sampler.make_params(rows, 1.0, 0, 0.95, 0.0)
    params["temperature"][1::3] = 0.7
    params["min_p"][2::7] = 0.01
    uniforms = rng.random(rows, dtype=np.float32)
    results = {}
    for fused in (True, False):
        batch_sampler.fused_bf16(fused)
        try:
            results[fused], _ = _check_rows(batch_sampler, bits, params, uniforms, dtype="bf16", vocab=vocab,
                                            context="bf16 full nucleus, fused %s" % fused)
        finally:
            batch_sampler.fused_bf16(True)
    assert results[True].tobytes() == results[False].tobytes()


@pytest.mark.parametrize("tied", [0, 700, 1500, 2600])
def test_wide_windows_with_ties_at_the_cut(batch_sampler, tied):
    """Top-K windows of several hundred to a thousand whose K-th value is shared by `tied` further logits: the
    list that the wide select orders is then K + tied entries long (its bitonic sort runs over 1024, 2048 or
    4096 slots), and the ties resolve toward the lower token index."""
    rng = np.random.default_rng(4242 + tied)
    rows, vocab = 24, 60013
    logits = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    params = hip_sampler.make_params(rows, 0.9, 0, 0.97, 0.0)
    params["top_k"] = np.array([(300, 700, 1000, 1024)[i % 4] for i in range(rows)], dtype=np.uint32)
    for row in range(rows):
        if tied:
            k = int(params["top_k"][row])
            order = np.argsort(-logits[row], kind="stable")
            cut_value = logits[row, order[k - 1 - (row % 3)]]      # the window's last value, or one just inside it
            lower = order[k + 50:]                                  # logits below the window take its value
            chosen = rng.choice(lower, size=tied, replace=False)
            logits[row, chosen] = cut_value
    uniforms = rng.random(rows, dtype=np.float32)
    gpu, cpu = _check_rows(batch_sampler, logits, params, uniforms, context="wide windows, %d ties at the cut" % tied)
    served = (gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH) == 0
    assert served.sum() >= (rows if tied <= 1500 else 0)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_sampled_zeros_of_both_signs(batch_sampler, dtype):
    """+0.0 and -0.0 tie (the reference compares logits with ==), so a row whose best logits are zeros of both
    signs orders them by index alone; the full-order path recovers the sampled token's index by comparing
    bit patterns and must treat the two patterns as one key.  Every draw lands on a zero."""
    rng = np.random.default_rng(31337)
    rows, vocab = 32, 70001
    logits = (-20.0 - 5.0 * rng.random((rows, vocab))).astype(np.float32)
    zeros_per_row = 40
    for row in range(rows):
        where = rng.choice(vocab, size=zeros_per_row, replace=False)
        logits[row, where] = np.where(rng.random(zeros_per_row) < 0.5, np.float32(0.0), np.float32(-0.0))
    data = workloads.float32_to_bf16_bits(logits) if dtype == "bf16" else logits
    if dtype == "bf16":
        assert (data == 0x8000).any() and (data == 0x0000).any()
    params = hip_sampler.make_params(rows, 1.0, 0, 1.0, 0.0)      # no window: full-order path
    params["top_k"][1::2] = 5000
    tokens = set()
    for trial in range(4):
        uniforms = rng.random(rows, dtype=np.float32)
        gpu, cpu = _check_rows(batch_sampler, data, params, uniforms, dtype=dtype, vocab=vocab,
                               context="zeros of both signs, %s, draw %d" % (dtype, trial))
        assert (gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH != 0).all()
        picked = logits[np.arange(rows), gpu["token_id"]]
        assert (picked == 0.0).all()
        tokens.update(int(t) for t in gpu["token_id"])
    assert len(tokens) > rows  # the draws spread over the zeros


def test_distribution_of_a_wide_window(batch_sampler):
    """The filtered distribution of a row with a window of several hundred tokens, exported by the wide select
    (all of its threads write the list): ids and probabilities bit for bit those of the oracle."""
    rng = np.random.default_rng(808)
    vocab = 90007
    logits = (rng.standard_normal((4, vocab)) * 2.5).astype(np.float32)
    batch_sampler.upload_logits(logits, vocab=vocab)
    for row, options in enumerate([dict(temperature=0.9, top_k=700, top_p=1.0, min_p=0.0),
                                   dict(temperature=1.3, top_k=1024, top_p=0.99, min_p=0.0),
                                   dict(temperature=0.7, top_k=300, top_p=0.95, min_p=0.001),
                                   dict(temperature=1.0, top_k=65, top_p=1.0, min_p=0.0)]):
        _announce("distribution of a wide window, row %d" % row)
        status, ids, probabilities, count = batch_sampler.distribution(row, **options)
        oracle_status, oracle_ids, oracle_probabilities = oracle_lib.oracle_distribution(logits[row], **options)
        assert status == oracle_status
        assert count == len(oracle_ids) and count > 64
        assert np.array_equal(ids[:count], oracle_ids)
        assert np.array_equal(probabilities[:count].view(np.uint32), np.asarray(oracle_probabilities, dtype=np.float32).view(np.uint32))
