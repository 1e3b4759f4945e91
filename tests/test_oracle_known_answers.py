"""The CPU oracle against the reference's own sampler checks (tests/test_runtime.cpp:4332-4362) and
the known answers recorded from the reference library."""
import numpy as np
import pytest

import oracle_lib as ol

NAN, INF = np.nan, np.inf
# logf of {0.4, 0.3, 0.2, 0.1} in fp32, as bit patterns
LN_4321 = np.array([3211432455, 3214547912, 3217949200, 3222494606], dtype=np.uint32).view(np.float32)


def test_reference_own_vectors():
    # tests/test_runtime.cpp:4333-4339: greedy argmax, probability 1
    r = ol.oracle_sample([1, 2, 3], 0.5, temperature=0.0)
    assert r["status"] == 0 and r["token_id"] == 2 and r["probability"] == 1.0
    # :4341-4344: greedy skips NaN, ties go to the lower index
    assert ol.oracle_sample([3, NAN, 3], 0.5, temperature=0.0)["token_id"] == 0
    # :4346-4349: no finite logit
    r = ol.oracle_sample([NAN, INF], 0.5, temperature=0.0)
    assert r["status"] == ol.STATUS_NO_FINITE_LOGIT and r["token_id"] == -1
    # :4351-4356: top_k = 1
    r = ol.oracle_sample([1, 2, 3], 0.5, top_k=1)
    assert r["token_id"] == 2 and r["draw_consumed"] == 0
    # :4358-4362: top_p = 0 is invalid
    assert ol.oracle_sample([1, 2, 3], 0.5, top_p=0.0)["status"] == ol.STATUS_BAD_TOP_P


@pytest.mark.parametrize("logits,options,ids,probabilities", [
    (LN_4321, dict(min_p=0.45, top_p=0.75), [0, 1, 2], [0.444444478, 0.333333313, 0.222222209]),
    (LN_4321, dict(min_p=0.5, top_p=0.75), [0, 1], [0.571428597, 0.428571403]),
    (LN_4321, dict(top_p=0.5), [0, 1], [0.571428597, 0.428571403]),
    ([1, 2, 3], dict(top_k=7), [2, 1, 0], [0.665240943, 0.244728476, 0.0900305733]),
    ([1, 2, 3, 4, 5], dict(temperature=0.5, top_k=3, top_p=0.9, min_p=0.05), [4, 3], [0.880797088, 0.119202919]),
    ([2, 2, 1], dict(min_p=1.0), [0, 1], [0.5, 0.5]),
    ([5, 7, 7, 7], dict(top_k=2), [1, 2], [0.5, 0.5]),
    ([1, 1], dict(top_p=0.5), [0], [1.0]),
    ([3, -INF, -INF], dict(top_k=2), [0], [1.0]),
    ([0.0, -0.0], dict(top_k=1), [0], [1.0]),
    ([-0.0, 0.0], dict(top_k=1), [0], [1.0]),
    ([1, 2], dict(temperature=1e-30), [1], [1.0]),
])
def test_recorded_distributions(logits, options, ids, probabilities):
    status, got_ids, got_probabilities = ol.oracle_distribution(logits, **options)
    assert status == 0
    assert got_ids.tolist() == ids
    assert np.array_equal(got_probabilities, np.array(probabilities, dtype=np.float32))


@pytest.mark.parametrize("logits,options,status", [
    ([-INF, -INF], dict(temperature=0.0), ol.STATUS_NO_FINITE_LOGIT),
    ([-INF, -INF], dict(temperature=1.0), ol.STATUS_NO_FINITE_LOGIT),
    ([1, INF, 2], dict(temperature=0.7, top_k=20, top_p=0.8), ol.STATUS_NO_FINITE_LOGIT),
    ([1, 2], dict(temperature=1e-39), ol.STATUS_INVALID_DISTRIBUTION),
    ([1, 2], dict(temperature=-1.0), ol.STATUS_BAD_TEMPERATURE),
    ([1, 2], dict(temperature=INF), ol.STATUS_BAD_TEMPERATURE),
    ([1, 2], dict(temperature=NAN), ol.STATUS_BAD_TEMPERATURE),
    ([1, 2], dict(top_p=1.0000001), ol.STATUS_BAD_TOP_P),
    ([1, 2], dict(top_p=NAN), ol.STATUS_BAD_TOP_P),
    ([1, 2], dict(min_p=-1e-9), ol.STATUS_BAD_MIN_P),
    ([1, 2], dict(min_p=1.5), ol.STATUS_BAD_MIN_P),
    ([], dict(), ol.STATUS_EMPTY_LOGITS),
])
def test_recorded_errors(logits, options, status):
    r = ol.oracle_sample(np.array(logits, dtype=np.float32), 0.5, **options)
    assert r["status"] == status and r["token_id"] == -1 and r["probability"] == 0.0
    assert ol.oracle().oracle_status_message(status).decode() == ol.STATUS_MESSAGES[status]


def test_negative_zero_temperature_is_greedy():
    r = ol.oracle_sample([1, 3, 2], 0.9, temperature=-0.0)
    assert r["status"] == 0 and r["token_id"] == 1 and r["probability"] == 1.0


def test_greedy_skips_positive_infinity():
    assert ol.oracle_sample([1, INF, 2], 0.9, temperature=0.0)["token_id"] == 2


def test_rng_lockstep_known_answer():
    """{0,5,5,-1}, seed 1234, Top-K 2: the reference picked token 1 iff u < 0.5 on 2000/2000 draws, and
    a Top-K 1 call in between consumed no draw."""
    rng = ol.OracleRng(1234)
    logits = np.array([0, 5, 5, -1], dtype=np.float32)
    for _ in range(200):
        u = rng.uniform()
        r = ol.oracle_sample(logits, u, top_k=2)
        assert r["token_id"] == (1 if u < 0.5 else 2) and r["probability"] == 0.5 and r["draw_consumed"] == 1
        assert ol.oracle_sample(logits, u, top_k=1)["draw_consumed"] == 0


def test_rng_first_draws_are_the_mt19937_64_stream():
    """uniform_real_distribution<float>(0,1) over mt19937_64 takes one 64-bit draw per float.  The
    10000th output of mt19937_64 seeded with 5489 is 9981545732273789042 (C++ standard, [rand.predef])."""
    rng = ol.OracleRng(5489)
    draws = [rng.uniform() for _ in range(10000)]
    expected = np.float32(9981545732273789042) * np.float32(2.0 ** -64)
    assert draws[-1] == expected
    assert all(0.0 <= u < 1.0 for u in draws)


def test_bf16_helpers_exhaustive():
    lib = ol.oracle()
    bits = np.arange(65536, dtype=np.uint32)
    widened = (bits << np.uint32(16)).view(np.float32)
    for b in range(0, 65536, 257):
        assert np.isnan(widened[b]) or np.float32(lib.oracle_bfloat16_to_float(b)).view(np.uint32) == np.uint32(b << 16)
    # round trip: every non-NaN bf16 value survives widen -> narrow
    finite = ~np.isnan(widened)
    assert np.array_equal(ol.quantize_bf16(widened[finite]), bits[finite].astype(np.uint16))
    # round to nearest even on the 16 dropped bits
    base = np.uint32(0x3F800000)  # 1.0
    assert lib.oracle_float_to_bfloat16(np.uint32(base + 0x7FFF).view(np.float32)) == 0x3F80
    assert lib.oracle_float_to_bfloat16(np.uint32(base + 0x8000).view(np.float32)) == 0x3F80  # tie -> even
    assert lib.oracle_float_to_bfloat16(np.uint32(base + 0x8001).view(np.float32)) == 0x3F81
    assert lib.oracle_float_to_bfloat16(np.uint32(base + 0x18000).view(np.float32)) == 0x3F82  # tie -> even (up)


def test_restated_expf_equals_libm_on_a_dense_sample():
    lib = ol.oracle()
    # every 211th bit pattern of the negative floats down to -110 and of the positive floats up to 90
    assert lib.oracle_expf_compare_range(0x80000000, 0xC2DC0000, 211) == 0
    assert lib.oracle_expf_compare_range(0x00000000, 0x42B40000, 211) == 0
    # the two inputs on which the unfused argument reduction differs from libm
    for x in (float.fromhex('-0x1.f8cbb2p+5'), float.fromhex('0x1.04845ep+5')):
        assert lib.oracle_expf_restated(x) == lib.oracle_expf_libm(x)
