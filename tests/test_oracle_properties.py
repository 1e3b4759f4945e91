"""What the mathematics fixes about the sampler, checked on the CPU oracle: brute-force selection,
an fp64 softmax over the kept set, the definition of Min-P / Top-P / the inverse-CDF draw, and
invariants.  None of these retypes the oracle's own loop."""
import numpy as np
import pytest

import oracle_lib as ol


def brute_force_order(logits):
    """(logit descending, index ascending) by a direct O(n log n) lexicographic sort in fp64."""
    logits = np.asarray(logits, dtype=np.float64)
    return np.lexsort((np.arange(logits.size), -logits))


def reference_model(logits, temperature, top_k, top_p, min_p):
    """fp64 model of the pipeline: Top-K -> softmax -> Min-P -> Top-P -> renormalise."""
    order = brute_force_order(logits)
    if 0 < top_k < len(order):
        order = order[:top_k]
    x = np.asarray(logits, dtype=np.float64)[order] / temperature
    e = np.exp(x - x[0])
    p = e / e.sum()
    keep = p >= p[0] * min_p if min_p > 0 else np.ones_like(p, dtype=bool)
    order, p = order[keep], p[keep]
    cumulative = np.cumsum(p)
    reached = np.nonzero(cumulative >= top_p)[0]
    count = reached[0] + 1 if reached.size else len(p)
    order, p = order[:count], p[:count]
    return order, p / p.sum(), cumulative[:count]


@pytest.mark.parametrize("seed", range(12))
def test_distribution_matches_fp64_model(seed):
    rng = np.random.default_rng(seed)
    vocab = int(rng.integers(5, 3000))
    logits = (rng.standard_normal(vocab) * rng.uniform(0.5, 4)).astype(np.float32)
    temperature = float(rng.uniform(0.2, 1.6))
    top_k = int(rng.choice([0, 1, 5, 50, vocab + 3]))
    top_p = float(rng.uniform(0.3, 1.0))
    min_p = float(rng.choice([0.0, 0.01, 0.2]))
    status, ids, probabilities = ol.oracle_distribution(logits, temperature, top_k, top_p, min_p)
    assert status == 0
    model_ids, model_probabilities, cumulative = reference_model(logits, temperature, top_k, top_p, min_p)
    # the cut positions agree unless a cumulative sum or a Min-P ratio lies within rounding of its threshold
    near_cut = np.min(np.abs(cumulative - top_p)) < 1e-5
    if not near_cut and min_p == 0.0:
        assert ids.tolist() == model_ids.tolist()
        np.testing.assert_allclose(probabilities, model_probabilities, rtol=2e-5)
    else:
        n = min(len(ids), len(model_ids))
        assert ids[:n].tolist() == model_ids[:n].tolist()
    assert abs(float(probabilities.astype(np.float64).sum()) - 1.0) < 1e-5
    assert (np.diff(probabilities) <= 0).all()


def test_top_k_selects_by_value_then_lower_index():
    rng = np.random.default_rng(1)
    logits = np.round(rng.standard_normal(500) * 3).astype(np.float32)  # many ties
    for top_k in (1, 2, 7, 33, 100):
        status, ids, _ = ol.oracle_distribution(logits, 1.0, top_k, 1.0, 0.0)
        assert status == 0
        assert ids.tolist() == brute_force_order(logits)[:top_k].tolist()


def test_greedy_is_first_argmax_over_finite():
    rng = np.random.default_rng(2)
    for _ in range(50):
        logits = np.round(rng.standard_normal(200) * 2).astype(np.float32)
        logits[rng.integers(0, 200, 20)] = np.nan
        logits[rng.integers(0, 200, 5)] = np.inf
        logits[rng.integers(0, 200, 5)] = -np.inf
        finite = np.isfinite(logits)
        expected = int(np.nonzero(finite & (logits == logits[finite].max()))[0][0])
        r = ol.oracle_sample(logits, 0.3, temperature=0.0)
        assert r["token_id"] == expected and r["probability"] == 1.0 and r["kept_count"] == 1


def test_draw_is_the_inverse_cdf():
    rng = np.random.default_rng(3)
    logits = (rng.standard_normal(300) * 2).astype(np.float32)
    status, ids, probabilities = ol.oracle_distribution(logits, 0.9, 40, 0.95, 0.0)
    cumulative = np.cumsum(probabilities, dtype=np.float32)  # sequential fp32 running sum
    for u in np.linspace(0.0, 0.999999, 97, dtype=np.float32):
        r = ol.oracle_sample(logits, float(u), 0.9, 40, 0.95, 0.0)
        position = int(np.searchsorted(cumulative, u, side="right"))
        position = min(position, len(ids) - 1)  # falls through to the last candidate
        assert r["token_id"] == ids[position] and r["probability"] == probabilities[position]
        assert r["draw_consumed"] == 1 and r["kept_count"] == len(ids)


def test_no_ops_and_invariances():
    rng = np.random.default_rng(4)
    logits = (rng.standard_normal(777) * 2).astype(np.float32)
    base = ol.oracle_distribution(logits, 0.7, 0, 1.0, 0.0)
    # top_k >= vocab is the same as no Top-K
    for top_k in (777, 778, 100000):
        other = ol.oracle_distribution(logits, 0.7, top_k, 1.0, 0.0)
        assert np.array_equal(base[1], other[1]) and np.array_equal(base[2], other[2])
    # scaling logits and temperature by two leaves every quotient logit / T unchanged
    scaled = ol.oracle_distribution(logits * np.float32(2), 1.4, 0, 1.0, 0.0)
    assert np.array_equal(base[1], scaled[1]) and np.array_equal(base[2], scaled[2])
    # a single survivor is returned with probability one and consumes no draw
    r = ol.oracle_sample(logits, 0.5, 0.7, 0, 1e-6, 0.0)
    assert r["kept_count"] == 1 and r["probability"] == 1.0 and r["draw_consumed"] == 0
    # adding a constant that is exact in fp32 does not change the order
    status, ids, _ = ol.oracle_distribution(np.round(logits * 4) / 4 + np.float32(8), 1.0, 10, 1.0, 0.0)
    status2, ids2, _ = ol.oracle_distribution(np.round(logits * 4) / 4, 1.0, 10, 1.0, 0.0)
    assert ids.tolist() == ids2.tolist()


def test_min_p_is_not_renormalised_before_top_p():
    # p = .4/.3/.2/.1; Min-P 0.45 drops the last; Top-P 0.75 then needs all three survivors
    logits = np.array([3211432455, 3214547912, 3217949200, 3222494606], dtype=np.uint32).view(np.float32)
    status, ids, _ = ol.oracle_distribution(logits, 1.0, 0, 0.75, 0.45)
    assert ids.tolist() == [0, 1, 2]


def test_batch_matches_single_rows_and_stop_flags():
    rng = np.random.default_rng(5)
    rows, vocab = 12, 400
    logits = (rng.standard_normal((rows, vocab)) * 2).astype(np.float32)
    params = np.zeros(rows, dtype=ol.ROW_PARAMS_DTYPE)
    params["temperature"] = rng.uniform(0, 1.5, rows)
    params["temperature"][::4] = 0.0
    params["top_k"] = rng.choice([0, 1, 20], rows)
    params["top_p"] = rng.uniform(0.5, 1.0, rows)
    params["min_p"] = rng.uniform(0, 0.1, rows)
    params["stop_begin"] = np.arange(rows) * 2
    params["stop_count"] = 2
    uniforms = rng.random(rows).astype(np.float32)
    singles = [ol.oracle_sample(logits[i], uniforms[i], params["temperature"][i], int(params["top_k"][i]),
                                params["top_p"][i], params["min_p"][i]) for i in range(rows)]
    stop_ids = rng.integers(0, vocab, rows * 2).astype(np.int32)
    stop_ids[0::4] = [s["token_id"] for s in singles[0::2]]
    for threads in (1, 3):
        batch = ol.oracle_sample_batch(logits, params, uniforms, stop_ids, threads=threads)
        for i in range(rows):
            assert batch["token_id"][i] == singles[i]["token_id"]
            assert batch["probability"][i] == singles[i]["probability"]
            expected_stop = singles[i]["token_id"] in stop_ids[2 * i:2 * i + 2].tolist()
            assert bool(batch["is_stop"][i]) == expected_stop
    # bf16 rows are widened with bits << 16
    bits = ol.quantize_bf16(logits)
    widened = ol.widen_bf16(bits)
    a = ol.oracle_sample_batch(bits, params, uniforms, stop_ids)
    b = ol.oracle_sample_batch(widened, params, uniforms, stop_ids)
    assert np.array_equal(a["token_id"], b["token_id"]) and np.array_equal(a["probability"], b["probability"])
