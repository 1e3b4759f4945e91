"""The oracle's expert router (src/graph/expert_dispatcher.cpp:12-157) against the reference's own
ExpertDispatcher (public class, called through the harness where the reference builds), against the
reference's test vectors (tests/test_runtime.cpp:3362-3540) and against what the mathematics fixes."""
import numpy as np
import pytest

import oracle_lib as ol

needs_reference = pytest.mark.skipif(not ol.reference_available(), reason="reference library not built here")
REF_INVALID_ARGUMENT, REF_INVALID_MODEL = 1 + 0, 1 + 2   # 1 + ErrorCode (include/ncnn/moe/result.h:12-19)


def test_reference_test_vectors():
    """tests/test_runtime.cpp:3362-3430: four tokens, Top-1 of 6 experts; then Top-2 of 3 with renormalised weights."""
    logits = np.zeros((4, 6), dtype=np.float32)
    logits[0, 1], logits[1, 5], logits[1, 1], logits[2, 1], logits[2, 3], logits[3, 5] = 5.0, 5.0, 4.0, 1.0, 1.0, 4.0
    logits[1, 1] = 0.0
    logits[1, 3] = 4.0
    status, offsets, routes = ol.oracle_router_dispatch(logits, 1)
    assert status == 0 and routes.size == 4
    populated = [e for e in range(6) if offsets[e + 1] > offsets[e]]
    assert populated == [1, 5]
    assert routes["token_index"][offsets[1]:offsets[2]].tolist() == [0, 2]      # ties: expert 1 before expert 3
    assert routes["token_index"][offsets[5]:offsets[6]].tolist() == [1, 3]
    assert routes["weight"][offsets[1]] == 1.0
    status, offsets, routes = ol.oracle_router_dispatch(np.array([[2.0, 1.0, 0.0]], dtype=np.float32), 2)
    assert status == 0 and routes["rank"].tolist() == [0, 1]
    assert abs(float(routes["weight"].sum()) - 1.0) < 1e-6
    # tests/test_runtime.cpp:3506-3530: sqrt-softplus scores, a bias that forces expert 1, scaling 1.5
    status, offsets, routes = ol.oracle_router_dispatch(
        np.array([[4.0, -4.0, 3.0, 2.0]], dtype=np.float32), 2, ol.ROUTER_SQRT_SOFTPLUS, True, 1.5,
        selection_bias=[0.0, 100.0, 0.0, 0.0])
    assert status == 0 and [e for e in range(4) if offsets[e + 1] > offsets[e]] == [0, 1]
    assert abs(float(routes["weight"].sum()) - 1.5) < 1e-5
    status, offsets, routes = ol.oracle_router_dispatch(
        np.array([[4.0, -4.0, 3.0, 2.0]], dtype=np.float32), 2, ol.ROUTER_SQRT_SOFTPLUS, True, 1.5,
        explicit_expert_ids=[3, 2])
    assert [e for e in range(4) if offsets[e + 1] > offsets[e]] == [2, 3]
    assert routes["rank"].tolist() == [1, 0]


def test_scores_against_float64_models():
    rng = np.random.default_rng(3)
    for _ in range(50):
        logits = (rng.standard_normal(int(rng.integers(1, 300))) * rng.uniform(0.1, 8)).astype(np.float32)
        x = logits.astype(np.float64)
        softmax = np.exp(x - x.max()) / np.exp(x - x.max()).sum()
        np.testing.assert_allclose(ol.oracle_router_scores(logits, ol.ROUTER_SOFTMAX), softmax, rtol=3e-6, atol=1e-12)
        np.testing.assert_allclose(ol.oracle_router_scores(logits, ol.ROUTER_SIGMOID), 1 / (1 + np.exp(-x)), rtol=3e-7)
        np.testing.assert_allclose(ol.oracle_router_scores(logits, ol.ROUTER_SQRT_SOFTPLUS),
                                   np.sqrt(np.logaddexp(0.0, x)), rtol=5e-7)


def test_selection_is_the_brute_force_order_and_weights_renormalise():
    rng = np.random.default_rng(4)
    for _ in range(100):
        tokens, experts = int(rng.integers(1, 9)), int(rng.integers(1, 70))
        top_k = int(rng.integers(1, experts + 1))
        logits = np.round(rng.standard_normal((tokens, experts)) * 2, 1).astype(np.float32)   # many ties
        bias = np.round(rng.standard_normal(experts), 1).astype(np.float32) if rng.random() < 0.5 else None
        scaling = float(rng.choice([1.0, 2.5]))
        status, offsets, routes = ol.oracle_router_dispatch(logits, top_k, ol.ROUTER_SIGMOID, True, scaling, selection_bias=bias)
        assert status == 0 and routes.size == tokens * top_k
        expert_of = np.repeat(np.arange(experts), np.diff(offsets.astype(np.int64)))
        for token in range(tokens):
            scores = ol.oracle_router_scores(logits[token], ol.ROUTER_SIGMOID)
            keyed = scores + (bias if bias is not None else np.float32(0))
            order = sorted(range(experts), key=lambda e: (-float(keyed[e]), e))[:top_k]
            mine = routes["token_index"] == token
            assert expert_of[mine][np.argsort(routes["rank"][mine])].tolist() == order
            assert abs(float(routes["weight"][mine].sum()) - scaling) < 1e-5
        # every expert's routes are in token order
        for expert in range(experts):
            group = routes["token_index"][offsets[expert]:offsets[expert + 1]]
            assert (np.diff(group.astype(np.int64)) > 0).all()


def test_error_statuses():
    logits = np.zeros((2, 4), dtype=np.float32)
    assert ol.oracle_router_dispatch(logits, 0)[0] == 2
    assert ol.oracle_router_dispatch(logits, 5)[0] == 2
    assert ol.oracle_router_dispatch(logits, 2, routed_scaling_factor=0.0)[0] == 3
    assert ol.oracle_router_dispatch(logits, 2, routed_scaling_factor=float("inf"))[0] == 3
    broken = logits.copy()
    broken[1, 2] = np.nan
    assert ol.oracle_router_dispatch(broken, 2)[0] == 4
    assert ol.oracle_router_dispatch(logits, 2, explicit_expert_ids=[0, 1, 2, 4])[0] == 5
    assert ol.oracle_router_dispatch(np.full((1, 4), -200.0, dtype=np.float32), 2, ol.ROUTER_SIGMOID)[0] == 6
    assert ol.oracle_router_dispatch(np.zeros((0, 4), dtype=np.float32), 2)[0] == 1


def _random_case(rng):
    tokens = int(rng.choice([1, 1, 2, 7, 64, 300]))
    experts = int(rng.choice([1, 2, 8, 20, 64, 65, 128, 256, 384, 512]))
    top_k = int(min(experts, rng.choice([1, 2, 4, 6, 8, 16, 17])))
    kind = int(rng.integers(0, 4))
    logits = (rng.standard_normal((tokens, experts)) * rng.uniform(0.2, 6)).astype(np.float32)
    if kind == 1:
        logits = np.round(logits)
    elif kind == 2:
        logits[:] = logits[0, 0]
    elif kind == 3:
        logits *= np.float32(8.0)     # saturating sigmoids, softplus branches beyond +-20
    options = dict(score_function=int(rng.integers(0, 3)), routed_scaling_factor=float(rng.choice([1.0, 2.5, 0.125])))
    bias = (rng.standard_normal(experts) * 0.3).astype(np.float32) if rng.random() < 0.4 else None
    explicit = None
    if rng.random() < 0.2:
        explicit = rng.integers(0, experts, size=(tokens, top_k)).astype(np.uint32)   # duplicates allowed
    return logits, top_k, options, bias, explicit


@needs_reference
@pytest.mark.reference
@pytest.mark.parametrize("seed", range(30))
def test_dispatch_matches_reference(seed):
    rng = np.random.default_rng(700 + seed)
    for _ in range(8):
        logits, top_k, options, bias, explicit = _random_case(rng)
        renormalize = bool(rng.random() < 0.7)
        normalization, flags = (1, 1) if renormalize else (0, 0)
        rc, ref_offsets, ref_routes, message = ol.reference_router_dispatch(
            logits, top_k, options["score_function"], normalization, flags, options["routed_scaling_factor"], bias, explicit)
        status, offsets, routes = ol.oracle_router_dispatch(
            logits, top_k, options["score_function"], renormalize, options["routed_scaling_factor"], bias, explicit)
        if rc != 0:
            assert rc in (REF_INVALID_ARGUMENT, REF_INVALID_MODEL) and ol.ROUTER_MESSAGES[status] == message
            assert (status == 6) == (rc == REF_INVALID_MODEL)
            continue
        assert status == 0
        assert np.array_equal(offsets, ref_offsets)
        assert np.array_equal(routes["token_index"], ref_routes["token_index"])
        assert np.array_equal(routes["rank"], ref_routes["rank"])
        assert np.array_equal(routes["weight"].view(np.uint32), ref_routes["weight"].view(np.uint32))


@needs_reference
@pytest.mark.reference
def test_single_token_entry_of_the_reference_agrees():
    """dispatch_into (src/graph/expert_dispatcher.cpp:159-301) is the reference's one-token fast path."""
    rng = np.random.default_rng(9)
    for _ in range(200):
        logits, top_k, options, bias, explicit = _random_case(rng)
        logits = logits[:1]
        explicit = None if explicit is None else explicit[:1]
        rc, ref_offsets, ref_routes, _ = ol.reference_router_dispatch(
            logits, top_k, options["score_function"], 1, 1, options["routed_scaling_factor"], bias, explicit, use_dispatch_into=True)
        status, offsets, routes = ol.oracle_router_dispatch(
            logits, top_k, options["score_function"], True, options["routed_scaling_factor"], bias, explicit)
        if rc != 0:
            assert status != 0
            continue
        assert status == 0 and np.array_equal(offsets, ref_offsets)
        assert np.array_equal(routes["rank"], ref_routes["rank"])
        assert np.array_equal(routes["weight"].view(np.uint32), ref_routes["weight"].view(np.uint32))


@needs_reference
@pytest.mark.reference
def test_reference_error_messages():
    logits = np.zeros((2, 4), dtype=np.float32)
    cases = [
        (dict(top_k=0), 2), (dict(top_k=5), 2), (dict(top_k=2, routed_scaling_factor=-1.0), 3),
        (dict(top_k=2, explicit_expert_ids=np.array([[0, 1], [2, 9]], dtype=np.uint32)), 5),
    ]
    for arguments, status in cases:
        rc, _, _, message = ol.reference_router_dispatch(logits, **arguments)
        assert rc == REF_INVALID_ARGUMENT and message == ol.ROUTER_MESSAGES[status]
        assert ol.oracle_router_dispatch(logits, **arguments)[0] == status
    broken = logits.copy()
    broken[0, 0] = np.inf
    rc, _, _, message = ol.reference_router_dispatch(broken, 2)
    assert rc == REF_INVALID_ARGUMENT and message == ol.ROUTER_MESSAGES[4]
    rc, _, _, message = ol.reference_router_dispatch(np.full((1, 4), -200.0, dtype=np.float32), 2, ol.ROUTER_SIGMOID)
    assert rc == REF_INVALID_MODEL and message == ol.ROUTER_MESSAGES[6]
