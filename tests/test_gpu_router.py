"""GPU parity of the expert router (ncnn_moe_hip_router_dispatch through the C ABI) against the CPU
oracle on identical seeded inputs: status, expert offsets, and every route's token, rank and weight
(weights bit for bit)."""
import ctypes

import numpy as np
import pytest

import oracle_lib
from ncnn_moe_runtime_amd import hip_router

pytestmark = pytest.mark.gpu

# imported before the router library is loaded, so that both bind the same HIP runtime
torch = pytest.importorskip("torch")


def _announce(text):
    print("[case] " + text, flush=True)


@pytest.fixture(scope="module")
def router():
    handle = hip_router.HipRouter(8192)
    yield handle
    handle.close()


def _compare(router, logits, top_k, context, **options):
    _announce(context)
    gpu_status, gpu_offsets, gpu_routes = router.dispatch(logits, top_k, **options)
    cpu_status, cpu_offsets, cpu_routes = oracle_lib.oracle_router_dispatch(logits, top_k, **options)
    assert gpu_status == cpu_status, (context, gpu_status, cpu_status)
    if cpu_status != 0:
        assert hip_router.status_message(gpu_status) == oracle_lib.ROUTER_MESSAGES[cpu_status]
        return gpu_status
    assert np.array_equal(gpu_offsets, cpu_offsets), context
    assert len(gpu_routes) == len(cpu_routes) == logits.shape[0] * top_k
    assert np.array_equal(gpu_routes["token_index"], cpu_routes["token_index"]), context
    assert np.array_equal(gpu_routes["rank"], cpu_routes["rank"]), context
    assert np.array_equal(gpu_routes["weight"].view(np.uint32), cpu_routes["weight"].view(np.uint32)), context
    return gpu_status


def _logits(rng, tokens, experts, scale):
    return (rng.standard_normal((tokens, experts)) * scale).astype(np.float32)


@pytest.mark.parametrize("experts,top_k", [(1, 1), (8, 2), (60, 4), (64, 8), (65, 6), (128, 8), (160, 6),
                                           (256, 8), (384, 8), (512, 10), (1000, 64), (1024, 1)])
@pytest.mark.parametrize("score", [hip_router.SOFTMAX, hip_router.SIGMOID, hip_router.SQRT_SOFTPLUS])
def test_random_dispatch_matches_oracle(router, experts, top_k, score):
    rng = np.random.default_rng(experts * 131 + top_k * 7 + score)
    for case, tokens in enumerate([1, 3, 64, 257, 1500]):
        scale = float(rng.choice([0.5, 2.0, 8.0]))
        logits = _logits(rng, tokens, experts, scale)
        bias = None if case % 2 == 0 else (rng.standard_normal(experts) * 0.3).astype(np.float32)
        options = dict(score_function=score, renormalize=bool(case % 3 != 1),
                       routed_scaling_factor=float(rng.choice([1.0, 2.5, 0.125, 16.0])), selection_bias=bias)
        status = _compare(router, logits, top_k, "E=%d K=%d score=%d T=%d scale=%g %s" % (
            experts, top_k, score, tokens, scale, {k: v for k, v in options.items() if k != "selection_bias"}), **options)
        assert status == 0


def test_ties_resolve_to_the_lower_expert_id(router):
    rng = np.random.default_rng(3)
    for experts, top_k in [(16, 4), (128, 8), (300, 17)]:
        logits = rng.integers(-2, 3, size=(200, experts)).astype(np.float32)  # a handful of distinct values
        for score in (hip_router.SOFTMAX, hip_router.SIGMOID, hip_router.SQRT_SOFTPLUS):
            _compare(router, logits, top_k, "tied logits E=%d K=%d score=%d" % (experts, top_k, score), score_function=score)
        flat = np.zeros((5, experts), dtype=np.float32)
        _, offsets, routes = router.dispatch(flat, top_k)
        assert np.array_equal(offsets[:top_k + 1], np.arange(top_k + 1) * 5) and offsets[-1] == 5 * top_k
        _compare(router, flat, top_k, "all logits equal E=%d" % experts)


def test_selection_bias_picks_but_does_not_weigh(router):
    """The bias moves the choice; the weights come from the unbiased scores (expert_dispatcher.cpp:61-77, 137-150)."""
    logits = np.array([[2.0, 1.0, 0.0, -1.0]], dtype=np.float32)
    bias = np.array([-10.0, 0.0, 0.0, 10.0], dtype=np.float32)
    status, offsets, routes = router.dispatch(logits, 2, selection_bias=bias, renormalize=False)
    assert status == 0 and list(np.diff(offsets.astype(np.int64))) == [0, 1, 0, 1]
    scores = oracle_lib.oracle_router_scores(logits[0], oracle_lib.ROUTER_SOFTMAX)
    assert routes["weight"][0] == scores[1] and routes["weight"][1] == scores[3]
    assert list(routes["rank"]) == [1, 0]
    _compare(router, logits, 2, "bias picks", selection_bias=bias, renormalize=False)


def test_explicit_expert_ids(router):
    rng = np.random.default_rng(4)
    for experts, top_k, tokens in [(8, 2, 10), (128, 8, 300), (256, 64, 40), (1024, 3, 700)]:
        logits = _logits(rng, tokens, experts, 2.0)
        explicit = rng.integers(0, experts, size=(tokens, top_k)).astype(np.uint32)  # repeats within a token allowed
        for score in (hip_router.SOFTMAX, hip_router.SIGMOID, hip_router.SQRT_SOFTPLUS):
            _compare(router, logits, top_k, "explicit ids E=%d K=%d T=%d score=%d" % (experts, top_k, tokens, score),
                     score_function=score, explicit_expert_ids=explicit)
    # an id out of range fails the call
    explicit = np.zeros((10, 2), dtype=np.uint32)
    explicit[7, 1] = 8
    status = _compare(router, _logits(rng, 10, 8, 1.0), 2, "explicit id out of range", explicit_expert_ids=explicit)
    assert status == hip_router.STATUS_EXPERT_OUT_OF_RANGE


def test_error_statuses_and_their_precedence(router):
    rng = np.random.default_rng(5)
    logits = _logits(rng, 6, 8, 1.0)
    assert _compare(router, logits, 0, "top_k zero") == hip_router.STATUS_BAD_TOP_K
    assert _compare(router, logits, 9, "top_k above the expert count") == hip_router.STATUS_BAD_TOP_K
    assert _compare(router, logits, 2, "zero scaling factor", routed_scaling_factor=0.0) == hip_router.STATUS_BAD_SCALING
    assert _compare(router, logits, 2, "infinite scaling factor", routed_scaling_factor=float("inf")) == hip_router.STATUS_BAD_SCALING
    assert _compare(router, np.zeros((0, 8), dtype=np.float32), 2, "no tokens") == hip_router.STATUS_NO_TOKENS
    for bad in (np.nan, np.inf, -np.inf):
        broken = logits.copy()
        broken[4, 3] = bad
        assert _compare(router, broken, 2, "logit %r" % bad) == hip_router.STATUS_NON_FINITE_LOGIT
    # a non-finite logit in a later token outranks an out-of-range id in an earlier one
    broken = logits.copy()
    broken[5, 0] = np.nan
    explicit = np.zeros((6, 2), dtype=np.uint32)
    explicit[0, 0] = 99
    assert _compare(router, broken, 2, "NaN behind a bad id", explicit_expert_ids=explicit) == hip_router.STATUS_NON_FINITE_LOGIT
    # selected scores that sum to zero: sigmoid of very negative logits, chosen explicitly
    low = np.full((4, 8), -200.0, dtype=np.float32)
    low[:, 0] = 0.0
    explicit = np.tile(np.array([1, 2], dtype=np.uint32), (4, 1))
    assert _compare(router, low, 2, "zero selected sum", score_function=hip_router.SIGMOID,
                    explicit_expert_ids=explicit) == hip_router.STATUS_NON_POSITIVE_SUM
    assert _compare(router, low, 2, "zero selected sum, no renormalisation", score_function=hip_router.SIGMOID,
                    explicit_expert_ids=explicit, renormalize=False) == hip_router.STATUS_OK
    # the earliest failing token decides: token 1 has a bad id, token 0 a zero sum
    explicit[1, 0] = 8
    assert _compare(router, low, 2, "zero sum before a bad id", score_function=hip_router.SIGMOID,
                    explicit_expert_ids=explicit) == hip_router.STATUS_NON_POSITIVE_SUM
    explicit[0, 0] = 8
    assert _compare(router, low, 2, "bad id first", score_function=hip_router.SIGMOID,
                    explicit_expert_ids=explicit) == hip_router.STATUS_EXPERT_OUT_OF_RANGE
    # a good call after failed ones is unaffected
    assert _compare(router, logits, 2, "good call after failures") == hip_router.STATUS_OK


def test_extreme_logits(router):
    rng = np.random.default_rng(6)
    logits = _logits(rng, 64, 128, 1.0)
    logits[::2] *= 60.0       # saturating sigmoid / softplus branches (|x| > 20) and softmax underflow
    logits[1::4] = logits[1::4] * 1e-3
    logits[5, :] = 3.0e38
    logits[6, :] = -3.0e38
    for score in (hip_router.SOFTMAX, hip_router.SIGMOID, hip_router.SQRT_SOFTPLUS):
        for renormalize in (True, False):
            cpu_status, _, _ = oracle_lib.oracle_router_dispatch(logits, 4, score_function=score, renormalize=renormalize)
            _compare(router, logits, 4, "extreme logits score=%d renormalize=%s (oracle status %d)" % (score, renormalize, cpu_status),
                     score_function=score, renormalize=renormalize)


def test_device_log1pf_is_libm(router):
    """Every exponent range of positive floats, plus the branch points of the routine."""
    rng = np.random.default_rng(7)
    bits = rng.integers(1, 0x7f800000, size=2_000_000, dtype=np.uint32)
    edges = np.array([0x24800000, 0x247fffff, 0x31000000, 0x30ffffff, 0x3ed413d7, 0x3ed413d6, 0x5a000000, 0x59ffffff,
                      0x3f800000, 0x3f000000, 0x00000001, 0x7f7fffff, 0x7f800000, 0x3504f7 | 0x3f800000], dtype=np.uint32)
    values = np.concatenate([bits, edges]).view(np.float32)
    expected = oracle_lib.log1pf_libm(values)
    got = router.debug_log1pf(values)
    mismatches = int((got.view(np.uint32) != expected.view(np.uint32)).sum())
    assert mismatches == 0, "device log1pf differs from libm on %d of %d values" % (mismatches, values.size)


def test_device_entry_on_a_stream(router):
    """dispatch_device with torch-owned device arrays on a side stream, twice in a row with different sizes."""
    rng = np.random.default_rng(8)
    stream = torch.cuda.Stream()
    for tokens, experts, top_k in [(3000, 256, 8), (100, 64, 6)]:
        _announce("device entry T=%d E=%d K=%d" % (tokens, experts, top_k))
        logits = _logits(rng, tokens, experts, 2.0)
        device_logits = torch.from_numpy(logits).cuda()
        offsets = torch.zeros(experts + 1, dtype=torch.int32, device="cuda")
        routes = torch.zeros(tokens * top_k * 3, dtype=torch.int32, device="cuda")
        status = torch.full((1,), 77, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        options = hip_router.make_options(experts, top_k, hip_router.SIGMOID, True, 2.5)
        with torch.cuda.stream(stream):
            host_status = router.dispatch_device(device_logits.data_ptr(), tokens, options, offsets.data_ptr(),
                                                 routes.data_ptr(), status.data_ptr(), stream=stream.cuda_stream)
        stream.synchronize()
        assert host_status == 0 and int(status.item()) == 0
        cpu_status, cpu_offsets, cpu_routes = oracle_lib.oracle_router_dispatch(
            logits, top_k, score_function=hip_router.SIGMOID, routed_scaling_factor=2.5)
        assert np.array_equal(offsets.cpu().numpy().view(np.uint32), cpu_offsets)
        got = routes.cpu().numpy().view(np.uint32).reshape(-1, 3)
        assert np.array_equal(got[:, 0], cpu_routes["token_index"]) and np.array_equal(got[:, 1], cpu_routes["rank"])
        assert np.array_equal(got[:, 2], cpu_routes["weight"].view(np.uint32))


def test_capacity_limits_are_reported(router):
    with pytest.raises(hip_router.RouterError):
        router.dispatch(np.zeros((8193, 4), dtype=np.float32), 2)
    with pytest.raises(hip_router.RouterError):
        router.dispatch(np.zeros((4, 1025), dtype=np.float32), 2)
    with pytest.raises(hip_router.RouterError):
        router.dispatch(np.zeros((4, 128), dtype=np.float32), 65)
    with pytest.raises(hip_router.RouterError):
        hip_router.HipRouter(16, max_experts=2048)
