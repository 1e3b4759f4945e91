"""ctypes bindings for the CPU oracle (oracle/libsampler_oracle.so) and, where it has been built,
the reference library driver (oracle/_ref/libref_sampler.so).  Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libsampler_oracle.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libref_sampler.so")

STATUS_OK = 0
STATUS_EMPTY_LOGITS = 1
STATUS_BAD_TEMPERATURE = 2
STATUS_BAD_TOP_P = 3
STATUS_BAD_MIN_P = 4
STATUS_NO_FINITE_LOGIT = 5
STATUS_INVALID_DISTRIBUTION = 6

STATUS_MESSAGES = {
    STATUS_EMPTY_LOGITS: "cannot sample empty logits",
    STATUS_BAD_TEMPERATURE: "temperature must be finite and non-negative",
    STATUS_BAD_TOP_P: "top_p must be in the range (0, 1]",
    STATUS_BAD_MIN_P: "min_p must be in the range [0, 1]",
    STATUS_NO_FINITE_LOGIT: "sampling requires at least one finite logit",
    STATUS_INVALID_DISTRIBUTION: "sampling distribution is invalid",
}


class SamplingOptions(ctypes.Structure):
    _fields_ = [("temperature", ctypes.c_float), ("top_k", ctypes.c_uint32),
                ("top_p", ctypes.c_float), ("min_p", ctypes.c_float)]


ROW_PARAMS_DTYPE = np.dtype([("temperature", "<f4"), ("top_k", "<u4"), ("top_p", "<f4"),
                             ("min_p", "<f4"), ("stop_begin", "<u4"), ("stop_count", "<u4")])

VERIFY_RESULT_DTYPE = np.dtype([("accepted", "<u4"), ("next_token_id", "<i4"), ("next_probability", "<f4"),
                                ("status", "<u4"), ("row_status", "<u4"), ("accept_draws", "<u4"),
                                ("final_draw_consumed", "<u4"), ("next_is_residual", "<u4")])
VERIFY_MESSAGES = {
    2: "sampled draft token has zero probability",
    3: "speculative residual distribution is empty",
    4: "speculative residual sampling failed",
}

ORACLE_RESULT_DTYPE = np.dtype([("token_id", "<i4"), ("probability", "<f4"), ("kept_count", "<u4"),
                                ("status", "u1"), ("is_stop", "u1"), ("draw_consumed", "u1"),
                                ("has_nan", "u1"), ("cdf_gap", "<f4"), ("top_p_gap", "<f4")])


def build_oracle():
    subprocess.run(["make", "-C", ORACLE_DIR, "oracle"], check=True, stdout=subprocess.DEVNULL)


_oracle = None


def oracle():
    global _oracle
    if _oracle is not None:
        return _oracle
    if not os.path.exists(ORACLE_SO):
        build_oracle()
    lib = ctypes.CDLL(ORACLE_SO)
    f32p = ctypes.POINTER(ctypes.c_float)
    lib.oracle_status_message.restype = ctypes.c_char_p
    lib.oracle_status_message.argtypes = [ctypes.c_int]
    lib.oracle_validate_sampling_options.argtypes = [ctypes.POINTER(SamplingOptions)]
    lib.oracle_sampling_distribution.argtypes = [
        ctypes.c_void_p, ctypes.c_size_t, ctypes.POINTER(SamplingOptions),
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_size_t)]
    lib.oracle_sample.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.POINTER(SamplingOptions),
                                  ctypes.c_float, ctypes.c_void_p]
    lib.oracle_sample_batch.argtypes = [
        ctypes.c_void_p, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64,
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
    lib.oracle_candidate_probability.restype = ctypes.c_float
    lib.oracle_candidate_probability.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32]
    lib.oracle_sample_residual_distribution.argtypes = [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
        ctypes.c_size_t, ctypes.c_float, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_float)]
    lib.oracle_speculative_verify.argtypes = [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32, ctypes.POINTER(SamplingOptions),
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.oracle_router_status_message.restype = ctypes.c_char_p
    lib.oracle_router_status_message.argtypes = [ctypes.c_int]
    lib.oracle_router_scores.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p]
    lib.oracle_log1pf_libm_array.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
    lib.oracle_log1pf_libm_array.restype = None
    lib.oracle_router_dispatch.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.oracle_bfloat16_to_float.restype = ctypes.c_float
    lib.oracle_bfloat16_to_float.argtypes = [ctypes.c_uint16]
    lib.oracle_float_to_bfloat16.restype = ctypes.c_uint16
    lib.oracle_float_to_bfloat16.argtypes = [ctypes.c_float]
    lib.oracle_quantize_bfloat16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
    lib.oracle_rng_create.restype = ctypes.c_void_p
    lib.oracle_rng_create.argtypes = [ctypes.c_uint64]
    lib.oracle_rng_destroy.argtypes = [ctypes.c_void_p]
    lib.oracle_rng_uniform.restype = ctypes.c_float
    lib.oracle_rng_uniform.argtypes = [ctypes.c_void_p]
    lib.oracle_expf_libm.restype = ctypes.c_float
    lib.oracle_expf_libm.argtypes = [ctypes.c_float]
    lib.oracle_expf_restated.restype = ctypes.c_float
    lib.oracle_expf_restated.argtypes = [ctypes.c_float]
    lib.oracle_expf_libm_array.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
    lib.oracle_expf_compare_range.restype = ctypes.c_uint64
    lib.oracle_expf_compare_range.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32]
    _oracle = lib
    return lib


def oracle_distribution(logits, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0):
    """Returns (status, ids, probabilities) for one fp32 row."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    options = SamplingOptions(temperature, top_k, top_p, min_p)
    cap = max(1, logits.size)
    ids = np.empty(cap, dtype=np.int32)
    probs = np.empty(cap, dtype=np.float32)
    count = ctypes.c_size_t(0)
    status = oracle().oracle_sampling_distribution(
        logits.ctypes.data, logits.size, ctypes.byref(options),
        ids.ctypes.data, probs.ctypes.data, cap, ctypes.byref(count))
    return status, ids[:count.value].copy(), probs[:count.value].copy()


def oracle_sample(logits, uniform, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0):
    """Returns a 1-element ORACLE_RESULT_DTYPE record for one fp32 row."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    options = SamplingOptions(temperature, top_k, top_p, min_p)
    result = np.zeros(1, dtype=ORACLE_RESULT_DTYPE)
    oracle().oracle_sample(logits.ctypes.data, logits.size, ctypes.byref(options),
                           ctypes.c_float(uniform), result.ctypes.data)
    return result[0]


def oracle_sample_batch(logits, params, uniforms, stop_ids=None, threads=1, vocab=None):
    """logits: [rows, stride] float32 or uint16 (bf16 bits); params: ROW_PARAMS_DTYPE[rows]."""
    logits = np.ascontiguousarray(logits)
    assert logits.ndim == 2 and logits.dtype in (np.float32, np.uint16)
    rows, stride = logits.shape
    vocab = stride if vocab is None else vocab
    params = np.ascontiguousarray(params, dtype=ROW_PARAMS_DTYPE)
    uniforms = np.ascontiguousarray(uniforms, dtype=np.float32)
    assert params.shape == (rows,) and uniforms.shape == (rows,)
    stops = None if stop_ids is None else np.ascontiguousarray(stop_ids, dtype=np.int32)
    results = np.zeros(rows, dtype=ORACLE_RESULT_DTYPE)
    rc = oracle().oracle_sample_batch(
        logits.ctypes.data, 0 if logits.dtype == np.float32 else 1, rows, vocab, stride,
        params.ctypes.data, uniforms.ctypes.data,
        None if stops is None else stops.ctypes.data, results.ctypes.data, threads)
    assert rc == 0
    return results


def oracle_candidate_probability(ids, probabilities, token_id):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    probabilities = np.ascontiguousarray(probabilities, dtype=np.float32)
    return oracle().oracle_candidate_probability(ids.ctypes.data, probabilities.ctypes.data, ids.size, int(token_id))


def oracle_sample_residual(target_ids, target_probabilities, draft_ids, draft_probabilities, vocab, canonical_uniform):
    """Returns (status, token_id, probability)."""
    target_ids = np.ascontiguousarray(target_ids, dtype=np.int32)
    target_probabilities = np.ascontiguousarray(target_probabilities, dtype=np.float32)
    draft_ids = np.ascontiguousarray(draft_ids, dtype=np.int32)
    draft_probabilities = np.ascontiguousarray(draft_probabilities, dtype=np.float32)
    token = ctypes.c_int32(-1)
    probability = ctypes.c_float(0.0)
    status = oracle().oracle_sample_residual_distribution(
        target_ids.ctypes.data, target_probabilities.ctypes.data, target_ids.size,
        draft_ids.ctypes.data, draft_probabilities.ctypes.data, draft_ids.size,
        vocab, ctypes.c_float(canonical_uniform), ctypes.byref(token), ctypes.byref(probability))
    return status, token.value, probability.value


def oracle_speculative_verify(target_logits, draft_logits, proposed_token_ids, uniforms,
                              temperature=1.0, top_k=0, top_p=1.0, min_p=0.0):
    """target_logits [D + 1, V], draft_logits [D, V] fp32.  Returns (VERIFY_RESULT_DTYPE record, accepted[D])."""
    target_logits = np.ascontiguousarray(target_logits, dtype=np.float32)
    draft_logits = np.ascontiguousarray(draft_logits, dtype=np.float32)
    proposed = np.ascontiguousarray(proposed_token_ids, dtype=np.int32)
    uniforms = np.ascontiguousarray(uniforms, dtype=np.float32)
    drafts = proposed.size
    assert target_logits.shape[0] == drafts + 1 and draft_logits.shape[0] == drafts and uniforms.size == drafts + 1
    options = SamplingOptions(temperature, top_k, top_p, min_p)
    accepted = np.zeros(max(drafts, 1), dtype=np.float32)
    result = np.zeros(1, dtype=VERIFY_RESULT_DTYPE)
    oracle().oracle_speculative_verify(
        target_logits.ctypes.data, draft_logits.ctypes.data, target_logits.shape[1], drafts,
        ctypes.byref(options), proposed.ctypes.data, uniforms.ctypes.data, accepted.ctypes.data, result.ctypes.data)
    return result[0], accepted[:drafts]


def expf_libm(values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty_like(values)
    oracle().oracle_expf_libm_array(values.ctypes.data, out.ctypes.data, values.size)
    return out


def quantize_bf16(values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(values.shape, dtype=np.uint16)
    oracle().oracle_quantize_bfloat16(values.ctypes.data, out.ctypes.data, values.size)
    return out


def widen_bf16(bits):
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


class OracleRng:
    """std::mt19937_64(seed) + std::uniform_real_distribution<float>(0, 1), one draw per call."""

    def __init__(self, seed):
        self._handle = oracle().oracle_rng_create(seed)

    def uniform(self):
        return float(oracle().oracle_rng_uniform(self._handle))

    def __del__(self):
        if getattr(self, "_handle", None):
            oracle().oracle_rng_destroy(self._handle)
            self._handle = None


_ref = None


def reference_available():
    return os.path.exists(REF_SO)


def reference():
    """The reference library driver; only present where the reference checkout was built."""
    global _ref
    if _ref is not None:
        return _ref
    lib = ctypes.CDLL(REF_SO)
    lib.ref_session_create.restype = ctypes.c_void_p
    lib.ref_session_create.argtypes = [ctypes.c_uint64, ctypes.c_char_p, ctypes.c_size_t]
    lib.ref_session_destroy.argtypes = [ctypes.c_void_p]
    lib.ref_session_sample.argtypes = [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_uint32,
        ctypes.c_float, ctypes.c_float, ctypes.POINTER(ctypes.c_int32),
        ctypes.POINTER(ctypes.c_float), ctypes.c_char_p, ctypes.c_size_t]
    lib.ref_sampling_distribution.argtypes = [
        ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_uint32, ctypes.c_float,
        ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
        ctypes.POINTER(ctypes.c_size_t), ctypes.c_char_p, ctypes.c_size_t]
    lib.ref_sample_rows.argtypes = [ctypes.c_void_p] * 2 + [ctypes.c_uint32, ctypes.c_uint32,
                                                            ctypes.c_uint64] + [ctypes.c_void_p] * 11 + [ctypes.c_int]
    lib.ref_candidate_probability.restype = ctypes.c_float
    lib.ref_candidate_probability.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32]
    lib.ref_sample_residual_distribution.argtypes = [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
        ctypes.c_size_t, ctypes.c_uint64, ctypes.c_uint64, ctypes.POINTER(ctypes.c_int32),
        ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_uint64), ctypes.c_char_p, ctypes.c_size_t]
    lib.ref_router_dispatch.argtypes = [
        ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
        ctypes.c_uint32, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64), ctypes.c_char_p, ctypes.c_size_t]
    lib.ref_bfloat16_to_float.restype = ctypes.c_float
    lib.ref_bfloat16_to_float.argtypes = [ctypes.c_uint16]
    lib.ref_float_to_bfloat16.restype = ctypes.c_uint16
    lib.ref_float_to_bfloat16.argtypes = [ctypes.c_float]
    _ref = lib
    return lib


class ReferenceSession:
    """A real reference Session (seeded) whose sample() is called on arbitrary rows."""

    def __init__(self, seed):
        message = ctypes.create_string_buffer(256)
        self._handle = reference().ref_session_create(seed, message, 256)
        if not self._handle:
            raise RuntimeError("reference session: " + message.value.decode())

    @property
    def handle(self):
        return self._handle

    def sample(self, logits, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0):
        """Returns (error_code_plus_one_or_zero, token_id, probability, message)."""
        logits = np.ascontiguousarray(logits, dtype=np.float32)
        token = ctypes.c_int32(-1)
        prob = ctypes.c_float(0.0)
        message = ctypes.create_string_buffer(256)
        rc = reference().ref_session_sample(
            self._handle, logits.ctypes.data, logits.size, temperature, top_k, top_p, min_p,
            ctypes.byref(token), ctypes.byref(prob), message, 256)
        return rc, token.value, prob.value, message.value.decode()

    def __del__(self):
        if getattr(self, "_handle", None):
            reference().ref_session_destroy(self._handle)
            self._handle = None


def reference_distribution(logits, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0):
    """Returns (rc, ids, probabilities, message) from the reference's own sampling_distribution."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    cap = max(1, logits.size)
    ids = np.empty(cap, dtype=np.int32)
    probs = np.empty(cap, dtype=np.float32)
    count = ctypes.c_size_t(0)
    message = ctypes.create_string_buffer(256)
    rc = reference().ref_sampling_distribution(
        logits.ctypes.data, logits.size, temperature, top_k, top_p, min_p,
        ids.ctypes.data, probs.ctypes.data, cap, ctypes.byref(count), message, 256)
    return rc, ids[:count.value].copy(), probs[:count.value].copy(), message.value.decode()


def reference_sample_residual(target_ids, target_probabilities, draft_ids, draft_probabilities, vocab, seed, discard=0):
    """The reference's own sample_residual_distribution with mt19937_64(seed) advanced by `discard`.
    Returns (rc, token_id, probability, draws consumed, message)."""
    target_ids = np.ascontiguousarray(target_ids, dtype=np.int32)
    target_probabilities = np.ascontiguousarray(target_probabilities, dtype=np.float32)
    draft_ids = np.ascontiguousarray(draft_ids, dtype=np.int32)
    draft_probabilities = np.ascontiguousarray(draft_probabilities, dtype=np.float32)
    token = ctypes.c_int32(-1)
    probability = ctypes.c_float(0.0)
    draws = ctypes.c_uint64(0)
    message = ctypes.create_string_buffer(256)
    rc = reference().ref_sample_residual_distribution(
        target_ids.ctypes.data, target_probabilities.ctypes.data, target_ids.size,
        draft_ids.ctypes.data, draft_probabilities.ctypes.data, draft_ids.size,
        vocab, seed, discard, ctypes.byref(token), ctypes.byref(probability), ctypes.byref(draws), message, 256)
    return rc, token.value, probability.value, draws.value, message.value.decode()


def reference_candidate_probability(ids, probabilities, token_id):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    probabilities = np.ascontiguousarray(probabilities, dtype=np.float32)
    return reference().ref_candidate_probability(ids.ctypes.data, probabilities.ctypes.data, ids.size, int(token_id))


# ---- expert router (MoE token dispatch)

ROUTER_SOFTMAX, ROUTER_SIGMOID, ROUTER_SQRT_SOFTPLUS = 0, 1, 2
ROUTER_OPTIONS_DTYPE = np.dtype([("expert_count", "<u4"), ("top_k", "<u4"), ("score_function", "<u4"),
                                 ("renormalize", "<u4"), ("routed_scaling_factor", "<f4")])
ROUTE_DTYPE = np.dtype([("token_index", "<u4"), ("rank", "<u4"), ("weight", "<f4")])
ROUTER_MESSAGES = {
    1: "expert dispatch requires at least one token",
    2: "expert dispatch requires 0 < top_k <= expert_count",
    3: "routed scaling factor must be finite and positive",
    4: "router logits must be finite",
    5: "explicit expert id is out of range",
    6: "selected router weights have a non-positive sum",
}


def router_options(expert_count, top_k, score_function=ROUTER_SOFTMAX, renormalize=True, routed_scaling_factor=1.0):
    options = np.zeros(1, dtype=ROUTER_OPTIONS_DTYPE)
    options[0] = (expert_count, top_k, score_function, 1 if renormalize else 0, routed_scaling_factor)
    return options


def log1pf_libm(values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty_like(values)
    oracle().oracle_log1pf_libm_array(values.ctypes.data, out.ctypes.data, values.size)
    return out


def oracle_router_scores(logits, score_function):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    scores = np.empty_like(logits)
    oracle().oracle_router_scores(logits.ctypes.data, logits.size, score_function, scores.ctypes.data)
    return scores


def oracle_router_dispatch(router_logits, top_k, score_function=ROUTER_SOFTMAX, renormalize=True,
                           routed_scaling_factor=1.0, selection_bias=None, explicit_expert_ids=None):
    """router_logits [tokens, experts] fp32.  Returns (status, expert_offsets[experts + 1], routes ROUTE_DTYPE)."""
    router_logits = np.ascontiguousarray(router_logits, dtype=np.float32)
    tokens, experts = router_logits.shape
    options = router_options(experts, top_k, score_function, renormalize, routed_scaling_factor)
    bias = None if selection_bias is None else np.ascontiguousarray(selection_bias, dtype=np.float32)
    explicit = None if explicit_expert_ids is None else np.ascontiguousarray(explicit_expert_ids, dtype=np.uint32)
    offsets = np.zeros(experts + 1, dtype=np.uint32)
    routes = np.zeros(max(1, tokens * max(top_k, 1)), dtype=ROUTE_DTYPE)
    status = oracle().oracle_router_dispatch(
        router_logits.ctypes.data, tokens, options.ctypes.data, None if bias is None else bias.ctypes.data,
        None if explicit is None else explicit.ctypes.data, offsets.ctypes.data, routes.ctypes.data)
    count = int(offsets[-1]) if status == 0 else 0
    return status, offsets, routes[:count].copy()


def reference_router_dispatch(router_logits, top_k, score_function=ROUTER_SOFTMAX, normalization=1, flags=1,
                              routed_scaling_factor=1.0, selection_bias=None, explicit_expert_ids=None,
                              use_dispatch_into=False):
    """The reference's own ExpertDispatcher.  Returns (rc, expert_offsets, routes ROUTE_DTYPE, message)."""
    router_logits = np.ascontiguousarray(router_logits, dtype=np.float32)
    tokens, experts = router_logits.shape
    bias = None if selection_bias is None else np.ascontiguousarray(selection_bias, dtype=np.float32)
    explicit = None if explicit_expert_ids is None else np.ascontiguousarray(explicit_expert_ids, dtype=np.uint32)
    cap = max(1, tokens * max(top_k, 1))
    offsets = np.zeros(experts + 1, dtype=np.uint32)
    route_tokens = np.zeros(cap, dtype=np.uint32)
    route_ranks = np.zeros(cap, dtype=np.uint32)
    route_weights = np.zeros(cap, dtype=np.float32)
    assignments = ctypes.c_uint64(0)
    message = ctypes.create_string_buffer(256)
    rc = reference().ref_router_dispatch(
        router_logits.ctypes.data, tokens, experts, top_k, score_function, normalization, flags,
        ctypes.c_float(routed_scaling_factor), None if bias is None else bias.ctypes.data,
        None if explicit is None else explicit.ctypes.data, 1 if use_dispatch_into else 0,
        offsets.ctypes.data, route_tokens.ctypes.data, route_ranks.ctypes.data, route_weights.ctypes.data,
        ctypes.byref(assignments), message, 256)
    count = int(offsets[-1]) if rc == 0 else 0
    routes = np.zeros(count, dtype=ROUTE_DTYPE)
    routes["token_index"], routes["rank"], routes["weight"] = route_tokens[:count], route_ranks[:count], route_weights[:count]
    return rc, offsets, routes, message.value.decode()
