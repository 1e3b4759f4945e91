"""ctypes binding of libncnn_moe_hip_sampler.so (include/ncnn_moe_hip_sampler.h).

There is no CPU fallback: if the library is missing or no GPU is visible, calls raise.
"""
import ctypes
import os

import numpy as np

PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(PACKAGE_DIR, "libncnn_moe_hip_sampler.so")
TESTING_LIBRARY_PATH = os.path.join(PACKAGE_DIR, "libncnn_moe_hip_sampler_testing.so")

LOGITS_F32 = 0
LOGITS_BF16 = 1

RC_SUCCESS = 0
RC_INVALID_ARGUMENT = 1
RC_HIP_ERROR = 2
RC_NO_DEVICE = 3

ROW_OK = 0
ROW_EMPTY_LOGITS = 1
ROW_BAD_TEMPERATURE = 2
ROW_BAD_TOP_P = 3
ROW_BAD_MIN_P = 4
ROW_NO_FINITE_LOGIT = 5
ROW_INVALID_DISTRIBUTION = 6
ROW_NEEDS_FULL_ORDER = 7

VERIFY_OK = 0
VERIFY_ROW_ERROR = 1
VERIFY_ZERO_DRAFT_PROBABILITY = 2
VERIFY_RESIDUAL_EMPTY = 3
VERIFY_RESIDUAL_FAILED = 4
VERIFY_UNSUPPORTED_WINDOW = 5
PASSES_FULL_ORDER = 1     # sample_device: the later passes are enqueued as well
PASSES_SIDE_BY_SIDE = 2   # ... and run side by side (rows with wide windows and rows without a window are both present)
PASSES_NO_WIDE_WINDOWS = 4  # ... but no row has 64 < top_k <= 1024: the select kernel for such windows is left out
MAX_DRAFT_TOKENS = 16

FLAG_HAS_NAN = 1
FLAG_GENERAL_PATH = 2
FLAG_FALLBACK = 4

PARAMS_DTYPE = np.dtype([("temperature", "<f4"), ("top_k", "<u4"), ("top_p", "<f4"),
                         ("min_p", "<f4"), ("stop_begin", "<u4"), ("stop_count", "<u4")])
RESULT_DTYPE = np.dtype([("token_id", "<i4"), ("probability", "<f4"), ("kept_count", "<u4"),
                         ("status", "u1"), ("is_stop", "u1"), ("draw_consumed", "u1"), ("flags", "u1")])
VERIFY_RESULT_DTYPE = np.dtype([("accepted", "<u4"), ("next_token_id", "<i4"), ("next_probability", "<f4"),
                                ("status", "<u4"), ("row_status", "<u4"), ("accept_draws", "<u4"),
                                ("final_draw_consumed", "<u4"), ("next_is_residual", "<u4")])

EXPORTED_SYMBOLS = [
    "ncnn_moe_hip_sampler_create",
    "ncnn_moe_hip_sampler_destroy",
    "ncnn_moe_hip_sampler_logits_buffer",
    "ncnn_moe_hip_sampler_upload_logits",
    "ncnn_moe_hip_sampler_sample",
    "ncnn_moe_hip_sampler_sample_device",
    "ncnn_moe_hip_sampler_sample_device_static",
    "ncnn_moe_hip_sampler_distribution",
    "ncnn_moe_hip_sampler_speculative_verify",
    "ncnn_moe_hip_sampler_verify_status_message",
    "ncnn_moe_hip_sampler_last_error",
    "ncnn_moe_hip_sampler_status_message",
    "ncnn_moe_hip_sampler_device_count",
]

# include/ncnn_moe_hip_sampler_testing.h: hooks for this repository's tests
TESTING_SYMBOLS = [
    "ncnn_moe_hip_sampler_debug_force_general",
    "ncnn_moe_hip_sampler_debug_scatter_segments",
    "ncnn_moe_hip_sampler_debug_spread_sort",
    "ncnn_moe_hip_sampler_debug_fused_bf16",
    "ncnn_moe_hip_sampler_debug_partial_sort",
    "ncnn_moe_hip_sampler_debug_sort_lengths",
    "ncnn_moe_hip_sampler_debug_skip_low_digit",
    "ncnn_moe_hip_sampler_debug_wide_sampled_bound",
    "ncnn_moe_hip_sampler_debug_disordered_rows",
    "ncnn_moe_hip_sampler_debug_chunk_steps",
    "ncnn_moe_hip_sampler_debug_stream_only",
    "ncnn_moe_hip_sampler_debug_set_row_epochs",
    "ncnn_moe_hip_sampler_debug_expf",
    "ncnn_moe_hip_sampler_debug_exp2_table",
    "ncnn_moe_hip_sampler_debug_select_geometry",
]


class SamplerError(RuntimeError):
    pass


_library = None
_testing_library = None


def _bind(lib, testing):
    vp = ctypes.c_void_p
    lib.ncnn_moe_hip_sampler_create.argtypes = [ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(vp)]
    lib.ncnn_moe_hip_sampler_destroy.argtypes = [vp]
    lib.ncnn_moe_hip_sampler_destroy.restype = None
    lib.ncnn_moe_hip_sampler_logits_buffer.argtypes = [
        vp, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(vp), ctypes.POINTER(ctypes.c_uint64)]
    lib.ncnn_moe_hip_sampler_upload_logits.argtypes = [vp, vp, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64]
    lib.ncnn_moe_hip_sampler_sample.argtypes = [vp, ctypes.c_uint32, vp, vp, vp, ctypes.c_uint32, vp]
    lib.ncnn_moe_hip_sampler_sample_device.argtypes = [
        vp, vp, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64, vp, vp, vp, vp, ctypes.c_int, vp]
    lib.ncnn_moe_hip_sampler_sample_device_static.argtypes = [
        ctypes.c_int, vp, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64, vp, vp, vp, vp, vp]
    lib.ncnn_moe_hip_sampler_distribution.argtypes = [
        vp, ctypes.c_uint32, vp, ctypes.c_uint32, vp, vp, ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32)]
    lib.ncnn_moe_hip_sampler_speculative_verify.argtypes = [vp, ctypes.c_uint32, vp, vp, vp, vp, vp]
    lib.ncnn_moe_hip_sampler_verify_status_message.argtypes = [ctypes.c_int]
    lib.ncnn_moe_hip_sampler_verify_status_message.restype = ctypes.c_char_p
    lib.ncnn_moe_hip_sampler_last_error.argtypes = [vp]
    lib.ncnn_moe_hip_sampler_last_error.restype = ctypes.c_char_p
    lib.ncnn_moe_hip_sampler_status_message.argtypes = [ctypes.c_int]
    lib.ncnn_moe_hip_sampler_status_message.restype = ctypes.c_char_p
    lib.ncnn_moe_hip_sampler_device_count.argtypes = []
    if not testing:
        return lib
    lib.ncnn_moe_hip_sampler_debug_force_general.argtypes = [vp, ctypes.c_int]
    lib.ncnn_moe_hip_sampler_debug_scatter_segments.argtypes = [vp, ctypes.c_int]
    lib.ncnn_moe_hip_sampler_debug_spread_sort.argtypes = [vp, ctypes.c_int]
    lib.ncnn_moe_hip_sampler_debug_partial_sort.argtypes = [vp, ctypes.c_int]
    lib.ncnn_moe_hip_sampler_debug_sort_lengths.argtypes = [vp, vp, ctypes.c_uint32]
    lib.ncnn_moe_hip_sampler_debug_skip_low_digit.argtypes = [vp, ctypes.c_int]
    lib.ncnn_moe_hip_sampler_debug_wide_sampled_bound.argtypes = [vp, ctypes.c_int]
    lib.ncnn_moe_hip_sampler_debug_disordered_rows.argtypes = [vp, vp, ctypes.c_uint32]
    lib.ncnn_moe_hip_sampler_debug_fused_bf16.argtypes = [vp, ctypes.c_int]
    lib.ncnn_moe_hip_sampler_debug_chunk_steps.argtypes = [vp, ctypes.c_int]
    lib.ncnn_moe_hip_sampler_debug_stream_only.argtypes = [vp, vp, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64, vp]
    lib.ncnn_moe_hip_sampler_debug_set_row_epochs.argtypes = [vp, ctypes.c_int, ctypes.c_uint32]
    lib.ncnn_moe_hip_sampler_debug_expf.argtypes = [vp, vp, vp, ctypes.c_size_t]
    lib.ncnn_moe_hip_sampler_debug_exp2_table.argtypes = [vp]
    lib.ncnn_moe_hip_sampler_debug_exp2_table.restype = None
    lib.ncnn_moe_hip_sampler_debug_select_geometry.argtypes = [
        ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32),
        ctypes.POINTER(ctypes.c_uint32)]
    return lib


def load_library():
    """Loads the C-ABI library (the boundary of include/ncnn_moe_hip_sampler.h); raises if it has not been built."""
    global _library
    if _library is not None:
        return _library
    if not os.path.exists(LIBRARY_PATH):
        raise SamplerError(
            "%s is missing: build it with `make -C %s` (or __graft_entry__.build())" % (LIBRARY_PATH, PACKAGE_DIR))
    _library = _bind(ctypes.CDLL(LIBRARY_PATH), False)
    return _library


def load_testing_library():
    """Loads the testing build of the library: the same source with the hooks of
    include/ncnn_moe_hip_sampler_testing.h compiled in.  For this repository's tests and the benchmark's probes."""
    global _testing_library
    if _testing_library is not None:
        return _testing_library
    if not os.path.exists(TESTING_LIBRARY_PATH):
        raise SamplerError(
            "%s is missing: build it with `make -C %s` (or __graft_entry__.build())" % (TESTING_LIBRARY_PATH, PACKAGE_DIR))
    _testing_library = _bind(ctypes.CDLL(TESTING_LIBRARY_PATH), True)
    return _testing_library


def status_message(row_status):
    """The CPU sampler's message for a per-row status."""
    return load_library().ncnn_moe_hip_sampler_status_message(int(row_status)).decode()


def verify_status_message(verify_status):
    return load_library().ncnn_moe_hip_sampler_verify_status_message(int(verify_status)).decode()


GEOMETRY_WHOLE_ROW = 0
GEOMETRY_SPLIT_ONE_CHUNK = 1
GEOMETRY_SPLIT_LOOPED = 2


def select_geometry(dtype, rows, vocab):
    """(workgroups per row, chunks per workgroup, kernel variant) of the first select kernel for this shape."""
    segments, chunks, variant = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()
    rc = load_testing_library().ncnn_moe_hip_sampler_debug_select_geometry(
        dtype, rows, vocab, ctypes.byref(segments), ctypes.byref(chunks), ctypes.byref(variant))
    if rc != RC_SUCCESS:
        raise SamplerError("select_geometry: rc=%d" % rc)
    return segments.value, chunks.value, variant.value


def exp2_table():
    out = np.zeros(32, dtype=np.uint64)
    load_testing_library().ncnn_moe_hip_sampler_debug_exp2_table(out.ctypes.data)
    return out


def make_params(rows, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0):
    params = np.zeros(rows, dtype=PARAMS_DTYPE)
    params["temperature"] = temperature
    params["top_k"] = top_k
    params["top_p"] = top_p
    params["min_p"] = min_p
    return params


class HipSampler:
    """One sampler handle on one device.  testing=True creates it in the testing build of the library, whose
    handles take the test hooks (force_general, scatter_segments, ...)."""

    def __init__(self, max_rows, max_vocab, device=0, testing=False):
        self._testing = bool(testing)
        self._lib = load_testing_library() if testing else load_library()
        self._handle = ctypes.c_void_p()
        rc = self._lib.ncnn_moe_hip_sampler_create(device, max_rows, max_vocab, ctypes.byref(self._handle))
        if rc != RC_SUCCESS:
            self._handle = ctypes.c_void_p()
            raise SamplerError("ncnn_moe_hip_sampler_create failed with code %d (no GPU or out of memory?)" % rc)
        self.max_rows = max_rows
        self.max_vocab = max_vocab

    def close(self):
        if getattr(self, "_handle", None) and self._handle.value:
            self._lib.ncnn_moe_hip_sampler_destroy(self._handle)
            self._handle = ctypes.c_void_p()

    def __del__(self):
        self.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def handle(self):
        return self._handle

    def _check(self, rc):
        if rc != RC_SUCCESS:
            raise SamplerError("rc=%d: %s" % (rc, self._lib.ncnn_moe_hip_sampler_last_error(self._handle).decode()))

    def logits_buffer(self, dtype, rows, vocab):
        pointer = ctypes.c_void_p()
        stride = ctypes.c_uint64()
        self._check(self._lib.ncnn_moe_hip_sampler_logits_buffer(
            self._handle, dtype, rows, vocab, ctypes.byref(pointer), ctypes.byref(stride)))
        return pointer.value, stride.value

    def upload_logits(self, logits, vocab=None):
        """logits: [rows, stride] float32, or uint16 holding bf16 bit patterns."""
        logits = np.ascontiguousarray(logits)
        if logits.ndim != 2 or logits.dtype not in (np.float32, np.uint16):
            raise ValueError("logits must be a 2-D float32 or uint16 (bf16 bits) array")
        rows, stride = logits.shape
        vocab = stride if vocab is None else vocab
        dtype = LOGITS_F32 if logits.dtype == np.float32 else LOGITS_BF16
        pointer = logits.ctypes.data if logits.size else ctypes.c_void_p(8)
        self._check(self._lib.ncnn_moe_hip_sampler_upload_logits(self._handle, pointer, dtype, rows, vocab, stride))

    def sample(self, params, uniforms, stop_ids=None):
        params = np.ascontiguousarray(params, dtype=PARAMS_DTYPE)
        uniforms = np.ascontiguousarray(uniforms, dtype=np.float32)
        rows = params.shape[0]
        if uniforms.shape != (rows,):
            raise ValueError("one uniform per row is required")
        stops = None if stop_ids is None else np.ascontiguousarray(stop_ids, dtype=np.int32)
        results = np.zeros(rows, dtype=RESULT_DTYPE)
        self._check(self._lib.ncnn_moe_hip_sampler_sample(
            self._handle, rows, params.ctypes.data, uniforms.ctypes.data,
            None if stops is None or stops.size == 0 else stops.ctypes.data,
            0 if stops is None else stops.size, results.ctypes.data))
        return results

    def sample_device(self, logits_ptr, dtype, rows, vocab, row_stride, params_ptr, uniforms_ptr,
                      stop_ids_ptr, results_ptr, may_need_full_order=True, stream=None):
        """All pointers are device addresses (ints); enqueues and returns."""
        self._check(self._lib.ncnn_moe_hip_sampler_sample_device(
            self._handle, logits_ptr, dtype, rows, vocab, row_stride, params_ptr, uniforms_ptr,
            stop_ids_ptr, results_ptr, int(may_need_full_order), stream))

    def distribution(self, row, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, cap=None):
        """Returns (row_status, ids, probabilities) for one row of the uploaded logits."""
        params = make_params(1, temperature, top_k, top_p, min_p)
        cap = self.max_vocab if cap is None else cap
        ids = np.empty(max(cap, 1), dtype=np.int32)
        probabilities = np.empty(max(cap, 1), dtype=np.float32)
        count = ctypes.c_uint32()
        status = ctypes.c_uint32()
        self._check(self._lib.ncnn_moe_hip_sampler_distribution(
            self._handle, row, params.ctypes.data, cap, ids.ctypes.data, probabilities.ctypes.data,
            ctypes.byref(count), ctypes.byref(status)))
        n = min(count.value, cap)
        return status.value, ids[:n].copy(), probabilities[:n].copy(), count.value

    def speculative_verify(self, proposed_token_ids, uniforms, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0):
        """One verification step over the uploaded logits (rows [0, D]: target, rows [D + 1, 2 D]: draft).
        uniforms: D + 1 canonical draws.  Returns (VERIFY_RESULT_DTYPE record, accepted probabilities[D])."""
        proposed = np.ascontiguousarray(proposed_token_ids, dtype=np.int32)
        uniforms = np.ascontiguousarray(uniforms, dtype=np.float32)
        drafts = proposed.size
        assert uniforms.shape == (drafts + 1,)
        options = make_params(1, temperature, top_k, top_p, min_p)
        accepted = np.zeros(max(drafts, 1), dtype=np.float32)
        result = np.zeros(1, dtype=VERIFY_RESULT_DTYPE)
        self._check(self._lib.ncnn_moe_hip_sampler_speculative_verify(
            self._handle, drafts, options.ctypes.data, proposed.ctypes.data, uniforms.ctypes.data,
            accepted.ctypes.data, result.ctypes.data))
        return result[0], accepted[:drafts]

    def _hooks(self, enabling=True):
        if not self._testing and not enabling:
            return None  # switching off what the shipped library never switches on
        if not self._testing:
            raise SamplerError("test hooks live in the testing build of the library: create the sampler with testing=True")
        return self._lib

    def force_general(self, enabled):
        hooks = self._hooks(bool(enabled))
        if hooks is not None:
            self._check(hooks.ncnn_moe_hip_sampler_debug_force_general(self._handle, 1 if enabled else 0))

    def scatter_segments(self, enabled):
        """Test hook: split rows are launched without the XCD-aware numbering of the workgroups."""
        hooks = self._hooks(bool(enabled))
        if hooks is not None:
            self._check(hooks.ncnn_moe_hip_sampler_debug_scatter_segments(self._handle, 1 if enabled else 0))

    def stream_only(self, logits_ptr, dtype, rows, vocab, row_stride, stream=None):
        """Test hook: a launch with the split kernel's grid and loads and nothing behind them."""
        self._check(self._hooks().ncnn_moe_hip_sampler_debug_stream_only(self._handle, logits_ptr, dtype, rows, vocab, row_stride, stream))

    def chunk_steps(self, enabled):
        """Test hook: whole chunks of a sorted fp32 row added in one precomputed step (default) or round by round."""
        self._check(self._hooks().ncnn_moe_hip_sampler_debug_chunk_steps(self._handle, 1 if enabled else 0))

    def spread_sort(self, enabled):
        """Test hook: the radix sort of long full-order rows on several workgroups (default) or on one."""
        self._check(self._hooks().ncnn_moe_hip_sampler_debug_spread_sort(self._handle, 1 if enabled else 0))

    def partial_sort(self, enabled):
        """Test hook: full-order fp32 rows sorted only as far as their terms can move a sum (default) or whole."""
        self._check(self._hooks().ncnn_moe_hip_sampler_debug_partial_sort(self._handle, 1 if enabled else 0))

    def sort_lengths(self, rows):
        """Test hook: elements sorted of each of the last call's first `rows` rows (SORT_WHOLE_ROW: all of them)."""
        out = np.empty(rows, dtype=np.uint32)
        self._check(self._hooks(True).ncnn_moe_hip_sampler_debug_sort_lengths(self._handle, out.ctypes.data, rows))
        return out

    def skip_low_digit(self, enabled):
        """Test hook: the spread sort of full-order fp32 rows in three passes over the keys' upper 24 bits, the lowest
        byte put in order on the way to the terms (default), or in four passes."""
        self._check(self._hooks().ncnn_moe_hip_sampler_debug_skip_low_digit(self._handle, 1 if enabled else 0))

    def wide_sampled_bound(self, enabled):
        """Test hook: the wide select bounds a window wider than 512 from a sample of the whole row (default) or from
        the row's first chunk."""
        self._check(self._hooks().ncnn_moe_hip_sampler_debug_wide_sampled_bound(self._handle, 1 if enabled else 0))

    def disordered_rows(self, rows):
        """Test hook: which of the last call's first `rows` rows the three-pass sort could not finish (1: the row was
        sorted whole by the launch behind it)."""
        out = np.empty(rows, dtype=np.uint32)
        self._check(self._hooks(True).ncnn_moe_hip_sampler_debug_disordered_rows(self._handle, out.ctypes.data, rows))
        return out

    def fused_bf16(self, enabled):
        """Test hook: bf16 full-order rows counted and walked by one kernel (default) or by two."""
        self._check(self._hooks().ncnn_moe_hip_sampler_debug_fused_bf16(self._handle, 1 if enabled else 0))

    def set_row_epochs(self, epoch):
        """Test hook: the launch number that tags the split kernel's hand-over records, for every row (1 .. LAST_EPOCH)."""
        self._check(self._hooks().ncnn_moe_hip_sampler_debug_set_row_epochs(self._handle, 0, epoch))

    def expf(self, values):
        values = np.ascontiguousarray(values, dtype=np.float32)
        out = np.empty_like(values)
        self._check(self._hooks().ncnn_moe_hip_sampler_debug_expf(self._handle, values.ctypes.data, out.ctypes.data, values.size))
        return out


STATIC_MAX_ROWS = 1024
LAST_EPOCH = 8191  # the launch numbers of the split kernel's records run 1 .. LAST_EPOCH and start over
SORT_WHOLE_ROW = 0xFFFFFFFF  # sort_lengths(): the row is sorted whole


def set_static_row_epochs(device, epoch):
    """Test hook: set_row_epochs for the scratch of the entry that allocates nothing (after its first call on the device)."""
    return load_testing_library().ncnn_moe_hip_sampler_debug_set_row_epochs(None, device, epoch)


def sample_device_static(device, logits_ptr, dtype, rows, vocab, row_stride, params_ptr, uniforms_ptr,
                         stop_ids_ptr, results_ptr, stream=None, testing=False):
    """The select pass without a handle and without any allocation (static device scratch); all pointers
    are device addresses.  Returns the call's return code; last_static_error() has the reason.  (Each build of
    the library has a static array of its own: testing=True calls the testing build's.)"""
    return (load_testing_library() if testing else load_library()).ncnn_moe_hip_sampler_sample_device_static(
        device, logits_ptr, dtype, rows, vocab, row_stride, params_ptr, uniforms_ptr, stop_ids_ptr, results_ptr, stream)


def last_static_error(testing=False):
    return (load_testing_library() if testing else load_library()).ncnn_moe_hip_sampler_last_error(None).decode()


def device_count():
    return load_library().ncnn_moe_hip_sampler_device_count()
