"""ctypes binding of libncnn_moe_hip_router.so (include/ncnn_moe_hip_router.h): the expert router of a
MoE layer (ExpertDispatcher::dispatch, src/graph/expert_dispatcher.cpp:76-157) on the GPU.

There is no CPU fallback: if the library is missing or no GPU is visible, calls raise.
"""
import ctypes
import os

import numpy as np

PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(PACKAGE_DIR, "libncnn_moe_hip_router.so")

SOFTMAX, SIGMOID, SQRT_SOFTPLUS = 0, 1, 2

STATUS_OK = 0
STATUS_NO_TOKENS = 1
STATUS_BAD_TOP_K = 2
STATUS_BAD_SCALING = 3
STATUS_NON_FINITE_LOGIT = 4
STATUS_EXPERT_OUT_OF_RANGE = 5
STATUS_NON_POSITIVE_SUM = 6

RC_SUCCESS = 0
RC_INVALID_ARGUMENT = 1
RC_HIP_ERROR = 2
RC_NO_DEVICE = 3

MAX_EXPERTS = 1024
MAX_TOP_K = 64

OPTIONS_DTYPE = np.dtype([("expert_count", "<u4"), ("top_k", "<u4"), ("score_function", "<u4"),
                          ("renormalize", "<u4"), ("routed_scaling_factor", "<f4")])
ROUTE_DTYPE = np.dtype([("token_index", "<u4"), ("rank", "<u4"), ("weight", "<f4")])

EXPORTED_SYMBOLS = [
    "ncnn_moe_hip_router_create",
    "ncnn_moe_hip_router_destroy",
    "ncnn_moe_hip_router_dispatch",
    "ncnn_moe_hip_router_dispatch_device",
    "ncnn_moe_hip_router_status_message",
    "ncnn_moe_hip_router_last_error",
    "ncnn_moe_hip_router_debug_log1pf",
]


class RouterError(RuntimeError):
    pass


_library = None


def load_library():
    """Loads the C-ABI library; raises if it has not been built."""
    global _library
    if _library is not None:
        return _library
    if not os.path.exists(LIBRARY_PATH):
        raise RouterError(
            "%s is missing: build it with `make -C %s` (or __graft_entry__.build())" % (LIBRARY_PATH, PACKAGE_DIR))
    lib = ctypes.CDLL(LIBRARY_PATH)
    vp = ctypes.c_void_p
    u32 = ctypes.c_uint32
    lib.ncnn_moe_hip_router_create.argtypes = [ctypes.c_int, u32, u32, u32, ctypes.POINTER(vp)]
    lib.ncnn_moe_hip_router_destroy.argtypes = [vp]
    lib.ncnn_moe_hip_router_destroy.restype = None
    lib.ncnn_moe_hip_router_dispatch.argtypes = [vp, vp, u32, vp, vp, vp, vp, vp, ctypes.POINTER(u32)]
    lib.ncnn_moe_hip_router_dispatch_device.argtypes = [vp, vp, u32, vp, vp, vp, vp, vp, vp, ctypes.POINTER(u32), vp]
    lib.ncnn_moe_hip_router_status_message.argtypes = [ctypes.c_int]
    lib.ncnn_moe_hip_router_status_message.restype = ctypes.c_char_p
    lib.ncnn_moe_hip_router_last_error.argtypes = [vp]
    lib.ncnn_moe_hip_router_last_error.restype = ctypes.c_char_p
    lib.ncnn_moe_hip_router_debug_log1pf.argtypes = [vp, vp, vp, ctypes.c_size_t]
    _library = lib
    return lib


def status_message(status):
    return load_library().ncnn_moe_hip_router_status_message(int(status)).decode()


def make_options(expert_count, top_k, score_function=SOFTMAX, renormalize=True, routed_scaling_factor=1.0):
    options = np.zeros(1, dtype=OPTIONS_DTYPE)
    options[0] = (expert_count, top_k, score_function, 1 if renormalize else 0, routed_scaling_factor)
    return options


class HipRouter:
    """One ncnn_moe_hip_router handle.  dispatch() mirrors ExpertDispatcher::dispatch on host arrays;
    dispatch_device() takes device pointers (integers) and enqueues on a stream."""

    def __init__(self, max_tokens, max_experts=MAX_EXPERTS, max_top_k=MAX_TOP_K, device=0):
        self._lib = load_library()
        self._handle = ctypes.c_void_p()
        rc = self._lib.ncnn_moe_hip_router_create(device, max_tokens, max_experts, max_top_k, ctypes.byref(self._handle))
        if rc != RC_SUCCESS:
            self._handle = ctypes.c_void_p()
            raise RouterError("ncnn_moe_hip_router_create failed with code %d (%s)" % (
                rc, {RC_INVALID_ARGUMENT: "invalid argument", RC_HIP_ERROR: "HIP error", RC_NO_DEVICE: "no GPU"}.get(rc, "?")))
        self.max_tokens, self.max_experts, self.max_top_k = max_tokens, max_experts, max_top_k

    def close(self):
        if self._handle:
            self._lib.ncnn_moe_hip_router_destroy(self._handle)
            self._handle = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc, what):
        if rc != RC_SUCCESS:
            raise RouterError("%s failed with code %d: %s" % (
                what, rc, self._lib.ncnn_moe_hip_router_last_error(self._handle).decode()))

    def dispatch(self, router_logits, top_k, score_function=SOFTMAX, renormalize=True, routed_scaling_factor=1.0,
                 selection_bias=None, explicit_expert_ids=None):
        """router_logits [tokens, experts] fp32.  Returns (status, expert_offsets[experts + 1], routes ROUTE_DTYPE)."""
        router_logits = np.ascontiguousarray(router_logits, dtype=np.float32)
        tokens, experts = router_logits.shape
        options = make_options(experts, top_k, score_function, renormalize, routed_scaling_factor)
        bias = None if selection_bias is None else np.ascontiguousarray(selection_bias, dtype=np.float32)
        explicit = None if explicit_expert_ids is None else np.ascontiguousarray(explicit_expert_ids, dtype=np.uint32)
        if bias is not None and bias.size != experts:
            raise RouterError("selection_bias must hold one value per expert")
        if explicit is not None and explicit.size != tokens * top_k:
            raise RouterError("explicit_expert_ids must hold tokens * top_k ids")
        offsets = np.zeros(experts + 1, dtype=np.uint32)
        routes = np.zeros(max(1, tokens * max(top_k, 1)), dtype=ROUTE_DTYPE)
        status = ctypes.c_uint32(0)
        rc = self._lib.ncnn_moe_hip_router_dispatch(
            self._handle, router_logits.ctypes.data, tokens, options.ctypes.data,
            None if bias is None else bias.ctypes.data, None if explicit is None else explicit.ctypes.data,
            offsets.ctypes.data, routes.ctypes.data, ctypes.byref(status))
        self._check(rc, "ncnn_moe_hip_router_dispatch")
        count = tokens * top_k if status.value == STATUS_OK else 0
        return int(status.value), offsets, routes[:count]

    def dispatch_device(self, logits_pointer, tokens, options, offsets_pointer, routes_pointer, status_pointer,
                        bias_pointer=None, explicit_pointer=None, stream=None):
        """Enqueues one dispatch over device arrays; returns the host-side status of the argument checks."""
        host_status = ctypes.c_uint32(0)
        rc = self._lib.ncnn_moe_hip_router_dispatch_device(
            self._handle, logits_pointer, tokens, options.ctypes.data, bias_pointer, explicit_pointer,
            offsets_pointer, routes_pointer, status_pointer, ctypes.byref(host_status), stream)
        self._check(rc, "ncnn_moe_hip_router_dispatch_device")
        return int(host_status.value)

    def debug_log1pf(self, values):
        values = np.ascontiguousarray(values, dtype=np.float32)
        out = np.empty_like(values)
        self._check(self._lib.ncnn_moe_hip_router_debug_log1pf(self._handle, values.ctypes.data, out.ctypes.data, values.size),
                    "ncnn_moe_hip_router_debug_log1pf")
        return out


def device_count():
    from . import hip_sampler
    return hip_sampler.device_count()
