"""ctypes binding of libratchet_hip.so, the C ABI declared in include/ratchet_hip.h.

The library is loaded from this directory only (built in-tree by ratchet_amd.build); a missing library is an
error, never a fallback to another implementation.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libratchet_hip.so")

# names and order follow include/ratchet_hip.h
F32, F16, BF16, I32, U32 = 0, 1, 2, 3, 4
ADD, SUB, MUL, DIV = 0, 1, 2, 3
UNARY_OPS = ["gelu", "tanh", "exp", "log", "sin", "cos", "abs", "sqrt", "relu", "floor", "ceil", "neg", "silu", "sigmoid"]
BINARY_OPS = ["add", "sub", "mul", "div"]
SOFTMAX_REFERENCE, SOFTMAX_STABLE = 0, 1

STATUS_NAMES = {
    0: "RT_OK", 1: "RT_ERR_NULL_POINTER", 2: "RT_ERR_DTYPE", 3: "RT_ERR_OP", 4: "RT_ERR_SHAPE", 5: "RT_ERR_PERM",
    6: "RT_ERR_SIZE", 7: "RT_ERR_ARG", 8: "RT_ERR_NULL_DEVICE", 9: "RT_ERR_ALIGN",
    10: "RT_ERR_CAPTURE",
}

EXPORTS = [
    "rt_device_count", "rt_device_create", "rt_device_destroy", "rt_sync", "rt_last_error", "rt_status_name", "rt_debug_hip_status", "rt_debug_softmax_pace", "rt_malloc",
    "rt_free", "rt_pool_trim", "rt_pool_begin_pass", "rt_pool_stats", "rt_pool_peak", "rt_capture_begin", "rt_capture_end", "rt_graph_launch", "rt_graph_destroy", "rt_memset0", "rt_h2d", "rt_d2h", "rt_d2d", "rt_event_create", "rt_event_destroy", "rt_event_record",
    "rt_event_elapsed_ms", "rt_binary", "rt_binary_bcast", "rt_unary", "rt_cast", "rt_permute", "rt_slice", "rt_broadcast",
    "rt_concat", "rt_cache", "rt_index_select", "rt_index_select_q8_0", "rt_index_write", "rt_rope", "rt_softmax", "rt_softmax_masked", "rt_layer_norm", "rt_rms_norm", "rt_group_norm", "rt_group_norm_static", "rt_norm_via_f32", "rt_softmax_via_f32", "rt_unary_via_f32", "rt_gated_mul_via_f32",
]


class RatchetError(RuntimeError):
    def __init__(self, status, message):
        name = STATUS_NAMES.get(status, "HIP_ERROR" if status < 0 else "RT_ERR_UNKNOWN")
        super().__init__(f"{name} ({status}): {message}")
        self.status = status


_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `python -m ratchet_amd.build` (needs hipcc)")
    L = ctypes.CDLL(LIB_PATH)
    vp, sz, i, f = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_float
    u64, u32 = ctypes.c_uint64, ctypes.c_uint32
    pp = ctypes.POINTER(ctypes.c_void_p)
    sh = ctypes.POINTER(u32)
    L.rt_device_count.argtypes = [ctypes.POINTER(i)]
    L.rt_device_create.argtypes = [i, pp]
    L.rt_device_destroy.argtypes = [vp]
    L.rt_sync.argtypes = [vp]
    L.rt_last_error.argtypes = []
    L.rt_last_error.restype = ctypes.c_char_p
    L.rt_status_name.argtypes = [i]
    L.rt_status_name.restype = ctypes.c_char_p
    L.rt_debug_softmax_pace.argtypes = [vp, u32]
    L.rt_malloc.argtypes = [vp, sz, pp]
    L.rt_free.argtypes = [vp, vp]
    L.rt_pool_trim.argtypes = [vp]
    L.rt_pool_begin_pass.argtypes = [vp]
    L.rt_capture_begin.argtypes = [vp]
    L.rt_capture_end.argtypes = [vp, pp]
    L.rt_graph_launch.argtypes = [vp, vp]
    L.rt_graph_destroy.argtypes = [vp]
    L.rt_pool_stats.argtypes = [vp] + [ctypes.POINTER(ctypes.c_uint64)] * 4
    L.rt_memset0.argtypes = [vp, vp, sz]
    L.rt_h2d.argtypes = [vp, vp, vp, sz]
    L.rt_d2h.argtypes = [vp, vp, vp, sz]
    L.rt_d2d.argtypes = [vp, vp, vp, sz]
    L.rt_event_create.argtypes = [vp, pp]
    L.rt_event_destroy.argtypes = [vp]
    L.rt_event_record.argtypes = [vp, vp]
    L.rt_event_elapsed_ms.argtypes = [vp, vp, ctypes.POINTER(f)]
    L.rt_binary.argtypes = [vp, i, i, vp, vp, vp, u64]
    L.rt_binary_bcast.argtypes = [vp, i, i, vp, sh, vp, sh, vp, sh]
    L.rt_unary.argtypes = [vp, i, i, vp, vp, u64]
    L.rt_cast.argtypes = [vp, i, i, vp, vp, u64]
    L.rt_permute.argtypes = [vp, i, vp, vp, sh, sh]
    L.rt_slice.argtypes = [vp, i, vp, vp, sh, sh, sh]
    L.rt_broadcast.argtypes = [vp, i, vp, vp, sh, sh]
    L.rt_concat.argtypes = [vp, i, i, pp, vp, i, vp]
    L.rt_cache.argtypes = [vp, i, vp, sh, vp, sh, i, u32, vp]
    L.rt_index_select.argtypes = [vp, i, vp, sh, vp, u32, i, vp]
    L.rt_index_select_q8_0.argtypes = [vp, i, vp, vp, sh, vp, u32, i, vp]
    L.rt_index_write.argtypes = [vp, i, vp, sh, vp, u64, sh]
    L.rt_rope.argtypes = [vp, i, vp, vp, sh, u32, f, u32]
    L.rt_softmax.argtypes = [vp, i, vp, vp, u64, u32, i]
    L.rt_softmax_masked.argtypes = [vp, i, vp, sh, vp, sh, vp, i]
    L.rt_layer_norm.argtypes = [vp, i, vp, vp, vp, vp, u64, u32, f]
    L.rt_rms_norm.argtypes = [vp, i, vp, vp, vp, u64, u32, f]
    L.rt_group_norm.argtypes = [vp, i, vp, vp, vp, vp, u32, u32, u32, u32, f]
    L.rt_group_norm_static.argtypes = [vp, i, vp, vp, vp, vp, u32, u32, u32, u32, f]
    L.rt_norm_via_f32.argtypes = [vp, i, i, vp, vp, vp, vp, u64, u32, f]
    L.rt_softmax_via_f32.argtypes = [vp, i, vp, sh, vp, sh, vp, i]
    L.rt_unary_via_f32.argtypes = [vp, i, i, vp, vp, u64]
    L.rt_gated_mul_via_f32.argtypes = [vp, i, i, vp, u64, vp, u64, vp, u64, u32]
    for name in EXPORTS:
        fn = getattr(L, name)
        if name not in ("rt_last_error", "rt_status_name"):
            fn.restype = i
    _lib = L
    return L


def check(status):
    if status != 0:
        raise RatchetError(status, load().rt_last_error().decode("utf-8", "replace"))


def shape4(shape):
    """Shape::promote(shape, 4): left-pad with 1s (crates/ratchet-core/src/shape.rs:92-96)."""
    shape = [int(s) for s in shape]
    if len(shape) > 4:
        raise ValueError("rank > 4 is not supported")
    return (ctypes.c_uint32 * 4)(*([1] * (4 - len(shape)) + shape))
