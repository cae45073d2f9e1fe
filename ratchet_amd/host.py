"""ctypes binding of libratchet_host.so: the C++ mirror of ratchet-core's lazy Tensor API (include/ratchet_host.h).

    dev = HostDevice(0)
    y = Tensor.from_numpy(x, dev).add(Tensor.from_numpy(b, dev)).gelu().layer_norm(w, bias, 1e-5).resolve()
    y.to_numpy()

Method names and argument order follow crates/ratchet-core/src/tensor.rs.  All graph logic (broadcast rules, guards,
topological order, in-place rule, broadcast fusion) lives in the C++ library; this file only marshals arguments.
"""
import ctypes
import os

import numpy as np

from . import _lib

HERE = os.path.dirname(os.path.abspath(__file__))
# RATCHET_HOST_LIB names another build of the same library (the sanitizer build of tests/test_sanitizers.py)
HOST_LIB_PATH = os.environ.get("RATCHET_HOST_LIB") or os.path.join(HERE, "libratchet_host.so")

_NP_TO_DT = {np.dtype(np.float32): _lib.F32, np.dtype(np.float16): _lib.F16, np.dtype(np.int32): _lib.I32,
             np.dtype(np.uint32): _lib.U32}
_DT_TO_NP = {_lib.F32: np.float32, _lib.F16: np.float16, _lib.BF16: np.uint16, _lib.I32: np.int32, _lib.U32: np.uint32}

Q8_0F, Q8_0H = 5, 6            # the quantized types of the host mirror (sources of index_select only)

_h = None


class HostError(RuntimeError):
    def __init__(self, kind, message):
        super().__init__(message)
        self.kind = kind


def load():
    global _h
    if _h is not None:
        return _h
    _lib.load()                                   # libratchet_hip.so first: the host library links against it
    if not os.path.exists(HOST_LIB_PATH):
        raise ImportError(f"{HOST_LIB_PATH} is missing: build it with `python -m ratchet_amd.build`")
    H = ctypes.CDLL(HOST_LIB_PATH)
    vp, i, f, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
    u64p = ctypes.POINTER(ctypes.c_uint64)
    H.rth_last_error.restype = ctypes.c_char_p
    H.rth_last_error_kind.restype = ctypes.c_char_p
    H.rth_op_name.restype = ctypes.c_char_p
    H.rth_op_name.argtypes = [vp]
    H.rth_device_request.restype = vp
    H.rth_device_request.argtypes = [i]
    H.rth_device_release.argtypes = [vp]
    H.rth_device_release.restype = None
    H.rth_release.argtypes = [vp]
    H.rth_release.restype = None
    for name, args in {
        "rth_from_host": [vp, vp, i, u64p, i], "rth_from_quantized": [vp, vp, i, u64p, i], "rth_placeholder": [i, u64p, i], "rth_binary": [vp, vp, i], "rth_unary": [vp, i],
        "rth_cast": [vp, i], "rth_layer_norm": [vp, vp, vp, f], "rth_rms_norm": [vp, vp, f], "rth_group_norm": [vp, sz, vp, vp, f],
        "rth_softmax": [vp, sz, i], "rth_slice": [vp, i, u64p, u64p], "rth_view": [vp, i, u64p],
        "rth_cat": [ctypes.POINTER(vp), i, sz], "rth_cache": [vp, vp, sz, sz], "rth_rope": [vp, sz, f, sz], "rth_index_select": [vp, vp, sz],
        "rth_index_write": [vp, vp, i, u64p], "rth_permute": [vp, i, u64p], "rth_broadcast_to": [vp, i, u64p],
    }.items():
        fn = getattr(H, name)
        fn.argtypes = args
        fn.restype = vp
    for name, args in {"rth_rank": [vp], "rth_shape": [vp, u64p], "rth_dtype": [vp], "rth_resolved": [vp], "rth_resolve": [vp],
                       "rth_to_host": [vp, vp], "rth_execution_order": [vp, u64p, i]}.items():
        fn = getattr(H, name)
        fn.argtypes = args
        fn.restype = i
    H.rth_memory_plan.argtypes = [vp, u64p, i, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int64), i]
    H.rth_memory_plan.restype = i
    H.rth_last_resolve_launches.argtypes = [vp]
    H.rth_last_resolve_launches.restype = ctypes.c_long
    H.rth_id.argtypes = [vp]
    H.rth_id.restype = ctypes.c_uint64
    H.rth_pool_stats.argtypes = [vp, u64p]
    H.rth_pool_stats.restype = i
    H.rth_pool_peak.argtypes = [vp, u64p, i]
    H.rth_pool_peak.restype = i
    H.rth_set_pattern_fusion.argtypes = [i]
    H.rth_set_pattern_fusion.restype = None
    H.rth_storage_bytes.argtypes = [i, u64p, i]
    H.rth_storage_bytes.restype = ctypes.c_uint64
    H.rth_compile.argtypes = [vp]
    H.rth_compile.restype = vp
    H.rth_executable_dispatch.argtypes = [vp, i]
    H.rth_executable_dispatch.restype = i
    H.rth_executable_launches.argtypes = [vp]
    H.rth_executable_launches.restype = ctypes.c_long
    H.rth_executable_held_bytes.argtypes = [vp]
    H.rth_executable_held_bytes.restype = ctypes.c_uint64
    H.rth_executable_release.argtypes = [vp]
    H.rth_executable_release.restype = None
    H.rth_update_from_host.argtypes = [vp, vp]
    H.rth_update_from_host.restype = i
    _h = H
    return H


def set_pattern_fusion(on):
    """resolve() folds full() -> norm / softmax / activation -> cast(dt) sequences into one launch each (default on)."""
    load().rth_set_pattern_fusion(int(bool(on)))


def _raise():
    H = load()
    raise HostError(H.rth_last_error_kind().decode(), H.rth_last_error().decode())


def _u64(v):
    v = [int(x) for x in v]
    return (ctypes.c_uint64 * max(len(v), 1))(*v)


class HostDevice:
    def __init__(self, ordinal=0):
        self.H = load()
        self.handle = self.H.rth_device_request(ordinal)
        if not self.handle:
            _raise()

    def pool_stats(self):
        """(bytes handed out, bytes parked for reuse, requests served by the pool, requests passed to hipMalloc)"""
        out = (ctypes.c_uint64 * 4)()
        if self.H.rth_pool_stats(self.handle, out) != 0:
            _raise()
        return tuple(int(v) for v in out)

    def pool_peak(self, reset=False):
        """the most bytes handed out at one time since the last reset"""
        out = (ctypes.c_uint64 * 1)()
        if self.H.rth_pool_peak(self.handle, out, int(bool(reset))) != 0:
            _raise()
        return int(out[0])

    def close(self):
        if self.handle:
            self.H.rth_device_release(self.handle)
            self.handle = None


class Executable:
    """The recorded launch list of a compiled graph (the reference's Executable, executable.rs:13-59, as a HIP graph)."""

    def __init__(self, handle):
        self.H = load()
        self.handle = handle

    def dispatch(self, wait=True):
        if self.H.rth_executable_dispatch(self.handle, int(bool(wait))) != 0:
            _raise()
        return self

    @property
    def launches(self):
        return int(self.H.rth_executable_launches(self.handle))

    @property
    def held_bytes(self):
        return int(self.H.rth_executable_held_bytes(self.handle))

    def close(self):
        if self.handle:
            self.H.rth_executable_release(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Tensor:
    def __init__(self, handle):
        if not handle:
            _raise()
        self.H = load()
        self.handle = handle

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                self.H.rth_release(self.handle)
                self.handle = None
        except Exception:
            pass

    # ---- construction
    @staticmethod
    def from_numpy(a, device, bf16=False):
        a = np.ascontiguousarray(a)
        dt = _lib.BF16 if bf16 else _NP_TO_DT[a.dtype]
        return Tensor(load().rth_from_host(device.handle, a.ctypes.data_as(ctypes.c_void_p), a.ndim, _u64(a.shape), dt))

    @staticmethod
    def from_quantized(words, scales, shape, device):
        """Tensor::from_quantized (tensor.rs:618-628): `words` are the packed signed bytes (uint32, numel / 4 of them),
        `scales` one f32 (Q8_0F) or f16 (Q8_0H) per group of 32; they are laid out as the reference's quantized buffer is
        (quant.rs:19-49: each segment padded to 256 bytes)."""
        words, scales = np.ascontiguousarray(words, np.uint32), np.ascontiguousarray(scales)
        dt = {np.dtype(np.float32): Q8_0F, np.dtype(np.float16): Q8_0H}[scales.dtype]
        total = int(load().rth_storage_bytes(len(shape), _u64(shape), dt))
        buf = np.zeros(total, np.uint8)
        scale_at = (words.nbytes + 255) & ~255
        if scale_at + scales.nbytes > total:
            raise ValueError("from_quantized: words / scales do not match the shape")
        buf[:words.nbytes] = words.view(np.uint8).ravel()
        buf[scale_at:scale_at + scales.nbytes] = scales.view(np.uint8).ravel()
        return Tensor(load().rth_from_quantized(device.handle, buf.ctypes.data_as(ctypes.c_void_p), len(shape), _u64(shape), dt))

    @staticmethod
    def placeholder(shape, dt=_lib.F32):
        return Tensor(load().rth_placeholder(len(shape), _u64(shape), dt))

    # ---- metadata
    @property
    def shape(self):
        r = self.H.rth_rank(self.handle)
        d = (ctypes.c_uint64 * max(r, 1))()
        self.H.rth_shape(self.handle, d)
        return tuple(int(d[k]) for k in range(r))

    @property
    def dt(self):
        return self.H.rth_dtype(self.handle)

    @property
    def id(self):
        return int(self.H.rth_id(self.handle))

    def resolved(self):
        return bool(self.H.rth_resolved(self.handle))

    def op_name(self):
        return self.H.rth_op_name(self.handle).decode()

    # ---- op builders (names as in tensor.rs)
    def _bin(self, other, op):
        return Tensor(self.H.rth_binary(self.handle, other.handle, op))

    def add(self, other): return self._bin(other, _lib.ADD)
    def sub(self, other): return self._bin(other, _lib.SUB)
    def mul(self, other): return self._bin(other, _lib.MUL)
    def div(self, other): return self._bin(other, _lib.DIV)

    def unary(self, name):
        return Tensor(self.H.rth_unary(self.handle, _lib.UNARY_OPS.index(name)))

    def gelu(self): return self.unary("gelu")
    def tanh(self): return self.unary("tanh")
    def exp(self): return self.unary("exp")
    def log(self): return self.unary("log")
    def sin(self): return self.unary("sin")
    def cos(self): return self.unary("cos")
    def abs(self): return self.unary("abs")
    def sqrt(self): return self.unary("sqrt")
    def relu(self): return self.unary("relu")
    def floor(self): return self.unary("floor")
    def ceil(self): return self.unary("ceil")
    def neg(self): return self.unary("neg")
    def silu(self): return self.unary("silu")
    def sigmoid(self): return self.unary("sigmoid")

    def cast(self, dst_dt): return Tensor(self.H.rth_cast(self.handle, dst_dt))
    def full(self): return self.cast(_lib.F32)
    def half(self): return self.cast(_lib.F16)

    def layer_norm(self, weight, bias, eps):
        return Tensor(self.H.rth_layer_norm(self.handle, weight.handle, bias.handle if bias is not None else None, eps))

    def rms_norm(self, weight, eps):
        return Tensor(self.H.rth_rms_norm(self.handle, weight.handle, eps))

    def group_norm(self, num_groups, weight, bias, eps):
        return Tensor(self.H.rth_group_norm(self.handle, num_groups, weight.handle, bias.handle if bias is not None else None, eps))

    def softmax(self, dim, mode=_lib.SOFTMAX_REFERENCE):
        return Tensor(self.H.rth_softmax(self.handle, dim, mode))

    def slice(self, ranges):
        return Tensor(self.H.rth_slice(self.handle, len(ranges), _u64(r[0] for r in ranges), _u64(r[1] for r in ranges)))

    def view(self, shape):
        return Tensor(self.H.rth_view(self.handle, len(shape), _u64(shape)))

    @staticmethod
    def cat(tensors, dim):
        arr = (ctypes.c_void_p * len(tensors))(*[t.handle for t in tensors])
        return Tensor(load().rth_cat(arr, len(tensors), dim))

    def cache(self, source, dim, offset):
        return Tensor(self.H.rth_cache(self.handle, source.handle, dim, offset))

    def rope(self, dim, base, offset):
        return Tensor(self.H.rth_rope(self.handle, dim, base, offset))

    def index_select(self, indices, dim):
        return Tensor(self.H.rth_index_select(self.handle, indices.handle, dim))

    def index_write(self, src, write_start):
        return Tensor(self.H.rth_index_write(self.handle, src.handle, len(write_start), _u64(write_start)))

    def permute(self, dims):
        return Tensor(self.H.rth_permute(self.handle, len(dims), _u64(dims)))

    def broadcast_to(self, shape):
        return Tensor(self.H.rth_broadcast_to(self.handle, len(shape), _u64(shape)))

    # ---- execution
    def resolve(self):
        if self.H.rth_resolve(self.handle) != 0:
            _raise()
        return self

    def to_numpy(self):
        out = np.empty(self.shape, dtype=_DT_TO_NP[self.dt])
        if self.H.rth_to_host(self.handle, out.ctypes.data_as(ctypes.c_void_p)) != 0:
            _raise()
        return out

    def last_resolve_launches(self):
        return int(self.H.rth_last_resolve_launches(self.handle))

    def compile(self):
        """resolve() that also records its launches: returns the Executable that replays them with one graph launch"""
        h = self.H.rth_compile(self.handle)
        if not h:
            _raise()
        return Executable(h)

    def update(self, a):
        """overwrite the contents of a tensor that has storage (an input of a compiled graph) with array `a`"""
        a = np.ascontiguousarray(a)
        if a.nbytes != int(np.prod(self.shape, dtype=np.int64)) * np.dtype(_DT_TO_NP[self.dt]).itemsize:
            raise ValueError("update: the array does not have the tensor's size")
        if self.H.rth_update_from_host(self.handle, a.ctypes.data_as(ctypes.c_void_p)) != 0:
            _raise()
        return self

    def memory_plan(self):
        """(object_bytes, entries) of the plan resolve() would follow; entries are dicts id / bytes / object / source in
        execution order (object -1: own allocation, -2: in place in a buffer that exists already)"""
        nobj = ctypes.c_int(0)
        n = self.H.rth_memory_plan(self.handle, None, 0, ctypes.byref(nobj), None, 0)
        if n < 0:
            _raise()
        objs = (ctypes.c_uint64 * max(nobj.value, 1))()
        ent = (ctypes.c_int64 * max(4 * n, 1))()
        self.H.rth_memory_plan(self.handle, objs, nobj.value, ctypes.byref(nobj), ent, n)
        entries = [dict(id=int(ent[4 * k]), bytes=int(ent[4 * k + 1]), object=int(ent[4 * k + 2]), source=int(ent[4 * k + 3])) for k in range(n)]
        return [int(objs[k]) for k in range(nobj.value)], entries

    def execution_order(self):
        n = self.H.rth_execution_order(self.handle, _u64([0]), 0)
        ids = (ctypes.c_uint64 * max(n, 1))()
        self.H.rth_execution_order(self.handle, ids, n)
        return [int(ids[k]) for k in range(n)]
