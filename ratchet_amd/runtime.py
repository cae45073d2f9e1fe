"""Thin object layer over the C ABI: Device (one HIP stream), Buffer (hipMalloc'd storage), op launchers.

This mirrors the storage/dispatch seam of ratchet-core that the native library replaces:
  Device  ~ WgpuDevice          (crates/ratchet-core/src/gpu/device.rs:18-30)
  Buffer  ~ GPUBuffer           (crates/ratchet-core/src/storage/gpu_buffer.rs:20-27): ref-counted by Python, freed on drop
  op methods ~ one CompiledOp dispatch each (crates/ratchet-core/src/executable.rs:33-59)
Every method enqueues on the device's single stream; Device.sync() / Buffer.to_numpy() block.
"""
import ctypes

import numpy as np

from . import _lib
from ._lib import RatchetError, check, shape4  # noqa: F401

_NP_TO_DT = {np.dtype(np.float32): _lib.F32, np.dtype(np.float16): _lib.F16, np.dtype(np.int32): _lib.I32,
             np.dtype(np.uint32): _lib.U32}
_DT_BYTES = {_lib.F32: 4, _lib.F16: 2, _lib.BF16: 2, _lib.I32: 4, _lib.U32: 4}
_DT_TO_NP = {_lib.F32: np.float32, _lib.F16: np.float16, _lib.BF16: np.uint16, _lib.I32: np.int32, _lib.U32: np.uint32}


def dtype_code(np_dtype, bf16=False):
    if bf16:
        return _lib.BF16
    return _NP_TO_DT[np.dtype(np_dtype)]


class Buffer:
    """A device allocation with a dtype code and a shape; owns its memory."""

    def __init__(self, device, shape, dt):
        self.device = device
        self.shape = tuple(int(s) for s in shape)
        self.dt = dt
        self.numel = int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1
        self.nbytes = self.numel * _DT_BYTES[dt]
        p = ctypes.c_void_p()
        check(device.lib.rt_malloc(device.handle, self.nbytes, ctypes.byref(p)))
        self.ptr = p

    def __del__(self):
        try:
            if getattr(self, "ptr", None) is not None and self.device.handle is not None:
                self.device.lib.rt_free(self.device.handle, self.ptr)
                self.ptr = None
        except Exception:
            pass

    def to_numpy(self):
        out = np.empty(self.shape, dtype=_DT_TO_NP[self.dt])
        check(self.device.lib.rt_d2h(self.device.handle, out.ctypes.data_as(ctypes.c_void_p), self.ptr, self.nbytes))
        return out

    def view(self, offset, shape):
        return BufferView(self, offset, shape)

    def reshape(self, shape):
        return BufferView(self, 0, shape)

    def zero_(self):
        check(self.device.lib.rt_memset0(self.device.handle, self.ptr, self.nbytes))
        return self


def _unary_code(op):
    return _lib.UNARY_OPS.index(op) if isinstance(op, str) else op


class BufferView:
    """A window into a Buffer starting `offset` elements in (keeps the parent alive); used for offset / misaligned operands."""

    def __init__(self, parent, offset, shape):
        self.device = parent.device
        self.parent = parent
        self.dt = parent.dt
        self.shape = tuple(int(s) for s in shape)
        self.numel = int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1
        self.nbytes = self.numel * _DT_BYTES[self.dt]
        assert (offset + self.numel) <= parent.numel
        self.ptr = ctypes.c_void_p(parent.ptr.value + offset * _DT_BYTES[self.dt])

    def to_numpy(self):
        out = np.empty(self.shape, dtype=_DT_TO_NP[self.dt])
        check(self.device.lib.rt_d2h(self.device.handle, out.ctypes.data_as(ctypes.c_void_p), self.ptr, self.nbytes))
        return out

    def upload(self, array):
        a = np.ascontiguousarray(array)
        assert a.nbytes == self.nbytes
        check(self.device.lib.rt_h2d(self.device.handle, self.ptr, a.ctypes.data_as(ctypes.c_void_p), a.nbytes))
        return self


class Graph:
    """A replayable list of launches recorded on a device (a HIP graph); the buffers it touches must outlive it."""

    def __init__(self, device, handle):
        self.device, self.handle = device, handle

    def launch(self):
        check(self.device.lib.rt_graph_launch(self.device.handle, self.handle))

    def __del__(self):
        try:
            if self.handle is not None and self.device.handle is not None:
                self.device.lib.rt_graph_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


class _Capture:
    def __init__(self, device):
        self.device = device
        self.graph = None

    def __enter__(self):
        check(self.device.lib.rt_capture_begin(self.device.handle))
        return self

    def __exit__(self, exc_type, exc, tb):
        p = ctypes.c_void_p()
        rc = self.device.lib.rt_capture_end(self.device.handle, ctypes.byref(p))
        if exc_type is None:
            check(rc)
            self.graph = Graph(self.device, p)
        elif rc == 0:
            self.device.lib.rt_graph_destroy(p)
        return False

    def launch(self):
        self.graph.launch()


class Event:
    def __init__(self, device):
        self.device = device
        p = ctypes.c_void_p()
        check(device.lib.rt_event_create(device.handle, ctypes.byref(p)))
        self.ptr = p

    def record(self):
        check(self.device.lib.rt_event_record(self.device.handle, self.ptr))
        return self

    def elapsed_ms(self, stop):
        ms = ctypes.c_float()
        check(self.device.lib.rt_event_elapsed_ms(self.ptr, stop.ptr, ctypes.byref(ms)))
        return float(ms.value)

    def __del__(self):
        try:
            if getattr(self, "ptr", None) is not None:
                self.device.lib.rt_event_destroy(self.ptr)
                self.ptr = None
        except Exception:
            pass


class Device:
    def __init__(self, ordinal=0):
        self.lib = _lib.load()
        self.handle = None
        h = ctypes.c_void_p()
        check(self.lib.rt_device_create(ordinal, ctypes.byref(h)))
        self.handle = h
        self.ordinal = ordinal

    @staticmethod
    def count():
        n = ctypes.c_int()
        lib = _lib.load()
        status = lib.rt_device_count(ctypes.byref(n))
        return n.value if status == 0 else 0

    def close(self):
        if self.handle is not None:
            self.lib.rt_device_destroy(self.handle)
            self.handle = None

    def sync(self):
        check(self.lib.rt_sync(self.handle))

    def capture(self):
        """with dev.capture() as g: <launch ops> ... then g.launch() replays them with one submission."""
        return _Capture(self)

    def pool_stats(self):
        """(bytes handed out, bytes parked for reuse, requests served by the pool, requests passed to hipMalloc)"""
        v = [ctypes.c_uint64() for _ in range(4)]
        check(self.lib.rt_pool_stats(self.handle, *[ctypes.byref(x) for x in v]))
        return tuple(int(x.value) for x in v)

    def pool_trim(self):
        check(self.lib.rt_pool_trim(self.handle))

    def pool_begin_pass(self):
        """What the reference does at the top of every resolve: blocks freed before the previous call and not reused since
        go back to the driver."""
        check(self.lib.rt_pool_begin_pass(self.handle))

    # ---- storage
    def empty(self, shape, dt):
        return Buffer(self, shape, dt)

    def upload(self, array, bf16=False):
        a = np.ascontiguousarray(array)
        buf = Buffer(self, a.shape, dtype_code(a.dtype, bf16))
        check(self.lib.rt_h2d(self.handle, buf.ptr, a.ctypes.data_as(ctypes.c_void_p), a.nbytes))
        return buf

    def event(self):
        return Event(self)

    # ---- ops (out may alias the first input where the C ABI allows it)
    def binary(self, op, a, b, out=None):
        op = _lib.BINARY_OPS.index(op) if isinstance(op, str) else op
        if a.shape == b.shape:
            out = out or Buffer(self, a.shape, a.dt)
            check(self.lib.rt_binary(self.handle, op, a.dt, a.ptr, b.ptr, out.ptr, a.numel))
            return out
        shape = tuple(np.broadcast_shapes(a.shape, b.shape))
        out = out or Buffer(self, shape, a.dt)
        check(self.lib.rt_binary_bcast(self.handle, op, a.dt, a.ptr, shape4(a.shape), b.ptr, shape4(b.shape), out.ptr,
                                       shape4(shape)))
        return out

    def unary(self, op, x, out=None):
        op = _lib.UNARY_OPS.index(op) if isinstance(op, str) else op
        out = out or Buffer(self, x.shape, x.dt)
        check(self.lib.rt_unary(self.handle, op, x.dt, x.ptr, out.ptr, x.numel))
        return out

    def cast(self, x, dst_dt, out=None):
        out = out or Buffer(self, x.shape, dst_dt)
        check(self.lib.rt_cast(self.handle, x.dt, dst_dt, x.ptr, out.ptr, x.numel))
        return out

    def permute(self, x, dims, out=None):
        dims = [int(d) for d in dims]
        pad = 4 - len(dims)
        perm = (ctypes.c_uint32 * 4)(*(list(range(pad)) + [d + pad for d in dims]))   # Permute::promote
        out_shape = [x.shape[d] for d in dims]
        out = out or Buffer(self, out_shape, x.dt)
        check(self.lib.rt_permute(self.handle, _DT_BYTES[x.dt], x.ptr, out.ptr, shape4(x.shape), perm))
        return out

    def slice(self, x, ranges, out=None):
        start = [int(r[0]) for r in ranges]
        dst = [int(r[1]) - int(r[0]) for r in ranges]
        out = out or Buffer(self, dst, x.dt)
        pad = 4 - len(start)
        check(self.lib.rt_slice(self.handle, _DT_BYTES[x.dt], x.ptr, out.ptr, shape4(x.shape),
                                (ctypes.c_uint32 * 4)(*([0] * pad + start)), shape4(dst)))
        return out

    def broadcast_to(self, x, shape, out=None):
        out = out or Buffer(self, shape, x.dt)
        check(self.lib.rt_broadcast(self.handle, _DT_BYTES[x.dt], x.ptr, out.ptr, shape4(x.shape), shape4(shape)))
        return out

    def concat(self, xs, dim, out=None):
        rank = len(xs[0].shape)
        out_shape = list(xs[0].shape)
        out_shape[dim] = sum(x.shape[dim] for x in xs)
        out = out or Buffer(self, out_shape, xs[0].dt)
        ptrs = (ctypes.c_void_p * len(xs))(*[x.ptr.value for x in xs])
        shapes = ((ctypes.c_uint32 * 4) * len(xs))(*[shape4(x.shape) for x in xs])
        check(self.lib.rt_concat(self.handle, _DT_BYTES[xs[0].dt], len(xs), ptrs, shapes, dim + (4 - rank), out.ptr))
        return out

    def cache(self, cache, source, dim, offset, out=None):
        """KV-cache append: returns cat(cache[:offset], source) along dim and writes source into cache at offset."""
        rank = len(cache.shape)
        out_shape = list(cache.shape)
        out_shape[dim] = offset + source.shape[dim]
        out = out or Buffer(self, out_shape, cache.dt)
        check(self.lib.rt_cache(self.handle, _DT_BYTES[cache.dt], cache.ptr, shape4(cache.shape), source.ptr, shape4(source.shape),
                                dim + (4 - rank), offset, out.ptr))
        return out

    def index_select(self, src, indices, dim, out=None):
        """indices: 1-D I32 buffer."""
        rank = len(src.shape)
        out_shape = list(src.shape)
        out_shape[dim] = indices.numel
        out = out or Buffer(self, out_shape, src.dt)
        check(self.lib.rt_index_select(self.handle, _DT_BYTES[src.dt], src.ptr, shape4(src.shape), indices.ptr, indices.numel,
                                       dim + (4 - rank), out.ptr))
        return out

    def index_select_q8_0(self, packed, scales, src_shape, indices, dim, out=None):
        """IndexSelect from a Q8_0 source: packed is the U32 word segment, scales the F32 (Q8_0F) or F16 (Q8_0H) segment of the
        reference's quantized buffer, src_shape the logical shape; the result has the scales' dtype."""
        rank = len(src_shape)
        out_shape = list(src_shape)
        out_shape[dim] = indices.numel
        out = out or Buffer(self, out_shape, scales.dt)
        check(self.lib.rt_index_select_q8_0(self.handle, scales.dt, packed.ptr, scales.ptr, shape4(src_shape), indices.ptr, indices.numel,
                                            dim + (4 - rank), out.ptr))
        return out

    def index_write(self, dst, src, write_start):
        """dst is modified in place and returned."""
        pad = 4 - len(dst.shape)
        check(self.lib.rt_index_write(self.handle, _DT_BYTES[dst.dt], dst.ptr, shape4(dst.shape), src.ptr, src.numel,
                                      (ctypes.c_uint32 * 4)(*([0] * pad + [int(w) for w in write_start]))))
        return dst

    def rope(self, x, dim, base, offset, out=None):
        """x [B, H, S, D]; out may be x."""
        out = out or Buffer(self, x.shape, x.dt)
        check(self.lib.rt_rope(self.handle, x.dt, x.ptr, out.ptr, shape4(x.shape), dim, base, offset))
        return out

    def softmax(self, x, out=None, mode=_lib.SOFTMAX_REFERENCE):
        cols = x.shape[-1]
        out = out or Buffer(self, x.shape, x.dt)
        check(self.lib.rt_softmax(self.handle, x.dt, x.ptr, out.ptr, x.numel // cols, cols, mode))
        return out

    def softmax_masked(self, x, mask, out=None, mode=_lib.SOFTMAX_REFERENCE):
        """softmax over the last dim of x + mask (mask broadcast over x's leading dims), in x's own arithmetic."""
        out = out or Buffer(self, x.shape, x.dt)
        check(self.lib.rt_softmax_masked(self.handle, x.dt, x.ptr, shape4(x.shape), mask.ptr, shape4(mask.shape), out.ptr, mode))
        return out

    def layer_norm(self, x, scale, bias, eps=1e-5, out=None):
        cols = x.shape[-1]
        out = out or Buffer(self, x.shape, x.dt)
        check(self.lib.rt_layer_norm(self.handle, x.dt, x.ptr, scale.ptr, bias.ptr if bias is not None else None, out.ptr,
                                     x.numel // cols, cols, eps))
        return out

    def rms_norm(self, x, scale, eps=1e-5, out=None):
        cols = x.shape[-1]
        out = out or Buffer(self, x.shape, x.dt)
        check(self.lib.rt_rms_norm(self.handle, x.dt, x.ptr, scale.ptr, out.ptr, x.numel // cols, cols, eps))
        return out

    # ---- caller patterns in one pass: what full() -> op -> cast(dt) yields on a 16-bit tensor
    def norm_via_f32(self, kind, x, scale, bias=None, eps=1e-5, out=None):
        """kind 'layer' | 'rms'; x 16-bit, scale / bias f32 buffers."""
        cols = x.shape[-1]
        out = out or Buffer(self, x.shape, x.dt)
        check(self.lib.rt_norm_via_f32(self.handle, {"layer": 0, "rms": 1}[kind], x.dt, x.ptr, scale.ptr,
                                       bias.ptr if bias is not None else None, out.ptr, x.numel // cols, cols, eps))
        return out

    def softmax_via_f32(self, x, mask=None, out=None, mode=_lib.SOFTMAX_REFERENCE):
        """softmax over the last dim of (x + mask) with the mask broadcast over x's leading dims."""
        out = out or Buffer(self, x.shape, x.dt)
        check(self.lib.rt_softmax_via_f32(self.handle, x.dt, x.ptr, shape4(x.shape), mask.ptr if mask is not None else None,
                                          shape4(mask.shape) if mask is not None else None, out.ptr, mode))
        return out

    def unary_via_f32(self, op, x, out=None):
        out = out or Buffer(self, x.shape, x.dt)
        check(self.lib.rt_unary_via_f32(self.handle, _unary_code(op), x.dt, x.ptr, out.ptr, x.numel))
        return out

    def gated_mul_via_f32(self, op, gate, up, rows, cols, gate_row_stride=None, up_row_stride=None, out=None):
        """out[r, c] = up[r, c] * cast(op(full(gate[r, c]))); gate / up may be views with a row stride (elements)."""
        out = out or Buffer(self, (rows, cols), gate.dt)
        check(self.lib.rt_gated_mul_via_f32(self.handle, _unary_code(op), gate.dt, gate.ptr, gate_row_stride or cols, up.ptr,
                                            up_row_stride or cols, out.ptr, rows, cols))
        return out

    def group_norm(self, x, groups, scale, bias, eps=1e-5, out=None, static_scratch=False):
        """static_scratch=True calls rt_group_norm_static, which never allocates (pass `out`, or the Buffer made here does)."""
        B, C = x.shape[0], x.shape[1]
        L = x.numel // (B * C)
        out = out or Buffer(self, x.shape, x.dt)
        fn = self.lib.rt_group_norm_static if static_scratch else self.lib.rt_group_norm
        check(fn(self.handle, x.dt, x.ptr, scale.ptr if scale is not None else None,
                 bias.ptr if bias is not None else None, out.ptr, B, C, L, groups, eps))
        return out
