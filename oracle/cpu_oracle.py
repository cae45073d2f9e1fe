"""TEST INFRASTRUCTURE ONLY: numpy-facing loader for the CPU oracle (libratchet_cpu_oracle.so).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module.
The shipped package (ratchet_amd) never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# RATCHET_ORACLE_LIB names another build of the same library (the sanitizer build, oracle/_asan/, in tests/test_sanitizers.py)
_LIB_PATH = os.environ.get("RATCHET_ORACLE_LIB") or os.path.join(_HERE, "libratchet_cpu_oracle.so")

F32, F16, BF16, I32, U32 = 0, 1, 2, 3, 4
ADD, SUB, MUL, DIV = 0, 1, 2, 3
UNARY_OPS = ["gelu", "tanh", "exp", "log", "sin", "cos", "abs", "sqrt", "relu", "floor", "ceil", "neg", "silu", "sigmoid"]
BINARY_OPS = ["add", "sub", "mul", "div"]


def build(force=False):
    """Compile the oracle with the Makefile beside this file (g++ only, a few seconds)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE, "-j4"], check=True, capture_output=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, sz, i, f, d = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_float, ctypes.c_double
        L.orc_binary.argtypes = [i, i, vp, vp, vp, sz]
        L.orc_unary.argtypes = [i, i, vp, vp, sz]
        L.orc_cast.argtypes = [i, i, vp, vp, sz]
        L.orc_permute.argtypes = [i, vp, vp, i, vp, vp]
        L.orc_slice.argtypes = [i, vp, vp, i, vp, vp, vp]
        L.orc_broadcast.argtypes = [i, vp, vp, i, vp, i, vp, i]
        L.orc_concat.argtypes = [i, i, vp, i, vp, i, vp]
        L.orc_cache.argtypes = [i, vp, i, vp, vp, vp, i, ctypes.c_uint64, vp]
        L.orc_rope.argtypes = [i, vp, vp, vp, ctypes.c_uint64, f, ctypes.c_uint64]
        L.orc_index_select.argtypes = [i, vp, i, vp, vp, ctypes.c_uint64, i, vp]
        L.orc_index_write.argtypes = [i, vp, i, vp, vp, ctypes.c_uint64, vp]
        L.orc_q8_0_quantize.argtypes = [i, vp, ctypes.c_uint64, vp, vp]
        L.orc_q8_0_dequantize.argtypes = [i, vp, vp, ctypes.c_uint64, vp]
        L.orc_softmax.argtypes = [i, vp, vp, sz, sz]
        L.orc_layer_norm.argtypes = [i, vp, vp, vp, vp, sz, sz, f, sz]
        L.orc_rms_norm.argtypes = [i, vp, vp, vp, sz, sz, f, sz]
        L.orc_group_norm.argtypes = [i, vp, vp, vp, vp, sz, sz, sz, sz, f]
        L.orc_count_not_close.argtypes = [i, vp, vp, sz, d, d, ctypes.POINTER(d)]
        L.orc_count_not_close.restype = sz
        L.orc_f32_to_f16.argtypes = [f]
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f16_to_f32.restype = f
        L.orc_f32_to_bf16.argtypes = [f]
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_bf16_to_f32.restype = f
        for fn in (L.orc_set_reference_copies, L.orc_set_f16_sum_mode, L.orc_set_hw_f16):
            fn.argtypes = [i]
            fn.restype = None
        _lib = L
    return _lib


def dt_code(dtype, bf16=False):
    dtype = np.dtype(dtype)
    if bf16:
        assert dtype == np.uint16
        return BF16
    return {np.dtype(np.float32): F32, np.dtype(np.float16): F16, np.dtype(np.int32): I32, np.dtype(np.uint32): U32}[dtype]


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _c(a):
    return np.ascontiguousarray(a)


def _u64(v):
    return np.asarray(list(v), dtype=np.uint64)


def _check(rc, what):
    if rc != 0:
        raise ValueError(f"oracle rejected {what} (rc={rc})")


def set_reference_copies(on):
    lib().orc_set_reference_copies(int(bool(on)))


def set_f16_sum_mode(sequential):
    lib().orc_set_f16_sum_mode(int(bool(sequential)))


def set_hw_f16(on):
    lib().orc_set_hw_f16(int(bool(on)))


def binary(op, a, b, bf16=False):
    a, b = _c(a), _c(b)
    assert a.shape == b.shape and a.dtype == b.dtype
    y = np.empty_like(a)
    op = BINARY_OPS.index(op) if isinstance(op, str) else op
    _check(lib().orc_binary(op, dt_code(a.dtype, bf16), _p(a), _p(b), _p(y), a.size), "binary")
    return y


def unary(op, x, bf16=False):
    x = _c(x)
    y = np.empty_like(x)
    op = UNARY_OPS.index(op) if isinstance(op, str) else op
    _check(lib().orc_unary(op, dt_code(x.dtype, bf16), _p(x), _p(y), x.size), "unary")
    return y


def cast(x, dst_dtype, src_bf16=False, dst_bf16=False):
    x = _c(x)
    y = np.empty(x.shape, dtype=dst_dtype)
    _check(lib().orc_cast(dt_code(x.dtype, src_bf16), dt_code(dst_dtype, dst_bf16), _p(x), _p(y), x.size), "cast")
    return y


def permute(x, dims):
    x = _c(x)
    dims = list(dims)
    y = np.empty([x.shape[d] for d in dims], dtype=x.dtype)
    shape = _u64(x.shape)
    d32 = np.asarray(dims, dtype=np.uint32)
    _check(lib().orc_permute(x.dtype.itemsize, _p(x), _p(y), x.ndim, _p(shape), _p(d32)), "permute")
    return y


def slice_(x, ranges):
    x = _c(x)
    start = _u64(r[0] for r in ranges)
    stop = _u64(r[1] for r in ranges)
    y = np.empty([int(b - a) for a, b in zip(start, stop)], dtype=x.dtype)
    _check(lib().orc_slice(x.dtype.itemsize, _p(x), _p(y), x.ndim, _p(_u64(x.shape)), _p(start), _p(stop)), "slice")
    return y


def broadcast(x, to_shape, numpy_semantics=False):
    x = _c(x)
    y = np.empty(tuple(to_shape), dtype=x.dtype)
    _check(lib().orc_broadcast(x.dtype.itemsize, _p(x), _p(y), x.ndim, _p(_u64(x.shape)), len(to_shape),
                               _p(_u64(to_shape)), int(numpy_semantics)), "broadcast")
    return y


def concat(xs, dim):
    xs = [_c(x) for x in xs]
    rank = xs[0].ndim
    shapes = _u64(s for x in xs for s in x.shape)
    out_shape = list(xs[0].shape)
    out_shape[dim] = sum(x.shape[dim] for x in xs)
    y = np.empty(out_shape, dtype=xs[0].dtype)
    ptrs = (ctypes.c_void_p * len(xs))(*[x.ctypes.data for x in xs])
    _check(lib().orc_concat(xs[0].dtype.itemsize, len(xs), ptrs, rank, _p(shapes), dim, _p(y)), "concat")
    return y


def cache(cache_arr, source, dim, offset):
    """KV-cache append: returns dst; cache_arr (C-contiguous, writable) is updated in place as the reference's kernel does."""
    assert cache_arr.flags["C_CONTIGUOUS"] and cache_arr.flags["WRITEABLE"]
    source = _c(source)
    out_shape = list(cache_arr.shape)
    out_shape[dim] = offset + source.shape[dim]
    y = np.empty(out_shape, dtype=cache_arr.dtype)
    _check(lib().orc_cache(cache_arr.dtype.itemsize, _p(cache_arr), cache_arr.ndim, _p(_u64(cache_arr.shape)), _p(source),
                           _p(_u64(source.shape)), dim, offset, _p(y)), "cache")
    return y


def rope(x, dim, base, offset):
    """x [B, H, S, D] float32 (the only dtype the reference's CPU path implements)."""
    x = _c(x)
    assert x.ndim == 4
    y = np.empty_like(x)
    _check(lib().orc_rope(dt_code(x.dtype), _p(x), _p(y), _p(_u64(x.shape)), dim, base, offset), "rope")
    return y


def index_select(src, indices, dim):
    src = _c(src)
    indices = np.ascontiguousarray(indices, dtype=np.int32)
    out_shape = list(src.shape)
    out_shape[dim] = indices.shape[0]
    y = np.empty(out_shape, dtype=src.dtype)
    _check(lib().orc_index_select(src.dtype.itemsize, _p(src), src.ndim, _p(_u64(src.shape)), _p(indices), indices.shape[0], dim, _p(y)),
           "index_select")
    return y


def q8_0_quantize(x):
    """quantize::<Q8_0F / Q8_0H>(x) by x's dtype (float32 / float16): (words uint32 [numel / 4], scales [numel / 32])"""
    x = _c(x)
    fp = 1 if x.dtype == np.float16 else 0
    words = np.empty(x.size // 4, np.uint32)
    scales = np.empty(x.size // 32, x.dtype)
    _check(lib().orc_q8_0_quantize(fp, _p(x), x.size, _p(words), _p(scales)), "q8_0_quantize")
    return words, scales


def q8_0_dequantize(words, scales, shape):
    """dequantize of a Q8_0F (float32 scales) / Q8_0H (float16 scales) buffer to an array of `shape`"""
    words, scales = np.ascontiguousarray(words, np.uint32), _c(scales)
    fp = 1 if scales.dtype == np.float16 else 0
    y = np.empty(shape, scales.dtype)
    _check(lib().orc_q8_0_dequantize(fp, _p(words), _p(scales), y.size, _p(y)), "q8_0_dequantize")
    return y


def q8_0_index_select(words, scales, shape, indices, dim):
    """IndexSelect from a quantized source: dequantize everything, then index_select (cpu/mod.rs:86-103)"""
    return index_select(q8_0_dequantize(words, scales, shape), indices, dim)


def index_write(dst, src, write_start):
    """Writes src (flattened) into dst (C-contiguous, writable, modified in place) from the element write_start addresses."""
    assert dst.flags["C_CONTIGUOUS"] and dst.flags["WRITEABLE"]
    src = _c(src)
    _check(lib().orc_index_write(dst.dtype.itemsize, _p(dst), dst.ndim, _p(_u64(dst.shape)), _p(src), src.size, _p(_u64(write_start))),
           "index_write")
    return dst


def softmax(x, bf16=False):
    x = _c(x)
    cols = x.shape[-1]
    y = np.empty_like(x)
    _check(lib().orc_softmax(dt_code(x.dtype, bf16), _p(x), _p(y), x.size // cols, cols), "softmax")
    return y


def layer_norm(x, scale, bias, eps=1e-5, bf16=False, intended=False):
    """intended=True ignores the reference's scale/bias vector-broadcast special case (shape[0] == N)."""
    x, scale = _c(x), _c(scale)
    bias = _c(bias) if bias is not None else None
    cols = x.shape[-1]
    y = np.empty_like(x)
    shape0 = 1 if intended else x.shape[0]
    _check(lib().orc_layer_norm(dt_code(x.dtype, bf16), _p(x), _p(scale), _p(bias), _p(y), x.size // cols, cols, eps,
                                shape0), "layer_norm")
    return y


def rms_norm(x, scale, eps=1e-5, bf16=False, intended=False):
    x, scale = _c(x), _c(scale)
    cols = x.shape[-1]
    y = np.empty_like(x)
    shape0 = 1 if intended else x.shape[0]
    _check(lib().orc_rms_norm(dt_code(x.dtype, bf16), _p(x), _p(scale), _p(y), x.size // cols, cols, eps, shape0),
           "rms_norm")
    return y


def group_norm(x, groups, scale, bias, eps=1e-5, bf16=False):
    x = _c(x)
    scale = _c(scale) if scale is not None else None
    bias = _c(bias) if bias is not None else None
    B, C = x.shape[0], x.shape[1]
    L = x.size // (B * C)
    y = np.empty_like(x)
    _check(lib().orc_group_norm(dt_code(x.dtype, bf16), _p(x), _p(scale), _p(bias), _p(y), B, C, L, groups, eps),
           "group_norm")
    return y


def count_not_close(a, b, atol, rtol, bf16=False):
    """The reference's all_close rule; returns (failures, max_abs_diff)."""
    a, b = _c(a), _c(b)
    assert a.shape == b.shape and a.dtype == b.dtype
    mx = ctypes.c_double(0.0)
    bad = lib().orc_count_not_close(dt_code(a.dtype, bf16), _p(a), _p(b), a.size, atol, rtol, ctypes.byref(mx))
    return int(bad), float(mx.value)
