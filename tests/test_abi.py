"""CPU-only checks of the C ABI: the library loads without a GPU, exports every symbol the headers under include/ declare, and
rejects bad arguments before touching HIP (so these paths are testable here; no compute call needs a device).

Error behaviour mirrors the reference's guards: Permute duplicate dims (ops/reindex/permute.rs:49-52), Broadcast shape
rule (ops/reindex/broadcast.rs:31-58), Slice bounds (ops/reindex/slice.rs:38-51), Concat arity/shape rule
(ops/concat.rs:131-152), float-only dtypes for binary/unary/softmax/norm (ops/binary.rs:247-270, ops/softmax.rs:36-39).
"""
import ctypes
import os
import re

import pytest

from ratchet_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def u4(*v):
    return (ctypes.c_uint32 * 4)(*v)


HEADERS = ("ratchet_hip.h", "ratchet_hip_debug.h")     # the seam a -sys crate binds, and the library's test hooks


def c_declarations(name):
    """{entry point: argument list} of one header under include/, comments removed"""
    header = open(os.path.join(ROOT, "include", name)).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    return {m.group(1): m.group(2) for m in re.finditer(r"\b(rt_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", header)}


def test_headers_and_library_agree(lib):
    declared = []
    for h in HEADERS:
        names = sorted(c_declarations(h))
        assert names, f"no declarations parsed in {h}"
        declared += names
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared under include/ but not exported"
    assert sorted(_lib.EXPORTS) == sorted(declared)
    # the product header holds no test hook, the debug header nothing else
    assert not [n for n in c_declarations("ratchet_hip.h") if n.startswith("rt_debug_")]
    assert all(n.startswith("rt_debug_") for n in c_declarations("ratchet_hip_debug.h"))


def test_rust_bindings_in_integration_md_list_the_headers_entry_points():
    """the integration guide at the repository root shows the `extern "C"` blocks a ratchet maintainer would put into the
    -sys crate: the first has to name every entry point ratchet_hip.h declares, no other, each with as many arguments as
    the C declaration has; the second (behind a feature) does the same for ratchet_hip_debug.h"""
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = []
    at = 0
    while True:
        at = doc.find('extern "C" {', at)
        if at < 0:
            break
        end = doc.index("\n}\n", at)
        blocks.append(re.sub(r"//[^\n]*", "", doc[at:end]))
        at = end
    assert len(blocks) == len(HEADERS)

    def count(args, void_word):
        args = args.strip()
        return 0 if args in ("", void_word) else args.count(",") + 1

    for h, block in zip(HEADERS, blocks):
        c_decls = c_declarations(h)
        rust_decls = {m.group(1): m.group(2) for m in re.finditer(r"pub fn (rt_[a-z0-9_]+)\s*\((.*?)\)\s*->", block, flags=re.S)}
        assert sorted(rust_decls) == sorted(c_decls), h
        for name in c_decls:
            assert count(rust_decls[name], "") == count(c_decls[name], "void"), name


def test_status_names(lib):
    for code, name in _lib.STATUS_NAMES.items():
        assert lib.rt_status_name(code).decode() == name
    assert lib.rt_status_name(-2).decode() == "HIP_ERROR"


def test_hip_errors_map_to_negative_status_with_the_runtime_s_name(lib):
    """every entry point turns a failed HIP call into -hipError_t and a message that names the call and the runtime's
    own error string; injected here through the test hook, since nothing fails on demand without a GPU"""
    lib.rt_debug_hip_status.argtypes = [ctypes.c_int, ctypes.c_char_p]
    assert lib.rt_debug_hip_status(0, b"nothing") == 0
    for code, name in ((1, b"hipErrorInvalidValue"), (2, b"hipErrorOutOfMemory"), (100, b"hipErrorNoDevice"), (101, b"hipErrorInvalidDevice"),
                       (700, b"hipErrorIllegalAddress"), (719, b"hipErrorLaunchFailure")):
        rc = lib.rt_debug_hip_status(code, b"hipFakeCall(args)")
        assert rc == -code
        msg = lib.rt_last_error()
        assert msg.startswith(b"hipFakeCall(args): ") and name in msg, msg
        assert lib.rt_status_name(rc).decode() == "HIP_ERROR"
    # an argument error reported afterwards replaces the message (the HIP failure is not sticky in the library)
    assert lib.rt_device_create(-1, ctypes.byref(ctypes.c_void_p())) == 7           # RT_ERR_ARG
    assert b"negative ordinal" in lib.rt_last_error()


def test_no_device_is_reported_not_hidden(lib):
    n = ctypes.c_int(-1)
    rc = lib.rt_device_count(ctypes.byref(n))
    if rc != 0:                       # this container has no GPU: a HIP error code, never a silent fallback
        assert rc < 0 and n.value == 0
        h = ctypes.c_void_p()
        assert lib.rt_device_create(0, ctypes.byref(h)) < 0
        assert h.value is None
        assert b"hip" in lib.rt_last_error().lower()


SOME = ctypes.c_void_p(0x1000)        # a non-null, 16-byte aligned fake pointer: validation must reject before using it
ODD = ctypes.c_void_p(0x1001)


def test_binary_validation(lib):
    assert lib.rt_binary(None, 9, _lib.F32, SOME, SOME, SOME, 8) == 3                 # RT_ERR_OP
    assert lib.rt_binary(None, _lib.ADD, _lib.I32, SOME, SOME, SOME, 8) == 2          # RT_ERR_DTYPE
    assert lib.rt_binary(None, _lib.ADD, _lib.F32, None, SOME, SOME, 8) == 1          # RT_ERR_NULL_POINTER
    assert lib.rt_binary(None, _lib.ADD, _lib.F32, SOME, SOME, ODD, 8) == 9           # RT_ERR_ALIGN
    assert lib.rt_binary(None, _lib.ADD, _lib.F32, SOME, SOME, SOME, 1 << 41) == 6    # RT_ERR_SIZE
    assert lib.rt_binary(None, _lib.ADD, _lib.F32, SOME, SOME, SOME, 8) == 8          # all fine but no device
    assert b"NULL" in lib.rt_last_error()


def test_broadcast_binary_validation(lib):
    ok = (None, _lib.MUL, _lib.F16, SOME, u4(1, 32, 64, 1), SOME, u4(1, 1, 1, 64), SOME, u4(1, 32, 64, 64))
    assert lib.rt_binary_bcast(*ok) == 8
    bad = (None, _lib.MUL, _lib.F16, SOME, u4(1, 32, 64, 3), SOME, u4(1, 1, 1, 64), SOME, u4(1, 32, 64, 64))
    assert lib.rt_binary_bcast(*bad) == 4                                             # BroadcastingFailed
    bad = (None, _lib.MUL, _lib.F16, SOME, u4(1, 32, 64, 1), SOME, u4(1, 1, 1, 64), SOME, u4(1, 32, 64, 128))
    assert lib.rt_binary_bcast(*bad) == 4
    zero = (None, _lib.MUL, _lib.F16, SOME, u4(1, 0, 64, 1), SOME, u4(1, 1, 1, 64), SOME, u4(1, 0, 64, 64))
    assert lib.rt_binary_bcast(*zero) == 4


def test_unary_and_cast_validation(lib):
    assert lib.rt_unary(None, 14, _lib.F32, SOME, SOME, 8) == 3
    assert lib.rt_unary(None, 0, _lib.U32, SOME, SOME, 8) == 2
    assert lib.rt_unary(None, 0, _lib.F16, SOME, None, 8) == 1
    assert lib.rt_unary(None, 0, _lib.F16, SOME, SOME, 8) == 8
    assert lib.rt_cast(None, _lib.F16, _lib.I32, SOME, SOME, 8) == 2                  # unimplemented!() in the reference
    assert lib.rt_cast(None, _lib.F16, _lib.BF16, SOME, SOME, 8) == 2
    assert lib.rt_cast(None, 7, _lib.F32, SOME, SOME, 8) == 2
    assert lib.rt_cast(None, _lib.F32, _lib.F16, SOME, SOME, 8) == 8
    assert lib.rt_cast(None, _lib.F32, _lib.U32, SOME, SOME, 8) == 8


def test_reindex_validation(lib):
    shp = u4(2, 3, 4, 5)
    assert lib.rt_permute(None, 4, SOME, SOME, shp, u4(0, 1, 1, 3)) == 5              # DuplicateDims
    assert lib.rt_permute(None, 4, SOME, SOME, shp, u4(0, 1, 2, 4)) == 5
    assert lib.rt_permute(None, 3, SOME, SOME, shp, u4(0, 1, 2, 3)) == 7              # elem_bytes
    assert lib.rt_permute(None, 4, SOME, SOME, shp, u4(3, 2, 1, 0)) == 8
    assert lib.rt_slice(None, 2, SOME, SOME, shp, u4(0, 0, 0, 3), u4(2, 3, 4, 3)) == 4   # 3 + 3 > 5
    assert lib.rt_slice(None, 2, SOME, SOME, shp, u4(0, 0, 0, 0), u4(2, 3, 4, 0)) == 4   # empty range
    assert lib.rt_slice(None, 2, SOME, SOME, shp, u4(1, 0, 0, 2), u4(1, 3, 4, 3)) == 8
    assert lib.rt_broadcast(None, 4, SOME, SOME, u4(1, 3, 1, 5), u4(2, 3, 4, 6)) == 4
    assert lib.rt_broadcast(None, 4, SOME, SOME, u4(1, 3, 1, 5), u4(2, 3, 4, 5)) == 8
    shapes = ((ctypes.c_uint32 * 4) * 2)(u4(1, 2, 3, 4), u4(1, 2, 5, 4))
    ptrs = (ctypes.c_void_p * 2)(0x1000, 0x2000)
    assert lib.rt_concat(None, 4, 2, ptrs, shapes, 2, SOME) == 8
    assert lib.rt_concat(None, 4, 2, ptrs, shapes, 1, SOME) == 4                      # differs outside the concat dim
    assert lib.rt_concat(None, 4, 1, ptrs, shapes, 2, SOME) == 7                      # needs 2..8 inputs
    assert lib.rt_concat(None, 4, 9, ptrs, shapes, 2, SOME) == 7
    assert lib.rt_concat(None, 4, 2, ptrs, shapes, 4, SOME) == 7
    cs, ss = u4(1, 2, 6, 16), u4(1, 2, 1, 16)
    assert lib.rt_cache(None, 4, SOME, cs, SOME, ss, 2, 2, SOME) == 8
    assert lib.rt_cache(None, 4, SOME, cs, SOME, ss, 2, 6, SOME) == 4                 # offset 6 + 1 row > 6
    assert lib.rt_cache(None, 4, SOME, cs, SOME, ss, 2, 7, SOME) == 4                 # offset > cache extent (ops/cache.rs:127)
    assert lib.rt_cache(None, 4, SOME, cs, SOME, u4(1, 3, 1, 16), 2, 0, SOME) == 4    # differs outside dim
    assert lib.rt_cache(None, 4, SOME, cs, SOME, ss, 4, 0, SOME) == 7
    assert lib.rt_cache(None, 8, SOME, cs, SOME, ss, 2, 0, SOME) == 7
    assert lib.rt_cache(None, 4, None, cs, SOME, ss, 2, 0, SOME) == 1


def test_reduction_validation(lib):
    assert lib.rt_softmax(None, _lib.I32, SOME, SOME, 4, 8, 0) == 2
    assert lib.rt_softmax(None, _lib.F32, SOME, SOME, 4, 8, 5) == 7                   # unknown mode
    assert lib.rt_softmax(None, _lib.F32, SOME, SOME, 4, 0, 0) == 4
    assert lib.rt_softmax(None, _lib.F32, SOME, SOME, 4, 8, 0) == 8
    assert lib.rt_layer_norm(None, _lib.F32, SOME, None, None, SOME, 4, 8, 1e-5) == 1   # scale is required
    assert lib.rt_layer_norm(None, _lib.F32, SOME, SOME, None, SOME, 4, 8, 1e-5) == 8   # bias is optional
    assert lib.rt_layer_norm(None, _lib.F32, SOME, SOME, None, SOME, 4, 8, float("nan")) == 7
    assert lib.rt_rms_norm(None, _lib.U32, SOME, SOME, SOME, 4, 8, 1e-5) == 2
    assert lib.rt_group_norm(None, _lib.F16, SOME, None, None, SOME, 1, 6, 4, 4, 1e-5) == 7   # 6 channels, 4 groups
    assert lib.rt_group_norm(None, _lib.F16, SOME, None, None, SOME, 1, 8, 4, 4, 1e-5) == 8


def test_rope_and_index_validation(lib):
    shp = u4(1, 2, 4, 24)
    assert lib.rt_rope(None, _lib.F32, SOME, SOME, shp, 16, 10000.0, 0) == 8
    assert lib.rt_rope(None, _lib.F32, SOME, SOME, shp, 12, 10000.0, 0) == 4                 # dim % 8 (ops/rope.rs:57)
    assert lib.rt_rope(None, _lib.F32, SOME, SOME, shp, 32, 10000.0, 0) == 4                 # dim > head_dim (ops/rope.rs:56)
    assert lib.rt_rope(None, _lib.I32, SOME, SOME, shp, 16, 10000.0, 0) == 2
    assert lib.rt_rope(None, _lib.F32, SOME, SOME, shp, 16, -1.0, 0) == 7
    assert lib.rt_index_select(None, 4, SOME, u4(1, 1, 8, 4), SOME, 3, 2, SOME) == 8
    assert lib.rt_index_select(None, 4, SOME, u4(1, 1, 8, 4), SOME, 0, 2, SOME) == 4
    assert lib.rt_index_select(None, 4, SOME, u4(1, 1, 8, 4), None, 3, 2, SOME) == 1
    assert lib.rt_index_select(None, 1, SOME, u4(1, 1, 8, 4), SOME, 3, 2, SOME) == 7
    # quantized source: whole groups of 32 elements, runs of whole 4-element words (quant.rs:20-21, ops/select.rs:144-161)
    assert lib.rt_index_select_q8_0(None, _lib.F32, SOME, SOME, u4(1, 1, 8, 32), SOME, 3, 2, SOME) == 8
    assert lib.rt_index_select_q8_0(None, _lib.F16, SOME, SOME, u4(1, 1, 8, 32), SOME, 3, 2, SOME) == 8
    assert lib.rt_index_select_q8_0(None, _lib.BF16, SOME, SOME, u4(1, 1, 8, 32), SOME, 3, 2, SOME) == 2
    assert lib.rt_index_select_q8_0(None, _lib.F32, SOME, SOME, u4(1, 1, 8, 30), SOME, 3, 2, SOME) == 4    # 240 elements: not whole groups
    assert lib.rt_index_select_q8_0(None, _lib.F32, SOME, SOME, u4(1, 1, 32, 2), SOME, 3, 2, SOME) == 4    # runs of 2 elements
    assert lib.rt_index_select_q8_0(None, _lib.F32, SOME, None, u4(1, 1, 8, 32), SOME, 3, 2, SOME) == 1
    assert lib.rt_index_select_q8_0(None, _lib.F32, SOME, SOME, u4(1, 1, 8, 32), SOME, 0, 2, SOME) == 4
    assert lib.rt_index_select_q8_0(None, _lib.F32, SOME, SOME, u4(1, 1, 8, 32), SOME, 3, 4, SOME) == 7
    assert lib.rt_index_write(None, 4, SOME, u4(1, 1, 3, 2), SOME, 2, u4(0, 0, 2, 0)) == 8
    assert lib.rt_index_write(None, 4, SOME, u4(1, 1, 3, 2), SOME, 3, u4(0, 0, 2, 0)) == 4   # the run would leave dst
    assert lib.rt_index_write(None, 4, SOME, u4(1, 1, 3, 2), SOME, 1, u4(0, 0, 3, 0)) == 4   # write_start outside dst


def test_fused_pattern_validation(lib):
    f32p = ctypes.cast(ctypes.c_void_p(0x1000), ctypes.c_void_p)
    assert lib.rt_norm_via_f32(None, 0, _lib.F16, SOME, f32p, None, SOME, 4, 8, 1e-5) == 8
    assert lib.rt_norm_via_f32(None, 2, _lib.F16, SOME, f32p, None, SOME, 4, 8, 1e-5) == 7      # kind
    assert lib.rt_norm_via_f32(None, 0, _lib.F32, SOME, f32p, None, SOME, 4, 8, 1e-5) == 2      # f32 needs no full()/cast()
    assert lib.rt_norm_via_f32(None, 1, _lib.BF16, SOME, None, None, SOME, 4, 8, 1e-5) == 1
    shp = u4(1, 2, 4, 8)
    assert lib.rt_softmax_via_f32(None, _lib.F16, SOME, shp, None, None, SOME, 0) == 8
    assert lib.rt_softmax_via_f32(None, _lib.F16, SOME, shp, SOME, u4(1, 1, 4, 8), SOME, 0) == 8
    assert lib.rt_softmax_via_f32(None, _lib.F16, SOME, shp, SOME, u4(1, 3, 4, 8), SOME, 0) == 4
    assert lib.rt_softmax_via_f32(None, _lib.F16, SOME, shp, SOME, None, SOME, 0) == 1
    assert lib.rt_softmax_via_f32(None, _lib.F32, SOME, shp, None, None, SOME, 0) == 2
    assert lib.rt_softmax_via_f32(None, _lib.F16, SOME, shp, None, None, SOME, 3) == 7
    assert lib.rt_unary_via_f32(None, 0, _lib.F16, SOME, SOME, 16) == 8
    assert lib.rt_unary_via_f32(None, 14, _lib.F16, SOME, SOME, 16) == 3
    assert lib.rt_unary_via_f32(None, 0, _lib.I32, SOME, SOME, 16) == 2
    assert lib.rt_gated_mul_via_f32(None, 12, _lib.F16, SOME, 16, SOME, 16, SOME, 4, 8) == 8
    assert lib.rt_gated_mul_via_f32(None, 12, _lib.F16, SOME, 4, SOME, 16, SOME, 4, 8) == 4      # stride shorter than a row
    assert lib.rt_gated_mul_via_f32(None, 12, _lib.F32, SOME, 16, SOME, 16, SOME, 4, 8) == 2


def test_graph_validation(lib):
    assert lib.rt_capture_begin(None) == 8
    p = ctypes.c_void_p()
    assert lib.rt_capture_end(None, ctypes.byref(p)) == 8
    assert lib.rt_capture_end(None, None) == 1
    assert lib.rt_graph_launch(None, None) == 1
    assert lib.rt_graph_destroy(None) == 0
    assert lib.rt_status_name(10) == b"RT_ERR_CAPTURE"


def test_pool_validation(lib):
    assert lib.rt_pool_trim(None) == 8
    assert lib.rt_pool_begin_pass(None) == 8
    assert lib.rt_pool_stats(None, None, None, None, None) == 8


def test_storage_validation(lib):
    p = ctypes.c_void_p()
    assert lib.rt_malloc(None, 16, ctypes.byref(p)) == 8
    assert lib.rt_malloc(None, 16, None) == 1
    assert lib.rt_sync(None) == 8
    assert lib.rt_h2d(None, None, None, 16) == 1
    assert lib.rt_event_elapsed_ms(None, None, None) == 1


def test_python_binding_fails_loudly_without_library(tmp_path, monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "missing.so"))
    with pytest.raises(ImportError):
        _lib.load()
