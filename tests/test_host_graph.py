"""CPU-only checks of the C++ host mirror's graph building: shape/dtype rules, the errors the reference raises, and the
topological order.  Tensors here are placeholders (no storage), so no GPU is needed.

Known answers come from the reference's own rules: Shape::multi_broadcast (shape.rs:118-136, numpy rules), Permute output
shape (ops/reindex/permute.rs:53-56), Concat output shape (ops/concat.rs:116-124), Strides [2,3,4] -> [12,4,1]
(strides.rs:173-179 is the reference's own unit test).
"""
import numpy as np
import pytest

from ratchet_amd import _lib
from ratchet_amd.host import HostError, Tensor

F32, F16 = _lib.F32, _lib.F16


def test_host_header_and_library_agree():
    import os
    import re

    from ratchet_amd import host

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    header = open(os.path.join(root, "include", "ratchet_host.h")).read()
    declared = sorted(set(re.findall(r"\b(rth_[a-z0-9_]+)\(", header)))
    assert len(declared) > 30
    H = host.load()
    for name in declared:
        assert hasattr(H, name), f"{name} is declared in ratchet_host.h but not exported by libratchet_host.so"


def P(*shape, dt=F32):
    return Tensor.placeholder(shape, dt)


@pytest.mark.parametrize("a,b", [((1, 1500, 384), (384,)), ((1, 32, 2048, 1), (1, 1, 1, 2048)), ((3, 1, 5), (1, 7, 1)), ((5, 7), (1,)),
                                 ((1,), (2, 9)), ((4, 1, 8), (4, 6, 8)), ((2, 3), (2, 3))])
def test_binary_shape_is_numpy_broadcast(a, b):
    y = P(*a).add(P(*b))
    assert y.shape == tuple(np.broadcast_shapes(a, b))
    assert y.op_name() == "Add" and not y.resolved()


def test_binary_errors():
    with pytest.raises(HostError) as e:
        P(2, 3).mul(P(2, 4))
    assert e.value.kind == "BroadcastingFailed"                      # InvariantError::BroadcastingFailed (tensor.rs:258-261)
    with pytest.raises(HostError) as e:
        P(2, 3).mul(P(2, 3, dt=F16))
    assert e.value.kind == "DTypeMismatch"                           # Binary::check_dtypes (ops/binary.rs:142-144)
    with pytest.raises(HostError) as e:
        P(2, 3, dt=_lib.I32).add(P(2, 3, dt=_lib.I32))
    assert e.value.kind == "UnsupportedDType"


def test_cast_rules():
    x = P(2, 3)
    assert x.cast(F32).id == x.id                                    # same dtype returns self (tensor.rs:316-318)
    assert x.half().dt == F16 and x.half().full().dt == F32
    assert x.cast(_lib.U32).dt == _lib.U32
    with pytest.raises(HostError) as e:
        P(2, 3, dt=F16).cast(_lib.I32)                               # unimplemented!() in cpu_cast (cpu/mod.rs:152)
    assert e.value.kind == "UnsupportedCast"


def test_permute_rules():
    x = P(1, 1500, 6, 64)
    assert x.permute((0, 2, 1, 3)).shape == (1, 6, 1500, 64)
    assert P(4, 5, 6).permute((2, 0, 1)).shape == (6, 4, 5)
    with pytest.raises(HostError) as e:
        x.permute((0, 1, 1, 3))
    assert e.value.kind == "DuplicateDims"                           # InvariantError::DuplicateDims (permute.rs:49-52)
    with pytest.raises(HostError) as e:
        x.permute((0, 1, 2))
    assert e.value.kind == "RankMismatch"                            # assert!(rank == dims.len()) (permute.rs:69)


def test_slice_broadcast_view_cat_rules():
    x = P(6, 5, 9, 40)
    assert x.slice([(1, 4), (0, 5), (3, 8), (8, 32)]).shape == (3, 5, 5, 24)
    for ranges, kind in (([(0, 7), (0, 5), (0, 9), (0, 40)], "SliceOutOfBounds"), ([(2, 2), (0, 5), (0, 9), (0, 40)], "EmptySlice"),
                         ([(0, 6), (0, 5)], "RankMismatch")):
        with pytest.raises(HostError) as e:
            x.slice(ranges)
        assert e.value.kind == kind
    assert P(1, 5, 1, 16).broadcast_to((3, 5, 4, 16)).shape == (3, 5, 4, 16)
    assert P(7).broadcast_to((2, 7)).shape == (2, 7)
    for src, dst in (((2, 3), (2, 4)), ((2, 3, 4), (3, 4))):
        with pytest.raises(HostError) as e:
            P(*src).broadcast_to(dst)
        assert e.value.kind == "InvalidBroadcast"                    # Broadcast::check_shapes panics (broadcast.rs:31-58)
    assert P(2, 6).view((3, 4)).shape == (3, 4)
    with pytest.raises(HostError) as e:
        P(2, 6).view((12,))                                          # View::check_shapes asserts equal rank (ops/view.rs:19-23)
    assert e.value.kind == "RankMismatch"
    with pytest.raises(HostError) as e:
        P(2, 6).view((3, 5))
    assert e.value.kind == "ShapeMismatch"
    xs = [P(4, 2, k, 128) for k in (50, 13, 77, 55, 11)]             # the reference's concat test (ops/concat.rs:273-359)
    assert Tensor.cat(xs, 2).shape == (4, 2, 206, 128)
    with pytest.raises(HostError) as e:
        Tensor.cat([P(2, 3)], 0)
    assert e.value.kind == "ConcatArity"
    with pytest.raises(HostError) as e:
        Tensor.cat([P(2, 3), P(3, 4)], 0)
    assert e.value.kind == "ConcatShapeMismatch"
    with pytest.raises(HostError) as e:
        Tensor.cat([P(2, 3)] * 9, 0)
    assert e.value.kind == "ConcatArity"


def test_cache_rules():
    # Cache::compute_view and check_shapes (ops/cache.rs:124-147)
    kv = P(1, 32, 2048, 80, dt=F16)
    y = kv.cache(P(1, 32, 1, 80, dt=F16), 2, 17)
    assert y.shape == (1, 32, 18, 80) and y.op_name() == "Cache"
    assert P(1, 1500, 384).cache(P(1, 3, 384), 1, 0).shape == (1, 3, 384)     # whisper's layout (models/whisper/mha.rs:72-79)
    for cache, src, dim, off, kind in ((P(64, 80), P(1, 80), 0, 0, "RankMismatch"), (kv, P(1, 32, 1, 80), 2, 0, "DTypeMismatch"),
                                       (kv, P(1, 32, 1, 80, dt=F16), 2, 2049, "CacheOverflow"), (kv, P(1, 32, 2, 80, dt=F16), 2, 2047, "CacheOverflow"),
                                       (kv, P(1, 16, 1, 80, dt=F16), 2, 0, "ShapeMismatch"), (kv, P(1, 32, 1, 80, dt=F16), 4, 0, "DimOutOfRange")):
        with pytest.raises(HostError) as e:
            cache.cache(src, dim, off)
        assert e.value.kind == kind, (kind, e.value.kind)


def test_rope_and_index_rules():
    q = P(1, 32, 4096, 96)
    assert q.rope(96, 10000.0, 0).shape == q.shape and q.rope(32, 10000.0, 7).op_name() == "RoPE"
    for t, dim, kind in ((P(32, 4096, 96), 96, "RankMismatch"), (q, 128, "ShapeMismatch"), (q, 20, "ShapeMismatch"),
                         (P(1, 2, 3, 8, dt=_lib.I32), 8, "UnsupportedDType")):     # RoPE::check_shapes / check_dtypes (ops/rope.rs:52-66)
        with pytest.raises(HostError) as e:
            t.rope(dim, 10000.0, 0)
        assert e.value.kind == kind
    table, ids = P(51865, 384, dt=F16), P(7, dt=_lib.I32)
    y = table.index_select(ids, 0)                                               # IndexSelect::compute_view (ops/select.rs:48-60)
    assert y.shape == (7, 384) and y.dt == F16 and y.op_name() == "IndexSelect"
    assert table.index_select(ids, 1).shape == (51865, 7)
    for src, idx, dim, kind in ((P(2, 3, 4), ids, 0, "RankMismatch"), (table, P(7, 1, dt=_lib.I32), 0, "RankMismatch"),
                                (table, P(7), 0, "DTypeMismatch"), (table, ids, 2, "DimOutOfRange")):   # ops/select.rs:67-79
        with pytest.raises(HostError) as e:
            src.index_select(idx, dim)
        assert e.value.kind == kind
    dst = P(3, 2)
    assert dst.index_write(P(1, 2), [2, 0]).shape == (3, 2)                      # the reference's test (ops/index_write.rs:203-224)
    for src, ws, kind in ((P(1, 2), [3, 0], "IndexOutOfBounds"), (P(2, 2), [2, 0], "IndexOutOfBounds"), (P(1, 2), [2], "RankMismatch"),
                          (P(1, 2, dt=F16), [2, 0], "DTypeMismatch")):
        with pytest.raises(HostError) as e:
            dst.index_write(src, ws)
        assert e.value.kind == kind


def test_softmax_and_norm_rules():
    x = P(1, 6, 1500, 1500)
    assert x.softmax(3).shape == x.shape
    for t, dim, kind in ((P(8), 0, "RankMismatch"), (x, 4, "DimOutOfRange"), (x, 1, "UnsupportedSoftmaxDim"),
                         (P(2, 3, dt=_lib.I32), 1, "UnsupportedDType")):
        with pytest.raises(HostError) as e:
            t.softmax(dim)
        assert e.value.kind == kind
    h = P(1, 2048, 2560, dt=F16)
    w, b = P(2560, dt=F16), P(2560, dt=F16)
    assert h.layer_norm(w, b, 1e-5).shape == h.shape and h.layer_norm(w, None, 1e-5).op_name() == "Norm"
    assert h.rms_norm(w, 1e-5).shape == h.shape
    with pytest.raises(HostError) as e:
        h.layer_norm(P(2560), b, 1e-5)
    assert e.value.kind == "DTypeMismatch"                           # apply_layer_norm's dtype check (cpu/norm.rs:34-49)
    with pytest.raises(HostError) as e:
        h.rms_norm(P(2561, dt=F16), 1e-5)
    assert e.value.kind == "ShapeMismatch"
    g = P(1, 512, 3000, dt=F16)
    assert g.group_norm(32, P(512, dt=F16), P(512, dt=F16), 1e-5).shape == g.shape
    with pytest.raises(HostError) as e:
        g.group_norm(30, P(512, dt=F16), None, 1e-5)
    assert e.value.kind == "InvalidGroups"


def test_execution_order_is_topological_and_dedups_shared_nodes():
    a, b = P(4, 8), P(8)
    s = a.add(b)                    # Broadcast(b) + Add
    g = s.gelu()
    y = g.mul(s)                    # s is used twice
    order = y.execution_order()
    assert len(order) == len(set(order))
    pos = {i: k for k, i in enumerate(order)}
    assert pos[a.id] < pos[s.id] and pos[b.id] < pos[s.id] < pos[g.id] < pos[y.id]
    assert order[-1] == y.id
    assert len(order) == 6          # a, b, Broadcast(b), s, g, y


def test_placeholders_cannot_be_resolved():
    with pytest.raises(HostError) as e:
        P(2, 3).gelu().resolve()
    assert e.value.kind == "Unresolved"


def test_placeholders_cannot_be_compiled():
    # compile() is resolve() plus a recording of its launches: the same precondition, checked before anything is allocated
    with pytest.raises(HostError) as e:
        P(2, 3).gelu().tanh().compile()
    assert e.value.kind == "Unresolved"


def test_quantized_tensors_are_sources_of_index_select_only():
    # dtype/mod.rs:99-107 (activation_dt), ops/select.rs:48-60: the gather's result has the scales' type; nothing else
    # computes on the packed bytes
    from ratchet_amd.host import Q8_0F, Q8_0H

    ids = Tensor.placeholder((5,), _lib.I32)
    for qdt, act in ((Q8_0F, _lib.F32), (Q8_0H, _lib.F16)):
        q = Tensor.placeholder((64, 32), qdt)
        y = q.index_select(ids, 0)
        assert y.shape == (5, 32) and y.dt == act
        for bad in (lambda: q.gelu(), lambda: q.add(q), lambda: q.full(), lambda: q.softmax(1), lambda: q.permute((1, 0)),
                    lambda: q.view((32, 64)), lambda: q.slice(((0, 1), (0, 32))), lambda: Tensor.cat([q, q], 0),
                    lambda: q.broadcast_to((2, 64, 32)), lambda: q.rms_norm(Tensor.placeholder((32,), _lib.F32), 1e-5)):
            with pytest.raises(HostError) as e:
                bad()
            assert e.value.kind in ("UnsupportedDType", "UnsupportedCast", "DTypeMismatch"), e.value.kind
        with pytest.raises(HostError) as e:
            q.index_select(ids, 1)                                   # rows only
        assert e.value.kind == "ShapeMismatch"
        with pytest.raises(HostError) as e:
            Tensor.placeholder((64, 30), qdt).index_select(ids, 0)   # whole words of four along the row
        assert e.value.kind == "ShapeMismatch"
