"""GPU tests through the C++ host mirror of ratchet's Tensor API: the reference's own per-op trials (same problem spaces,
torch as referee, the reference's tolerances) plus graph-level behaviour (multi-op graphs, the in-place rule, fused
broadcasts) checked against the CPU oracle.

Reference trials mirrored: ops/binary.rs:275-334, ops/unary.rs:365-461, ops/softmax.rs:308-365, ops/norm/mod.rs:400-512,
ops/norm/groupnorm.rs:11-87, ops/cast.rs:217-282, ops/concat.rs:273-359, ops/reindex/{permute,slice,broadcast}.rs tests,
and the multi-op attention graph of crates/ratchet-core/tests/attn_tests.rs (without its matmuls).
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from gpu_util import same_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hdev():
    from ratchet_amd.host import HostDevice

    d = HostDevice(0)
    yield d
    d.close()


def T(a, dev):
    from ratchet_amd.host import Tensor

    return Tensor.from_numpy(a, dev)


def close(oracle, got, want, tol):
    bad, mx = oracle.count_not_close(np.ascontiguousarray(got), np.ascontiguousarray(want), tol, tol)
    return bad == 0, (bad, mx)


def test_binary_trials(hdev, oracle):
    rng = np.random.default_rng(400)
    for _ in range(8):
        shape = (int(rng.integers(1, 5)), int(rng.integers(1, 5)), 1, int(rng.integers(1, 257)))
        a, b = rng.standard_normal(shape).astype(np.float32), rng.standard_normal(shape).astype(np.float32)
        for name, tf in (("add", torch.add), ("sub", torch.sub), ("mul", torch.mul), ("div", torch.div)):
            got = getattr(T(a, hdev), name)(T(b, hdev)).resolve().to_numpy()
            ok, info = close(oracle, got, tf(torch.from_numpy(a), torch.from_numpy(b)).numpy(), 1e-4)
            assert ok, (name, shape, info)
            assert same_bits(got, oracle.binary(name, a, b))


def test_unary_trials(hdev, oracle):
    rng = np.random.default_rng(401)
    tf = {"gelu": lambda t: F.gelu(t, approximate="tanh"), "tanh": torch.tanh, "exp": torch.exp, "log": torch.log, "sin": torch.sin,
          "cos": torch.cos, "abs": torch.abs, "sqrt": torch.sqrt, "relu": torch.relu, "floor": torch.floor, "ceil": torch.ceil,
          "neg": torch.neg, "silu": F.silu, "sigmoid": torch.sigmoid}
    for name, fn in tf.items():
        x = rng.standard_normal((int(rng.integers(1, 3)), int(rng.integers(1, 129)))).astype(np.float32)
        got = getattr(T(x, hdev), name)().resolve().to_numpy()
        with np.errstate(all="ignore"):
            want = fn(torch.from_numpy(x)).numpy()
        tol = 5e-2 if name in ("gelu", "tanh") else 1e-4
        ok, info = close(oracle, got, want, tol)
        assert ok, (name, info)


def test_softmax_norm_groupnorm_trials(hdev, oracle):
    rng = np.random.default_rng(402)
    for _ in range(6):
        shape = (int(rng.integers(1, 4)), int(rng.integers(1, 257)), int(rng.integers(1, 257)))
        x = rng.standard_normal(shape).astype(np.float32)
        n = shape[-1]
        got = T(x, hdev).softmax(2).resolve().to_numpy()
        ok, info = close(oracle, got, F.softmax(torch.from_numpy(x), dim=-1).numpy(), 1e-6)
        assert ok, ("softmax", shape, info)
        w, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
        got = T(x, hdev).layer_norm(T(w, hdev), T(b, hdev), 1e-5).resolve().to_numpy()
        want = F.layer_norm(torch.from_numpy(x), (n,), torch.from_numpy(w), torch.from_numpy(b), eps=1e-5).numpy()
        ok, info = close(oracle, got, want, 1e-4)
        assert ok, ("layer_norm", shape, info)
        t = torch.from_numpy(x)
        want = (t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + 1e-5) * torch.from_numpy(w)).numpy()
        got = T(x, hdev).rms_norm(T(w, hdev), 1e-5).resolve().to_numpy()
        ok, info = close(oracle, got, want, 1e-4)
        assert ok, ("rms_norm", shape, info)
    for B, C, L, G in ((1, 3, 1, 1), (2, 8, 5, 4), (1, 64, 40, 32)):
        x = rng.standard_normal((B, C, L)).astype(np.float32)
        w, b = rng.standard_normal(C).astype(np.float32), rng.standard_normal(C).astype(np.float32)
        got = T(x, hdev).group_norm(G, T(w, hdev), T(b, hdev), 1e-5).resolve().to_numpy()
        want = F.group_norm(torch.from_numpy(x), G, torch.from_numpy(w), torch.from_numpy(b), eps=1e-5).numpy()
        ok, info = close(oracle, got, want, 1e-4)
        assert ok, ("group_norm", (B, C, L, G), info)


def test_cast_and_reindex_trials(hdev, oracle):
    from ratchet_amd import _lib
    from ratchet_amd.host import Tensor

    rng = np.random.default_rng(403)
    x = rng.standard_normal((2, 100, 77)).astype(np.float32)
    h = T(x, hdev).cast(_lib.F16).resolve().to_numpy()
    assert same_bits(h, x.astype(np.float16))
    assert np.array_equal(T(x, hdev).cast(_lib.I32).resolve().to_numpy(), x.view(np.int32))
    assert same_bits(T(h, hdev).full().resolve().to_numpy(), h.astype(np.float32))
    xs = [rng.standard_normal((4, 2, k, 128)).astype(np.float32) for k in (50, 13, 77, 55, 11)]
    got = Tensor.cat([T(a, hdev) for a in xs], 2).resolve().to_numpy()
    assert np.array_equal(got, np.concatenate(xs, axis=2))
    for _ in range(8):
        shape = (int(rng.integers(1, 3)), int(rng.integers(1, 5)), int(rng.integers(1, 257)), int(rng.integers(1, 257)))
        perm = [int(p) for p in rng.permutation(4)]
        a = rng.standard_normal(shape).astype(np.float32)
        assert np.array_equal(T(a, hdev).permute(perm).resolve().to_numpy(), np.ascontiguousarray(a.transpose(perm))), (shape, perm)
    for _ in range(8):
        shape = [int(rng.integers(2, 17)) for _ in range(3)] + [int(rng.integers(2, 129))]
        a = rng.standard_normal(shape).astype(np.float32)
        ranges = []
        for s in shape:
            lo = int(rng.integers(0, s))
            ranges.append((lo, int(rng.integers(lo + 1, s + 1))))
        want = a[tuple(slice(lo, hi) for lo, hi in ranges)]
        assert np.array_equal(T(a, hdev).slice(ranges).resolve().to_numpy(), want), (shape, ranges)
    for _ in range(8):
        src = [int(rng.integers(1, 3)), int(rng.integers(1, 9)), int(rng.integers(1, 3)), int(rng.integers(1, 129))]
        dst = [s if s != 1 else int(rng.integers(1, 9)) for s in src]
        a = rng.standard_normal(src).astype(np.float32)
        assert np.array_equal(T(a, hdev).broadcast_to(dst).resolve().to_numpy(), np.broadcast_to(a, dst)), (src, dst)
    one = np.array([3.5], np.float32)                                 # the reference's debug case [1] -> [4,32,128,128]
    assert np.all(T(one, hdev).broadcast_to((4, 32, 128, 128)).resolve().to_numpy() == 3.5)
    v = rng.standard_normal((2, 6)).astype(np.float32)
    assert np.array_equal(T(v, hdev).view((3, 4)).gelu().resolve().to_numpy(), oracle.unary("gelu", v.reshape(3, 4)))


def test_whisper_bias_gelu_layer_norm_graph(hdev, oracle):
    # the reference-runnable benchmark case as ONE lazy graph: bias add (broadcast fused) -> tanh GELU -> LayerNorm, f32
    rng = np.random.default_rng(404)
    x = rng.standard_normal((1, 1500, 384)).astype(np.float32)
    bias = (0.02 * rng.standard_normal(384)).astype(np.float32)
    g = (1 + 0.02 * rng.standard_normal(384)).astype(np.float32)
    b = (0.02 * rng.standard_normal(384)).astype(np.float32)
    y = T(x, hdev).add(T(bias, hdev)).gelu().layer_norm(T(g, hdev), T(b, hdev), 1e-5).resolve()
    # three kernels: the Broadcast node is absorbed by the add, GELU runs in place on the add's buffer
    assert y.last_resolve_launches() == 3
    h = oracle.unary("gelu", oracle.binary("add", x, np.ascontiguousarray(np.broadcast_to(bias, x.shape))))
    want = oracle.layer_norm(h, g, b, 1e-5)
    ok, info = close(oracle, y.to_numpy(), want, 1e-5)
    assert ok, info


def test_phi3_style_attention_tail_graph(hdev, oracle):
    # scores.add(mask) -> full -> softmax(3) -> cast(f16), the pattern of models/phi3/attn.rs:148-153, and SwiGLU
    # up.mul(gate.full().silu().cast(f16)) of models/phi3/mlp.rs:37, in f16 with an f32 mask broadcast over heads
    from ratchet_amd import _lib

    rng = np.random.default_rng(405)
    S, H = 128, 4
    scores = (2 * rng.standard_normal((1, H, S, S))).astype(np.float32)
    mask = np.triu(np.full((S, S), -np.inf, np.float32), k=1)
    y = T(scores, hdev).add(T(mask, hdev)).softmax(3).cast(_lib.F16).resolve()
    want = oracle.cast(oracle.softmax(oracle.binary("add", scores, np.ascontiguousarray(np.broadcast_to(mask, scores.shape)))),
                       np.float16)
    ok, info = close(oracle, y.to_numpy(), want, 1e-3)
    assert ok, info
    assert y.last_resolve_launches() == 2                            # add + softmax go through one call, then the cast
    gate = rng.standard_normal((1, 64, 512)).astype(np.float16)
    up = rng.standard_normal((1, 64, 512)).astype(np.float16)
    z = T(up, hdev).mul(T(gate, hdev).full().silu().cast(_lib.F16)).resolve().to_numpy()
    want = oracle.binary("mul", up, oracle.cast(oracle.unary("silu", oracle.cast(gate, np.float32)), np.float16))
    assert same_bits(z, want)


def test_two_sided_broadcast_and_inplace_rule(hdev, oracle):
    rng = np.random.default_rng(406)
    a = rng.standard_normal((1, 8, 64, 1)).astype(np.float16)
    b = rng.standard_normal((1, 1, 1, 96)).astype(np.float16)
    y = T(a, hdev).mul(T(b, hdev)).resolve()                        # the reference mis-builds this graph (tensor.rs:266-272)
    assert y.shape == (1, 8, 64, 96) and y.last_resolve_launches() == 1
    want = oracle.binary("mul", np.ascontiguousarray(np.broadcast_to(a, y.shape)), np.ascontiguousarray(np.broadcast_to(b, y.shape)))
    assert same_bits(y.to_numpy(), want)
    # in-place rule (tensor.rs:823-824): a source somebody else still holds must keep its contents
    x = rng.standard_normal((4, 100)).astype(np.float32)
    tx = T(x, hdev)
    g = tx.gelu().resolve()
    assert same_bits(tx.resolve().to_numpy(), x)                    # tx is held here, so gelu must not have written into it
    assert same_bits(g.to_numpy(), oracle.unary("gelu", x))
    s = tx.add(tx).resolve()                                        # both operands are the same tensor
    assert same_bits(s.to_numpy(), x + x) and same_bits(tx.to_numpy(), x)
    # a materialised broadcast held by the caller stays a separate tensor
    bt = T(b, hdev).broadcast_to((1, 8, 64, 96))
    y2 = T(a, hdev).mul(bt).resolve()
    assert same_bits(y2.to_numpy(), want)
    assert same_bits(bt.resolve().to_numpy(), np.broadcast_to(b, (1, 8, 64, 96)))


def test_cache_decode_loop(hdev, oracle):
    """phi2's KV append (models/phi2/attn.rs:129-135): the cache tensor is reused across steps and each step's result is
    cat(cache[:offset], new rows); ground truth as in the reference's test (ops/cache.rs:162-217)."""
    from ratchet_amd import _lib

    rng = np.random.default_rng(405)
    cache_np = np.zeros((1, 4, 24, 80), np.float16)
    cache = T(cache_np, hdev)
    rows, off = [], 0
    for n in (7, 1, 1, 1):
        src = rng.standard_normal((1, 4, n, 80)).astype(np.float16)
        rows.append(src)
        got = cache.cache(T(src, hdev), 2, off).resolve().to_numpy()
        off += n
        assert np.array_equal(got, np.concatenate(rows, axis=2))
        assert np.array_equal(got, oracle.cache(cache_np, src, 2, off - n))
    assert np.array_equal(cache.to_numpy(), cache_np)


def test_caller_patterns_resolve_in_one_launch(hdev, oracle):
    """The models' full() -> op -> cast(dt) sequences (ratchet-nn/src/norm.rs:35-44, ratchet-models/src/phi3/attn.rs:143-153,
    phi3/mlp.rs:32-38) are folded by resolve() when nobody else sees the intermediate tensors; results stay within the op
    sequence's own bars and the graph the user built is unchanged."""
    from ratchet_amd import _lib
    from ratchet_amd.host import set_pattern_fusion

    F16, F32 = _lib.F16, _lib.F32
    rng = np.random.default_rng(406)
    x = (rng.standard_normal((2, 64, 2560)) * 2).astype(np.float16)
    w = rng.standard_normal(2560).astype(np.float32)
    b = rng.standard_normal(2560).astype(np.float32)
    S, H = 128, 4
    scores = (2 * rng.standard_normal((1, H, S, S))).astype(np.float16)
    mask = np.triu(np.full((S, S), -np.inf, np.float16), k=1)
    proj = rng.standard_normal((1, 64, 1024)).astype(np.float16)

    def graphs():
        ln = T(x, hdev).full().layer_norm(T(w, hdev), T(b, hdev), 1e-5).cast(F16)
        rms = T(x, hdev).full().rms_norm(T(w, hdev), 1e-5).cast(F16)
        attn = T(scores, hdev).add(T(mask, hdev)).full().softmax(3).cast(F16)
        attn16 = T(scores, hdev).add(T(mask, hdev)).softmax(3)
        act = T(x, hdev).full().gelu().cast(F16)
        p = T(proj, hdev)
        gate, up = p.slice([(0, 1), (0, 64), (0, 512)]), p.slice([(0, 1), (0, 64), (512, 1024)])
        glu = up.mul(gate.full().silu().cast(F16))
        return {"ln": ln, "rms": rms, "attn": attn, "attn16": attn16, "act": act, "glu": glu}

    set_pattern_fusion(False)
    try:
        plain = {k: (g.resolve().to_numpy(), g.last_resolve_launches()) for k, g in graphs().items()}
    finally:
        set_pattern_fusion(True)
    fused = {k: (g.resolve().to_numpy(), g.last_resolve_launches()) for k, g in graphs().items()}
    assert {k: v[1] for k, v in plain.items()} == {"ln": 3, "rms": 3, "attn": 4, "attn16": 2, "act": 3, "glu": 6}
    assert {k: v[1] for k, v in fused.items()} == {"ln": 1, "rms": 1, "attn": 1, "attn16": 1, "act": 1, "glu": 1}
    for k in ("act", "glu", "attn16"):
        assert same_bits(fused[k][0], plain[k][0]), k
    for k in ("ln", "rms", "attn"):
        ok, info = close(oracle, fused[k][0], plain[k][0], 1e-3)
        assert ok, (k, info)
    # against the oracle's op sequence as well
    x32 = oracle.cast(x, np.float32)
    ok, info = close(oracle, fused["ln"][0], oracle.cast(oracle.layer_norm(x32, w, b, 1e-5, intended=True), np.float16), 1e-3)
    assert ok, info
    want = oracle.cast(oracle.softmax(oracle.cast(oracle.binary("add", scores, np.ascontiguousarray(np.broadcast_to(mask, scores.shape))),
                                                  np.float32)), np.float16)
    ok, info = close(oracle, fused["attn"][0], want, 1e-3)
    assert ok, info
    gate_np, up_np = np.ascontiguousarray(proj[..., :512]), np.ascontiguousarray(proj[..., 512:])
    want = oracle.binary("mul", up_np, oracle.cast(oracle.unary("silu", oracle.cast(gate_np, np.float32)), np.float16))
    assert same_bits(fused["glu"][0], want)


def test_masked_softmax_on_a_prompt_of_odd_length_is_one_launch(hdev, oracle):
    """scores.add(mask).softmax(3) in f16 with 1001 tokens (rows that are not whole 16-byte vectors): still folded into
    one launch, still the bits of the two separate ops; the f32-intermediate attention pattern on the same shape too"""
    from ratchet_amd import _lib
    from ratchet_amd.host import set_pattern_fusion

    rng = np.random.default_rng(409)
    S, H = 1001, 3
    scores = (2 * rng.standard_normal((1, H, S, S))).astype(np.float16)
    mask = np.triu(np.full((S, S), -np.inf, np.float16), k=1)
    full_mask = np.ascontiguousarray(np.broadcast_to(mask, scores.shape))
    g = T(scores, hdev).add(T(mask, hdev)).softmax(3).resolve()
    assert g.last_resolve_launches() == 1
    want = oracle.softmax(oracle.binary("add", scores, full_mask))
    assert same_bits(g.to_numpy(), want)
    set_pattern_fusion(False)
    try:
        plain = T(scores, hdev).add(T(mask, hdev)).softmax(3).resolve()
        assert plain.last_resolve_launches() == 2 and same_bits(plain.to_numpy(), want)
    finally:
        set_pattern_fusion(True)
    g32 = T(scores, hdev).add(T(mask, hdev)).full().softmax(3).cast(_lib.F16).resolve()
    assert g32.last_resolve_launches() == 1
    want32 = oracle.cast(oracle.softmax(oracle.cast(oracle.binary("add", scores, full_mask), np.float32)), np.float16)
    ok, info = close(oracle, g32.to_numpy(), want32, 1e-3)
    assert ok, info


def test_pattern_with_a_visible_intermediate_is_not_folded(hdev, oracle):
    from ratchet_amd import _lib

    rng = np.random.default_rng(407)
    x = rng.standard_normal((4, 256)).astype(np.float16)
    w = rng.standard_normal(256).astype(np.float32)
    wide = T(x, hdev).full()                                   # the caller keeps the f32 tensor: it must be materialised
    y = wide.rms_norm(T(w, hdev), 1e-5).cast(_lib.F16).resolve()
    assert y.last_resolve_launches() == 3
    assert wide.resolved() and same_bits(wide.to_numpy(), x.astype(np.float32))
    want = oracle.cast(oracle.rms_norm(oracle.cast(x, np.float32), w, 1e-5, intended=True), np.float16)
    ok, info = close(oracle, y.to_numpy(), want, 1e-3)
    assert ok, info


def test_rope_index_select_index_write_graphs(hdev, oracle):
    """phi3's attention head prep (ratchet-models/src/phi3/attn.rs:118-133): x.full().rope(dim, base, offset).cast(dt); the embedding
    lookup (index_select, dim 0); index_write with the reference's own case (ops/index_write.rs:203-224)."""
    from ratchet_amd import _lib

    rng = np.random.default_rng(408)
    q = rng.standard_normal((1, 8, 33, 96)).astype(np.float32)
    got = T(q, hdev).rope(96, 10000.0, 5).resolve().to_numpy()
    bad, mx = oracle.count_not_close(got, oracle.rope(q, 96, 10000.0, 5), 1e-6, 1e-6)
    assert bad == 0, (bad, mx)
    q16 = q.astype(np.float16)
    got16 = T(q16, hdev).full().rope(96, 10000.0, 5).cast(_lib.F16).resolve().to_numpy()
    want16 = oracle.cast(oracle.rope(oracle.cast(q16, np.float32), 96, 10000.0, 5), np.float16)
    ok, info = close(oracle, got16, want16, 1e-3)
    assert ok, info
    table = rng.standard_normal((1000, 64)).astype(np.float16)
    ids = rng.integers(0, 1000, 19).astype(np.int32)
    got = T(table, hdev).index_select(T(ids, hdev), 0).resolve().to_numpy()
    assert np.array_equal(got, table[ids])
    dst = T(np.array([1, 2, 3, 4, 5, 6], np.float32).reshape(3, 2), hdev)
    out = dst.index_write(T(np.array([[7, 8]], np.float32), hdev), [2, 0]).resolve()
    assert np.array_equal(out.to_numpy(), np.array([[1, 2], [3, 4], [7, 8]], np.float32))
    assert np.array_equal(dst.to_numpy(), out.to_numpy())                      # in place: the destination's buffer is the result


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_embedding_lookup_from_a_quantized_table(hdev, oracle, dtype):
    """Tensor::from_quantized + index_select (tensor.rs:618-628, ops/select.rs:48-60,107-111): the result has the scales'
    type and is, bit for bit, dequantize-then-gather (cpu/mod.rs:86-103); followed by the models' next op on it."""
    from ratchet_amd.host import Tensor

    rng = np.random.default_rng(409)
    for shape, idx in (((256, 32), [64, 192, 255]),                              # the reference's test shape (ops/select.rs:350-357)
                       ((6400, 2560), rng.integers(0, 6400, 77))):               # embedding-table rows, prefill-sized gather
        table = (rng.standard_normal(shape) * 0.05).astype(dtype)
        words, scales = oracle.q8_0_quantize(table)
        ids = np.asarray(idx, np.int32)
        q = Tensor.from_quantized(words, scales, shape, hdev)
        y = q.index_select(T(ids, hdev), 0)
        assert y.shape == (len(ids), shape[1]) and y.dt == (0 if dtype == np.float32 else 1)
        want = oracle.q8_0_index_select(words, scales, shape, ids, 0)
        assert same_bits(y.resolve().to_numpy(), want) and y.last_resolve_launches() == 1
        g = (1 + 0.1 * rng.standard_normal(shape[1])).astype(dtype)
        z = q.index_select(T(ids, hdev), 0).rms_norm(T(g, hdev), 1e-5).resolve().to_numpy()
        ok, info = close(oracle, z, oracle.rms_norm(want, g, 1e-5, intended=True), 1e-5 if dtype == np.float32 else 1e-3)
        assert ok, info


def test_intermediates_return_their_buffers_during_resolve(oracle):
    """What the reference's allocation planner achieves (gpu/buffer_allocator/allocator.rs:141-271): a long graph holds a few
    live buffers, not one per node.  Twelve alternating casts of an 8 MiB tensor (Cast never runs in place) need three
    buffers from the driver, not twelve, and only the result stays allocated afterwards."""
    from ratchet_amd import _lib
    from ratchet_amd.host import HostDevice, set_pattern_fusion

    d = HostDevice(0)
    try:
        rng = np.random.default_rng(409)
        x = rng.standard_normal((1024, 4096)).astype(np.float16)
        tx = T(x, d)
        live0, _, _, misses0 = d.pool_stats()
        set_pattern_fusion(False)                               # keep all twelve casts as launches
        try:
            y = tx
            for _ in range(6):
                y = y.full().half()
            y.resolve()
        finally:
            set_pattern_fusion(True)
        assert y.last_resolve_launches() == 12
        assert same_bits(y.to_numpy(), x)
        live, parked, _, misses = d.pool_stats()
        assert misses - misses0 <= 3, misses - misses0
        assert live - live0 == x.nbytes                         # the result; every intermediate is back in the pool
        # a tensor the caller still holds keeps its buffer
        mid = tx.full()
        z = mid.neg().half().resolve()
        assert mid.resolved() and same_bits(mid.to_numpy(), x.astype(np.float32))
        assert same_bits(z.to_numpy(), oracle.cast(oracle.unary("neg", x.astype(np.float32)), np.float16))
        # a resolved tensor whose inputs were released can still be built upon
        w = y.full().neg().half().resolve()
        assert same_bits(w.to_numpy(), (-x.astype(np.float32)).astype(np.float16))
    finally:
        d.close()
