"""GPU parity of the one-pass caller patterns against the oracle's op sequence (cast -> f32 op -> cast).

Patterns and where the models emit them: LayerNorm / RMSNorm modules (crates/ratchet-nn/src/norm.rs:35-44, 61-70), attention
softmax (crates/ratchet-models/src/phi3/attn.rs:143-153), activations between full() and cast() (phi2/mlp.rs), the gated
feed-forward of phi3 (phi3/mlp.rs:32-38).  Bars: bit-exact where the f32 op itself is bit-exact on the GPU (elementwise),
the reference's 16-bit tolerance 1e-3 (|a-b| <= tol + tol*|b|) where the f32 sums are tree-ordered (norms, softmax).
"""
import numpy as np
import pytest

from gpu_util import randn, same_bits, describe_mismatch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    from ratchet_amd import Device

    return Device(0)


def close(oracle, got, want, tol):
    bad, mx = oracle.count_not_close(got, want, tol, tol)
    return bad == 0, (bad, mx)


EXACT = ["gelu", "tanh", "exp", "abs", "sqrt", "relu", "floor", "ceil", "neg", "silu", "sigmoid"]


@pytest.mark.parametrize("op", EXACT + ["log", "sin", "cos"])
def test_unary_via_f32_all_f16_inputs(dev, oracle, op):
    x = np.arange(65536, dtype=np.uint16).view(np.float16)
    want = oracle.cast(oracle.unary(op, oracle.cast(x, np.float32)), np.float16)
    got = dev.unary_via_f32(op, dev.upload(x)).to_numpy()
    if op in EXACT:
        assert same_bits(got, want), describe_mismatch(got, want)
    else:                                                     # the f32 op is within 1 ulp of the oracle's: a few roundings may flip
        diff = np.abs(got.view(np.int16).astype(np.int32) - want.view(np.int16).astype(np.int32))
        both_nan = np.isnan(got) & np.isnan(want)
        assert ((diff <= 1) | both_nan).all() and (diff[~both_nan] != 0).sum() <= 64


@pytest.mark.parametrize("op", ["gelu", "silu"])
def test_unary_via_f32_large_tensor_table_path(dev, oracle, op):
    rng = np.random.default_rng(501)
    x = randn(rng, (3, 1024, 1031), np.float16) * np.float16(3)
    x.reshape(-1)[:65536] = np.arange(65536, dtype=np.uint16).view(np.float16)
    want = oracle.cast(oracle.unary(op, oracle.cast(x, np.float32)), np.float16)
    d = dev.upload(x)
    assert same_bits(dev.unary_via_f32(op, d).to_numpy(), want)
    assert same_bits(dev.unary_via_f32(op, d, out=d).to_numpy(), want)          # in place


def test_unary_via_f32_bf16(dev, oracle):
    x = np.arange(65536, dtype=np.uint16)
    for op in ("silu", "gelu", "exp"):
        want = oracle.cast(oracle.unary(op, oracle.cast(x, np.float32, src_bf16=True)), np.uint16, dst_bf16=True)
        got = dev.unary_via_f32(op, dev.upload(x, bf16=True)).to_numpy()
        assert np.array_equal(got[~_bf16_nan(want)], want[~_bf16_nan(want)]) and _bf16_nan(got)[_bf16_nan(want)].all(), op


def _bf16_nan(u):
    return (u & 0x7fff) > 0x7f80


@pytest.mark.parametrize("shape,split", [((2, 1024, 4096), True), ((1, 7, 48), True), ((3, 5, 22), True), ((600, 4096), False),
                                         ((33, 77), False), ((1, 64, 16384), True), ((100, 512), False), ((1, 30, 144), True)])
def test_gated_mul_matches_the_op_sequence(dev, oracle, shape, split):
    """phi3's MLP: up_states.slice(second half).mul(up_states.slice(first half).full().silu().cast(dt))."""
    rng = np.random.default_rng(502)
    if split:
        proj = randn(rng, shape, np.float16) * np.float16(2)
        z = shape[-1]
        gate_np, up_np = np.ascontiguousarray(proj[..., : z // 2]), np.ascontiguousarray(proj[..., z // 2:])
        d = dev.upload(proj)
        from ratchet_amd.runtime import BufferView
        rows = proj.size // z
        gate = BufferView(d, 0, (proj.size - z // 2,))
        up = BufferView(d, z // 2, (proj.size - z // 2,))
        got = dev.gated_mul_via_f32("silu", gate, up, rows, z // 2, gate_row_stride=z, up_row_stride=z).to_numpy()
    else:
        gate_np, up_np = randn(rng, shape, np.float16) * np.float16(2), randn(rng, shape, np.float16)
        got = dev.gated_mul_via_f32("silu", dev.upload(gate_np), dev.upload(up_np), shape[0], shape[1]).to_numpy()
    act = oracle.cast(oracle.unary("silu", oracle.cast(gate_np, np.float32)), np.float16)
    want = oracle.binary("mul", up_np, act)
    assert same_bits(got.reshape(want.shape), want), describe_mismatch(got.reshape(want.shape), want)


@pytest.mark.parametrize("kind", ["layer", "rms"])
@pytest.mark.parametrize("rows,cols", [(64, 2560), (100, 3072), (257, 384), (9, 4096), (5, 1000), (3, 77), (2, 8192), (3, 5120), (2, 16384),
                                       (2, 16392),
                                       # enough rows that a LayerNorm wave (a block, beyond 4096 columns) takes two of them and loads the
                                       # weights once for both; odd row counts leave the last one a row short
                                       (32771, 512), (16385, 1536), (16385, 3072), (16387, 4096), (2049, 8192), (4099, 5120)])
def test_norm_via_f32(dev, oracle, kind, rows, cols):
    rng = np.random.default_rng(503)
    x = (randn(rng, (rows, cols), np.float16) * np.float16(3) + np.float16(0.5)).astype(np.float16)
    w = rng.standard_normal(cols).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    x32 = oracle.cast(x, np.float32)
    if kind == "layer":
        want = oracle.cast(oracle.layer_norm(x32, w, b, 1e-5, intended=True), np.float16)
        got = dev.norm_via_f32("layer", dev.upload(x), dev.upload(w), dev.upload(b), 1e-5).to_numpy()
        want_nb = oracle.cast(oracle.layer_norm(x32, w, None, 1e-5, intended=True), np.float16)
        got_nb = dev.norm_via_f32("layer", dev.upload(x), dev.upload(w), None, 1e-5).to_numpy()
        ok, info = close(oracle, got_nb, want_nb, 1e-3)
        assert ok, ("no bias", info)
    else:
        want = oracle.cast(oracle.rms_norm(x32, w, 1e-5, intended=True), np.float16)
        got = dev.norm_via_f32("rms", dev.upload(x), dev.upload(w), None, 1e-5).to_numpy()
    ok, info = close(oracle, got, want, 1e-3)
    assert ok, info
    # tighter than the bar: the f32 results before the final rounding agree to float rounding, so only the few values that sit
    # on a 16-bit rounding boundary may differ (by one ulp; more only where scale * x + bias cancels towards zero)
    assert (got.view(np.uint16) != want.view(np.uint16)).mean() < 0.01


def _attn_case(rng, B, H, S, T, mask_kind, dtype=np.float16):
    x = (randn(rng, (B, H, S, T), dtype) * dtype(2)).astype(dtype)
    if mask_kind == "causal":
        mask = np.triu(np.full((S, T), -np.inf, dtype), k=1 + T - S)
    elif mask_kind == "causal4":
        mask = np.triu(np.full((S, T), -np.inf, dtype), k=1 + T - S).reshape(1, 1, S, T)
    elif mask_kind == "holes":                                 # finite values with -inf in three places of ten, any S and T
        mask = np.where(rng.random((S, T)) < 0.3, -np.inf, rng.standard_normal((S, T))).astype(dtype)
    elif mask_kind == "per_batch":
        mask = (rng.standard_normal((B, 1, 1, T)) * 2).astype(dtype)
    elif mask_kind == "row_scalar":
        mask = (rng.standard_normal((1, 1, S, 1))).astype(dtype)
    else:
        mask = None
    return x, mask


@pytest.mark.parametrize("B,H,S,T,mask_kind", [(1, 4, 128, 128, "causal"), (2, 3, 64, 200, "causal4"), (1, 6, 100, 1500, None),
                                               (2, 2, 33, 77, "per_batch"), (1, 2, 40, 64, "row_scalar"), (1, 8, 512, 1024, "causal"),
                                               (1, 2, 7, 4096, "causal"), (1, 1, 3, 8200, None), (1, 3, 5, 4100, "causal"),
                                               (1, 2, 6, 8192, "causal"), (2, 1, 3, 16384, "per_batch"), (1, 2, 4, 6000, None),
                                               (1, 1, 2, 16392, None),
                                               # masks of 1 to 8 MiB under several heads (the L2s keep them: plain block order)
                                               (2, 2, 2048, 2048, "causal"), (1, 3, 160, 4096, "causal"),
                                               # masks of 28 MiB and more: the XCD-aware block order (chunks of 64, 4 and 1 row blocks; wave and block per row)
                                               (1, 2, 6144, 2560, "holes"), (1, 2, 5888, 2560, "holes"), (1, 2, 5792, 2560, "holes"),
                                               (1, 2, 3840, 4096, "causal"),
                                               # rows that are not whole vectors (prompts of 1001, 333, 13 tokens): the span kernel
                                               (1, 4, 1001, 1001, "causal"), (2, 3, 333, 333, "causal4"), (1, 2, 5, 13, "causal"),
                                               (2, 2, 9, 1004, "per_batch"), (1, 3, 1, 2047, None), (1, 2, 3, 4101, "causal"),
                                               (1, 2, 2, 9001, None), (1, 1, 3, 1, None), (3, 1, 7, 7, "row_scalar")])
def test_softmax_via_f32(dev, oracle, B, H, S, T, mask_kind):
    rng = np.random.default_rng(504)
    x, mask = _attn_case(rng, B, H, S, T, mask_kind)
    scores = x
    if mask is not None:
        scores = oracle.binary("add", x, np.ascontiguousarray(np.broadcast_to(mask, x.shape)))
    want = oracle.cast(oracle.softmax(oracle.cast(scores, np.float32)), np.float16)
    got = dev.softmax_via_f32(dev.upload(x), dev.upload(mask) if mask is not None else None).to_numpy()
    ok, info = close(oracle, got, want, 1e-3)
    assert ok, info
    ulp = np.abs(got.view(np.int16).astype(np.int32) - want.view(np.int16).astype(np.int32))
    assert ulp.max() <= 1
    if mask_kind and mask_kind.startswith("causal"):
        assert (got[..., 0, 1 + T - S:] == 0).all()           # masked entries are exactly zero
    from ratchet_amd import _lib
    stable = dev.softmax_via_f32(dev.upload(x), dev.upload(mask) if mask is not None else None, mode=_lib.SOFTMAX_STABLE).to_numpy()
    ok, info = close(oracle, stable, want, 1e-3)
    assert ok, ("stable", info)
    dx = dev.upload(x)                                        # in place: a row's ragged ends share vectors with its neighbours
    dev.softmax_via_f32(dx, dev.upload(mask) if mask is not None else None, out=dx)
    assert same_bits(dx.to_numpy(), got)


def test_softmax_via_f32_overflow_and_fully_masked_rows(dev, oracle):
    # exp(100) overflows f32: inf / inf = NaN at that element, 0 elsewhere in the row, as the op sequence gives
    x = np.zeros((1, 1, 4, 16), np.float16)
    x[0, 0, 1, 3] = 100
    x[0, 0, 2, :] = -np.inf                                   # fully masked row: 0 / 0
    want = oracle.cast(oracle.softmax(oracle.cast(x, np.float32)), np.float16)
    got = dev.softmax_via_f32(dev.upload(x)).to_numpy()
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])


def test_fused_entry_points_reject_bad_arguments(dev):
    from ratchet_amd import RatchetError

    x = dev.upload(np.zeros((2, 3, 4, 8), np.float32))
    with pytest.raises(RatchetError) as e:
        dev.softmax_via_f32(x)                                # f32 has no full()/cast() to fold
    assert e.value.status == 2
    h = dev.upload(np.zeros((2, 3, 4, 8), np.float16))
    with pytest.raises(RatchetError) as e:
        dev.softmax_via_f32(h, dev.upload(np.zeros((2, 3, 4, 5), np.float16)))
    assert e.value.status == 4


def test_bf16_patterns(dev, oracle):
    """The same four entry points on bf16 (carried as uint16 bit patterns on the host)."""
    rng = np.random.default_rng(505)

    def bf(a):
        return oracle.cast(np.ascontiguousarray(a, dtype=np.float32), np.uint16, dst_bf16=True)

    def wide(u):
        return oracle.cast(u, np.float32, src_bf16=True)

    def close_bf16(got, want, tol):
        bad, mx = oracle.count_not_close(got, want, tol, tol, bf16=True)
        return bad == 0, (bad, mx)

    # norms: f32 arithmetic, one rounding to bf16 (8 significand bits: the bar is the reference's 16-bit one, relative 1e-2 here)
    x = bf(rng.standard_normal((33, 1024)) * 2 + 0.25)
    w, b = rng.standard_normal(1024).astype(np.float32), rng.standard_normal(1024).astype(np.float32)
    want = bf(oracle.layer_norm(wide(x), w, b, 1e-5, intended=True))
    got = dev.norm_via_f32("layer", dev.upload(x, bf16=True), dev.upload(w), dev.upload(b), 1e-5).to_numpy()
    ok, info = close_bf16(got, want, 1e-2)
    assert ok, info
    assert (got != want).mean() < 0.01
    want = bf(oracle.rms_norm(wide(x), w, 1e-5, intended=True))
    got = dev.norm_via_f32("rms", dev.upload(x, bf16=True), dev.upload(w), None, 1e-5).to_numpy()
    assert (got != want).mean() < 0.01
    # masked softmax
    s = bf(rng.standard_normal((1, 3, 40, 256)) * 2)
    mask = bf(np.triu(np.full((40, 256), -np.inf, np.float32), k=217))
    masked = oracle.binary("add", s, np.ascontiguousarray(np.broadcast_to(mask, s.shape)), bf16=True)
    want = bf(oracle.softmax(wide(masked)))
    got = dev.softmax_via_f32(dev.upload(s, bf16=True), dev.upload(mask, bf16=True)).to_numpy()
    ok, info = close_bf16(got, want, 1e-2)
    assert ok, info
    assert (got != want).mean() < 0.01
    # gated multiply: bit-exact (table path and direct path)
    for shape in ((600, 4096), (5, 24), (40, 512)):
        gate, up = bf(rng.standard_normal(shape) * 2), bf(rng.standard_normal(shape))
        act = bf(oracle.unary("silu", wide(gate)))
        want = oracle.binary("mul", up, act, bf16=True)
        got = dev.gated_mul_via_f32("silu", dev.upload(gate, bf16=True), dev.upload(up, bf16=True), shape[0], shape[1]).to_numpy()
        nan = ((want & 0x7fff) > 0x7f80)
        assert np.array_equal(got[~nan], want[~nan]), shape
