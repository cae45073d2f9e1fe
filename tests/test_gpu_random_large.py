"""Seeded random shapes at the sizes where the row kernels and the reindex kernels change strategy: thousands of rows
(the streaming 16-bit softmax, with every mask broadcast pattern), tens of thousands of narrow rows (one lane per row),
ragged rows, rows beyond 4096 columns, and transposes / concats / casts / RoPE / table-driven unaries over a few million
elements.  The small-shape random tests never reach these paths.  Same bars as the fixed-shape tests: bit-exact for the
reference f16 / bf16 softmax, reindex and casts; the all_close bars for norms, f32-intermediate softmax, RoPE, unaries."""
import numpy as np
import pytest

from gpu_util import randn, same_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    from ratchet_amd import Device

    d = Device(0)
    yield d
    d.close()


@pytest.mark.parametrize("seed", range(12))
def test_rows_random_large(dev, oracle, seed):
    rng = np.random.default_rng(5000 + seed)
    kind = seed % 4
    if kind == 0:      # streaming sizes, whole vectors
        b, h = int(rng.integers(1, 4)), int(rng.integers(1, 9))
        t = int(rng.integers(30, 1200))
        cols = int(rng.integers(1, 1100)) * 8
        shape = (b, h, t, cols)
    elif kind == 1:    # many narrow rows
        shape = (int(rng.integers(32768, 90000)), int(rng.integers(1, 17)) * 8)
    elif kind == 2:    # ragged
        shape = (int(rng.integers(1, 3)), int(rng.integers(1, 9)), int(rng.integers(30, 700)), int(rng.integers(1, 3000)))
    else:              # long rows
        shape = (int(rng.integers(1, 40)), int(rng.integers(513, 4000)) * 8)
    while np.prod(shape) > 24_000_000:
        k = int(np.argmax(shape[:-1]))
        shape = shape[:k] + (max(1, shape[k] // 2),) + shape[k + 1:]
    x = randn(rng, shape, np.float16, 2.0)
    dx = dev.upload(x)
    want = oracle.softmax(x)
    assert same_bits(dev.softmax(dx).to_numpy(), want), ("softmax", shape)
    xb = oracle.cast(x.astype(np.float32), np.uint16, dst_bf16=True)
    got = dev.softmax(dev.upload(xb, bf16=True)).to_numpy()
    wb = oracle.softmax(xb, bf16=True)
    nan = (wb & 0x7fff) > 0x7f80
    assert np.array_equal(got[~nan], wb[~nan]), ("bf16", shape)
    if len(shape) == 4:
        for mshape in ((1, 1) + shape[2:], (shape[0], 1) + shape[2:], shape, (1, 1, 1, shape[3])):
            mask = randn(rng, mshape, np.float16)
            mask[rng.random(mshape) < 0.3] = -np.inf
            want = oracle.softmax(oracle.binary("add", x, np.ascontiguousarray(np.broadcast_to(mask, shape))))
            assert same_bits(dev.softmax_masked(dx, dev.upload(mask)).to_numpy(), want), ("masked", shape, mshape)
            got = dev.softmax_via_f32(dx, dev.upload(mask)).to_numpy()
            w2 = oracle.cast(oracle.softmax(oracle.binary("add", x, np.ascontiguousarray(np.broadcast_to(mask, shape))).astype(np.float32)), np.float16)
            bad, mx = oracle.count_not_close(got, w2, 1e-3, 1e-3)
            assert bad == 0, ("via32 masked", shape, mshape, mx)
    cols = shape[-1]
    w, bb = randn(rng, (cols,), np.float16), randn(rng, (cols,), np.float16)
    got = dev.layer_norm(dx, dev.upload(w), dev.upload(bb), 1e-5).to_numpy()
    want = oracle.layer_norm(x, w, bb, 1e-5, intended=True)
    bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
    assert bad == 0, ("ln", shape, mx)
    got = dev.rms_norm(dx, dev.upload(w), 1e-5).to_numpy()
    want = oracle.rms_norm(x, w, 1e-5, intended=True)
    bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
    assert bad == 0, ("rms", shape, mx)


def dims(rng, rank):
    pool = [1, 2, 3, 4, 5, 8, 12, 16, 24, 32, 40, 64, 80, 96, 100, 128, 160, 200, 256, 333, 512]
    while True:
        s = tuple(int(rng.choice(pool)) for _ in range(rank))
        if 1000 < np.prod(s) < 6_000_000:
            return s


@pytest.mark.parametrize("seed", range(10))
def test_reindex_random_large(dev, oracle, seed):
    rng = np.random.default_rng(7000 + seed)
    for _ in range(6):
        dtype = (np.float32, np.float16)[int(rng.integers(0, 2))]
        rank = int(rng.integers(2, 5))
        shape = dims(rng, rank)
        x = randn(rng, shape, dtype)
        dx = dev.upload(x)
        perm = [int(p) for p in rng.permutation(rank)]
        assert np.array_equal(dev.permute(dx, perm).to_numpy(), x.transpose(perm)), ("permute", shape, perm)
        ranges = []
        for s in shape:
            lo = int(rng.integers(0, s)) if rng.random() < 0.5 else 0
            ranges.append((lo, int(rng.integers(lo + 1, s + 1)) if rng.random() < 0.5 else s))
        assert np.array_equal(dev.slice(dx, ranges).to_numpy(), x[tuple(slice(a, b) for a, b in ranges)]), ("slice", shape, ranges)
        dim = int(rng.integers(0, rank))
        parts = []
        for _k in range(int(rng.integers(2, 6))):
            s = list(shape)
            s[dim] = int(rng.integers(1, 20))
            parts.append(randn(rng, s, dtype))
        assert np.array_equal(dev.concat([dev.upload(p) for p in parts], dim).to_numpy(), np.concatenate(parts, axis=dim)), ("concat", shape, dim)
        # casts
        if dtype == np.float32:
            assert same_bits(dev.cast(dx, 1).to_numpy(), x.astype(np.float16)), ("cast", shape)
        else:
            assert same_bits(dev.cast(dx, 0).to_numpy(), x.astype(np.float32)), ("cast", shape)
        # rope on the last two dims
        if rank == 4 and shape[-1] % 8 == 0:
            hd = shape[-1]
            rd = int(rng.choice([d for d in (hd, hd // 2, 8, 16, 32) if d <= hd and d % 8 == 0 and d > 0]))
            off = int(rng.integers(0, 3000))
            if dtype == np.float32:
                want = oracle.rope(x, rd, 10000.0, off)
                got = dev.rope(dx, rd, 10000.0, off).to_numpy()
                bad, mx = oracle.count_not_close(got, want, 1e-5, 1e-5)
                assert bad == 0, ("rope", shape, rd, off, mx)
            else:
                want = oracle.cast(oracle.rope(x.astype(np.float32), rd, 10000.0, off), np.float16)
                got = dev.rope(dx, rd, 10000.0, off).to_numpy()
                bad, mx = oracle.count_not_close(got, want, 2e-3, 2e-3)
                assert bad == 0, ("rope16", shape, rd, off, mx)
        # unaries across the table / gather / direct size thresholds
        if dtype == np.float16:
            for op in ("gelu", "silu", "tanh", "exp"):
                got = dev.unary(op, dx).to_numpy()
                want = oracle.unary(op, x)
                bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
                assert bad == 0, (op, shape, mx)


@pytest.mark.parametrize("seed", range(12))
def test_ragged_rows_masked_softmax_random(dev, oracle, seed):
    """16-bit softmax with and without a mask on rows that are not whole vectors: every mask broadcast pattern, mask periods on
    both sides of the 240 rows where groups stop running across periods, masks at 16-byte offsets inside an allocation"""
    from ratchet_amd.runtime import BufferView
    rng = np.random.default_rng(11000 + seed)
    b, h = int(rng.integers(1, 3)), int(rng.integers(1, 7))
    s = int(rng.choice([1, 2, 7, 30, 31, 100, 239, 240, 241, 500]))
    t = int(rng.choice([193, 199, 255, 257, 511, 513, 1001, 1023, 1535, 2047, 2049, 3001, 4095, int(rng.integers(192, 4096))]))
    shape = (b, h, s, t)
    bf = bool(rng.integers(0, 2))
    xf = (rng.standard_normal(shape) * 2).astype(np.float32)
    x = oracle.cast(xf, np.uint16, dst_bf16=True) if bf else xf.astype(np.float16)
    dx = dev.upload(x, bf16=bf)
    isnan = (lambda v: (v & 0x7fff) > 0x7f80) if bf else (lambda v: (v.view(np.uint16) & 0x7fff) > 0x7c00)
    for mshape in ((1, 1, s, t), (b, 1, s, t), (b, h, s, t), (1, 1, 1, t)):
        mf = rng.standard_normal(mshape).astype(np.float32)
        mf[rng.random(mshape) < 0.3] = -np.inf
        mask = oracle.cast(mf, np.uint16, dst_bf16=True) if bf else mf.astype(np.float16)
        full = np.ascontiguousarray(np.broadcast_to(mask, shape))
        want = oracle.softmax(oracle.binary("add", x, full, bf16=bf), bf16=bf)
        moff = int(rng.choice([0, 8, 16]))
        mbuf = dev.empty((mask.size + 24,), 2 if bf else 1)
        mv = BufferView(mbuf, moff, mshape).upload(mask)
        got = dev.softmax_masked(dx, mv).to_numpy()
        bad = (got.view(np.uint16) != want.view(np.uint16)) & ~(isnan(got) & isnan(want))
        assert not bad.any(), (shape, mshape, moff, int(bad.sum()), np.argwhere(bad)[:5])
    want = oracle.softmax(x, bf16=bf)
    got = dev.softmax(dx).to_numpy()
    bad = (got.view(np.uint16) != want.view(np.uint16)) & ~(isnan(got) & isnan(want))
    assert not bad.any(), (shape, "plain", int(bad.sum()))


@pytest.mark.parametrize("seed", range(9))
def test_f32_rows_random_large(dev, oracle, seed):
    """f32 softmax, norms and unaries over thousands of rows, tens of thousands of narrow rows and rows of up to 20000 columns
    (most of them not whole vectors).  Layer norm is held to 1e-4 here: the reference's one-pass variance amplifies the
    rounding of the sums by mean^2 / variance, and among a few hundred thousand random short rows some are ill conditioned."""
    rng = np.random.default_rng(8000 + seed)
    kind = seed % 3
    if kind == 0:
        shape = (int(rng.integers(200, 6000)), int(rng.integers(1, 600)) * 4)
    elif kind == 1:
        shape = (int(rng.integers(20000, 70000)), int(rng.integers(1, 40)))
    else:
        shape = (int(rng.integers(1, 300)), int(rng.integers(1, 20000)))
    while np.prod(shape) > 12_000_000:
        shape = (max(1, shape[0] // 2), shape[1])
    x = randn(rng, shape, np.float32, 2.0)
    dx = dev.upload(x)
    got = dev.softmax(dx).to_numpy()
    bad, mx = oracle.count_not_close(got, oracle.softmax(x), 1e-5, 1e-5)
    assert bad == 0, ("softmax", shape, mx)
    cols = shape[-1]
    w, b = randn(rng, (cols,), np.float32), randn(rng, (cols,), np.float32)
    got = dev.layer_norm(dx, dev.upload(w), dev.upload(b), 1e-5).to_numpy()
    bad, mx = oracle.count_not_close(got, oracle.layer_norm(x, w, b, 1e-5, intended=True), 1e-4, 1e-4)
    assert bad == 0 or cols < 3, ("ln", shape, mx)
    got = dev.rms_norm(dx, dev.upload(w), 1e-5).to_numpy()
    bad, mx = oracle.count_not_close(got, oracle.rms_norm(x, w, 1e-5, intended=True), 1e-5, 1e-5)
    assert bad == 0, ("rms", shape, mx)
    for op in ("gelu", "tanh", "exp", "silu", "sigmoid", "sqrt", "neg", "abs", "relu", "log", "sin", "cos", "floor", "ceil"):
        want = oracle.unary(op, x)
        got = dev.unary(op, dx).to_numpy()
        bad, mx = oracle.count_not_close(got, want, 1e-5, 1e-5)
        assert bad == 0, (op, shape, mx)

@pytest.mark.parametrize("seed", range(8))
def test_group_norm_and_cache_random(dev, oracle, seed):
    rng = np.random.default_rng(8100 + seed)
    for dtype, tol in ((np.float32, 1e-4), (np.float16, 2e-3)):
        B, G = int(rng.integers(1, 4)), int(rng.choice([1, 2, 4, 8, 32]))
        cpg, L = int(rng.integers(1, 9)), int(rng.integers(1, 5000))
        C = G * cpg
        x = randn(rng, (B, C, L), dtype)
        w, b = randn(rng, (C,), dtype), randn(rng, (C,), dtype)
        got = dev.group_norm(dev.upload(x), G, dev.upload(w), dev.upload(b), 1e-5).to_numpy()
        want = oracle.group_norm(x, G, w, b, 1e-5)
        bad, mx = oracle.count_not_close(got, want, tol, tol)
        assert bad == 0, ("gn", B, C, L, G, dtype.__name__, mx)
        # cache
        bb, h, T, hd = int(rng.integers(1, 3)), int(rng.integers(1, 9)), int(rng.integers(4, 600)), int(rng.choice([8, 64, 80, 96, 128, 100]))
        n = int(rng.integers(1, T))
        off = int(rng.integers(0, T - n + 1))
        c, s = randn(rng, (bb, h, T, hd), dtype), randn(rng, (bb, h, n, hd), dtype)
        dc = dev.upload(c)
        got = dev.cache(dc, dev.upload(s), 2, off).to_numpy()
        c2 = c.copy()
        want = oracle.cache(c2, s, 2, off)
        assert same_bits(got, want) and same_bits(dc.to_numpy(), c2), ("cache", c.shape, n, off)

@pytest.mark.parametrize("seed", range(8))
def test_binary_broadcast_random_large(dev, oracle, seed):
    rng = np.random.default_rng(8200 + seed)
    pool = [1, 2, 3, 5, 8, 12, 32, 50, 64, 80, 128, 200, 256, 1000, 1001, 2560]
    for _ in range(8):
        dtype = (np.float32, np.float16)[int(rng.integers(0, 2))]
        rank = int(rng.integers(1, 5))
        while True:
            out = tuple(int(rng.choice(pool)) for _ in range(rank))
            if np.prod(out) < 8_000_000:
                break
        sa = tuple(s if rng.random() < 0.7 else 1 for s in out)
        sb = tuple(s if (rng.random() < 0.7 or sa[i] == 1) else 1 for i, s in enumerate(out))
        if rng.random() < 0.3:
            sb = tuple(sb[int(rng.integers(0, rank)):]) or (1,)
        try:
            oshape = np.broadcast_shapes(sa, sb)
        except ValueError:
            continue
        a, b = randn(rng, sa, dtype), randn(rng, sb, dtype)
        op = ("add", "sub", "mul", "div")[int(rng.integers(0, 4))]
        want = oracle.binary(op, np.ascontiguousarray(np.broadcast_to(a, oshape)), np.ascontiguousarray(np.broadcast_to(b, oshape)))
        got = dev.binary(op, dev.upload(a), dev.upload(b)).to_numpy()
        assert got.shape == tuple(oshape) and same_bits(got, want), (op, sa, sb)
