"""Properties at the full sizes of the benchmark configurations (too large for the oracle to walk in test time): round
trips, row sums, repetition over heads, agreement between two independent paths of the library.  Small-size parity against
the oracle lives in the other test_gpu_* files; here the question is whether indexing, chunking and grid mapping hold up
at 2^29-element tensors."""
import numpy as np
import pytest

from gpu_util import same_bits

pytestmark = pytest.mark.gpu

F32, F16 = 0, 1


@pytest.fixture(scope="module")
def dev():
    from ratchet_amd import Device

    d = Device(0)
    yield d
    d.close()


def test_whisper_scores_softmax_rows_sum_to_one_and_permute_round_trip(dev, oracle):
    rng = np.random.default_rng(701)
    scores = (3 * rng.standard_normal((1, 6, 1500, 1500))).astype(np.float32)
    y = dev.softmax(dev.upload(scores)).to_numpy()
    sums = y.sum(axis=-1, dtype=np.float64)
    assert np.abs(sums - 1).max() < 1e-5
    assert (y >= 0).all() and np.array_equal(y.argmax(-1), scores.argmax(-1))
    bad, mx = oracle.count_not_close(y[0, 3, 700:764], oracle.softmax(scores[0, 3, 700:764]), 1e-5, 1e-5)   # a slab from the middle
    assert bad == 0, mx
    q = rng.standard_normal((1, 1500, 6, 64)).astype(np.float32)
    dq = dev.upload(q)
    p = dev.permute(dq, (0, 2, 1, 3))
    assert np.array_equal(p.to_numpy(), q.transpose(0, 2, 1, 3))
    assert same_bits(dev.permute(p, (0, 2, 1, 3)).to_numpy(), q)


def test_f32_causal_softmax_at_a_2048_token_prompt(dev, oracle):
    """scores.add(mask).softmax(3) on f32 scores [1,32,2048,2048]: the one-launch path against the two ops (bits), the
    mask's zeros, row sums, and a slab of rows against the oracle"""
    rng = np.random.default_rng(702)
    H, S = 32, 2048
    scores = (2 * rng.standard_normal((1, H, S, S))).astype(np.float32)
    mask = np.triu(np.full((S, S), -np.inf, np.float32), k=1)
    dx, dm = dev.upload(scores), dev.upload(mask)
    dy = dev.softmax_masked(dx, dm)
    y = dy.to_numpy()
    two = dev.softmax(dev.binary("add", dx, dm))
    assert same_bits(y, two.to_numpy())
    del two
    upper = np.triu(np.ones((S, S), bool), k=1)
    assert not y[0, :, upper].any()                                    # masked entries are exactly zero in every head
    assert np.abs(y.sum(axis=-1, dtype=np.float64) - 1).max() < 1e-5
    sl = slice(1000, 1032)
    want = oracle.softmax(oracle.binary("add", scores[0, 17, sl], mask[sl]))
    bad, mx = oracle.count_not_close(y[0, 17, sl], want, 1e-5, 1e-5)
    assert bad == 0, mx


def test_phi2_block_identities(dev, oracle):
    rng = np.random.default_rng(702)
    x = rng.standard_normal((1, 2048, 2560)).astype(np.float16)
    a = (0.5 * rng.standard_normal((1, 2048, 2560))).astype(np.float16)
    dx, da = dev.upload(x), dev.upload(a)
    r = dev.binary("add", dx, da)
    assert same_bits(dev.binary("sub", r, da).to_numpy(), oracle.binary("sub", oracle.binary("add", x, a), a))    # whole tensor, exact
    assert same_bits(dev.cast(dev.cast(dx, F32), F16).to_numpy(), x)                                               # f16 -> f32 -> f16 is the identity
    g = (1 + 0.02 * rng.standard_normal(2560)).astype(np.float16)
    b = (0.02 * rng.standard_normal(2560)).astype(np.float16)
    ln = dev.layer_norm(r, dev.upload(g), dev.upload(b), 1e-5).to_numpy()
    rr = r.to_numpy()
    rows = [0, 1, 777, 2047]
    want = oracle.layer_norm(rr[0, rows], g, b, 1e-5, intended=True)
    assert same_bits(ln[0, rows], want)
    h = rng.standard_normal((1, 2048, 10240)).astype(np.float16)
    ge = dev.unary("gelu", dev.upload(h)).to_numpy()
    table = oracle.unary("gelu", np.arange(65536, dtype=np.uint16).view(np.float16))                               # every f16 input, once
    assert same_bits(ge, table[h.view(np.uint16)])


def test_phi3_attention_tail_at_full_size(dev, oracle):
    S, H = 4096, 32
    rng = np.random.default_rng(703)
    head = (2 * rng.standard_normal((S, S))).astype(np.float16)
    mask = np.triu(np.full((S, S), -np.inf, np.float16), k=1)
    scores = dev.empty((1, H, S, S), F16)
    dh = dev.upload(head)
    from ratchet_amd import _lib
    for h in range(H):
        _lib.check(dev.lib.rt_d2d(dev.handle, scores.ptr.value + h * head.nbytes, dh.ptr, head.nbytes))
    masked = dev.binary("add", scores, dev.upload(mask))
    # the add itself (from 1 GiB the broadcast kernel makes one access per thread), and the same size with a row operand
    mk = masked.to_numpy()
    assert all(same_bits(mk[0, h, 1000:1064], head[1000:1064] + mask[1000:1064]) for h in (0, 17, 31))
    del mk
    row = rng.standard_normal(S).astype(np.float16)
    biased = dev.binary("add", scores, dev.upload(row)).to_numpy()
    assert all(same_bits(biased[0, h, -64:], head[-64:] + row) for h in (0, 9, 31))
    del biased
    soft = dev.softmax(masked)
    out = soft.to_numpy()
    # every head holds the same data, so every head must hold the same result, bit for bit (catches any grid / chunk mapping slip)
    assert all(same_bits(out[0, h], out[0, 0]) for h in range(1, H))
    rows = list(range(0, 64)) + list(range(2016, 2080)) + list(range(4032, 4096))
    want = oracle.softmax(oracle.binary("add", head[rows], mask[rows]))
    assert same_bits(out[0, 0, rows], want)
    assert not out[0, 0][np.triu_indices(S, k=1)].any()                            # masked positions are exactly zero
    # no "rows sum to one" here: the reference accumulates the 4096 exp terms in f16, terms below half an ulp of the running
    # sum vanish, and long rows come out up to ~10 % heavy; the oracle rows above pin exactly that behaviour
    # the one-pass path (f32 inside) agrees with the f16 path within the 16-bit bar, and is again identical across heads
    fused = dev.softmax_via_f32(scores, dev.upload(mask)).to_numpy()
    assert all(same_bits(fused[0, h], fused[0, 0]) for h in (1, 13, 31))
    want = oracle.cast(oracle.softmax(oracle.cast(oracle.binary("add", head[rows], mask[rows]), np.float32)), np.float16)
    bad, mx = oracle.count_not_close(fused[0, 0, rows], want, 1e-3, 1e-3)
    assert bad == 0, mx
    assert np.abs(fused[0, 0].astype(np.float64).sum(-1) - 1).max() < 1e-3         # f32 sums inside: these rows do sum to one


def test_phi3_mlp_and_norm_at_full_size(dev, oracle):
    rng = np.random.default_rng(704)
    gate = rng.standard_normal((1, 4096, 8192)).astype(np.float16)
    up = rng.standard_normal((1, 4096, 8192)).astype(np.float16)
    dg, du = dev.upload(gate), dev.upload(up)
    table = oracle.unary("silu", np.arange(65536, dtype=np.uint16).view(np.float16))
    act = dev.unary("silu", dg)
    assert same_bits(act.to_numpy(), table[gate.view(np.uint16)])
    got = dev.binary("mul", du, act).to_numpy()
    assert same_bits(got[0, 1000:1016], oracle.binary("mul", up[0, 1000:1016], table[gate[0, 1000:1016].view(np.uint16)]))
    x = rng.standard_normal((1, 4096, 3072)).astype(np.float16)
    g = (1 + 0.02 * rng.standard_normal(3072)).astype(np.float16)
    rn = dev.rms_norm(dev.upload(x), dev.upload(g), 1e-5).to_numpy()
    rows = [0, 5, 2048, 4095]
    assert same_bits(rn[0, rows], oracle.rms_norm(x[0, rows], g, 1e-5, intended=True))


def test_reindex_stress_round_trips(dev, oracle):
    rng = np.random.default_rng(705)
    ka = rng.standard_normal((1, 32, 1984, 80)).astype(np.float16)
    kb = rng.standard_normal((1, 32, 64, 80)).astype(np.float16)
    cat = dev.concat([dev.upload(ka), dev.upload(kb)], 2)
    assert same_bits(dev.slice(cat, [(0, 1), (0, 32), (0, 1984), (0, 80)]).to_numpy(), ka)       # concat then slice gives the parts back
    assert same_bits(dev.slice(cat, [(0, 1), (0, 32), (1984, 2048), (0, 80)]).to_numpy(), kb)
    cache = dev.upload(np.concatenate([ka, np.zeros_like(kb)], axis=2))
    assert same_bits(dev.cache(cache, dev.upload(kb), 2, 1984).to_numpy(), cat.to_numpy())          # the KV append builds the same tensor
    a = rng.standard_normal((1, 32, 2048, 1)).astype(np.float16)
    b = rng.standard_normal((1, 1, 1, 2048)).astype(np.float16)
    m = dev.binary("mul", dev.upload(a), dev.upload(b)).to_numpy()
    assert same_bits(m, a * b)                                                                    # numpy's f16 product is correctly rounded too
    p = rng.standard_normal((1, 2048, 32, 80)).astype(np.float16)
    dp = dev.upload(p)
    t = dev.permute(dp, (0, 2, 1, 3))
    assert np.array_equal(t.to_numpy(), p.transpose(0, 2, 1, 3))
    assert same_bits(dev.permute(t, (0, 2, 1, 3)).to_numpy(), p)
    gx = rng.standard_normal((1, 512, 3000)).astype(np.float16)
    gw, gb = rng.standard_normal(512).astype(np.float16), rng.standard_normal(512).astype(np.float16)
    gn = dev.group_norm(dev.upload(gx), 32, dev.upload(gw), dev.upload(gb), 1e-5).to_numpy()
    bad, mx = oracle.count_not_close(gn, oracle.group_norm(gx, 32, gw, gb, 1e-5), 1e-3, 1e-3)
    assert bad == 0, mx


def test_casts_and_gathers_beyond_the_one_access_per_thread_thresholds(dev, oracle):
    """From 2^23 elements a cast, and from 48 MB a permute / slice without repeated source dims, run one access per
    thread instead of four / two: the same results, bit for bit, on sizes just past the switch (with a ragged tail)."""
    rng = np.random.default_rng(77)
    n = (1 << 23) + 5
    x32 = rng.standard_normal(n).astype(np.float32)
    got16 = dev.cast(dev.upload(x32), F16).to_numpy()
    assert same_bits(got16, x32.astype(np.float16))
    assert same_bits(got16, oracle.cast(x32, np.float16))
    assert same_bits(dev.cast(dev.upload(got16), F32).to_numpy(), got16.astype(np.float32))
    # 64 MB head swap and its way back; a slice of it with offsets in every dim
    q = rng.standard_normal((4, 1024, 64, 128)).astype(np.float16)
    dq = dev.upload(q)
    p = dev.permute(dq, (0, 2, 1, 3))
    assert same_bits(p.to_numpy(), q.transpose(0, 2, 1, 3))
    assert same_bits(dev.permute(p, (0, 2, 1, 3)).to_numpy(), q)
    big = rng.standard_normal((5, 1030, 64, 136)).astype(np.float16)
    got = dev.slice(dev.upload(big), [(1, 5), (3, 1027), (0, 64), (8, 136)]).to_numpy()
    assert same_bits(got, big[1:5, 3:1027, :, 8:136])


def test_large_transpose_takes_the_patch_kernel(dev):
    """From 128 MB on (and for source rows of 9-12 vectors, covered at small sizes in test_gpu_reindex.py) a permutation
    that moves the contiguous dim runs through the LDS patch kernel: K^T of eight Phi-2-sized layers at once, and the
    [B,T,H,D] -> [B,H,D,T] form with a ragged last patch."""
    rng = np.random.default_rng(78)
    k = rng.standard_normal((8, 32, 2048, 128)).astype(np.float16)
    dk = dev.upload(k)
    assert same_bits(dev.permute(dk, (0, 1, 3, 2)).to_numpy(), k.transpose(0, 1, 3, 2))
    x = rng.standard_normal((4, 2056, 32, 136)).astype(np.float16)
    assert same_bits(dev.permute(dev.upload(x), (0, 2, 3, 1)).to_numpy(), x.transpose(0, 2, 3, 1))
    # 32-bit tensors of that size: patches of 128 x 64 elements, ragged on both sides here (8200 = 64 * 128 + 8, 4100 = 64 * 64 + 4)
    m = rng.standard_normal((1, 8200, 4100)).astype(np.float32)
    assert same_bits(dev.permute(dev.upload(m), (0, 2, 1)).to_numpy(), m.transpose(0, 2, 1))
    h = rng.standard_normal((2, 2056, 32, 260)).astype(np.float32)
    assert same_bits(dev.permute(dev.upload(h), (0, 2, 3, 1)).to_numpy(), h.transpose(0, 2, 3, 1))
    # channels to planes and back at image-batch size (a contiguous dim of 5 that changes sides; H and W merge into one run)
    img = rng.standard_normal((4, 1024, 1024, 5)).astype(np.float16)
    planes = dev.permute(dev.upload(img), (0, 3, 1, 2))
    assert same_bits(planes.to_numpy(), img.transpose(0, 3, 1, 2))
    assert same_bits(dev.permute(planes, (0, 2, 3, 1)).to_numpy(), img)
    del planes
    # 16-bit tensors of that size whose rows are not whole 128-byte lines stay with the 64 x 64 patches in the widest units
    m16 = rng.standard_normal((1, 8200, 8200)).astype(np.float16)
    assert same_bits(dev.permute(dev.upload(m16), (0, 2, 1)).to_numpy(), m16.transpose(0, 2, 1))


def test_ops_across_the_4_gib_boundary(dev, oracle):
    """Tensors of 2^31 + 2^20 + 24 f16 elements (4.3 GB): element 2^31 lies at byte 2^32, where a 32-bit byte offset or
    element index would wrap.  The tensor repeats a 2^24-element pattern, so any window of it is known without holding
    4 GB on the host; the windows checked sit at the start, across the boundary and at the ragged end."""
    from ratchet_amd import _lib
    from ratchet_amd.runtime import BufferView

    P = 1 << 24
    n = (1 << 31) + (1 << 20) + 24
    rng = np.random.default_rng(707)
    pat = (2 * rng.standard_normal(P)).astype(np.float16)
    pat[:8] = [0.0, -0.0, np.inf, -np.inf, np.nan, 65504.0, 6e-8, -6e-8]
    x = dev.empty((n,), F16)
    dp = dev.upload(pat)
    for k in range(0, n, P):
        _lib.check(dev.lib.rt_d2d(dev.handle, x.ptr.value + 2 * k, dp.ptr, 2 * min(P, n - k)))
    windows = [(0, 64), ((1 << 31) - 40, (1 << 31) + 40), (n - 56, n)]

    def expect(lo, hi):
        return pat[np.arange(lo, hi) % P]

    def window(buf, lo, hi):
        return BufferView(buf, lo, (hi - lo,)).to_numpy()

    y = dev.binary("add", x, x)
    for lo, hi in windows:
        assert same_bits(window(y, lo, hi), oracle.binary("add", expect(lo, hi), expect(lo, hi))), ("add", lo)
    dev.unary("gelu", x, out=y)                                        # the table kernel
    for lo, hi in windows:
        assert same_bits(window(y, lo, hi), oracle.unary("gelu", expect(lo, hi))), ("gelu", lo)
    dev.unary("neg", x, out=y)                                         # the computing kernel
    for lo, hi in windows:
        assert same_bits(window(y, lo, hi), oracle.unary("neg", expect(lo, hi))), ("neg", lo)
    del y
    wide = dev.cast(x, F32)
    for lo, hi in windows:
        assert same_bits(window(wide, lo, hi), expect(lo, hi).astype(np.float32)), ("cast", lo)
    del wide
    # the last rows of the aligned part as a slice: source offsets beyond 2^32 bytes
    cols = 4096
    rows = ((1 << 31) + (1 << 20)) // cols
    tail = dev.slice(BufferView(x, 0, (1, 1, rows, cols)), [(0, 1), (0, 1), (rows - 300, rows), (0, cols)]).to_numpy()
    assert same_bits(tail.reshape(-1), expect((rows - 300) * cols, rows * cols))
    # row ops over the same bytes as [rows, 4096]: the rows on either side of byte 2^32 and the last ones
    xr = BufferView(x, 0, (rows, cols))
    at = [(1 << 31) // cols - 1, (1 << 31) // cols + 1, rows - 3, rows - 2, rows - 1]
    want_rows = np.stack([expect(r * cols, (r + 1) * cols) for r in at])
    g = (1 + 0.02 * rng.standard_normal(cols)).astype(np.float16)
    b = (0.02 * rng.standard_normal(cols)).astype(np.float16)

    def rows_of(buf):
        return np.stack([window(buf, r * cols, (r + 1) * cols) for r in at])

    out = dev.layer_norm(xr, dev.upload(g), dev.upload(b), 1e-5)
    assert same_bits(rows_of(out), oracle.layer_norm(want_rows, g, b, 1e-5, intended=True))
    dev.rms_norm(xr, dev.upload(g), 1e-5, out=out)
    assert same_bits(rows_of(out), oracle.rms_norm(want_rows, g, 1e-5, intended=True))
    dev.softmax(xr, out=out)                                           # split into launches of less than 2 GiB
    assert same_bits(rows_of(out), oracle.softmax(want_rows))
    dev.softmax_via_f32(xr, out=out)
    want = oracle.cast(oracle.softmax(oracle.cast(want_rows, np.float32)), np.float16)
    bad, mx = oracle.count_not_close(rows_of(out), want, 1e-3, 1e-3)
    assert bad == 0, mx
    g32 = g.astype(np.float32)
    dev.norm_via_f32("rms", xr, dev.upload(g32), None, 1e-5, out=out)
    want = oracle.cast(oracle.rms_norm(oracle.cast(want_rows, np.float32), g32, 1e-5, intended=True), np.float16)
    bad, mx = oracle.count_not_close(rows_of(out), want, 1e-3, 1e-3)
    assert bad == 0, mx


def test_reindex_across_the_4_gib_boundary(dev):
    """Permutes of a 4.3 GB f16 tensor (a repeated 2^24-element pattern): moving heads in front of the sequence (vector
    gather) and transposing the last two dims (LDS patches); windows of the result on either side of byte 2^32."""
    from ratchet_amd import _lib
    from ratchet_amd.runtime import BufferView

    P = 1 << 24
    n = (1 << 31) + (1 << 20)
    pat = np.random.default_rng(708).integers(0, 1 << 16, P, dtype=np.uint16).view(np.float16)     # any bits: nothing is computed
    x = dev.empty((n,), F16)
    dp = dev.upload(pat)
    for k in range(0, n, P):
        _lib.check(dev.lib.rt_d2d(dev.handle, x.ptr.value + 2 * k, dp.ptr, 2 * min(P, n - k)))

    def src(idx):
        return pat[np.asarray(idx, dtype=np.int64) % P]

    # [1, S, 32, 128] -> [1, 32, S, 128]: out[h, s, :] = in[s, h, :]
    S, H, D = n // (32 * 128), 32, 128
    y = dev.permute(BufferView(x, 0, (1, S, H, D)), (0, 2, 1, 3))
    for h, s in ((0, 0), (15, S // 2), (16, (1 << 31) // (H * D) - 1), (16, (1 << 31) // (H * D)), (31, S - 1)):
        got = BufferView(y, (h * S + s) * D, (D,)).to_numpy()
        assert same_bits(got, src((s * H + h) * D + np.arange(D))), (h, s)
    # [1, 2049, 4096, 256] -> [1, 2049, 256, 4096]: slab 2048 starts at byte 2^32
    A, R, C = n // (4096 * 256), 4096, 256
    dev.permute(BufferView(x, 0, (1, A, R, C)), (0, 1, 3, 2), out=BufferView(y, 0, (1, A, C, R)))
    for a, c in ((0, 0), (2047, 255), (2048, 0), (2048, 129), (A - 1, 255)):
        got = BufferView(y, (a * C + c) * R, (R,)).to_numpy()
        assert same_bits(got, src((a * R + np.arange(R)) * C + c)), (a, c)


def test_concat_cache_and_broadcast_across_the_4_gib_boundary(dev, oracle):
    """A 4.3 GB KV-cache-shaped tensor [1, 16, 32784, 4096] f16 built by concat from two halves, appended to through the
    cache op, and added to a row vector: windows of the results in the first head and in the last (beyond byte 2^32)."""
    from ratchet_amd import _lib
    from ratchet_amd.runtime import BufferView

    P = 1 << 24
    Hd, R, C = 16, 16392, 4096
    half = Hd * R * C                                                  # 2.1 GB each
    rng = np.random.default_rng(709)
    pat = rng.standard_normal(P).astype(np.float16)
    x = dev.empty((2 * half,), F16)
    dp = dev.upload(pat)
    for k in range(0, 2 * half, P):
        _lib.check(dev.lib.rt_d2d(dev.handle, x.ptr.value + 2 * k, dp.ptr, 2 * min(P, 2 * half - k)))

    def src(idx):
        return pat[np.asarray(idx, dtype=np.int64) % P]

    a, b = BufferView(x, 0, (1, Hd, R, C)), BufferView(x, half, (1, Hd, R, C))
    cat = dev.concat([a, b], 2)                                        # [1, 16, 32784, 4096]
    cols = np.arange(C)

    def cat_row(h, r):                                                 # what row r of head h of `cat` holds
        return src((h * R + r) * C + cols) if r < R else src(half + (h * R + r - R) * C + cols)

    def row_of(buf, h, r, rows_per_head=2 * R):
        return BufferView(buf, (h * rows_per_head + r) * C, (C,)).to_numpy()

    probes = [(0, 0), (0, R - 1), (0, R), (7, 2 * R - 1), (8, 0), (15, R - 1), (15, R), (15, 2 * R - 1)]
    for h, r in probes:
        assert same_bits(row_of(cat, h, r), cat_row(h, r)), ("concat", h, r)
    # append 8 new rows per head at row 32776 of the cache: dst = cat(cache[:32776], new), and the cache holds them too
    new = rng.standard_normal((1, Hd, 8, C)).astype(np.float16)
    dst = dev.cache(cat, dev.upload(new), 2, 2 * R - 8)
    for h, r in probes:
        want = new[0, h, r - (2 * R - 8)] if r >= 2 * R - 8 else cat_row(h, r)
        assert same_bits(row_of(dst, h, r), want), ("cache dst", h, r)
        assert same_bits(row_of(cat, h, r), want), ("cache", h, r)
    # the whole tensor plus a row vector
    row = rng.standard_normal(C).astype(np.float16)
    dev.binary("add", cat, dev.upload(row), out=dst)
    for h, r in probes:
        base = new[0, h, r - (2 * R - 8)] if r >= 2 * R - 8 else cat_row(h, r)
        assert same_bits(row_of(dst, h, r), oracle.binary("add", base, row)), ("add", h, r)


def test_rope_and_index_select_across_the_4_gib_boundary(dev, oracle):
    """RoPE on a 4.3 GB f32 tensor [1, 32, 349600, 96] and an embedding lookup from a 4.3 GB f16 table: positions and
    rows whose bytes lie beyond 2^32."""
    from ratchet_amd import _lib
    from ratchet_amd.runtime import BufferView

    P = 1 << 22
    H, S, D = 32, 349600, 96
    n = H * S * D                                                      # 1.07e9 f32 elements
    rng = np.random.default_rng(710)
    pat = rng.standard_normal(P).astype(np.float32)
    x = dev.empty((1, H, S, D), F32)
    dp = dev.upload(pat)
    for k in range(0, n, P):
        _lib.check(dev.lib.rt_d2d(dev.handle, x.ptr.value + 4 * k, dp.ptr, 4 * min(P, n - k)))
    y = dev.rope(x, 64, 10000.0, 3)                                    # rotate 64 of the 96 columns, positions from 3
    for h, s0 in ((0, 0), (15, S - 16), (16, 0), (31, S - 16)):
        first = (h * S + s0) * D
        win = pat[(first + np.arange(16 * D)) % P].reshape(1, 1, 16, D)
        got = BufferView(y, first, (1, 1, 16, D)).to_numpy()
        want = oracle.rope(win, 64, 10000.0, 3 + s0)
        bad, mx = oracle.count_not_close(got, want, 1e-5, 1e-5)
        assert bad == 0, (h, s0, mx)
    del y, x
    # embedding lookup: table [524544, 4096] f16
    V, C = 524544, 4096
    pat16 = rng.integers(0, 1 << 16, 1 << 24, dtype=np.uint16).view(np.float16)
    table = dev.empty((V, C), F16)
    dp = dev.upload(pat16)
    for k in range(0, V * C, 1 << 24):
        _lib.check(dev.lib.rt_d2d(dev.handle, table.ptr.value + 2 * k, dp.ptr, 2 * min(1 << 24, V * C - k)))
    ids = np.array([0, 524287, 524288, V - 1, 17, 524400, V - 2, 300000], np.int32)
    emb = dev.index_select(table, dev.upload(ids), 0).to_numpy()
    for i, r in enumerate(ids):
        assert same_bits(emb[i], pat16[(int(r) * C + np.arange(C)) % (1 << 24)]), r


def test_group_norm_across_the_4_gib_boundary(dev, oracle):
    """GroupNorm on a 4.3 GB f16 tensor [8, 512, 524544] with 32 groups (16 MB each, so every group is split over many
    blocks): the first group, the two on either side of byte 2^32 and the last one, against torch's definition in f64."""
    from ratchet_amd import _lib
    from ratchet_amd.runtime import BufferView

    P = 1 << 24
    B, C, L, G = 8, 512, 524544, 32
    n = B * C * L
    rng = np.random.default_rng(711)
    pat = (0.5 + rng.standard_normal(P)).astype(np.float16)
    x = dev.empty((B, C, L), F16)
    dp = dev.upload(pat)
    for k in range(0, n, P):
        _lib.check(dev.lib.rt_d2d(dev.handle, x.ptr.value + 2 * k, dp.ptr, 2 * min(P, n - k)))
    w = (1 + 0.1 * rng.standard_normal(C)).astype(np.float16)
    bi = (0.1 * rng.standard_normal(C)).astype(np.float16)
    y = dev.group_norm(x, G, dev.upload(w), dev.upload(bi), 1e-5)
    glen, cpg = (C // G) * L, C // G
    for pair in (0, (1 << 31) // glen - 1, (1 << 31) // glen, B * G - 1):
        first = pair * glen
        grp = pat[(first + np.arange(glen, dtype=np.int64)) % P].astype(np.float64)
        mu, var = grp.mean(), grp.var()
        g = pair % G
        for ch, l0 in ((0, 0), (cpg - 1, L - 64)):                     # 64 elements at the start and at the end of the group
            c = g * cpg + ch
            got = BufferView(y, first + ch * L + l0, (64,)).to_numpy()
            xs = grp[ch * L + l0: ch * L + l0 + 64]
            want = ((xs - mu) / np.sqrt(var + 1e-5) * float(w[c]) + float(bi[c])).astype(np.float16)
            bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
            assert bad == 0, (pair, ch, mx)


def test_f32_rows_broadcast_and_index_write_across_the_4_gib_boundary(dev, oracle):
    """f32 softmax and norms on [716800, 1500] (4.3 GB; rows of 6000 bytes, so most rows start off a 128-byte line), a
    broadcast to 4.3 GB and an index_write into the far end of a 4.3 GB destination."""
    from ratchet_amd import _lib
    from ratchet_amd.runtime import BufferView

    P = 1 << 22
    rows, cols = 716800, 1500
    n = rows * cols
    rng = np.random.default_rng(712)
    pat = rng.standard_normal(P).astype(np.float32)
    x = dev.empty((rows, cols), F32)
    dp = dev.upload(pat)
    for k in range(0, n, P):
        _lib.check(dev.lib.rt_d2d(dev.handle, x.ptr.value + 4 * k, dp.ptr, 4 * min(P, n - k)))
    at = [0, (1 << 32) // (4 * cols) - 1, (1 << 32) // (4 * cols), (1 << 32) // (4 * cols) + 1, rows - 2, rows - 1]
    want_rows = np.stack([pat[(r * cols + np.arange(cols, dtype=np.int64)) % P] for r in at])

    def rows_of(buf):
        return np.stack([BufferView(buf, r * cols, (cols,)).to_numpy() for r in at])

    g = (1 + 0.02 * rng.standard_normal(cols)).astype(np.float32)
    b = (0.02 * rng.standard_normal(cols)).astype(np.float32)
    out = dev.softmax(x)
    bad, mx = oracle.count_not_close(rows_of(out), oracle.softmax(want_rows), 1e-5, 1e-5)
    assert bad == 0, mx
    dev.layer_norm(x, dev.upload(g), dev.upload(b), 1e-5, out=out)
    bad, mx = oracle.count_not_close(rows_of(out), oracle.layer_norm(want_rows, g, b, 1e-5, intended=True), 1e-5, 1e-5)
    assert bad == 0, mx
    dev.rms_norm(x, dev.upload(g), 1e-5, out=out)
    bad, mx = oracle.count_not_close(rows_of(out), oracle.rms_norm(want_rows, g, 1e-5, intended=True), 1e-5, 1e-5)
    assert bad == 0, mx
    del out
    # broadcast [1, 1, 1500] over 716800 rows, then overwrite two rows at the far end through index_write
    row = rng.standard_normal((1, 1, cols)).astype(np.float32)
    big = dev.broadcast_to(dev.upload(row), (1, rows, cols))
    for r in at:
        assert same_bits(BufferView(big, r * cols, (cols,)).to_numpy(), row[0, 0]), r
    patch = rng.standard_normal((1, 2, cols)).astype(np.float32)
    dev.index_write(big, dev.upload(patch), (0, rows - 2, 0))
    assert same_bits(BufferView(big, (rows - 2) * cols, (2 * cols,)).to_numpy(), patch.reshape(-1))
    assert same_bits(BufferView(big, (rows - 3) * cols, (cols,)).to_numpy(), row[0, 0])
