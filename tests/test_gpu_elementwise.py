"""GPU parity: binary / unary / cast kernels against the CPU oracle, through the C ABI.

Bars (same seeded inputs on both sides):
  add/sub/mul/div, cast ......... bit-exact
  f32 transcendental unaries .... <= 2 ulp (tanh, gelu, exp, silu, sigmoid are expected to be bit-exact)
  f16 unaries ................... <= 1e-3 with the reference's all_close rule; checked exhaustively over all 65536 inputs
"""
import numpy as np
import pytest

from gpu_util import bits, mismatch_count, randn, same_bits, ulp_diff

pytestmark = pytest.mark.gpu

ALL_F16 = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16)
SPECIALS32 = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1.17549435e-38, 3.4e38, -3.4e38, 88.7, 88.8, -103.9,
                       -104.1, 1.0, -1.0, 0.5, 22.0, -22.0, 1e-8, 0.3465, 0.35, 1.04, 1.05], dtype=np.float32)


@pytest.fixture(scope="module")
def dev():
    from ratchet_amd import Device

    d = Device(0)
    yield d
    d.close()


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_binary_bit_exact(dev, oracle, op, dtype):
    rng = np.random.default_rng(100)
    for n in (1, 7, 8, 1000, 4096 + 3, (1 << 20) + 5):
        a = (rng.standard_normal(n) * 10 ** rng.uniform(-5, 4, n)).astype(dtype)
        b = (rng.standard_normal(n) * 10 ** rng.uniform(-5, 4, n)).astype(dtype)
        if n >= 1000:
            sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504, 6e-8, -6e-8, 1, -1], dtype=dtype)
            a[:100] = np.repeat(sp, 10)
            b[:100] = np.tile(sp, 10)
        want = oracle.binary(op, a, b)
        got = dev.binary(op, dev.upload(a), dev.upload(b)).to_numpy()
        assert same_bits(got, want), (op, dtype, n, mismatch_count(got, want))


def test_binary_f16_div_many_pairs(dev, oracle):
    rng = np.random.default_rng(101)
    a = ALL_F16[rng.integers(0, 65536, 4_000_000)]
    b = ALL_F16[rng.integers(0, 65536, 4_000_000)]
    got = dev.binary("div", dev.upload(a), dev.upload(b)).to_numpy()
    assert same_bits(got, oracle.binary("div", a, b))


def test_binary_bf16_bit_exact(dev, oracle):
    rng = np.random.default_rng(102)
    a = oracle.cast(rng.standard_normal(100003).astype(np.float32), np.uint16, dst_bf16=True)
    b = oracle.cast(rng.standard_normal(100003).astype(np.float32), np.uint16, dst_bf16=True)
    for op in ("add", "sub", "mul", "div"):
        want = oracle.binary(op, a, b, bf16=True)
        got = dev.binary(op, dev.upload(a, bf16=True), dev.upload(b, bf16=True)).to_numpy()
        assert np.array_equal(got, want), op


def test_binary_in_place_and_offset_pointers(dev, oracle):
    rng = np.random.default_rng(103)
    n = 70001
    a = randn(rng, n, np.float16)
    b = randn(rng, n, np.float16)
    want = oracle.binary("mul", a, b)
    da, db = dev.upload(a), dev.upload(b)
    dev.binary("mul", da, db, out=da)                          # y aliases a: the reference's in-place rule
    assert same_bits(da.to_numpy(), want)
    # operands that start 2 bytes past a 16-byte boundary take the scalar path
    big_a, big_b, big_y = dev.empty((n + 8,), da.dt), dev.empty((n + 8,), da.dt), dev.empty((n + 8,), da.dt)
    va, vb, vy = big_a.view(1, (n,)).upload(a), big_b.view(1, (n,)).upload(b), big_y.view(3, (n,))
    dev.binary("mul", va, vb, out=vy)
    assert same_bits(vy.to_numpy(), want)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_binary_broadcast_fused(dev, oracle, dtype):
    rng = np.random.default_rng(104)
    cases = [((1, 150, 384), (384,)), ((2, 3, 16, 16), (16, 16)), ((1, 4, 64, 1), (1, 1, 1, 64)), ((3, 1, 5), (1, 7, 1)),
             ((5, 7), (1,)), ((1,), (2, 9)), ((2, 3, 4, 10), (2, 1, 4, 1)), ((4, 1, 8), (4, 6, 8)), ((6, 130), (6, 1)),
             # an operand of 1 to 8 MiB repeated over the leading dims: the L2s keep it between the repeats, plain block order
             ((1, 3, 1024, 512), (1024, 512)), ((1024, 1024), (3, 1024, 1024)), ((5, 136, 4096), (136, 4096)),
             ((2, 2, 256, 2048), (1, 1, 256, 2048)),
             # from 28 MiB on such an operand takes the XCD-aware block order (walks of 64, 4 and 1 slabs, either side repeated)
             ((2, 4096, 4096), (4096, 4096)), ((3616, 4096), (2, 3616, 4096)), ((1, 2, 3592, 4096), (3592, 4096))]
    for sa, sb in cases:
        a, b = randn(rng, sa, dtype), randn(rng, sb, dtype)
        out_shape = np.broadcast_shapes(sa, sb)
        # the reference materialises broadcast_to on each side, then runs the equal-shape op
        want = oracle.binary("sub", np.ascontiguousarray(np.broadcast_to(a, out_shape)),
                             np.ascontiguousarray(np.broadcast_to(b, out_shape)))
        got = dev.binary("sub", dev.upload(a), dev.upload(b)).to_numpy()
        assert got.shape == tuple(out_shape)
        assert same_bits(got, want), (sa, sb)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_binary_broadcast_against_rows_that_are_not_whole_vectors(dev, oracle, dtype, op):
    """one operand of the output's shape, a last dim that is not a multiple of the vector length: the full operand and the output
    move as flat 16-byte vectors and the broadcast operand element by element; both operand orders, every broadcast pattern,
    a tensor whose size is not a whole vector, rows shorter than a vector, in place"""
    rng = np.random.default_rng(105)
    cases = [((4, 33, 1001), (1001,)), ((1001,), (4, 33, 1001)), ((4, 33, 1001), (4, 33, 1)), ((3, 7, 5, 13), (3, 1, 5, 1)),
             ((2, 3, 4, 5), (1, 3, 1, 1)), ((1, 3, 1, 1), (2, 3, 4, 5)), ((9, 3), (3,)), ((77, 1), (1,)), ((5, 6, 7), (6, 1)),
             ((2, 50, 3, 999), (2, 1, 3, 999)), ((64, 3, 31, 31), (1, 3, 1, 1))]
    for sa, sb in cases:
        a, b = randn(rng, sa, dtype), randn(rng, sb, dtype)
        if op == "div":
            b = np.where(np.abs(b) < 0.1, dtype(0.5), b)
        out_shape = np.broadcast_shapes(sa, sb)
        want = oracle.binary(op, np.ascontiguousarray(np.broadcast_to(a, out_shape)), np.ascontiguousarray(np.broadcast_to(b, out_shape)))
        da, db = dev.upload(a), dev.upload(b)
        got = dev.binary(op, da, db).to_numpy()
        assert same_bits(got, want), (op, sa, sb)
        full = da if tuple(sa) == tuple(out_shape) else db
        dev.binary(op, da, db, out=full)                                 # in place on the full operand
        assert same_bits(full.to_numpy(), want), (op, sa, sb, "in place")


UNARY = ["gelu", "tanh", "exp", "log", "sin", "cos", "abs", "sqrt", "relu", "floor", "ceil", "neg", "silu", "sigmoid"]
EXACT32 = {"gelu", "tanh", "exp", "log", "sin", "cos", "abs", "sqrt", "relu", "floor", "ceil", "neg", "silu", "sigmoid"}


@pytest.mark.parametrize("op", UNARY)
def test_unary_f32(dev, oracle, op):
    rng = np.random.default_rng(110)
    x = np.concatenate([rng.standard_normal(300_000) * 4, rng.standard_normal(100_000) * 40, rng.uniform(-1e-3, 1e-3, 50_000),
                        rng.standard_normal(50_003)]).astype(np.float32)
    x[: len(SPECIALS32)] = SPECIALS32
    if op in ("log", "sqrt"):
        x[len(SPECIALS32):] = np.abs(x[len(SPECIALS32):])
    if op in ("sin", "cos"):
        x[1000:2000] *= 1e4                                   # large arguments exercise range reduction
    want = oracle.unary(op, x)
    got = dev.unary(op, dev.upload(x)).to_numpy()
    d = ulp_diff(got, want)
    # relu(-0.0) and NaN payloads aside, signed zeros must agree too: compare zeros by value
    zero_both = (got == 0) & (want == 0)
    d = np.where(zero_both, 0, d)
    assert d.max() <= 2, (op, int(d.max()), x[np.argmax(d)], got[np.argmax(d)], want[np.argmax(d)])
    if op in EXACT32:
        assert d.max() == 0, (op, int(np.count_nonzero(d)), x[np.argmax(d)], got[np.argmax(d)], want[np.argmax(d)])


@pytest.mark.parametrize("op", UNARY)
def test_unary_f16_exhaustive(dev, oracle, op):
    want = oracle.unary(op, ALL_F16)
    got = dev.unary(op, dev.upload(ALL_F16)).to_numpy()
    bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
    assert bad == 0, (op, bad, mx)
    mism = mismatch_count(got, want)
    # every op is the C library's own algorithm: bit-exact
    assert mism == 0, (op, mism)
    assert ulp_diff(got, want).max() <= 1


def test_unary_in_place_and_tail(dev, oracle):
    rng = np.random.default_rng(111)
    for n in (1, 3, 9, 1027):
        x = randn(rng, n, np.float16)
        dx = dev.upload(x)
        dev.unary("silu", dx, out=dx)
        assert same_bits(dx.to_numpy(), oracle.unary("silu", x)), n
    x = randn(rng, 10001, np.float32)
    big = dev.empty((10010,), 0)
    v = big.view(1, (10001,)).upload(x)
    dev.unary("gelu", v, out=v)
    assert same_bits(v.to_numpy(), oracle.unary("gelu", x))


def test_unary_bf16(dev, oracle):
    rng = np.random.default_rng(112)
    x = oracle.cast((rng.standard_normal(50001) * 3).astype(np.float32), np.uint16, dst_bf16=True)
    for op in ("gelu", "silu", "exp", "abs", "relu", "sqrt"):
        want = oracle.unary(op, x, bf16=True)
        got = dev.unary(op, dev.upload(x, bf16=True)).to_numpy()
        assert np.array_equal(got, want) or np.count_nonzero(got != want) == np.count_nonzero(
            np.isnan(oracle.cast(got, np.float32, src_bf16=True)) & (got != want)), op


def test_cast(dev, oracle):
    from ratchet_amd import _lib

    rng = np.random.default_rng(113)
    # f16 -> f32, exhaustive
    got = dev.cast(dev.upload(ALL_F16), _lib.F32).to_numpy()
    assert same_bits(got, oracle.cast(ALL_F16, np.float32))
    # f32 -> f16: random bit patterns, every rounding boundary, subnormals, overflow
    rand = rng.integers(0, 2**32, size=3_000_001, dtype=np.uint64).astype(np.uint32).view(np.float32)
    fin = ALL_F16[np.isfinite(ALL_F16)].astype(np.float32)
    ties = ((fin[:-1].astype(np.float64) + fin[1:].astype(np.float64)) / 2).astype(np.float32)
    x = np.concatenate([rand, fin, ties, np.nextafter(ties, np.float32(np.inf)), np.nextafter(ties, np.float32(-np.inf)),
                        np.array([65504, 65519.99, 65520, 1e-8, 2.9802322e-8, 3e-8, 1e-5], dtype=np.float32)])
    got = dev.cast(dev.upload(x), _lib.F16).to_numpy()
    assert same_bits(got, oracle.cast(x, np.float16))
    # bf16 both ways
    y = rng.standard_normal(100_003).astype(np.float32)
    gb = dev.cast(dev.upload(y), _lib.BF16).to_numpy()
    assert np.array_equal(gb, oracle.cast(y, np.uint16, dst_bf16=True))
    back = dev.cast(dev.upload(gb, bf16=True), _lib.F32).to_numpy()
    assert same_bits(back, oracle.cast(gb, np.float32, src_bf16=True))
    # f32 -> bf16 over random bit patterns (NaNs with payloads, infinities, subnormals) and around every tie: the kernels
    # round with the chip's conversion instruction, the oracle on the bit pattern as half::bf16::from_f32 does
    hi = rng.integers(0, 2**16, size=200_000, dtype=np.uint64).astype(np.uint32) << 16
    around = np.concatenate([hi | 0x7fff, hi | 0x8000, hi | 0x8001, hi | 0xffff, hi])
    z = np.concatenate([rand.view(np.uint32), around]).view(np.float32)
    gz = dev.cast(dev.upload(z), _lib.BF16).to_numpy()
    wz = oracle.cast(z, np.uint16, dst_bf16=True)
    bad = np.flatnonzero(gz != wz)
    assert bad.size == 0, (bad.size, [hex(v) for v in z.view(np.uint32)[bad[:5]]], [hex(v) for v in gz[bad[:5]]], [hex(v) for v in wz[bad[:5]]])
    # f32 <-> i32/u32: bit reinterpretation, as the reference does (cpu/mod.rs:116-125)
    gi = dev.cast(dev.upload(y), _lib.I32).to_numpy()
    assert np.array_equal(gi, y.view(np.int32))
    gf = dev.cast(dev.upload(y.view(np.uint32)), _lib.F32).to_numpy()
    assert np.array_equal(gf.view(np.uint32), y.view(np.uint32))
    # odd lengths and offset pointers
    for n in (1, 5, 8, 13):
        z = randn(rng, n, np.float32)
        assert same_bits(dev.cast(dev.upload(z), _lib.F16).to_numpy(), oracle.cast(z, np.float16))
    big = dev.empty((1000,), _lib.F32)
    v = big.view(1, (777,)).upload(y[:777])
    assert same_bits(dev.cast(v, _lib.F16).to_numpy(), oracle.cast(y[:777], np.float16))


@pytest.mark.parametrize("op", ["gelu", "silu", "sigmoid", "tanh", "exp", "sqrt", "log"])
def test_unary_f16_large_tensor_table_path(dev, oracle, op):
    # tensors of 2^21 elements and more go through the LDS lookup table; it must equal the computed kernel bit for bit
    rng = np.random.default_rng(120)
    n = (1 << 22) + 5
    x = ALL_F16[rng.integers(0, 65536, n)]
    x[:65536] = ALL_F16
    want = oracle.unary(op, x)
    dx = dev.upload(x)
    got = dev.unary(op, dx).to_numpy()
    assert mismatch_count(got, want) == 0, (op, mismatch_count(got, want))
    small = dev.unary(op, dev.upload(ALL_F16)).to_numpy()        # computed path
    assert same_bits(got[:65536], small)
    dev.unary(op, dx, out=dx)                                    # in place
    assert same_bits(dx.to_numpy(), got)


def test_unary_bf16_large_tensor_table_path(dev, oracle):
    rng = np.random.default_rng(121)
    n = (1 << 21) + 3
    x = rng.integers(0, 65536, n).astype(np.uint16)
    x[:65536] = np.arange(65536, dtype=np.uint16)
    for op in ("gelu", "silu"):
        want = oracle.unary(op, x, bf16=True)
        got = dev.unary(op, dev.upload(x, bf16=True)).to_numpy()
        wf, gf = oracle.cast(want, np.float32, src_bf16=True), oracle.cast(got, np.float32, src_bf16=True)
        assert np.all((got == want) | (np.isnan(wf) & np.isnan(gf))), op


def test_storage_pool_reuses_blocks_in_stream_order(oracle):
    """rt_free parks a block, the next rt_malloc of about that size gets it back without a device synchronisation
    (the role of the reference's BufferPool, gpu/pools/buffer_pool.rs:60-112); results stay right because every launch of a
    device goes through one in-order stream."""
    from ratchet_amd import Device, RatchetError

    d = Device(0)
    try:
        rng = np.random.default_rng(120)
        x = randn(rng, (1 << 20,), np.float32)
        dx = d.upload(x)
        live0, parked0, hits0, misses0 = d.pool_stats()
        a = d.unary("neg", dx)
        pa = a.ptr.value
        del a                                                 # parked while the kernel may still be running
        b = d.unary("abs", dx)                                # same size: the parked block comes back
        assert b.ptr.value == pa
        assert np.array_equal(b.to_numpy(), np.abs(x))
        live, parked, hits, misses = d.pool_stats()
        assert hits == hits0 + 1 and misses == misses0 + 1 and live == live0 + 4 * (1 << 20) and parked == parked0
        # a chain that frees every intermediate immediately: correct values, two blocks cycle
        y = dx
        want = x
        for op in ("neg", "abs", "sqrt", "neg", "exp"):
            y = d.unary(op, y)
            want = oracle.unary(op, want)
        assert same_bits(y.to_numpy(), want)
        assert d.pool_stats()[3] <= misses + 2
        small = d.empty((3,), 0)                              # sizes are rounded: 12 bytes -> one 512-byte class
        ps = small.ptr.value
        del small
        assert d.empty((100,), 0).ptr.value == ps
        del b, y
        assert d.pool_stats()[1] > 0
        d.pool_trim()
        assert d.pool_stats()[1] == 0
        import ctypes
        assert d.lib.rt_free(d.handle, ctypes.c_void_p(0x1000)) == 7      # not a block of this pool
    finally:
        d.close()


def test_storage_pool_ages_unused_blocks_by_passes():
    """rt_pool_begin_pass is the reference's begin_pass (gpu/pools/dynamic_resource_pool.rs:140-190): a block freed during
    pass p can be taken again during passes p and p + 1 and goes back to the driver at the start of pass p + 2 if nobody
    did.  With sizes that drift from pass to pass the parked set therefore stays at the last two passes' blocks instead
    of growing; a program that repeats its sizes keeps hitting the pool and nothing is ever returned."""
    from ratchet_amd import Device

    d = Device(0)
    try:
        MB = 1 << 20
        d.pool_trim()
        parked_after = []
        for k in range(12):                                   # every pass wants a size no earlier pass had
            d.pool_begin_pass()
            b = d.empty(((8 + 3 * k) * MB // 4,), 0)
            c = d.empty(((100 + 20 * k) * MB // 4,), 0)              # apart by more than the pool's size classes (1/16)
            del b, c
            parked_after.append(d.pool_stats()[1])
        # pass k leaves its own two blocks and those of pass k - 1 (sizes are rounded up by at most 1/16)
        for k in range(1, 12):
            own = (8 + 3 * k + 100 + 20 * k) * MB
            before = (8 + 3 * (k - 1) + 100 + 20 * (k - 1)) * MB
            assert own + before <= parked_after[k] <= (own + before) * 17 // 16, (k, parked_after[k])
        d.pool_begin_pass()
        d.pool_begin_pass()
        assert d.pool_stats()[1] == 0                         # two passes without a taker: everything went back
        # steady state: the same two sizes every pass are served by the pool, and no block is returned
        live0, parked0, hits0, misses0 = d.pool_stats()
        for k in range(6):
            d.pool_begin_pass()
            b = d.empty((16 * MB // 4,), 0)
            c = d.empty((64 * MB // 4,), 0)
            del b, c
        live, parked, hits, misses = d.pool_stats()
        assert misses == misses0 + 2 and hits == hits0 + 10 and parked == 80 * MB
        # a block in use is not the pool's to return, however many passes go by
        keep = d.upload(np.arange(1024, dtype=np.float32))
        for k in range(4):
            d.pool_begin_pass()
        assert np.array_equal(keep.to_numpy(), np.arange(1024, dtype=np.float32))
        # while the device is capturing, a pass returns nothing (hipFree is not allowed there) and does not fail
        x = d.upload(np.ones(4096, np.float32))
        y = d.empty((4096,), 0)
        with d.capture() as g:
            d.pool_begin_pass()
            d.unary("neg", x, out=y)
        g.launch()
        assert (y.to_numpy() == -1).all()
    finally:
        d.close()


@pytest.mark.parametrize("n", [(1 << 21), (1 << 21) + 8, 5 * 32768 * 64 + 32768 * 7 + 8 * 100 + 5, 32768 * 300 - 1])
def test_unary_table_path_tiles_and_remainders(dev, oracle, n):
    """the table kernel walks whole 64 KiB tiles with the next tile's loads in flight and hands the rest (fewer vectors
    than a tile, fewer elements than a vector) to one block: every element once, none beyond the end"""
    rng = np.random.default_rng(123)
    x = rng.integers(0, 65536, n).astype(np.uint16).view(np.float16)
    want = oracle.unary("silu", x)
    big = dev.upload(np.full(n + 24, 7.25, np.float16))
    from ratchet_amd.runtime import BufferView

    out = BufferView(big, 8, (n,))
    dev.unary("silu", dev.upload(x), out=out)
    got = out.to_numpy()
    assert np.all((got.view(np.uint16) == want.view(np.uint16)) | (np.isnan(got) & np.isnan(want)))
    whole = big.to_numpy()
    assert (whole[:8] == 7.25).all() and (whole[8 + n:] == 7.25).all()


@pytest.mark.parametrize("a_shape,b_shape", [((1, 4, 256, 512), (1, 1, 256, 512)), ((1, 1, 256, 512), (1, 4, 256, 512)), ((1, 4, 256, 1), (1, 1, 1, 512)),
                                             ((2, 3, 64, 40), (2, 3, 64, 40)), ((1, 4, 256, 512), (512,)), ((3, 5, 7, 9), (1, 5, 1, 9))])
def test_broadcast_binary_streaming_variants(dev, oracle, a_shape, b_shape):
    """each side of rt_binary_bcast is streamed past the caches when it has no broadcast dim and cached when it repeats:
    the four instantiations (and the scalar one for odd rows) give the same bits as the oracle on materialised operands"""
    from ratchet_amd import _lib
    from ratchet_amd._lib import check
    from ratchet_amd.runtime import shape4

    rng = np.random.default_rng(124)
    a, b = randn(rng, a_shape, np.float16), randn(rng, b_shape, np.float16)
    shape = np.broadcast_shapes(a_shape, b_shape)
    for op in ("add", "mul", "div"):
        want = oracle.binary(op, np.ascontiguousarray(np.broadcast_to(a, shape)), np.ascontiguousarray(np.broadcast_to(b, shape)))
        da, db = dev.upload(a), dev.upload(b)
        out = dev.empty(shape, da.dt)
        # through rt_binary_bcast also when the shapes are equal (both sides streamed)
        check(dev.lib.rt_binary_bcast(dev.handle, _lib.BINARY_OPS.index(op), da.dt, da.ptr, shape4(a_shape), db.ptr, shape4(b_shape), out.ptr,
                                      shape4(shape)))
        assert same_bits(out.to_numpy(), want), (op, a_shape, b_shape)


def test_empty_tensors_are_no_ops(dev):
    """An op over no elements (or no rows) succeeds, launches nothing and leaves its output as it was; ops whose shape
    arguments hold a zero extent are refused with RT_ERR_SHAPE before anything runs (checked without a GPU in test_abi)."""
    import ctypes
    from ratchet_amd import _lib

    L, h = dev.lib, dev.handle
    keep = np.arange(64, dtype=np.float32)
    a, y = dev.upload(keep), dev.upload(keep)
    u4 = lambda *s: (ctypes.c_uint32 * 4)(*s)
    calls = [
        L.rt_binary(h, _lib.BINARY_OPS.index("add"), _lib.F32, a.ptr, a.ptr, y.ptr, 0),
        L.rt_unary(h, _lib.UNARY_OPS.index("gelu"), _lib.F32, a.ptr, y.ptr, 0),
        L.rt_unary_via_f32(h, _lib.UNARY_OPS.index("gelu"), _lib.F16, a.ptr, y.ptr, 0),
        L.rt_cast(h, _lib.F32, _lib.F16, a.ptr, y.ptr, 0),
        L.rt_softmax(h, _lib.F32, a.ptr, y.ptr, 0, 8, 0),
        L.rt_layer_norm(h, _lib.F32, a.ptr, a.ptr, a.ptr, y.ptr, 0, 8, 1e-5),
        L.rt_rms_norm(h, _lib.F32, a.ptr, a.ptr, y.ptr, 0, 8, 1e-5),
        L.rt_norm_via_f32(h, 0, _lib.F16, a.ptr, a.ptr, a.ptr, y.ptr, 0, 8, 1e-5),
        L.rt_gated_mul_via_f32(h, _lib.UNARY_OPS.index("silu"), _lib.F16, a.ptr, 8, a.ptr, 8, y.ptr, 0, 8),
        L.rt_index_write(h, 4, y.ptr, u4(1, 1, 8, 8), a.ptr, 0, u4(0, 0, 0, 0)),
    ]
    assert calls == [0] * len(calls), calls
    assert same_bits(y.to_numpy(), keep)
