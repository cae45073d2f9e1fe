"""GPU parity: softmax, layer_norm, rms_norm, group_norm against the CPU oracle, through the C ABI.

Bars: f32 <= 1e-5, f16 <= 1e-3 with the reference's all_close rule (|a-b| <= tol + tol*|b|, NaN == NaN).
f16 softmax replays the reference's sequential f16 accumulation and is expected to be bit-exact.
Problem spaces follow crates/ratchet-core/src/ops/softmax.rs:308-365 and ops/norm/mod.rs:400-512.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from gpu_util import describe_mismatch, mismatch_count, randn, same_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    from ratchet_amd import Device

    d = Device(0)
    yield d
    d.close()


SOFTMAX_SHAPES = [(3, 256, 256), (1, 7, 33), (2, 1, 1), (1, 5, 255), (2, 64, 1500), (1, 3, 2048), (1, 2, 2052), (1, 130, 8),
                  (1, 3, 5000), (2, 9, 4096), (1, 5, 3072), (1, 3, 8192), (1, 2, 8196), (1, 2, 6148),   # > 2048 columns: a block per row
                  (1, 5, 32064), (1, 3, 51200), (2, 65536), (2, 32001), (2, 65540)]                     # vocabulary-sized rows: 1024 threads per row up to 65536 columns


@pytest.mark.parametrize("shape", SOFTMAX_SHAPES)
def test_softmax_f32(dev, oracle, shape):
    rng = np.random.default_rng(300)
    x = randn(rng, shape, np.float32, 3.0)
    want = oracle.softmax(x)
    got = dev.softmax(dev.upload(x)).to_numpy()
    bad, mx = oracle.count_not_close(got, want, 1e-5, 1e-5)
    assert bad == 0, (shape, bad, mx)
    ref = F.softmax(torch.from_numpy(x), dim=-1).numpy()               # the reference test's own referee and tolerance
    bad, mx = oracle.count_not_close(got, ref, 1e-6, 1e-6)
    assert bad == 0, (shape, bad, mx)


@pytest.mark.parametrize("shape", [(2, 3, 101, 101), (1, 7, 33), (300, 5), (64, 1), (9, 1499), (5, 2047), (3, 5001), (2, 8190), (2, 8191), (40, 13)])
def test_softmax_f32_rows_that_are_not_whole_vectors(dev, oracle, shape):
    """ragged f32 rows run over the aligned vectors that cover them (8190 columns are the most that fit; 8191 take the
    scalar kernel): same results as for whole vectors, masked and overflowing rows included, and nothing written outside
    the tensor; reference and stable mode, also for f16 in stable mode"""
    from ratchet_amd import _lib
    from ratchet_amd.runtime import BufferView

    rng = np.random.default_rng(310)
    x = randn(rng, shape, np.float32, 3.0)
    flat = x.reshape(-1, shape[-1])
    flat[0, shape[-1] // 2 + 1:] = -np.inf
    flat[-1, :] = -np.inf                                              # 0 / 0 in the last row
    if flat.shape[0] > 2:
        flat[1, 0] = 100.0                                             # overflow in a row's first (shared) vector
    want = oracle.softmax(x)
    dx = dev.upload(x)
    fill = np.full(x.size + 12, 7.25, np.float32)
    big = dev.upload(fill)
    out = BufferView(big, 4, x.shape)
    dev.softmax(dx, out=out)
    got = out.to_numpy()
    bad, mx = oracle.count_not_close(got, want, 1e-5, 1e-5)
    assert bad == 0, (shape, bad, mx)
    whole = big.to_numpy()
    assert (whole[:4] == 7.25).all() and (whole[4 + x.size:] == 7.25).all()
    dev.softmax(dx, out=dx)                                             # in place
    assert same_bits(dx.to_numpy(), got)
    x[np.isinf(x) | (x == 100.0)] = -5.0
    with np.errstate(all="ignore"):
        ref = F.softmax(torch.from_numpy(x), dim=-1).numpy()
    got = dev.softmax(dev.upload(x), mode=_lib.SOFTMAX_STABLE).to_numpy()
    bad, mx = oracle.count_not_close(got, ref, 1e-6, 1e-6)
    assert bad == 0, ("stable", shape, bad, mx)
    got = dev.softmax(dev.upload(x.astype(np.float16)), mode=_lib.SOFTMAX_STABLE).to_numpy()
    ref = F.softmax(torch.from_numpy(x.astype(np.float16).astype(np.float32)), dim=-1).numpy()
    bad, mx = oracle.count_not_close(got.astype(np.float32), ref, 1e-3, 1e-3)
    assert bad == 0, ("stable f16", shape, bad, mx)


def test_softmax_f32_masks_overflow_in_place(dev, oracle):
    ninf = -np.inf
    x = np.zeros((4, 64), np.float32)
    x[0, 1:] = ninf
    x[1, 2:] = ninf
    x[1, :2] = 1.0
    x[2, 0] = 100.0                                                    # exp overflows: NaN there, 0 elsewhere
    x[3, :] = ninf                                                     # fully masked row: 0/0
    want = oracle.softmax(x)
    dx = dev.upload(x)
    dev.softmax(dx, out=dx)
    got = dx.to_numpy()
    assert same_bits(got, want)
    assert np.isnan(got[2, 0]) and np.all(got[2, 1:] == 0) and np.all(np.isnan(got[3]))


@pytest.mark.parametrize("cols", [64, 1500, 3000, 5001])
def test_softmax_f32_rows_whose_exponentials_are_subnormal(dev, oracle, cols):
    """known answers: every entry of a row at -95 (or -100) has a subnormal exponential, the row sums to a subnormal or tiny
    normal number and every probability is 1 / cols, as expf gives it on the CPU; an exp that flushes subnormals to zero
    returns 0 / 0 = NaN here.  Mixed rows around the threshold (-87.34) are compared with the oracle."""
    x = np.empty((6, cols), np.float32)
    x[0], x[1] = -95.0, -100.0
    rng = np.random.default_rng(cols)
    x[2] = -87.0 - 3.0 * rng.random(cols, dtype=np.float32)            # straddles the first subnormal result
    x[3] = -95.0 - 5.0 * rng.random(cols, dtype=np.float32)            # all subnormal: 3930 down to 26 units of 2^-149
    x[4] = -103.0 - 2.0 * rng.random(cols, dtype=np.float32)           # some round to zero
    x[5] = -95.0
    x[5, 0] = -90.0
    want = oracle.softmax(x)
    assert np.isfinite(want[:4]).all() and abs(want[0, 0] * cols - 1.0) < 1e-5
    got = dev.softmax(dev.upload(x)).to_numpy()
    assert np.isfinite(got[:4]).all() and np.isfinite(got[5]).all()
    # the subnormal grid is coarse: an exponential of a few units of 2^-149 carries a relative error of its own, in the
    # oracle and in the kernel alike, so rows 3 and 4 are held to the spacing of that grid instead of 1e-5
    bad, mx = oracle.count_not_close(got[[0, 1, 2, 5]], want[[0, 1, 2, 5]], 1e-5, 1e-5)
    assert bad == 0, (cols, bad, mx)
    assert np.allclose(got[0], 1.0 / cols, rtol=1e-5) and np.allclose(got[1], 1.0 / cols, rtol=1e-5)
    with np.errstate(all="ignore"):
        e3 = np.exp(x[3].astype(np.float64))
        ref3 = e3 / e3.sum()
    assert np.max(np.abs(got[3] - ref3) / ref3) < 0.05                 # half a unit of 2^-149 against values of 26 and more
    both_nan = np.isnan(got[4]) & np.isnan(want[4])
    assert (np.isfinite(got[4]) | both_nan).all()


@pytest.mark.parametrize("shape", [(3, 64, 256), (1, 7, 33), (2, 1, 1), (1, 70, 1000), (1, 65, 4096), (1, 3, 4100), (1, 129, 8)])
def test_softmax_f16_reference_sequence(dev, oracle, shape):
    rng = np.random.default_rng(301)
    x = randn(rng, shape, np.float16, 2.0)
    if shape[-1] >= 256:                                                # causal-style -inf tail and one overflow row
        x[0, 0, shape[-1] // 2:] = -np.inf
        x[0, 1, 5] = 12.0
    want = oracle.softmax(x)
    got = dev.softmax(dev.upload(x)).to_numpy()
    bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
    assert bad == 0, (shape, bad, mx)
    assert mismatch_count(got, want) == 0, (shape, mismatch_count(got, want))


@pytest.mark.parametrize("shape", [(1, 300, 4096), (2, 601, 1000), (1, 2100, 512), (1, 4099, 264), (7, 64, 2560), (2, 200, 3072), (1, 300, 2056), (3, 100, 1536), (2, 90, 1104),
                                   (32, 1, 4096), (32, 1, 1000), (1, 20, 8), (1, 257, 520), (1, 31, 2056), (16, 61, 72)])
def test_softmax_f16_streaming_kernel(dev, oracle, shape):
    # cols <= 4096 and cols % 8 == 0: the single-pass kernel (exp table in LDS, rows held in registers), from the large
    # prefill shapes down to a decode step's [B * H, 1, T] scores, where every row becomes a group of its own
    rng = np.random.default_rng(303)
    x = randn(rng, shape, np.float16, 2.0)
    n = shape[-1]
    flat = x.reshape(-1, n)
    for i in range(0, flat.shape[0], 3):                               # causal-style -inf tails of varying length
        flat[i, (i * 37) % n + 1:] = -np.inf
    flat[5, 7] = 12.0                                                  # overflow: inf sum, NaN at that element, 0 elsewhere
    flat[11, :] = -np.inf                                              # fully masked row: 0/0
    flat[13, 3] = np.nan
    flat[17, :] = -20.0                                                # every exp underflows to 0
    flat[19, :] = -16.0                                                # subnormal exps
    flat[-1, : n // 2] = -12.0                                         # the last row: tiny terms first, then ordinary ones
    want = oracle.softmax(x)
    dx = dev.upload(x)
    got = dev.softmax(dx).to_numpy()
    assert mismatch_count(got, want) == 0, (shape, describe_mismatch(got, want, x))
    dev.softmax(dx, out=dx)                                            # in place, as the reference runs it
    assert same_bits(dx.to_numpy(), want)


def test_softmax_streaming_kernel_leaves_a_wait_that_its_clock_never_ends(dev, oracle):
    """The paced kernel's walker waves wait for the device's wall clock; every such wait is bounded (4096 looks).  With the
    pace set far beyond what a step takes, each wait runs into that bound: the kernel must finish, every wave leaving it
    normally, with the bits of the run at the computed pace (which are the oracle's)."""
    from ratchet_amd import _lib

    rng = np.random.default_rng(310)
    x = randn(rng, (1, 8192, 4096), np.float16, 2.0)                   # 304 groups of 27 rows: a grid that fills the chip, so paced
    dx, dy = dev.upload(x), dev.empty(x.shape, _lib.F16)

    def timed_ms():
        e0, e1 = dev.event(), dev.event()
        e0.record()
        dev.softmax(dx, out=dy)
        e1.record()
        return e0.elapsed_ms(e1)

    timed_ms()
    usual = min(timed_ms() for _ in range(3))
    want = dy.to_numpy()
    assert mismatch_count(want[0, :64], oracle.softmax(x[0, :64])) == 0
    _lib.check(dev.lib.rt_debug_softmax_pace(dev.handle, 1 << 28))     # 2.7 s a step, if anything waited for it
    try:
        held = timed_ms()
        got = dy.to_numpy()
    finally:
        _lib.check(dev.lib.rt_debug_softmax_pace(dev.handle, 0))
    assert mismatch_count(got, want) == 0
    # 16 steps a block, each held for 4096 looks at the clock and no longer: milliseconds, not the 43 s of the pace asked for
    assert max(5 * usual, 0.5) < held < 2000.0, (usual, held)
    again = dev.softmax(dx).to_numpy()                                 # and the computed pace is back
    assert mismatch_count(again, want) == 0


@pytest.mark.parametrize("rows,n,split", [(262140 + 47, 4096, 262140), (262200 + 131, 4095, 262200)])
def test_softmax_f16_streaming_kernel_beyond_2_gib(dev, oracle, rows, n, split):
    # the kernel addresses a launch with 32-bit byte offsets below 2^31, so a larger tensor is split into row chunks
    # (262 140 rows of 4096 f16 each; 262 200 rows of 4095, a multiple of 120 so that the second chunk starts on a 16-byte
    # boundary); rows on both sides of the split and at the end are compared with the oracle
    rng = np.random.default_rng(304)
    block = randn(rng, (1021, n), np.float16, 2.0)
    block[::3, 1000:] = -np.inf
    x = np.tile(block, (rows // 1021 + 1, 1))[:rows]
    got = dev.softmax(dev.upload(x)).to_numpy()
    for lo, hi in ((0, 64), (split - 40, rows)):
        want = oracle.softmax(x[lo:hi])
        assert mismatch_count(got[lo:hi], want) == 0, (lo, hi)
    # every row equals the result of its source row in the repeated block
    want_block = oracle.softmax(block)
    reps = rows // 1021
    assert same_bits(got[: reps * 1021].reshape(reps, 1021, n), np.broadcast_to(want_block, (reps, 1021, n)))


def _bf16(oracle, a):
    return oracle.cast(np.asarray(a, np.float32), np.uint16, dst_bf16=True)


def _special_rows(flat, n):
    """the edge rows of test_softmax_f16_streaming_kernel, on an f32 array that is rounded to the 16-bit type afterwards"""
    for i in range(0, flat.shape[0], 3):
        flat[i, (i * 37) % n + 1:] = -np.inf
    flat[5, 7] = 95.0                                                   # overflows both 16-bit types' exp: inf sum, NaN there
    flat[11, :] = -np.inf
    flat[13, 3] = np.nan
    flat[17, :] = -110.0                                                # every exp underflows to 0 (bf16 and f16)
    flat[19, :] = -16.0                                                 # subnormal exps in f16
    flat[-1, : n // 2] = -12.0


@pytest.mark.parametrize("shape", [(1, 300, 4096), (2, 601, 1000), (1, 2100, 512), (32, 1, 4096), (1, 20, 8), (1, 31, 2056), (16, 61, 72)])
def test_softmax_bf16_streaming_kernel(dev, oracle, shape):
    """bf16 rows that are whole vectors take the same single-pass kernel: the sum is the reference's sequence of
    bf16(f32(sum) + f32(e)), the quotient bf16(f32(e) / f32(sum))."""
    rng = np.random.default_rng(305)
    n = shape[-1]
    xf = (rng.standard_normal(shape) * 2).astype(np.float32)
    _special_rows(xf.reshape(-1, n), n)
    xb = _bf16(oracle, xf)
    want = oracle.softmax(xb, bf16=True)
    dx = dev.upload(xb, bf16=True)
    got = dev.softmax(dx).to_numpy()
    isnan = lambda b: (b & 0x7fff) > 0x7f80
    bad = (got != want) & ~(isnan(got) & isnan(want))
    assert not bad.any(), (shape, int(bad.sum()), np.flatnonzero(bad.reshape(-1))[:8], got.reshape(-1)[bad.reshape(-1)][:8], want.reshape(-1)[bad.reshape(-1)][:8])
    dev.softmax(dx, out=dx)
    got2 = dx.to_numpy()
    assert not ((got2 != want) & ~(isnan(got2) & isnan(want))).any()


@pytest.mark.parametrize("shape,kind", [((1, 70, 8192), "f16"), ((2, 33, 4104), "f16"), ((1, 3, 51200), "f16"), ((1, 100, 6008), "f16"),
                                        ((1, 40, 8192), "bf16"), ((1, 5, 20000), "bf16")])
def test_softmax_16_bit_long_rows(dev, oracle, shape, kind):
    """rows of more than 4096 columns: the exp values are parked in y and read back once the row sum is known; also in place"""
    rng = np.random.default_rng(306)
    n = shape[-1]
    xf = (rng.standard_normal(shape) * 2).astype(np.float32)
    _special_rows(xf.reshape(-1, n), n) if xf.reshape(-1, n).shape[0] >= 20 else None
    xf.reshape(-1, n)[0, n // 3:] = -np.inf
    if kind == "f16":
        x = xf.astype(np.float16)
        want = oracle.softmax(x)
        dx = dev.upload(x)
        got = dev.softmax(dx).to_numpy()
        assert mismatch_count(got, want) == 0, (shape, describe_mismatch(got, want, x))
        dev.softmax(dx, out=dx)
        assert same_bits(dx.to_numpy(), want)
    else:
        xb = _bf16(oracle, xf)
        want = oracle.softmax(xb, bf16=True)
        dx = dev.upload(xb, bf16=True)
        isnan = lambda b: (b & 0x7fff) > 0x7f80
        got = dev.softmax(dx).to_numpy()
        assert not ((got != want) & ~(isnan(got) & isnan(want))).any(), shape
        dev.softmax(dx, out=dx)
        got = dx.to_numpy()
        assert not ((got != want) & ~(isnan(got) & isnan(want))).any(), shape


@pytest.mark.parametrize("shape,kind", [((2, 4, 333, 1001), "f16"), ((1, 3, 100, 199), "f16"), ((70, 4095), "f16"), ((7, 4097), "f16"), ((50, 2047), "f16"), ((90, 511), "f16"), ((40, 2305), "f16"), ((45, 1535), "f16"), ((33, 3071), "f16"), ((33, 513), "f16"),
                                        ((1000, 193), "f16"), ((61, 2561), "f16"), ((2, 2, 77, 1001), "bf16"), ((40, 3001), "bf16"), ((31, 1535), "bf16"), ((900, 250), "bf16")])
def test_softmax_16_bit_ragged_rows_stream(dev, oracle, shape, kind):
    """rows of 192 or more columns that are not whole 16-byte vectors (a prompt of 1001 tokens): streamed over the aligned
    vectors that cover each row, the vectors shared by two rows finished by a second small launch; bit-exact like the
    aligned rows, out of place and in place.  4095 columns fill the largest register-parked variant, 4097 are past it; rows
    of 511, 1535, 2047, 4095 columns can reach one vector past their last 512-column step."""
    from ratchet_amd.runtime import BufferView

    rng = np.random.default_rng(308)
    n = shape[-1]
    xf = (rng.standard_normal(shape) * 2).astype(np.float32)
    flat = xf.reshape(-1, n)
    if flat.shape[0] >= 20:
        _special_rows(flat, n)
    flat[0, n // 3:] = -np.inf
    flat[-1, :] = 95.0 if kind == "bf16" else 12.0                   # the last row overflows its sum
    flat[1, :7] = 11.0                                                # large terms in a row's first (shared) vector
    flat[2, -7:] = 11.0                                               # and in its last
    bf = kind == "bf16"
    x = _bf16(oracle, xf) if bf else xf.astype(np.float16)
    want = oracle.softmax(x, bf16=bf)
    isnan = (lambda b: (b & 0x7fff) > 0x7f80) if bf else (lambda b: (b.view(np.uint16) & 0x7fff) > 0x7c00)
    same = lambda g: not ((g.view(np.uint16) != want.view(np.uint16)) & ~(isnan(g) & isnan(want))).any()
    dx = dev.upload(x, bf16=bf)
    assert same(dev.softmax(dx).to_numpy()), shape
    # into the middle of a larger allocation: the elements next to the first and the last row stay as they were
    fill = np.full(x.size + 24, 0x1234, np.uint16)
    big = dev.upload(fill if bf else fill.view(np.float16), bf16=bf)
    out = BufferView(big, 8, x.shape)
    dev.softmax(dx, out=out)
    assert same(out.to_numpy()), shape
    whole = big.to_numpy().view(np.uint16)
    assert (whole[:8] == 0x1234).all() and (whole[8 + x.size:] == 0x1234).all()
    dev.softmax(dx, out=dx)
    assert same(dx.to_numpy()), shape


def test_softmax_f16_ragged_rows_many_rows_in_chunks(dev, oracle):
    """more rows than one launch of the ragged variant keeps sums for (2^19): the launches split on 16-byte boundaries"""
    from ratchet_amd.runtime import BufferView

    rng = np.random.default_rng(309)
    rows, cols = (1 << 19) + 4321, 193
    x = (rng.standard_normal((rows, cols)) * 2).astype(np.float16)
    want = oracle.softmax(x)
    big = dev.empty((rows * cols + 24,), 1)
    xv = BufferView(big, 8, (rows, cols)).upload(x)                    # 16 bytes into the allocation: still vector aligned
    got = dev.softmax(xv).to_numpy()
    assert mismatch_count(got, want) == 0, describe_mismatch(got, want, x)
    xo = BufferView(big, 3, (1000, cols)).upload(x[:1000])             # off the vector alignment: the tile walker, same results
    assert same_bits(dev.softmax(xo).to_numpy(), want[:1000])


@pytest.mark.parametrize("rows,cols,kind", [(40000, 8, "f16"), (33001, 72, "f16"), (32768 + 5, 128, "f16"), (50000, 24, "bf16"), (32800, 104, "bf16")])
def test_softmax_16_bit_many_narrow_rows(dev, oracle, rows, cols, kind):
    """tens of thousands of rows of at most 128 columns: the kernel with one lane per row; also in place"""
    rng = np.random.default_rng(307)
    xf = (rng.standard_normal((rows, cols)) * 2).astype(np.float32)
    _special_rows(xf, cols)
    xf[rows - 2, :] = 95.0 if kind == "bf16" else 12.0                  # a row in the last (partial) block that overflows
    bf = kind == "bf16"
    x = _bf16(oracle, xf) if bf else xf.astype(np.float16)
    want = oracle.softmax(x, bf16=bf)
    dx = dev.upload(x, bf16=bf)
    got = dev.softmax(dx).to_numpy()
    dev.softmax(dx, out=dx)
    got2 = dx.to_numpy()
    if bf:
        isnan = lambda b: (b & 0x7fff) > 0x7f80
        assert not ((got != want) & ~(isnan(got) & isnan(want))).any()
        assert not ((got2 != want) & ~(isnan(got2) & isnan(want))).any()
    else:
        assert mismatch_count(got, want) == 0, describe_mismatch(got, want, x)
        assert same_bits(got2, want)


def test_softmax_f16_order_dependence_is_reproduced(dev, oracle):
    # 2048 + 1 + 1 + ... never grows in f16: the kernel must reproduce that, not the mathematically exact sum
    row = np.zeros(512, np.float16)
    row[0] = np.float16(np.log(2048.0))
    x = np.stack([row, row[::-1]])
    want = oracle.softmax(x)
    got = dev.softmax(dev.upload(x)).to_numpy()
    assert same_bits(got, want)
    assert got[0, 1] != got[1, 0]


def test_softmax_bf16_and_stable_mode(dev, oracle):
    from ratchet_amd import _lib

    rng = np.random.default_rng(302)
    xb = oracle.cast((rng.standard_normal((2, 9, 320)) * 2).astype(np.float32), np.uint16, dst_bf16=True)
    got = dev.softmax(dev.upload(xb, bf16=True)).to_numpy()
    assert np.array_equal(got, oracle.softmax(xb, bf16=True))
    # stable mode: max-subtracted, f32 accumulation; compare with torch in f32
    for dtype, tol in ((np.float32, 1e-6), (np.float16, 1e-3)):
        x = randn(rng, (2, 33, 1000), dtype, 3.0)
        x[0, 0, 0] = 30000.0 if dtype == np.float16 else 1000.0         # would overflow without max subtraction
        got = dev.softmax(dev.upload(x), mode=_lib.SOFTMAX_STABLE).to_numpy()
        ref = F.softmax(torch.from_numpy(x.astype(np.float32)), dim=-1).numpy().astype(dtype)
        bad, mx = oracle.count_not_close(got, ref, tol, tol)
        assert bad == 0, (dtype, bad, mx)


NORM_SHAPES = [(3, 256, 256), (2, 57, 1001), (1, 1, 1), (1, 13, 7), (1, 150, 384), (2, 9, 2048), (1, 5, 2052), (1, 3, 6000),
               (2, 33, 2560), (1, 9, 3072), (1, 3, 8192), (1, 2, 8196),                             # > 2048 columns: a block per row
               (1, 5, 32064), (1, 3, 51200), (2, 65536), (2, 32001), (2, 65540)]                    # vocabulary-sized rows: 1024 threads per row up to 65536 columns


@pytest.mark.parametrize("shape", NORM_SHAPES)
def test_layer_norm_f32(dev, oracle, shape):
    rng = np.random.default_rng(310)
    n = shape[-1]
    x = randn(rng, shape, np.float32)
    w = randn(rng, n, np.float32)
    b = randn(rng, n, np.float32)
    # the oracle adds a row left to right in f32 as the reference's CPU code does; over 65536 terms that sum alone is off by
    # about 1e-5 of its value, which the kernel's tree sum is not: the reference test's own bar (1e-4) applies there
    tol = 1e-5 if n <= 60000 else 1e-4
    for bias in (b, None):
        want = oracle.layer_norm(x, w, bias, 1e-5, intended=True)
        got = dev.layer_norm(dev.upload(x), dev.upload(w), dev.upload(bias) if bias is not None else None, 1e-5).to_numpy()
        bad, mx = oracle.count_not_close(got, want, tol, tol)
        if n == 1:
            assert same_bits(got, want)
        else:
            assert bad == 0, (shape, bias is None, bad, mx)
    if n > 1:
        ref = F.layer_norm(torch.from_numpy(x), (n,), torch.from_numpy(w), torch.from_numpy(b), eps=1e-5).numpy()
        got = dev.layer_norm(dev.upload(x), dev.upload(w), dev.upload(b), 1e-5).to_numpy()
        bad, mx = oracle.count_not_close(got, ref, 1e-4, 1e-4)          # the reference test's tolerance
        assert bad == 0, (shape, bad, mx)


@pytest.mark.parametrize("shape", NORM_SHAPES)
def test_rms_norm_f32(dev, oracle, shape):
    rng = np.random.default_rng(311)
    n = shape[-1]
    x = randn(rng, shape, np.float32)
    w = randn(rng, n, np.float32)
    want = oracle.rms_norm(x, w, 1e-5, intended=True)
    got = dev.rms_norm(dev.upload(x), dev.upload(w), 1e-5).to_numpy()
    tol = 1e-5 if n <= 60000 else 1e-4                                  # (the oracle's left-to-right f32 sum over 65536 terms, as in test_layer_norm_f32)
    bad, mx = oracle.count_not_close(got, want, tol, tol)
    assert bad == 0, (shape, bad, mx)


@pytest.mark.parametrize("shape", [(3, 101, 101), (7, 33), (300, 5), (64, 1), (9, 1499), (5, 2047), (3, 5001), (2, 8190), (2, 8191), (4000, 13)])
def test_norms_f32_rows_that_are_not_whole_vectors(dev, oracle, shape):
    """ragged f32 rows run over the aligned vectors that cover them (8191 columns take the scalar kernel): results inside the
    f32 bar, nothing written outside the tensor; also with scale / bias 4 bytes off their vector alignment on whole-vector rows"""
    from ratchet_amd.runtime import BufferView

    rng = np.random.default_rng(311)
    cols = shape[-1]
    x = randn(rng, shape, np.float32, 1.5)
    w, b = randn(rng, (cols,), np.float32), randn(rng, (cols,), np.float32)
    dx, dw, db = dev.upload(x), dev.upload(w), dev.upload(b)
    for name, want, run in (("layer", oracle.layer_norm(x, w, b, 1e-5, intended=True), lambda o: dev.layer_norm(dx, dw, db, 1e-5, out=o)),
                            ("layer, no bias", oracle.layer_norm(x, w, None, 1e-5, intended=True), lambda o: dev.layer_norm(dx, dw, None, 1e-5, out=o)),
                            ("rms", oracle.rms_norm(x, w, 1e-5, intended=True), lambda o: dev.rms_norm(dx, dw, 1e-5, out=o))):
        big = dev.upload(np.full(x.size + 12, 7.25, np.float32))
        out = BufferView(big, 4, x.shape)
        run(out)
        bad, mx = oracle.count_not_close(out.to_numpy(), want, 1e-5, 1e-5)
        assert bad == 0 or cols == 1, (name, shape, bad, mx)
        whole = big.to_numpy()
        assert (whole[:4] == 7.25).all() and (whole[4 + x.size:] == 7.25).all(), (name, shape)
    x = randn(rng, (37, 512), np.float32, 1.5)
    w, b = randn(rng, (512,), np.float32), randn(rng, (512,), np.float32)
    wv = BufferView(dev.empty((516,), 0), 1, (512,)).upload(w)
    bv = BufferView(dev.empty((516,), 0), 3, (512,)).upload(b)
    got = dev.layer_norm(dev.upload(x), wv, bv, 1e-5).to_numpy()
    bad, mx = oracle.count_not_close(got, oracle.layer_norm(x, w, b, 1e-5, intended=True), 1e-5, 1e-5)
    assert bad == 0, (bad, mx)


@pytest.mark.parametrize("shape", [(2, 64, 2560), (1, 33, 3072), (1, 9, 384), (1, 7, 100), (1, 3, 4104), (16, 128, 256), (1, 5, 1)])
def test_norms_f16(dev, oracle, shape):
    rng = np.random.default_rng(312)
    n = shape[-1]
    x = randn(rng, shape, np.float16)
    w = (1 + 0.02 * rng.standard_normal(n)).astype(np.float16)
    b = (0.02 * rng.standard_normal(n)).astype(np.float16)
    want = oracle.layer_norm(x, w, b, 1e-5, intended=True)
    got = dev.layer_norm(dev.upload(x), dev.upload(w), dev.upload(b), 1e-5).to_numpy()
    bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
    assert bad == 0, ("layer", shape, bad, mx)
    # the rounding sequence and the f32 accumulation order are replayed exactly
    assert mismatch_count(got, want) == 0, mismatch_count(got, want)
    want = oracle.rms_norm(x, w, 1e-5, intended=True)
    got = dev.rms_norm(dev.upload(x), dev.upload(w), 1e-5).to_numpy()
    bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
    assert bad == 0, ("rms", shape, bad, mx)
    assert mismatch_count(got, want) == 0, mismatch_count(got, want)


@pytest.mark.parametrize("rows,cols,kind", [(13, 2560, "f16"), (2048, 4096, "f16"), (2051, 3072, "bf16"), (5, 8, "bf16"), (300, 264, "f16"),   # all blocks resident: output pass from LDS
                                            (40000, 256, "f16"), (9000, 1536, "bf16"), (64, 4104, "f16")])                              # more blocks than fit, rows too long: x re-read
def test_norms_16_bit_both_output_passes(dev, oracle, rows, cols, kind):
    """the 16-bit reference norms keep the raw rows, scale and bias in LDS for the output pass when every block of the
    launch is resident at once, and re-read x otherwise: same bits either way, with and without bias, ragged last block"""
    rng = np.random.default_rng(315)
    bf = kind == "bf16"
    conv = (lambda a: _bf16(oracle, a)) if bf else (lambda a: np.asarray(a, np.float32).astype(np.float16))
    x = conv(rng.standard_normal((rows, cols)) * 1.5 + 0.25)
    w = conv(1 + 0.02 * rng.standard_normal(cols))
    b = conv(0.02 * rng.standard_normal(cols))
    dx, dw, db = dev.upload(x, bf16=bf), dev.upload(w, bf16=bf), dev.upload(b, bf16=bf)
    for name, want, got in (("layer", oracle.layer_norm(x, w, b, 1e-5, bf16=bf, intended=True), dev.layer_norm(dx, dw, db, 1e-5).to_numpy()),
                            ("layer, no bias", oracle.layer_norm(x, w, None, 1e-5, bf16=bf, intended=True), dev.layer_norm(dx, dw, None, 1e-5).to_numpy()),
                            ("rms", oracle.rms_norm(x, w, 1e-5, bf16=bf, intended=True), dev.rms_norm(dx, dw, 1e-5).to_numpy())):
        assert np.array_equal(np.asarray(got).view(np.uint16), np.asarray(want).view(np.uint16)), (name, rows, cols, kind)


@pytest.mark.parametrize("cols", [256, 512, 1000, 1536, 2560, 3072, 4096])
@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_rms_norm_16_bit_row_sums_replayed_in_parallel(dev, oracle, cols, kind):
    """Rows of 256 to 4096 columns take a kernel that replays the reference's left-to-right f32 sum of T(x*x) with the 64
    lanes of a wave (pairs of sums per lane, composed across lanes) instead of walking it; the output must not differ in
    one bit from the walk.  Rows that stress what the kernel decides by: sums that land exactly on powers of two, ranges
    of 2^30 inside a row, heavy tails, squares that overflow the element type, NaN, rows of zeros, single large terms."""
    rng = np.random.default_rng(316 + cols)
    bf = kind == "bf16"
    conv = (lambda a: _bf16(oracle, a)) if bf else (lambda a: np.asarray(a, np.float32).astype(np.float16))
    rows = []
    rows += [rng.standard_normal(cols) * s for s in (1.0, 1.0, 1.0, 0.01, 0.3, 3.0, 20.0, 100.0)]
    rows += [np.ones(cols), np.full(cols, 0.5), np.full(cols, 2.0), np.full(cols, 0.0078125), np.zeros(cols)]
    rows += [np.concatenate([np.full(cols // 2, 2.5e-4), np.full(cols - cols // 2, 100.0)])]          # tiny terms, then large ones
    rows += [np.concatenate([np.full(cols // 2, 100.0), np.full(cols - cols // 2, 2.5e-4)])]          # large sum, then terms below its ulp
    rows += [np.clip(rng.standard_cauchy(cols), -200, 200)]
    one_big = rng.standard_normal(cols) * 0.1
    one_big[cols // 3] = 250.0
    rows += [one_big]
    overflow = rng.standard_normal(cols)
    overflow[cols // 2] = 300.0                                                                     # the square is inf in f16
    rows += [overflow]
    with_nan = rng.standard_normal(cols)
    with_nan[7] = np.nan
    rows += [with_nan]
    rows += [np.abs(rng.standard_normal(cols)) * 2.0 ** rng.integers(-12, 6, cols)]                   # every term its own binade
    rows += [np.arange(cols) % 7 * 0.125, np.linspace(0, 8, cols), np.linspace(8, 0, cols)]
    rows += [rng.standard_normal(cols) for _ in range(40)]
    x = conv(np.stack(rows))
    w = conv(1 + 0.02 * rng.standard_normal(cols))
    want = oracle.rms_norm(x, w, 1e-5, bf16=bf, intended=True)
    got = dev.rms_norm(dev.upload(x, bf16=bf), dev.upload(w, bf16=bf), 1e-5).to_numpy()
    g, t = np.asarray(got).view(np.uint16), np.asarray(want).view(np.uint16)
    nan = (lambda a: (a & 0x7f80) == 0x7f80) if bf else (lambda a: (a & 0x7c00) == 0x7c00)
    same = (g == t) | (nan(g) & nan(t) & ((g & (0x7f if bf else 0x3ff)) != 0) & ((t & (0x7f if bf else 0x3ff)) != 0))
    bad_rows = np.flatnonzero(~same.all(axis=1))
    assert bad_rows.size == 0, (kind, cols, bad_rows[:10].tolist())


@pytest.mark.parametrize("rows,cols,kind", [(20000, 8, "f16"), (16384 + 3, 64, "f16"), (17000, 128, "f16"), (30000, 24, "bf16"), (16500, 120, "bf16")])
def test_norms_16_bit_many_narrow_rows(dev, oracle, rows, cols, kind):
    """tens of thousands of rows of at most 128 columns take a kernel with one lane per row; same bits as the walkers"""
    rng = np.random.default_rng(314)
    bf = kind == "bf16"
    conv = (lambda a: _bf16(oracle, a)) if bf else (lambda a: np.asarray(a, np.float32).astype(np.float16))
    x = conv(rng.standard_normal((rows, cols)) * 1.5 + 0.25)
    w = conv(1 + 0.02 * rng.standard_normal(cols))
    b = conv(0.02 * rng.standard_normal(cols))
    dx, dw, db = dev.upload(x, bf16=bf), dev.upload(w, bf16=bf), dev.upload(b, bf16=bf)
    for name, want, got in (("layer", oracle.layer_norm(x, w, b, 1e-5, bf16=bf, intended=True), dev.layer_norm(dx, dw, db, 1e-5).to_numpy()),
                            ("layer, no bias", oracle.layer_norm(x, w, None, 1e-5, bf16=bf, intended=True), dev.layer_norm(dx, dw, None, 1e-5).to_numpy()),
                            ("rms", oracle.rms_norm(x, w, 1e-5, bf16=bf, intended=True), dev.rms_norm(dx, dw, 1e-5).to_numpy())):
        assert np.array_equal(np.asarray(got).view(np.uint16), np.asarray(want).view(np.uint16)), (name, rows, cols, kind)


def test_layer_norm_variance_form_matches_reference(dev, oracle):
    # E[x^2] - mu^2 loses digits with a large common offset; the kernel must lose them the same way (not use two passes)
    rng = np.random.default_rng(313)
    x = (rng.standard_normal((8, 256)) * 0.5 + 30).astype(np.float32)
    w = np.ones(256, np.float32)
    want = oracle.layer_norm(x, w, None, 1e-5, intended=True)
    got = dev.layer_norm(dev.upload(x), dev.upload(w), None, 1e-5).to_numpy()
    two_pass = F.layer_norm(torch.from_numpy(x), (256,), eps=1e-5).numpy()
    assert np.nanmax(np.abs(got - want)) < np.nanmax(np.abs(two_pass - want)) or np.allclose(two_pass, want, atol=1e-4)


# Three rows of five columns whose mean is far from zero next to their spread (mean 2.6-2.9, sigma 0.16-0.17), found by a
# search over random rows.  The reference's one-pass variance E[x^2] - mu^2 (cpu/norm.rs:116-122) amplifies the rounding of
# its two sums by mu^2 / var, so on these rows the reference formula itself lands about 3e-5 (in the all_close rule's
# units) from the float64 result whatever the summation order: the 1e-5 bar cannot be met against the true value there,
# and the bar of the reference's own test (1e-4, ops/norm/mod.rs:467) is the one that applies.
OFFSET_ROWS_BITS = [[0x40231C58, 0x4031057B, 0x4012EEA4, 0x40278F96, 0x402C5483],
                    [0x4039B87D, 0x403248EC, 0x402E5EA2, 0x40310982, 0x404CA049],
                    [0x403C178E, 0x4033E167, 0x401D0871, 0x402F6B91, 0x40287424]]


def test_layer_norm_f32_known_answer_rows_with_an_offset(dev, oracle):
    x = np.array(OFFSET_ROWS_BITS, dtype=np.uint32).view(np.float32)
    w, b = np.ones(5, np.float32), np.zeros(5, np.float32)
    x64 = x.astype(np.float64)
    exact = ((x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-5)).astype(np.float32)
    want = oracle.layer_norm(x, w, b, 1e-5, intended=True)
    bad5, _ = oracle.count_not_close(want, exact, 1e-5, 1e-5)
    assert bad5 > 0                                                    # the formula, not a kernel: the oracle itself misses 1e-5 here
    bad4, mx = oracle.count_not_close(want, exact, 1e-4, 1e-4)
    assert bad4 == 0, mx
    got = dev.layer_norm(dev.upload(x), dev.upload(w), dev.upload(b), 1e-5).to_numpy()
    for name, ref in (("float64 result", exact), ("oracle", want)):
        bad, mx = oracle.count_not_close(got, ref, 1e-4, 1e-4)
        assert bad == 0, (name, bad, mx)


@pytest.mark.parametrize("B,C,L,G", [(1, 3, 1, 1), (2, 8, 5, 4), (1, 6, 7, 6), (3, 4, 9, 1), (1, 64, 3000, 32), (2, 32, 17, 8),
                                     (1, 512, 3000, 32),          # the benchmark shape: 32 groups of 96 KB: eight blocks per group, each with the group in registers
                                     (9, 128, 40, 64),            # 576 groups of 80 elements, each staged in LDS by a block
                                     (1, 8, 40000, 2),            # groups larger than LDS
                                     (1, 4, 300000, 1),           # one group of 1.2 M elements: hundreds of slices, combined by a launch of their own
                                     (2, 16, 24, 4),
                                     (1, 64, 3000, 4),            # 4 groups of 96 KB (f16) / 187 KB (f32): 32 blocks per group, 6 / 12 vectors a thread
                                     (2, 256, 4096, 16),          # 32 groups of 128 (registers) / 256 KB (slices over the chip, two launches)
                                     (4, 576, 2040, 72),          # 288 groups of 32 / 64 KB f16/f32 staged in LDS
                                     (8, 512, 1504, 32),          # 256 groups of 47 KB (LDS) / 94 KB (LDS)
                                     (4, 1024, 2496, 32),         # 128 groups of 156 KB f16 / 312 KB f32: slices over the chip
                                     (16, 512, 4096, 32),         # 512 groups of 128 KB f16 (LDS) / 256 KB f32 (16 vectors a thread in registers)
                                     # rows that are not whole vectors (a 16-byte vector crosses into the next channel), groups that are:
                                     (2, 64, 1500, 4),            # f16 rows of 1500: slices in registers
                                     (16, 256, 100, 16),          # 256 groups in LDS, f16 rows of 100
                                     (12, 64, 3, 8),              # 96 groups in LDS, rows shorter than a vector: several channels in one
                                     (1, 256, 1, 8),              # rows of one element
                                     (4, 1024, 2500, 32),         # 128 groups of 156 KB f16 in slices, rows of 2500
                                     (4, 608, 2500, 32)])         # 128 groups of 93 KB f16 / 186 KB f32 in registers (two blocks / one block per group), rows of 2500
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_group_norm(dev, oracle, B, C, L, G, dtype):
    rng = np.random.default_rng(320)
    x = randn(rng, (B, C, L), dtype)
    w = randn(rng, C, dtype)
    b = randn(rng, C, dtype)
    tol = 1e-5 if dtype == np.float32 else 1e-3
    want = oracle.group_norm(x, G, w, b, 1e-5)
    got = dev.group_norm(dev.upload(x), G, dev.upload(w), dev.upload(b), 1e-5).to_numpy()
    bad, mx = oracle.count_not_close(got, want, tol, tol)
    assert bad == 0, (bad, mx)
    ref = F.group_norm(torch.from_numpy(x.astype(np.float32)), G, torch.from_numpy(w.astype(np.float32)),
                       torch.from_numpy(b.astype(np.float32)), eps=1e-5).numpy().astype(dtype)
    bad, mx = oracle.count_not_close(got, ref, max(tol, 1e-4), max(tol, 1e-4))      # the reference test's tolerance
    assert bad == 0, (bad, mx)
    got = dev.group_norm(dev.upload(x), G, None, None, 1e-5).to_numpy()
    bad, mx = oracle.count_not_close(got, oracle.group_norm(x, G, None, None, 1e-5), tol, tol)
    assert bad == 0, (bad, mx)


def test_group_norm_many_groups_too_large_for_lds(dev, oracle):
    """288 groups of 160 KB in f32 (more pairs than CUs, groups over what the LDS kernel stages): one block per group with the
    group in registers, two rounds of blocks; against the oracle"""
    rng = np.random.default_rng(323)
    B, C, L, G = 9, 320, 4096, 32
    x = randn(rng, (B, C, L), np.float32)
    w, b = randn(rng, C, np.float32), randn(rng, C, np.float32)
    got = dev.group_norm(dev.upload(x), G, dev.upload(w), dev.upload(b), 1e-5).to_numpy()
    bad, mx = oracle.count_not_close(got, oracle.group_norm(x, G, w, b, 1e-5), 1e-5, 1e-5)
    assert bad == 0, (bad, mx)


def test_group_norm_one_group_over_64_mib(dev, oracle):
    """One group of 72 MB per batch entry in f32: its 2048 slices are too large for the registers of a 256-thread block, so the
    looping stats and apply kernels run, and a launch of their own combines the partials; against the oracle"""
    rng = np.random.default_rng(324)
    B, C, L, G = 1, 2, 9_000_000, 1
    x = randn(rng, (B, C, L), np.float32)
    x += np.float32(0.5)
    w, b = randn(rng, C, np.float32), randn(rng, C, np.float32)
    got = dev.group_norm(dev.upload(x), G, dev.upload(w), dev.upload(b), 1e-5).to_numpy()
    bad, mx = oracle.count_not_close(got, oracle.group_norm(x, G, w, b, 1e-5), 1e-5, 1e-5)
    assert bad == 0, (bad, mx)


@pytest.mark.parametrize("shape,mshape", [((1, 8, 512, 512), (512, 512)), ((2, 4, 300, 1024), (1, 1, 300, 1024)), ((1, 32, 100, 4096), (100, 4096)),
                                          ((1, 6, 300, 3072), (300, 3072)), ((2, 2, 260, 2600), (1, 1, 260, 2600)), ((1, 4, 250, 1536), (250, 1536)), ((1, 3, 245, 2304), (245, 2304)),
                                          ((2, 3, 250, 1000), (2, 1, 250, 1000)), ((1, 5, 1000, 264), (1, 5, 1000, 264)),
                                          ((1, 16, 256, 256), (1, 1, 1, 256)), ((1, 2, 40, 64), (40, 64)), ((3, 2, 1031, 512), (1031, 512))])
def test_softmax_masked_equals_add_then_softmax(dev, oracle, shape, mshape):
    """scores.add(mask).softmax(3) in f16: one launch where the streaming kernel applies (a mask shared by periods of whole
    heads), two launches otherwise; always the bits of the two separate ops."""
    rng = np.random.default_rng(320)
    x = randn(rng, shape, np.float16, 2.0)
    S, T = mshape[-2], mshape[-1]
    mask = np.zeros(mshape, np.float16)
    m2 = mask.reshape(-1, S, T)
    m2[:] = np.triu(np.full((S, T), -np.inf, np.float16), k=1 + max(T - S, 0)) if S > 1 else (randn(rng, (T,), np.float16) * np.float16(3))
    m2[..., S // 2, :] = randn(rng, (T,), np.float16)                 # a finite row too: the 16-bit add must round as the separate op does
    full_mask = np.ascontiguousarray(np.broadcast_to(mask.reshape((1,) * (4 - mask.ndim) + mask.shape), shape))
    want = oracle.softmax(oracle.binary("add", x, full_mask))
    dx, dm = dev.upload(x), dev.upload(mask)
    got = dev.softmax_masked(dx, dm).to_numpy()
    assert mismatch_count(got, want) == 0, (shape, mshape, describe_mismatch(got, want, x))
    two = dev.softmax(dev.binary("add", dx, dm)).to_numpy()
    assert same_bits(got, two)
    dev.softmax_masked(dx, dm, out=dx)                                 # in place
    assert same_bits(dx.to_numpy(), got)


@pytest.mark.parametrize("shape,mshape", [((1, 2, 2048, 4096), (2048, 4096)), ((1, 3, 2048, 4096), (2048, 4096)), ((1, 2, 3300, 2560), (3300, 2560)),
                                          ((2, 1, 2400, 3584), (1, 1, 2400, 3584))])
def test_softmax_masked_large_masks_whose_uniform_tiles_are_not_loaded(dev, oracle, shape, mshape):
    """From 16 MiB on, a pass over the mask classifies its 512-column tiles first, and the streaming kernel loads only the
    tiles whose elements differ (a tile of equal elements is put together from its class word).  Masks here: causal, with
    a finite row across it, a stretch of rows that are one finite value throughout (uniform tiles that are neither 0 nor
    -inf), a tile that differs from its neighbours in its last element only, and NaN in one place.  Two and three heads
    under one mask take one mask row per pair of heads (the odd head out pairs with nothing); 2560 and 3584 columns take
    five and seven steps a row.  Always the bits of add-then-softmax."""
    rng = np.random.default_rng(322)
    x = randn(rng, shape, np.float16, 2.0)
    S, T = mshape[-2], mshape[-1]
    m2 = np.triu(np.full((S, T), -np.inf, np.float16), k=1)
    m2[S // 2, :] = randn(rng, (T,), np.float16)
    m2[S // 3:S // 3 + 40, :] = np.float16(-2.5)
    m2[S // 4, 1023] = np.float16(0.125)
    m2[S // 5, 700] = np.float16(np.nan)
    mask = np.ascontiguousarray(m2.reshape(mshape))
    assert mask.nbytes >= 16 << 20
    full_mask = np.ascontiguousarray(np.broadcast_to(mask.reshape((1,) * (4 - mask.ndim) + mask.shape), shape))
    want = oracle.softmax(oracle.binary("add", x, full_mask))
    dx, dm = dev.upload(x), dev.upload(mask)
    got = dev.softmax_masked(dx, dm).to_numpy()
    assert mismatch_count(got, want) == 0, (shape, mshape, describe_mismatch(got, want, x))
    dev.softmax_masked(dx, dm, out=dx)                                 # in place
    assert same_bits(dx.to_numpy(), got)


@pytest.mark.parametrize("shape,mshape,kind", [((1, 4, 333, 1001), (333, 1001), "f16"), ((2, 3, 77, 199), (1, 1, 77, 199), "f16"),
                                               ((1, 2, 50, 2047), (50, 2047), "f16"), ((2, 2, 40, 511), (2, 1, 40, 511), "f16"),
                                               ((1, 8, 9, 193), (1, 1, 1, 193), "f16"), ((1, 2, 30, 4089), (30, 4089), "f16"),
                                               ((1, 2, 30, 4095), (30, 4095), "f16"), ((1, 2, 30, 4097), (30, 4097), "f16"), ((1, 3, 50, 3001), (50, 3001), "f16"), ((1, 2, 40, 2303), (40, 2303), "f16"), ((1, 3, 1001, 1001), (1, 3, 1001, 1001), "f16"),
                                               ((1, 4, 250, 1003), (250, 1003), "bf16"), ((2, 2, 31, 1535), (1, 1, 31, 1535), "bf16"), ((1, 2, 64, 2047), (64, 2047), "bf16")])
def test_softmax_masked_rows_that_are_not_whole_vectors(dev, oracle, shape, mshape, kind):
    """the one-launch masked softmax on ragged rows (a prompt of 1001 tokens): the mask row that belongs to a row of scores
    has an alignment of its own, so every mask vector is assembled from two aligned ones; the bits of add-then-softmax.
    Rows of 511, 2047, 4095 columns can reach one vector past their last 512-column step (the walking wave adds it)."""
    rng = np.random.default_rng(323)
    bf = kind == "bf16"
    S, T = mshape[-2], mshape[-1]
    xf = (rng.standard_normal(shape) * 2).astype(np.float32)
    mf = np.zeros(mshape, np.float32)
    m2 = mf.reshape(-1, S, T)
    if S > 1:
        m2[:] = np.triu(np.full((S, T), -np.inf, np.float32), k=1 + max(T - S, 0))
        m2[:, S // 2, :] = rng.standard_normal(T).astype(np.float32)
        m2[:, S - 1, :] = 3 * rng.standard_normal(T).astype(np.float32)
        m2[:, 0, :9] = rng.standard_normal(9).astype(np.float32)   # finite values in the first elements of the mask (the vector before them does not exist)
    else:
        m2[:] = 3 * rng.standard_normal(T).astype(np.float32)
    x = _bf16(oracle, xf) if bf else xf.astype(np.float16)
    mask = _bf16(oracle, mf) if bf else mf.astype(np.float16)
    full_mask = np.ascontiguousarray(np.broadcast_to(mask.reshape((1,) * (4 - mask.ndim) + mask.shape), shape))
    want = oracle.softmax(oracle.binary("add", x, full_mask, bf16=bf), bf16=bf)
    isnan = (lambda b: (b & 0x7fff) > 0x7f80) if bf else (lambda b: (b.view(np.uint16) & 0x7fff) > 0x7c00)
    same = lambda g: not ((g.view(np.uint16) != want.view(np.uint16)) & ~(isnan(g) & isnan(want))).any()
    dx, dm = dev.upload(x, bf16=bf), dev.upload(mask, bf16=bf)
    got = dev.softmax_masked(dx, dm).to_numpy()
    assert same(got), (shape, mshape, kind, int(((got.view(np.uint16) != want.view(np.uint16)) & ~(isnan(got) & isnan(want))).sum()))
    dev.softmax_masked(dx, dm, out=dx)                                 # in place
    assert same(dx.to_numpy()), (shape, mshape, kind)


@pytest.mark.parametrize("shape,mshape,kind", [((1, 4, 50, 8192), (50, 8192), "f16"), ((2, 2, 33, 4200), (1, 1, 33, 4200), "f16"),
                                               ((1, 8, 128, 512), (128, 512), "bf16"), ((1, 3, 40, 6000), (40, 6000), "bf16")])
def test_softmax_masked_long_rows_and_bf16(dev, oracle, shape, mshape, kind):
    """the one-launch masked softmax beyond 4096 columns (values parked in y) and in bf16: the bits of add-then-softmax"""
    rng = np.random.default_rng(322)
    bf = kind == "bf16"
    S, T = mshape[-2], mshape[-1]
    xf = (rng.standard_normal(shape) * 2).astype(np.float32)
    mf = np.triu(np.full((S, T), -np.inf, np.float32), k=1 + max(T - S, 0))
    mf[S // 2, :] = rng.standard_normal(T).astype(np.float32)
    mf = np.ascontiguousarray(np.broadcast_to(mf, mshape))
    if bf:
        x, m = _bf16(oracle, xf), _bf16(oracle, mf)
    else:
        x, m = xf.astype(np.float16), mf.astype(np.float16)
    full_mask = np.ascontiguousarray(np.broadcast_to(m.reshape((1,) * (4 - m.ndim) + m.shape), shape))
    want = oracle.softmax(oracle.binary("add", x, full_mask, bf16=bf), bf16=bf)
    dx, dm = dev.upload(x, bf16=bf), dev.upload(m, bf16=bf)
    got = dev.softmax_masked(dx, dm).to_numpy()
    if bf:
        isnan = lambda b: (b & 0x7fff) > 0x7f80
        assert not ((got != want) & ~(isnan(got) & isnan(want))).any(), (shape, mshape)
    else:
        assert mismatch_count(got, want) == 0, (shape, mshape, describe_mismatch(got, want, x))
    dev.softmax_masked(dx, dm, out=dx)                                 # in place
    assert np.array_equal(dx.to_numpy().view(np.uint16), got.view(np.uint16))


@pytest.mark.parametrize("cols", [1536, 2048, 2056, 2560, 4096, 5000 // 8 * 8, 8192])
@pytest.mark.parametrize("masked", [False, True])
def test_softmax_f16_few_long_rows_sums_replayed_in_parallel(dev, oracle, cols, masked):
    """A few rows of 2048 to 8192 columns in f16 (a decode step's scores) take a kernel that replays the reference's
    left-to-right f16 sum of the exp values with the 64 lanes of a wave instead of walking it; not one bit may differ from the
    step-wise model.  Rows that stress what the kernel decides by: sums that stop growing (terms below half an ulp),
    sums that land on powers of two, tiny terms before and after large ones, overflow to inf, NaN, rows of -inf, a causal
    tail, every term in a binade of its own."""
    rng = np.random.default_rng(327 + cols)
    rows = [rng.standard_normal(cols) * s for s in (0.5, 1.0, 2.0, 3.0, 5.0)]
    rows += [np.zeros(cols), np.full(cols, -np.inf), np.full(cols, np.log(0.5)), np.full(cols, -8.0), np.full(cols, 3.0), np.full(cols, -17.5)]
    rows += [np.concatenate([np.full(cols // 2, -10.0), np.full(cols - cols // 2, 5.0)])]             # tiny terms, then large ones
    rows += [np.concatenate([np.full(cols // 2, 5.0), np.full(cols - cols // 2, -10.0)])]             # large sum, then terms below its ulp
    one_inf = rng.standard_normal(cols)
    one_inf[cols // 3] = 12.0                                                                        # exp overflows f16
    rows += [one_inf]
    late_big = rng.standard_normal(cols) - 4.0
    late_big[-5] = 10.0
    rows += [late_big]
    with_nan = rng.standard_normal(cols)
    with_nan[cols // 2 + 3] = np.nan
    rows += [with_nan]
    causal = rng.standard_normal(cols) * 2.0
    causal[cols // 4:] = -np.inf
    rows += [causal]
    rows += [rng.uniform(-16.0, 10.0, cols), np.linspace(-10, 10, cols), np.linspace(10, -10, cols), np.arange(cols) % 7 * 0.5 - 2.0]
    rows += [rng.standard_normal(cols) * 2.0 + m for m in (-6.0, -3.0, 0.0, 1.0) for _ in range(10)]
    x = np.stack(rows).astype(np.float16)
    dx = dev.upload(x)
    if masked:
        mask = np.zeros((1, cols), np.float16)
        mask[0, cols - cols // 5:] = -np.inf
        mask[0, ::3] = rng.standard_normal(len(mask[0, ::3])).astype(np.float16)                     # finite terms: the add rounds in f16
        want = oracle.softmax(oracle.binary("add", x, np.ascontiguousarray(np.broadcast_to(mask, x.shape))))
        got = dev.softmax_masked(dx, dev.upload(mask)).to_numpy()
    else:
        want = oracle.softmax(x)
        got = dev.softmax(dx).to_numpy()
    g, t = got.view(np.uint16), want.view(np.uint16)
    nan = lambda a: ((a & 0x7c00) == 0x7c00) & ((a & 0x3ff) != 0)
    same = (g == t) | (nan(g) & nan(t))
    bad_rows = np.flatnonzero(~same.all(axis=1))
    assert bad_rows.size == 0, (cols, masked, bad_rows[:10].tolist())
    if not masked:
        dev.softmax(dx, out=dx)                                                                      # in place
        assert same_bits(dx.to_numpy(), got)


@pytest.mark.parametrize("shape,mshape", [((2, 3, 33, 200), (33, 200)), ((1, 4, 100, 36), (100, 36)), ((2, 2, 64, 1500), (1, 1, 64, 1500)),
                                          ((1, 3, 20, 5120), (20, 5120)), ((2, 2, 3, 40000), (2, 1, 3, 40000)), ((1, 2, 50, 64), (1, 1, 1, 64)),
                                          ((1, 2, 17, 202), (17, 202))])
@pytest.mark.parametrize("np_dt,stable", [(np.float32, False), (np.float32, True), (np.float16, True), ("bf16", True)])
def test_softmax_masked_in_the_row_kernel_has_the_bits_of_add_then_softmax(dev, oracle, shape, mshape, np_dt, stable):
    """f32 scores, and the stable mode of every type: rows of whole vectors take one launch that adds the mask as it loads
    (each of the kernel's row widths: a few lanes, a wave, a block, a 1024-thread block); the last shape's rows are not
    whole vectors and take the two ops.  Bits of the two separate ops either way; f32 reference mode against the oracle."""
    from ratchet_amd import _lib

    rng = np.random.default_rng(326)
    bf = np_dt == "bf16"
    S, T = mshape[-2], mshape[-1]
    x32 = randn(rng, shape, np.float32, 2.0)
    m32 = np.zeros(mshape, np.float32)
    m2 = m32.reshape(-1, S, T)
    m2[:] = np.triu(np.full((S, T), -np.inf, np.float32), k=1 + max(T - S, 0)) if S > 1 else randn(rng, (T,), np.float32) * np.float32(3)
    m2[..., S // 2, :] = randn(rng, (T,), np.float32)                 # a finite row too: the add must round as the separate op does
    if bf:
        x, mask = _bf16(oracle, x32), _bf16(oracle, m32)
        dx, dm = dev.upload(x, bf16=True), dev.upload(mask, bf16=True)
    else:
        x, mask = x32.astype(np_dt), m32.astype(np_dt)
        dx, dm = dev.upload(x), dev.upload(mask)
    mode = _lib.SOFTMAX_STABLE if stable else _lib.SOFTMAX_REFERENCE
    got = dev.softmax_masked(dx, dm, mode=mode).to_numpy()
    two = dev.softmax(dev.binary("add", dx, dm), mode=mode).to_numpy()
    assert same_bits(got, two), (shape, mshape, np_dt, stable)
    if np_dt == np.float32 and not stable:
        full = np.ascontiguousarray(np.broadcast_to(mask.reshape((1,) * (4 - mask.ndim) + mask.shape), shape))
        bad, mx = oracle.count_not_close(got, oracle.softmax(oracle.binary("add", x, full)), 1e-5, 1e-5)
        assert bad == 0, mx
    dev.softmax_masked(dx, dm, out=dx, mode=mode)                      # in place
    assert same_bits(dx.to_numpy(), got)


def test_softmax_masked_other_types_and_modes(dev, oracle):
    from ratchet_amd import _lib, RatchetError

    rng = np.random.default_rng(321)
    x = randn(rng, (2, 3, 33, 200), np.float32, 2.0)
    mask = np.triu(np.full((33, 200), -np.inf, np.float32), k=168)
    got = dev.softmax_masked(dev.upload(x), dev.upload(mask)).to_numpy()
    want = oracle.softmax(oracle.binary("add", x, np.ascontiguousarray(np.broadcast_to(mask, x.shape))))
    bad, mx = oracle.count_not_close(got, want, 1e-5, 1e-5)
    assert bad == 0, mx
    h = x.astype(np.float16)
    got = dev.softmax_masked(dev.upload(h), dev.upload(mask.astype(np.float16)), mode=_lib.SOFTMAX_STABLE).to_numpy()
    ref = F.softmax(torch.from_numpy((h + mask.astype(np.float16)).astype(np.float32)), dim=-1).numpy().astype(np.float16)
    bad, mx = oracle.count_not_close(got, ref, 1e-3, 1e-3)
    assert bad == 0, mx
    with pytest.raises(RatchetError) as e:
        dev.softmax_masked(dev.upload(h), dev.upload(np.zeros((33, 100), np.float16)))
    assert e.value.status == 4
