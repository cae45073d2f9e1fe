"""GPU parity: permute / slice / broadcast_to / concat against the CPU oracle (bit-exact), through the C ABI.

Problem spaces follow the reference's own tests (crates/ratchet-core/src/ops/reindex/{permute,slice,broadcast}.rs,
ops/concat.rs) plus the benchmark shapes and alignment / odd-size edge cases.
"""
import itertools

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


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_permute_all_orders(dev, oracle, dtype):
    rng = np.random.default_rng(200)
    for shape in [(2, 3, 5, 7), (1, 4, 66, 130), (2, 1, 8, 64), (3, 5, 1, 16)]:
        x = randn(rng, shape, dtype)
        dx = dev.upload(x)
        for perm in itertools.permutations(range(4)):
            want = oracle.permute(x, perm)
            got = dev.permute(dx, perm).to_numpy()
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (shape, perm)


def test_permute_lower_rank_and_baseline_shapes(dev, oracle):
    rng = np.random.default_rng(201)
    x3 = randn(rng, (4, 100, 80), np.float16)
    for perm in itertools.permutations(range(3)):
        assert np.array_equal(dev.permute(dev.upload(x3), perm).to_numpy(), oracle.permute(x3, perm)), perm
    x2 = randn(rng, (257, 129), np.float32)
    assert np.array_equal(dev.permute(dev.upload(x2), (1, 0)).to_numpy(), x2.T)
    q = randn(rng, (1, 1500, 6, 64), np.float32)                       # Whisper-tiny heads
    p = dev.permute(dev.upload(q), (0, 2, 1, 3))
    assert np.array_equal(p.to_numpy(), oracle.permute(q, (0, 2, 1, 3)))
    assert np.array_equal(dev.permute(p, (0, 2, 1, 3)).to_numpy(), q)   # and back
    k = randn(rng, (1, 256, 32, 80), np.float16)                        # Phi-2 heads (shorter sequence)
    assert np.array_equal(dev.permute(dev.upload(k), (0, 2, 1, 3)).to_numpy(), oracle.permute(k, (0, 2, 1, 3)))
    assert np.array_equal(dev.permute(dev.upload(k), (0, 2, 3, 1)).to_numpy(), oracle.permute(k, (0, 2, 3, 1)))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_permute_transposes_of_whole_vectors(dev, oracle, dtype):
    """Permutations that move the contiguous dim, on shapes whose rows are whole 16-byte vectors on both sides
    (K^T in phi2/attn.rs:140, whisper/mha.rs:106, moondream/vision_encoder.rs:58): every order, head dims 64..128,
    extents that leave partial tiles, and a slice-shaped source offset through views of a larger upload."""
    rng = np.random.default_rng(202)
    # (the last three have rows of whole 128-byte lines on both sides in both types: the register transpose; the others go
    # through LDS patches in the type whose rows are off the lines)
    for shape in [(2, 3, 40, 80), (1, 6, 1504, 64), (2, 2, 264, 96), (1, 4, 72, 128), (3, 8, 16, 8), (1, 2, 520, 200), (2, 16, 8, 1032),
                  (1, 2, 320, 192), (2, 3, 64, 448), (1, 4, 128, 64)]:
        x = randn(rng, shape, dtype)
        dx = dev.upload(x)
        for perm in itertools.permutations(range(4)):
            if perm[3] == 3:
                continue                                    # the contiguous dim stays: covered above
            want = oracle.permute(x, perm)
            got = dev.permute(dx, perm).to_numpy()
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (shape, perm)
    # rank 3 ([B, C, T] -> [B, T, C]: whisper/encoder.rs:53) and rank 2
    x3 = randn(rng, (2, 384, 1504), dtype)
    assert np.array_equal(dev.permute(dev.upload(x3), (0, 2, 1)).to_numpy(), np.ascontiguousarray(x3.transpose(0, 2, 1)))
    x2 = randn(rng, (1000, 136), dtype)
    assert np.array_equal(dev.permute(dev.upload(x2), (1, 0)).to_numpy(), np.ascontiguousarray(x2.T))
    # channel-last image to channel-first and back (moondream/generate.rs:42,140): one side of the transpose is 3 long
    img = randn(rng, (378, 378, 3), dtype)
    chw = dev.permute(dev.upload(img), (2, 0, 1))
    assert np.array_equal(chw.to_numpy(), np.ascontiguousarray(img.transpose(2, 0, 1)))
    assert np.array_equal(dev.permute(chw, (1, 2, 0)).to_numpy(), img)
    wide = randn(rng, (2, 700, 12), dtype)
    assert np.array_equal(dev.permute(dev.upload(wide), (0, 2, 1)).to_numpy(), np.ascontiguousarray(wide.transpose(0, 2, 1)))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_permute_transposes_with_the_widest_access_each_side_allows(dev, oracle, dtype):
    """Permutations that move the contiguous dim on shapes whose rows are not whole 16-byte vectors on at least one side:
    the 64 x 64 patch is loaded and stored in units of 8, 4, 2 or 1 elements, whatever every row start and extent on that
    side is a multiple of.  K^T at whisper's 1500 frames (whisper/mha.rs:106), extents that leave ragged patches, every
    order that moves the last dim, and a source that starts off the 16-byte boundary."""
    rng = np.random.default_rng(203)
    # (the last four: source rows of 65 to 128 elements in whole vectors take one patch across the row, 80, 96 or 128 wide)
    for shape in [(2, 3, 1500, 64), (1, 2, 70, 66), (1, 3, 1502, 68), (2, 2, 129, 100), (1, 2, 67, 131), (1, 1, 1500, 1028), (2, 2, 36, 252),
                  (2, 3, 37, 80), (1, 3, 200, 104), (1, 2, 70, 120), (2, 2, 150, 72)]:
        x = randn(rng, shape, dtype)
        dx = dev.upload(x)
        for perm in itertools.permutations(range(4)):
            if perm[3] == 3:
                continue
            want = oracle.permute(x, perm)
            got = dev.permute(dx, perm).to_numpy()
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (shape, perm)
    from ratchet_amd.runtime import BufferView
    big = randn(rng, (1 + 4 * 300 * 72,), dtype)
    dbig = dev.upload(big)
    for skip in (1, 2, 4):                                             # element offsets: 2..16 bytes off the allocation's alignment
        view = BufferView(dbig, skip, (3, 300, 72))
        want = np.ascontiguousarray(big[skip:skip + 3 * 300 * 72].reshape(3, 300, 72).transpose(0, 2, 1))
        assert np.array_equal(dev.permute(view, (0, 2, 1)).to_numpy().view(np.uint8), want.view(np.uint8)), skip


def test_permute_rejects_duplicates(dev):
    from ratchet_amd import RatchetError

    x = dev.upload(np.zeros((2, 2, 2, 2), np.float32))
    with pytest.raises(RatchetError) as e:
        dev.permute(x, (0, 1, 1, 3))
    assert e.value.status == 5


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_slice(dev, oracle, dtype):
    rng = np.random.default_rng(202)
    x = randn(rng, (6, 5, 9, 40), dtype)
    dx = dev.upload(x)
    for ranges in [[(1, 4), (0, 5), (3, 8), (8, 32)], [(0, 6), (0, 5), (0, 9), (0, 40)], [(2, 3), (1, 2), (4, 5), (39, 40)],
                   [(0, 6), (0, 5), (0, 9), (1, 9)], [(3, 6), (0, 5), (0, 9), (0, 40)], [(0, 6), (2, 4), (0, 9), (0, 40)]]:
        want = oracle.slice_(x, ranges)
        got = dev.slice(dx, ranges).to_numpy()
        assert np.array_equal(got, want), ranges
    # random sub-ranges as in the reference test (ops/reindex/slice.rs:71-187)
    for _ in range(16):
        shape = [int(rng.integers(2, 17)) for _ in range(3)] + [int(rng.integers(2, 129))]
        y = randn(rng, shape, dtype)
        ranges = []
        for s in shape:
            a = int(rng.integers(0, s))
            b = int(rng.integers(a + 1, s + 1))
            ranges.append((a, b))
        assert np.array_equal(dev.slice(dev.upload(y), ranges).to_numpy(), oracle.slice_(y, ranges)), (shape, ranges)
    # Phi-3 style split of a fused projection: [1, S, 3*D] -> [1, S, D]
    z = randn(rng, (1, 64, 3 * 96), dtype)
    for k in range(3):
        r = [(0, 1), (0, 64), (k * 96, (k + 1) * 96)]
        assert np.array_equal(dev.slice(dev.upload(z), r).to_numpy(), oracle.slice_(z, r))


def test_slice_rejects_out_of_bounds(dev):
    from ratchet_amd import RatchetError

    x = dev.upload(np.zeros((2, 3), np.float32))
    with pytest.raises(RatchetError) as e:
        dev.slice(x, [(0, 2), (1, 4)])
    assert e.value.status == 4


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_broadcast(dev, oracle, dtype):
    rng = np.random.default_rng(203)
    cases = [((1, 5, 1, 16), (3, 5, 4, 16)), ((1,), (4, 32, 8, 8)), ((2, 1, 1, 1), (2, 3, 4, 5)), ((7,), (2, 7)), ((3, 1), (3, 4)),
             ((1, 1, 6), (2, 5, 6)), ((1, 32, 64, 1), (1, 32, 64, 64)), ((1, 1, 1, 64), (1, 4, 64, 64)), ((5, 1), (5, 3)),
             ((2, 1, 3), (2, 7, 3)), ((1, 8, 1, 128), (2, 8, 2, 128)), ((16, 16), (1, 8, 16, 16))]
    for src, dst in cases:
        x = randn(rng, src, dtype)
        want = oracle.broadcast(x, dst, numpy_semantics=True)
        got = dev.broadcast_to(dev.upload(x), dst).to_numpy()
        assert np.array_equal(got, want), (src, dst)
        assert np.array_equal(want, np.broadcast_to(x, dst))


def test_broadcast_rejects_invalid(dev):
    from ratchet_amd import RatchetError

    with pytest.raises(RatchetError) as e:
        dev.broadcast_to(dev.upload(np.zeros((2, 3), np.float32)), (2, 4))
    assert e.value.status == 4


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_concat(dev, oracle, dtype):
    rng = np.random.default_rng(204)
    # the reference's own case (ops/concat.rs:273-359)
    xs = [randn(rng, (4, 2, k, 128), dtype) for k in (50, 13, 77, 55, 11)]
    got = dev.concat([dev.upload(x) for x in xs], 2).to_numpy()
    assert np.array_equal(got, oracle.concat(xs, 2))
    for dim, shapes in [(0, [(2, 3), (5, 3), (1, 3)]), (1, [(3, 1), (3, 4)]), (3, [(2, 2, 3, 5), (2, 2, 3, 8)]),
                        (2, [(1, 4, 31, 80), (1, 4, 1, 80)]), (1, [(2, 7, 3), (2, 9, 3), (2, 1, 3), (2, 2, 3), (2, 5, 3), (2, 6, 3),
                                                                    (2, 1, 3), (2, 8, 3)])]:
        ys = [randn(rng, s, dtype) for s in shapes]
        got = dev.concat([dev.upload(y) for y in ys], dim).to_numpy()
        assert np.array_equal(got, oracle.concat(ys, dim)), (dim, shapes)
    # short segments take the kernel that walks the destination: the rotary / pass-through halves of a head
    # (phi2/attn.rs:119-127 via rope), eight narrow inputs, segments of 1..3 vectors, odd widths, many rows
    for dim, shapes in [(3, [(1, 32, 300, 32), (1, 32, 300, 48)]), (3, [(2, 4, 100, 16), (2, 4, 100, 64)]), (1, [(5000, 8), (5000, 8)]),
                        (1, [(3000, 3), (3000, 5)]), (1, [(1000, 33), (1000, 31)]), (2, [(7, 9, k, 4) for k in (1, 2, 3, 4, 5, 6, 7, 8)]),
                        (3, [(2, 3, 70, 24), (2, 3, 70, 8), (2, 3, 70, 40)]), (2, [(3, 500, 1, 8), (3, 500, 2, 8)])]:
        ys = [randn(rng, s, dtype) for s in shapes]
        got = dev.concat([dev.upload(y) for y in ys], dim).to_numpy()
        assert np.array_equal(got, oracle.concat(ys, dim)), (dim, shapes)


def test_concat_rejects_bad_arguments(dev):
    from ratchet_amd import RatchetError

    a = dev.upload(np.zeros((2, 3), np.float32))
    b = dev.upload(np.zeros((3, 4), np.float32))
    with pytest.raises(RatchetError) as e:
        dev.concat([a, b], 0)
    assert e.value.status == 4
    with pytest.raises(RatchetError) as e:
        dev.concat([a], 0)
    assert e.value.status == 7


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_cache(dev, oracle, dtype):
    rng = np.random.default_rng(205)
    # the reference's own case (ops/cache.rs:162-217)
    populated = randn(rng, (1, 2, 2, 16), dtype)
    source = randn(rng, (1, 2, 1, 16), dtype)
    cache = np.concatenate([populated, np.zeros((1, 2, 4, 16), dtype)], axis=2)
    d_cache = dev.upload(cache)
    got = dev.cache(d_cache, dev.upload(source), 2, 2).to_numpy()
    want = oracle.cache(cache, source, 2, 2)
    assert np.array_equal(got, want) and np.array_equal(got, np.concatenate([populated, source], axis=2))
    assert np.array_equal(d_cache.to_numpy(), cache)
    # decode loops in phi2's (dim 2) and whisper's (dim 1) layouts, odd extents for every vector width, prompt then single rows
    for dim, shape, chunks in ((2, (1, 32, 40, 80), (17, 1, 1, 1, 20)), (1, (1, 24, 384), (5, 1, 1, 17)), (2, (2, 3, 9, 5), (2, 3, 1, 3)),
                               (3, (1, 2, 3, 11), (4, 7)), (1, (2, 6, 4, 6), (1, 5)), (0, (6, 2, 4), (6,)), (2, (1, 1, 2048, 128), (2047, 1))):
        cache = randn(rng, shape, dtype)                       # stale contents beyond the fill must never reach dst
        d_cache = dev.upload(cache)
        off = 0
        for n in chunks:
            sshape = list(shape)
            sshape[dim] = n
            src = randn(rng, sshape, dtype)
            got = dev.cache(d_cache, dev.upload(src), dim, off).to_numpy()
            want = oracle.cache(cache, src, dim, off)
            off += n
            assert np.array_equal(got, want), (dim, shape, off)
            assert np.array_equal(d_cache.to_numpy(), cache), (dim, shape, off)


def test_cache_rejects_overflow(dev):
    from ratchet_amd import RatchetError

    c = dev.upload(np.zeros((1, 2, 4, 8), np.float32))
    s = dev.upload(np.zeros((1, 2, 2, 8), np.float32))
    with pytest.raises(RatchetError) as e:
        dev.cache(c, s, 2, 3)
    assert e.value.status == 4


@pytest.mark.parametrize("shape,perm", [((2, 37, 64, 3), (0, 3, 1, 2)), ((1, 33, 40, 5), (0, 3, 1, 2)), ((3, 5, 24, 2), (0, 3, 1, 2)),
                                        ((2, 8, 32, 16), (0, 3, 1, 2)), ((2, 3, 40, 4), (0, 1, 3, 2)), ((1, 1, 5000, 3), (0, 1, 3, 2)),
                                        ((2, 3, 16, 40), (0, 2, 3, 1)), ((1, 5, 33, 40), (0, 2, 3, 1)), ((2, 16, 8, 32), (0, 2, 3, 1)),
                                        ((2, 3, 4, 40), (0, 1, 3, 2)), ((1, 1, 3, 5000), (0, 1, 3, 2)), ((1, 2, 1031, 8, ), (0, 3, 1, 2)),
                                        ((1, 7, 9, 3), (0, 3, 1, 2)), ((1, 3, 7, 9), (0, 2, 3, 1)), ((1, 300, 300, 3), (0, 3, 1, 2))])
@pytest.mark.parametrize("np_dt", [np.float32, np.float16])
def test_permute_channels_to_planes_and_back(dev, shape, perm, np_dt):
    """[.., J, C] <-> [.., C, J] with 2 to 16 channels (images: [B,H,W,3] <-> [B,3,H,W]): the interleaved side moves as one
    contiguous run per tile, the planar side as C runs, both in 16-byte accesses; with and without the neighbouring dim
    merged into J, tiles that end early, and extents that are not whole vectors (which keep the element-wise tile kernel)"""
    rng = np.random.default_rng(95)
    x = rng.standard_normal(shape).astype(np_dt)
    got = dev.permute(dev.upload(x), perm).to_numpy()
    assert same_bits(got, np.ascontiguousarray(x.transpose(perm))), (shape, perm)


@pytest.mark.parametrize("shape", [(4, 6, 40, 24), (2, 3, 70, 5), (8, 16, 64, 80), (3, 33, 9, 130)])
@pytest.mark.parametrize("np_dt", [np.float32, np.float16])
def test_permute_every_order_of_four_dims(dev, shape, np_dt):
    """all 24 orders, among them those that end in a short dim behind one that is not the source's contiguous dim (the two
    are transposed as one merged dim whose source offset has two levels)"""
    rng = np.random.default_rng(96)
    x = rng.standard_normal(shape).astype(np_dt)
    dx = dev.upload(x)
    for perm in itertools.permutations(range(4)):
        got = dev.permute(dx, perm).to_numpy()
        assert same_bits(got, np.ascontiguousarray(x.transpose(perm))), (shape, perm)
