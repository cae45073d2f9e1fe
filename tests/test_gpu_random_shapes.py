"""Seeded random shapes, offsets and dtypes for the index-heavy ops against numpy / the oracle: the vector-width choice,
the dim merging of the reindex kernels and the broadcast index math all depend on divisibility and alignment, which
hand-picked cases sample thinly.  Every case is deterministic (fixed seeds) and small."""
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


def rand_shape(rng, rank, hi=(4, 6, 40, 70)):
    return tuple(int(rng.integers(1, hi[4 - rank + i] + 1)) for i in range(rank))


@pytest.mark.parametrize("seed", range(6))
def test_reindex_random(dev, oracle, seed):
    rng = np.random.default_rng(900 + seed)
    for _ in range(25):
        dtype = (np.float32, np.float16)[int(rng.integers(0, 2))]
        rank = int(rng.integers(1, 5))
        shape = rand_shape(rng, rank)
        x = randn(rng, shape, dtype)
        dx = dev.upload(x)
        perm = [int(p) for p in rng.permutation(rank)]
        assert np.array_equal(dev.permute(dx, perm).to_numpy(), x.transpose(perm)), ("permute", shape, perm)
        ranges = []
        for s in shape:
            lo = int(rng.integers(0, s))
            ranges.append((lo, int(rng.integers(lo + 1, s + 1))))
        assert np.array_equal(dev.slice(dx, ranges).to_numpy(), x[tuple(slice(a, b) for a, b in ranges)]), ("slice", shape, ranges)
        src = tuple(s if rng.random() < 0.6 else 1 for s in shape)
        b = randn(rng, src, dtype)
        dst = (int(rng.integers(1, 4)),) * (4 - rank) + shape if rng.random() < 0.5 else shape
        assert np.array_equal(dev.broadcast_to(dev.upload(b), dst).to_numpy(), np.broadcast_to(b, dst)), ("broadcast", src, dst)
        dim = int(rng.integers(0, rank))
        parts = []
        for _k in range(int(rng.integers(2, 6))):
            s = list(shape)
            s[dim] = int(rng.integers(1, 9))
            parts.append(randn(rng, s, dtype))
        assert np.array_equal(dev.concat([dev.upload(p) for p in parts], dim).to_numpy(), np.concatenate(parts, axis=dim)), ("concat", shape, dim)
        if rank <= 4:
            idx = rng.integers(0, shape[dim], size=int(rng.integers(1, 12))).astype(np.int32)
            assert np.array_equal(dev.index_select(dx, dev.upload(idx), dim).to_numpy(), np.take(x, idx, axis=dim)), ("select", shape, dim)


@pytest.mark.parametrize("seed", range(4))
def test_binary_broadcast_random(dev, oracle, seed):
    rng = np.random.default_rng(910 + seed)
    for _ in range(30):
        dtype = (np.float32, np.float16)[int(rng.integers(0, 2))]
        rank = int(rng.integers(1, 5))
        out = rand_shape(rng, rank, hi=(3, 5, 33, 130))
        sa = tuple(s if rng.random() < 0.7 else 1 for s in out)
        sb = tuple(s if (rng.random() < 0.7 or sa[i] == 1) else 1 for i, s in enumerate(out))     # every out dim comes from a or b
        if rng.random() < 0.3:
            sb = sb[int(rng.integers(0, rank)):] or (1,)                                           # lower rank on one side
            sb = tuple(sb)
        try:
            np.broadcast_shapes(sa, sb)
        except ValueError:
            continue
        a, b = randn(rng, sa, dtype), randn(rng, sb, dtype)
        op = ("add", "sub", "mul", "div")[int(rng.integers(0, 4))]
        oshape = np.broadcast_shapes(sa, sb)
        want = oracle.binary(op, np.ascontiguousarray(np.broadcast_to(a, oshape)), np.ascontiguousarray(np.broadcast_to(b, oshape)))
        got = dev.binary(op, dev.upload(a), dev.upload(b)).to_numpy()
        assert got.shape == tuple(oshape) and same_bits(got, want), (op, sa, sb)


@pytest.mark.parametrize("seed", range(4))
def test_rows_random(dev, oracle, seed):
    """softmax and norms over random row counts / lengths (every kernel selection boundary is crossed somewhere), f32 and f16,
    including operands that start at odd element offsets inside a larger allocation."""
    from ratchet_amd.runtime import BufferView

    rng = np.random.default_rng(920 + seed)
    for _ in range(12):
        rows = int(rng.integers(1, 70))
        cols = int(rng.choice([1, 2, 7, 8, 12, 33, 64, 255, 256, 520, 1000, 1001, 2047, 2048, 2056, 4096, 4104, 5000, 8200]))
        off = int(rng.choice([0, 0, 1, 3, 8]))
        for dtype, tol in ((np.float32, 1e-5), (np.float16, 0.0)):
            x = randn(rng, (rows, cols), dtype, 2.0)
            w, b = randn(rng, (cols,), dtype), randn(rng, (cols,), dtype)
            big = dev.empty((rows * cols + 16,), 0 if dtype == np.float32 else 1)
            xv = BufferView(big, off, (rows, cols)).upload(x)
            got = dev.softmax(xv).to_numpy()
            want = oracle.softmax(x)
            if tol:
                bad, mx = oracle.count_not_close(got, want, tol, tol)
                assert bad == 0, ("softmax", rows, cols, off, mx)
            else:
                assert same_bits(got, want), ("softmax f16", rows, cols, off)
            got = dev.layer_norm(xv, dev.upload(w), dev.upload(b), 1e-5).to_numpy()
            want = oracle.layer_norm(x, w, b, 1e-5, intended=True)
            bad, mx = oracle.count_not_close(got, want, tol or 1e-3, tol or 1e-3)
            assert bad == 0, ("layer_norm", rows, cols, off, dtype.__name__, mx)
            got = dev.rms_norm(xv, dev.upload(w), 1e-5).to_numpy()
            want = oracle.rms_norm(x, w, 1e-5, intended=True)
            bad, mx = oracle.count_not_close(got, want, tol or 1e-3, tol or 1e-3)
            assert bad == 0, ("rms_norm", rows, cols, off, dtype.__name__, mx)
            if dtype == np.float16:
                mask = randn(rng, (rows, cols), dtype)
                mask[rng.random((rows, cols)) < 0.3] = -np.inf
                want = oracle.softmax(oracle.binary("add", x, mask))
                assert same_bits(dev.softmax_masked(xv, dev.upload(mask)).to_numpy(), want), ("softmax_masked", rows, cols, off)
                w32, b32 = w.astype(np.float32), b.astype(np.float32)
                got = dev.norm_via_f32("layer", xv, dev.upload(w32), dev.upload(b32), 1e-5).to_numpy()
                want = oracle.cast(oracle.layer_norm(x.astype(np.float32), w32, b32, 1e-5, intended=True), np.float16)
                bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
                assert bad == 0 or cols == 1, ("norm_via_f32", rows, cols, off, mx)
                got = dev.softmax_via_f32(xv).to_numpy()
                want = oracle.cast(oracle.softmax(x.astype(np.float32)), np.float16)
                bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
                assert bad == 0, ("softmax_via_f32", rows, cols, off, mx)
                # with the mask, at an element offset of its own (the mask's alignment is independent of the rows')
                moff = int(rng.choice([0, 0, 5, 8]))
                mv = BufferView(dev.empty((rows * cols + 16,), 1), moff, (rows, cols)).upload(mask)
                got = dev.softmax_via_f32(xv, mv).to_numpy()
                want = oracle.cast(oracle.softmax(oracle.binary("add", x, mask).astype(np.float32)), np.float16)
                bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
                assert bad == 0, ("softmax_via_f32 masked", rows, cols, off, moff, mx)
                # bf16 reference softmax on the same numbers
                xb = oracle.cast(x.astype(np.float32), np.uint16, dst_bf16=True)
                bv = BufferView(dev.empty((rows * cols + 16,), 2), off, (rows, cols)).upload(xb)
                got = dev.softmax(bv).to_numpy()
                want = oracle.softmax(xb, bf16=True)
                nan = (want & 0x7fff) > 0x7f80
                assert np.array_equal(got[~nan], want[~nan]) and (((got & 0x7fff) > 0x7f80) == nan).all(), ("softmax bf16", rows, cols, off)
