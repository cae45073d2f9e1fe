"""GPU parity of RoPE, IndexSelect and IndexWrite against the oracle (crates/ratchet-core/src/cpu/rope.rs:23-143,
cpu/mod.rs:44-84, ops/index_write.rs:96-104).  IndexSelect / IndexWrite: bit-exact.  RoPE: the rounding points are the
oracle's and sin / cos are the host C library's algorithms, so the bits are the oracle's too (the reference tests at 1e-2)."""
import numpy as np
import pytest

from gpu_util import randn, same_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    from ratchet_amd import Device

    return Device(0)


@pytest.mark.parametrize("shape,dim,offset", [((1, 2, 5, 16), 16, 0), ((2, 3, 7, 32), 16, 5), ((1, 32, 128, 96), 96, 0), ((1, 32, 1, 96), 96, 4095),
                                              ((1, 4, 1, 80), 32, 1023), ((2, 1, 300, 128), 64, 17), ((1, 32, 512, 80), 32, 0),
                                              ((3, 37, 131, 80), 32, 5), ((2, 9, 77, 96), 64, 1), ((5, 7, 50, 72), 72, 0)])   # rows off 256-byte units: whole runs per block, ragged trips and positions
def test_rope_f32(dev, oracle, shape, dim, offset):
    rng = np.random.default_rng(601)
    x = rng.standard_normal(shape).astype(np.float32)
    want = oracle.rope(x, dim, 10000.0, offset)
    d = dev.upload(x)
    got = dev.rope(d, dim, 10000.0, offset).to_numpy()
    bad, mx = oracle.count_not_close(got, want, 1e-6, 1e-6)
    assert bad == 0, (bad, mx)
    assert same_bits(got, want)                                                              # sin / cos are the C library's algorithms: the same bits
    assert np.array_equal(got[..., dim:], x[..., dim:])
    inplace = dev.rope(d, dim, 10000.0, offset, out=d).to_numpy()                            # the reference's GPU kernel is in-place only
    assert same_bits(inplace, got)


def test_rope_16bit_is_widen_rotate_round(dev, oracle):
    rng = np.random.default_rng(602)
    x = randn(rng, (1, 8, 40, 96), np.float16)
    want = oracle.cast(oracle.rope(oracle.cast(x, np.float32), 96, 10000.0, 7), np.float16)
    got = dev.rope(dev.upload(x), 96, 10000.0, 7).to_numpy()
    bad, mx = oracle.count_not_close(got, want, 1e-3, 1e-3)
    assert bad == 0, (bad, mx)
    assert same_bits(got, want)


@pytest.mark.parametrize("shape,dim,offset", [((2, 5, 33, 80), 32, 3), ((1, 3, 9, 80), 40, 0), ((3, 7, 4, 128), 128, 100), ((1, 1, 70, 64), 48, 9),
                                              ((1, 19, 1, 96), 96, 2047), ((1, 2, 6, 24), 24, 1), ((3, 37, 131, 80), 32, 5), ((2, 40, 77, 64), 64, 1), ((1, 70, 50, 96), 64, 0)])
def test_rope_16bit_layouts(dev, oracle, shape, dim, offset):
    """f16 / bf16 in the vector layout (half the rotated width a multiple of 8) and outside it (dim 40, 24), odd
    batch * heads counts, with and without pass-through columns, out of place and in place"""
    rng = np.random.default_rng(605)
    xf = rng.standard_normal(shape).astype(np.float32)
    for bf in (False, True):
        x = oracle.cast(xf, np.uint16, dst_bf16=True) if bf else xf.astype(np.float16)
        x32 = oracle.cast(x, np.float32, src_bf16=bf)
        want = oracle.cast(oracle.rope(x32, dim, 10000.0, offset), np.uint16 if bf else np.float16, dst_bf16=bf)
        d = dev.upload(x, bf16=bf)
        got = dev.rope(d, dim, 10000.0, offset).to_numpy()
        diff = got.view(np.uint16) != np.asarray(want).view(np.uint16)
        assert diff.mean() < 0.002, (shape, dim, bf, diff.mean())                              # one sin / cos ulp may move a rounding
        bad, mx = oracle.count_not_close(got, want, 1e-2 if bf else 1e-3, 1e-2 if bf else 1e-3, bf16=bf)
        assert bad == 0, (shape, dim, bf, bad, mx)
        assert np.array_equal(got[..., dim:].view(np.uint16), x[..., dim:].view(np.uint16))
        inplace = dev.rope(d, dim, 10000.0, offset, out=d).to_numpy()
        assert np.array_equal(inplace.view(np.uint16), got.view(np.uint16))


def test_rope_f32_off_vector_alignment(dev, oracle):
    """an operand 4 bytes off 16-byte alignment takes the scalar kernel: same results as the aligned call"""
    rng = np.random.default_rng(606)
    shape = (1, 4, 37, 80)
    x = rng.standard_normal(shape).astype(np.float32)
    aligned = dev.rope(dev.upload(x), 32, 10000.0, 11).to_numpy()
    big = dev.empty((x.size + 4,), 0)
    view = big.view(1, shape)
    view.upload(x)
    out = dev.empty((x.size + 4,), 0).view(1, shape)
    dev.rope(view, 32, 10000.0, 11, out=out)
    assert same_bits(out.to_numpy(), aligned)


def test_rope_rejects_bad_arguments(dev):
    from ratchet_amd import RatchetError

    x = dev.upload(np.zeros((1, 2, 4, 24), np.float32))
    for dim, base in ((12, 10000.0), (32, 10000.0), (16, 0.0)):
        with pytest.raises(RatchetError) as e:
            dev.rope(x, dim, base, 0)
        assert e.value.status in (4, 7)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_index_select(dev, oracle, dtype):
    rng = np.random.default_rng(603)
    cases = [((256, 32), 0, [64, 192, 255]),                     # the reference's fixed case (ops/select.rs:350-357)
             ((32064, 256), 0, rng.integers(0, 32064, 77)),      # an embedding table
             ((51, 384), 0, rng.integers(0, 51, 1)), ((7, 9), 1, rng.integers(0, 9, 20)), ((3, 5, 11), 1, rng.integers(0, 5, 6)),
             ((2, 3, 4, 6), 2, rng.integers(0, 4, 9)), ((64, 3), 0, rng.integers(0, 64, 40)), ((10, 7), 0, rng.integers(0, 10, 5))]
    for shape, dim, idx in cases:
        src = randn(rng, shape, dtype)
        idx = np.asarray(idx, dtype=np.int32)
        got = dev.index_select(dev.upload(src), dev.upload(idx), dim).to_numpy()
        assert np.array_equal(got, oracle.index_select(src, idx, dim)), (shape, dim)
        assert np.array_equal(got, np.take(src, idx, axis=dim))
    src = randn(rng, (16, 8), dtype)
    got = dev.index_select(dev.upload(src), dev.upload(np.array([3, 16, -1, 0], np.int32)), 0).to_numpy()
    assert np.array_equal(got[[0, 3]], src[[3, 0]]) and not got[[1, 2]].any()                # out-of-range rows come back as zeros


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_index_select_from_q8_0_table(dev, oracle, dtype):
    """The embedding lookup of a quantized model (ops/select.rs:107-111,144-161): rows of a Q8_0F / Q8_0H table, bit for bit
    what dequantize-then-index_select gives (cpu/mod.rs:86-103); the packed words and the scales are the two segments of the
    reference's buffer, the scales starting at the next multiple of 256 bytes (quant.rs:8-17,46)."""
    rng = np.random.default_rng(607)
    for shape, dim, idx in [((256, 32), 0, [64, 192, 255]),                      # the reference's test shape (ops/select.rs:350-357)
                            ((51200 // 8, 2560), 0, rng.integers(0, 51200 // 8, 77)),   # an embedding table, prefill-sized gather
                            ((3, 50, 64), 1, [49, 0, 7, 7]), ((2, 4, 8, 12), 2, [3, 1])]:
        table = (rng.standard_normal(shape) * 0.05).astype(dtype)
        words, scales = oracle.q8_0_quantize(table)
        # one device buffer laid out as the reference lays it out
        nq = words.nbytes
        off = (nq + 255) // 256 * 256
        raw = np.zeros(off + scales.nbytes, np.uint8)
        raw[:nq] = words.view(np.uint8)
        raw[off:] = scales.view(np.uint8)
        buf = dev.upload(raw.view(np.uint32) if raw.nbytes % 4 == 0 else np.concatenate([raw, np.zeros(4 - raw.nbytes % 4, np.uint8)]).view(np.uint32))
        from ratchet_amd.runtime import BufferView
        packed = BufferView(buf, 0, (nq // 4,))
        sc = BufferView(buf, off // 4, (scales.nbytes // 4 if dtype == np.float32 else (scales.nbytes + 3) // 4,))
        sc.dt = 0 if dtype == np.float32 else 1
        ids = np.asarray(idx, np.int32)
        want = oracle.q8_0_index_select(words, scales, shape, ids, dim)
        got = dev.index_select_q8_0(packed, sc, shape, dev.upload(ids), dim).to_numpy()
        assert got.dtype == dtype and same_bits(got, want), (shape, dim)
    # an index outside the table gives a row of zeros
    got = dev.index_select_q8_0(packed, sc, shape, dev.upload(np.array([1, 99], np.int32)), dim).to_numpy()
    assert np.all(got[:, :, 1, :] == 0) and same_bits(got[:, :, 0, :], want[:, :, 1, :])


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_index_write(dev, oracle, dtype):
    rng = np.random.default_rng(604)
    dst = np.array([1, 2, 3, 4, 5, 6], dtype).reshape(3, 2)     # the reference's own test (ops/index_write.rs:203-224)
    d = dev.upload(dst)
    dev.index_write(d, dev.upload(np.array([[7, 8]], dtype)), [2, 0])
    assert np.array_equal(d.to_numpy(), np.array([[1, 2], [3, 4], [7, 8]], dtype))
    for shape, sshape, start in (((1, 32, 64, 80), (1, 32, 1, 80), (0, 0, 17, 0)), ((4, 100), (37,), (1, 3)), ((2, 3, 8), (2, 8), (0, 1, 0)),
                                 ((1024, 1024), (512, 1024), (512, 0)), ((5, 7), (1,), (4, 6))):
        dst, src = randn(rng, shape, dtype), randn(rng, sshape, dtype)
        d = dev.upload(dst)
        dev.index_write(d, dev.upload(src), start)
        assert np.array_equal(d.to_numpy(), oracle.index_write(dst.copy(), src, start)), (shape, sshape, start)
    from ratchet_amd import RatchetError
    with pytest.raises(RatchetError) as e:
        dev.index_write(dev.upload(np.zeros((2, 3), dtype)), dev.upload(np.zeros(3, dtype)), [1, 1])
    assert e.value.status == 4
