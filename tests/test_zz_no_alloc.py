"""rt_group_norm_static, the entry point that allocates nothing, against rt_group_norm through the C ABI.

The shapes split every group over several blocks, so the partial statistics pass through the fixed array in the
library's code object; the second call of each pair is smaller than the first and finds the first call's partials
still in the array.
"""
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


def _pair(dev, oracle, rng, shape, groups, dtype, tol):
    from ratchet_amd.runtime import Buffer

    B, C, L = shape
    x = randn(rng, shape, dtype)
    w = randn(rng, C, dtype)
    b = randn(rng, C, dtype)
    dx, dw, db = dev.upload(x), dev.upload(w), dev.upload(b)
    out_static = Buffer(dev, shape, dx.dt)
    out_plain = Buffer(dev, shape, dx.dt)
    before = dev.pool_stats()
    dev.group_norm(dx, groups, dw, db, 1e-5, out=out_static, static_scratch=True)
    after = dev.pool_stats()
    assert before == after, "rt_group_norm_static went to the storage pool"
    dev.group_norm(dx, groups, dw, db, 1e-5, out=out_plain)
    got, plain = out_static.to_numpy(), out_plain.to_numpy()
    assert same_bits(got, plain), shape
    bad, mx = oracle.count_not_close(got, oracle.group_norm(x, groups, w, b, 1e-5), tol, tol)
    assert bad == 0, (shape, bad, mx)


@pytest.mark.parametrize("dtype,tol", [(np.float16, 1e-3), (np.float32, 1e-5)])
def test_static_scratch_group_norm_two_calls_in_a_row(dev, oracle, dtype, tol):
    rng = np.random.default_rng(900)
    # groups of 512 KB / 1 MB: 16 (batch, group) pairs in 86 slices each, then a smaller problem with 4 pairs
    _pair(dev, oracle, rng, (2, 64, 32768), 8, dtype, tol)
    _pair(dev, oracle, rng, (1, 12, 40000), 4, dtype, tol)
    # one group of 1.2 M elements: hundreds of slices, combined by a launch of their own, then a handful of slices
    _pair(dev, oracle, rng, (1, 4, 300000), 1, dtype, tol)
    _pair(dev, oracle, rng, (1, 8, 40000), 2, dtype, tol)
    # shapes that need no scratch at all take the same single-launch kernels as rt_group_norm
    _pair(dev, oracle, rng, (1, 512, 3000), 32, dtype, tol)
    _pair(dev, oracle, rng, (9, 128, 40), 64, dtype, tol)


def test_static_scratch_group_norm_refuses_what_does_not_fit(dev):
    from ratchet_amd import RatchetError
    from ratchet_amd.runtime import Buffer

    # 24000 (batch, group) pairs, one slice each: 24000 * 2 * 12 bytes of partial and combined statistics > 256 KiB
    shape = (12000, 2, 40960)
    x = Buffer(dev, shape, 1)
    y = Buffer(dev, shape, 1)
    with pytest.raises(RatchetError) as e:
        dev.group_norm(x, 2, None, None, 1e-5, out=y, static_scratch=True)
    assert e.value.status == 6 and "fixed buffer" in str(e.value)      # RT_ERR_SIZE
    dev.group_norm(x, 2, None, None, 1e-5, out=y)                      # the growable entry point takes it
    dev.sync()


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_static_scratch_group_norm_records_into_a_graph_and_replays(dev, oracle, dtype):
    """While a device is capturing, every call that would allocate from the driver or wait for the device is refused
    (RT_ERR_CAPTURE), and hipMalloc itself is illegal: a capture of rt_group_norm_static that ends cleanly shows that the
    entry point stays away from the driver, which the pool's counters cannot (the growable scratch of rt_group_norm is
    grown with hipMalloc directly).  The shape splits every group over slices and needs more partials (98 304 bytes)
    than nothing, so the fixed array is really used.  Replays, with eager work between them, reproduce the eager bits."""
    from ratchet_amd.runtime import Buffer

    rng = np.random.default_rng(901)
    shape, groups = (2, 64, 32768), 8
    x = randn(rng, shape, dtype)
    w, b = randn(rng, shape[1], dtype), randn(rng, shape[1], dtype)
    dx, dw, db = dev.upload(x), dev.upload(w), dev.upload(b)
    eager, replayed = Buffer(dev, shape, dx.dt), Buffer(dev, shape, dx.dt)
    dev.group_norm(dx, groups, dw, db, 1e-5, out=eager, static_scratch=True)
    before = dev.pool_stats()
    with dev.capture() as g:
        dev.group_norm(dx, groups, dw, db, 1e-5, out=replayed, static_scratch=True)
    assert dev.pool_stats() == before
    want = eager.to_numpy()
    for k in range(3):
        replayed.zero_()
        g.launch()
        assert same_bits(replayed.to_numpy(), want), k
        # the program's own eager work between the replays: another problem through the same fixed array
        other = Buffer(dev, (1, 12, 40000), dx.dt)
        dev.group_norm(dev.upload(randn(rng, (1, 12, 40000), dtype)), 4, None, None, 1e-5, out=other, static_scratch=True)
        dev.sync()
    bad, mx = oracle.count_not_close(want, oracle.group_norm(x, groups, w, b, 1e-5), 1e-3 if dtype == np.float16 else 1e-5, 1e-3 if dtype == np.float16 else 1e-5)
    assert bad == 0, (bad, mx)
