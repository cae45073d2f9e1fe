"""Replayable launch lists (HIP graphs) through the C ABI: the counterpart of the reference's encode-all-then-submit-once
Executable::dispatch (crates/ratchet-core/src/executable.rs:33-59).  Every replay is compared bit for bit with eager execution,
with eager work and synchronisations between replays."""
import numpy as np
import pytest

from gpu_util import randn, same_bits

pytestmark = pytest.mark.gpu

F32, F16 = 0, 1


@pytest.fixture()
def dev():
    from ratchet_amd import Device

    d = Device(0)
    yield d
    d.close()


def test_replays_match_eager_execution(dev, oracle):
    rng = np.random.default_rng(801)
    x = randn(rng, (1, 1024, 2560), np.float16)
    bias = randn(rng, (2560,), np.float16, 0.02)
    g = randn(rng, (2560,), np.float16, 0.02) + np.float16(1)
    s = randn(rng, (1, 4, 512, 512), np.float16, 2.0)
    mask = np.triu(np.full((512, 512), -np.inf, np.float16), k=1)
    gx = randn(rng, (2, 64, 300), np.float16)
    gw = randn(rng, (64,), np.float16)
    dx, dbias, dg, ds, dmask, dgx, dgw = (dev.upload(a) for a in (x, bias, g, s, mask, gx, gw))
    h = dev.empty(x.shape, F16)
    act = dev.empty(x.shape, F16)
    ln = dev.empty(x.shape, F16)
    masked = dev.empty(s.shape, F16)
    soft = dev.empty(s.shape, F16)
    fused = dev.empty(s.shape, F16)
    gn = dev.empty(gx.shape, F16)
    cat = dev.empty((1, 2048, 2560), F16)
    scratch = dev.empty((1024,), F32)

    def sequence():
        scratch.zero_()                                        # a fill kernel, not a memset node
        dev.binary("add", dx, dbias, out=h)
        dev.unary("gelu", h, out=act)                          # table path (2.6M elements)
        dev.layer_norm(act, dg, dbias, 1e-5, out=ln)
        dev.binary("add", ds, dmask, out=masked)
        dev.softmax(masked, out=soft)                          # streaming kernel (1M elements)
        dev.softmax_via_f32(ds, dmask, out=fused)
        dev.group_norm(dgx, 8, dgw, None, 1e-5, out=gn)
        dev.concat([ln, act], 1, out=cat)

    outputs = (ln, soft, fused, gn, cat)
    sequence()                                                 # eager: builds the tables, sizes the scratch, gives the expected values
    want = [o.to_numpy() for o in outputs]
    assert same_bits(want[1], oracle.softmax(oracle.binary("add", s, np.ascontiguousarray(np.broadcast_to(mask, s.shape)))))
    with dev.capture() as cap:
        sequence()
    for o in outputs:                                          # capturing must not have run anything
        o.zero_()
    assert not soft.to_numpy().any()
    for replay in range(4):
        cap.launch()
        got = [o.to_numpy() for o in outputs]
        for k, (a, b) in enumerate(zip(got, want)):
            assert same_bits(a, b), (replay, k)
        # eager work and a synchronisation between replays, then scribble over the outputs so a replay that did nothing would show
        dev.unary("neg", dx, out=h)
        dev.sync()
        for o in outputs:
            o.zero_()
    # a new input value flows through the same graph (pointers are fixed, contents are not)
    x2 = randn(rng, x.shape, np.float16)
    from ratchet_amd import _lib
    import ctypes
    _lib.check(dev.lib.rt_h2d(dev.handle, dx.ptr, x2.ctypes.data_as(ctypes.c_void_p), x2.nbytes))
    cap.launch()
    got_ln = ln.to_numpy()
    sequence()
    assert same_bits(got_ln, ln.to_numpy())


def test_replays_of_ragged_row_softmax_match_eager_execution(dev, oracle):
    """rows that are not whole vectors: the streaming softmax leaves every row's sum in a buffer owned by the device and a second
    launch finishes the vectors shared by two rows; two such softmaxes (plain and masked) in one graph use that buffer one
    after the other, replay after replay"""
    rng = np.random.default_rng(802)
    a = randn(rng, (1, 4, 333, 1001), np.float16, 2.0)
    b = randn(rng, (2, 2, 70, 513), np.float16, 2.0)
    mask = np.triu(np.full((70, 513), -np.inf, np.float16), k=444)
    f = randn(rng, (3, 50, 1499), np.float32, 2.0)
    da, db, dm, df = (dev.upload(v) for v in (a, b, mask, f))
    ya, yb, yf = dev.empty(a.shape, F16), dev.empty(b.shape, F16), dev.empty(f.shape, F32)

    def sequence():
        dev.softmax(da, out=ya)
        dev.softmax_masked(db, dm, out=yb)
        dev.softmax(df, out=yf)

    sequence()
    want = [o.to_numpy() for o in (ya, yb, yf)]
    assert same_bits(want[0], oracle.softmax(a))
    assert same_bits(want[1], oracle.softmax(oracle.binary("add", b, np.ascontiguousarray(np.broadcast_to(mask, b.shape)))))
    with dev.capture() as cap:
        sequence()
    for replay in range(3):
        for o in (ya, yb, yf):
            o.zero_()
        cap.launch()
        for k, (o, w) in enumerate(zip((ya, yb, yf), want)):
            assert same_bits(o.to_numpy(), w), (replay, k)
        dev.softmax(db, out=yb)                                # eager use of the same row-sum buffer between replays
        dev.sync()


def test_replays_of_a_decode_step_softmax_match_eager_execution(dev, oracle):
    """[B * H, T] f16 scores of a decode step (one wave per row, the row sum replayed from per-lane pairs), plain and with
    a [1, T] mask, and the masked f32 row kernel, captured and replayed"""
    rng = np.random.default_rng(803)
    a = randn(rng, (1, 32, 1, 2304), np.float16, 2.0)
    m = np.zeros((1, 1, 1, 2304), np.float16)
    m[..., 2000:] = -np.inf
    f = randn(rng, (1, 8, 1, 2304), np.float32, 2.0)
    da, dm, df, dmf = dev.upload(a), dev.upload(m), dev.upload(f), dev.upload(m.astype(np.float32))
    ya, yb, yf = dev.empty(a.shape, F16), dev.empty(a.shape, F16), dev.empty(f.shape, F32)

    def sequence():
        dev.softmax(da, out=ya)
        dev.softmax_masked(da, dm, out=yb)
        dev.softmax_masked(df, dmf, out=yf)

    sequence()
    want = [o.to_numpy() for o in (ya, yb, yf)]
    assert same_bits(want[0], oracle.softmax(a))
    assert same_bits(want[1], oracle.softmax(oracle.binary("add", a, np.ascontiguousarray(np.broadcast_to(m, a.shape)))))
    with dev.capture() as cap:
        sequence()
    for replay in range(3):
        for o in (ya, yb, yf):
            o.zero_()
        cap.launch()
        for k, (o, w) in enumerate(zip((ya, yb, yf), want)):
            assert same_bits(o.to_numpy(), w), (replay, k)
        dev.softmax(da, out=yb)
        dev.sync()


def test_calls_that_cannot_be_captured_say_so(dev):
    from ratchet_amd import RatchetError

    x = dev.upload(np.ones((1 << 21,), np.float16))
    y = dev.empty(x.shape, F16)
    with pytest.raises(RatchetError) as e:
        with dev.capture():
            dev.sync()
    assert e.value.status == 10
    with pytest.raises(RatchetError) as e:
        with dev.capture():
            x.to_numpy()
    assert e.value.status == 10
    with pytest.raises(RatchetError) as e:
        with dev.capture():
            dev.empty((123457,), F32)                          # nothing of that size is parked in the pool
    assert e.value.status == 10
    # the device is usable again after each failed capture, and a nested begin is refused (first use of tanh here: no
    # lookup table exists yet, so the capture records the computing kernel)
    with dev.capture() as cap:
        dev.unary("tanh", x, out=y)
        assert dev.lib.rt_capture_begin(dev.handle) == 10
    y.zero_()
    cap.launch()
    assert np.allclose(y.to_numpy()[-4:].astype(np.float32), np.tanh(1.0), atol=1e-3)
    assert dev.lib.rt_capture_end(dev.handle, None) == 1


def test_first_use_inside_a_capture_takes_the_computing_kernels(dev, oracle):
    """An op whose lookup table does not exist yet cannot build it while a graph is being captured (building synchronises).
    On a fresh device the large unary, the one-pass unary, the gated multiply and the 16-bit softmaxes then record their
    table-free kernels, which give the same bits; replays are compared with the oracle and, afterwards, with eager execution
    (which builds the tables and takes the table kernels)."""
    from ratchet_amd.runtime import BufferView

    rng = np.random.default_rng(802)
    n = 1 << 21                                                # the size from which rt_unary looks values up in LDS
    x = randn(rng, (n,), np.float16)
    s = randn(rng, (2, 512, 1024), np.float16, 2.0)
    mask = np.triu(np.full((512, 1024), -np.inf, np.float16), k=1)
    gate_up = randn(rng, (256, 16384), np.float16)
    dx, ds, dmask, dgu = (dev.upload(a) for a in (x, s, mask, gate_up))
    y, y32, soft, msoft, gated = dev.empty(x.shape, F16), dev.empty(x.shape, F16), dev.empty(s.shape, F16), dev.empty(s.shape, F16), dev.empty((256, 8192), F16)

    def sequence():
        dev.unary("gelu", dx, out=y)
        dev.unary_via_f32("silu", dx, out=y32)
        dev.softmax(ds, out=soft)
        dev.softmax_masked(ds, dmask, out=msoft)
        dev.gated_mul_via_f32("silu", BufferView(dgu, 0, (256 * 16384 - 8192,)), BufferView(dgu, 8192, (256 * 16384 - 8192,)), 256, 8192,
                              gate_row_stride=16384, up_row_stride=16384, out=gated)

    outputs = (y, y32, soft, msoft, gated)
    with dev.capture() as cap:                                 # nothing has run on this device yet
        sequence()
    want = [oracle.unary("gelu", x),
            oracle.cast(oracle.unary("silu", oracle.cast(x, np.float32)), np.float16),
            oracle.softmax(s),
            oracle.softmax(oracle.binary("add", s, np.ascontiguousarray(np.broadcast_to(mask, s.shape)))),
            oracle.binary("mul", np.ascontiguousarray(gate_up[:, 8192:]),
                          oracle.cast(oracle.unary("silu", oracle.cast(np.ascontiguousarray(gate_up[:, :8192]), np.float32)), np.float16))]
    for _ in range(3):
        for o in outputs:
            o.zero_()
        dev.sync()
        cap.launch()
        dev.sync()
        for name, o, w in zip(("gelu", "silu via f32", "softmax", "masked softmax", "gated multiply"), outputs, want):
            assert same_bits(o.to_numpy(), w), name
    sequence()                                                 # eager: the tables are built now
    for name, o, w in zip(("gelu", "silu via f32", "softmax", "masked softmax", "gated multiply"), outputs, want):
        assert same_bits(o.to_numpy(), w), name + " (eager, table kernels)"
