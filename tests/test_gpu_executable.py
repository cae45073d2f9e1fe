"""GPU tests of the host mirror's Executable: a graph compiled once (buffers from the memory plan, launches recorded into a
HIP graph) and replayed with new input data must give, on every replay, the bits a fresh resolve() of the same graph
gives (the role of Executable::dispatch, executable.rs:33-59, under resolve_gpu, tensor.rs:795-859).  Replays are
interleaved with eager work and synchronisations, and every replay is checked.
"""
import numpy as np
import pytest

from gpu_util import same_bits
from ratchet_amd._lib import F16, F32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hdev():
    from ratchet_amd.host import HostDevice

    d = HostDevice(0)
    yield d
    d.close()


def T(a, dev):
    from ratchet_amd.host import Tensor

    return Tensor.from_numpy(a, dev)


@pytest.mark.parametrize("tail", [False, True], ids=["call_by_call", "hip_graph"])
def test_compiled_graph_replays_with_new_inputs(hdev, oracle, tail):
    # bias add (broadcast absorbed) -> tanh GELU (in place in the add's buffer) -> LayerNorm, f32; with `tail` five more
    # launches, which makes the list long enough to be recorded into a HIP graph (shorter lists are re-issued call by call)
    rng = np.random.default_rng(900)
    x = rng.standard_normal((1, 1500, 384)).astype(np.float32)
    bias = (0.02 * rng.standard_normal(384)).astype(np.float32)
    g = (1 + 0.02 * rng.standard_normal(384)).astype(np.float32)
    b = (0.02 * rng.standard_normal(384)).astype(np.float32)
    tx, tb, tg, tbb = T(x, hdev), T(bias, hdev), T(g, hdev), T(b, hdev)
    graph = lambda a, c: (lambda t: t.neg().exp().sqrt().neg().abs() if tail else t)(a.add(c).gelu().layer_norm(tg, tbb, 1e-5))
    y = graph(tx, tb)
    exe = y.compile()
    assert exe.launches == (8 if tail else 3) and y.last_resolve_launches() == exe.launches
    eager = graph(T(x, hdev), T(bias, hdev)).resolve().to_numpy()
    assert same_bits(y.to_numpy(), eager)                            # compile() leaves the tensor resolved
    for k in range(4):
        x2 = rng.standard_normal(x.shape).astype(np.float32)
        bias2 = (0.02 * rng.standard_normal(384)).astype(np.float32)
        tx.update(x2)
        tb.update(bias2)
        exe.dispatch()
        got = y.to_numpy()
        # the program's own eager work between the replays
        want = graph(T(x2, hdev), T(bias2, hdev)).resolve().to_numpy()
        assert same_bits(got, want), k
        assert same_bits(tx.to_numpy(), x2)                          # nothing ran in place in an input
    exe.close()


def test_compiled_attention_tail_and_swiglu_keep_the_one_launch_patterns(hdev, oracle):
    from ratchet_amd import _lib

    rng = np.random.default_rng(901)
    S, H = 256, 4
    mask = np.triu(np.full((S, S), -np.inf, np.float32), k=1).astype(np.float16)
    scores = (2 * rng.standard_normal((1, H, S, S))).astype(np.float16)
    gate = rng.standard_normal((1, 64, 1024)).astype(np.float16)
    up = rng.standard_normal((1, 64, 1024)).astype(np.float16)
    ts, tm, tgate, tup = T(scores, hdev), T(mask, hdev), T(gate, hdev), T(up, hdev)
    probs = ts.add(tm).full().softmax(3).cast(_lib.F16)
    act = tup.mul(tgate.full().silu().cast(_lib.F16))
    pe, ae = probs.compile(), act.compile()
    assert pe.launches == 1 and ae.launches == 1

    def eager(s, g_, u):
        p = T(s, hdev).add(T(mask, hdev)).full().softmax(3).cast(_lib.F16).resolve().to_numpy()
        a = T(u, hdev).mul(T(g_, hdev).full().silu().cast(_lib.F16)).resolve().to_numpy()
        return p, a

    for k in range(3):
        s2 = (2 * rng.standard_normal(scores.shape)).astype(np.float16)
        g2 = rng.standard_normal(gate.shape).astype(np.float16)
        u2 = rng.standard_normal(up.shape).astype(np.float16)
        ts.update(s2)
        tgate.update(g2)
        tup.update(u2)
        pe.dispatch(wait=False)
        ae.dispatch()
        wp, wa = eager(s2, g2, u2)
        assert same_bits(probs.to_numpy(), wp), k
        assert same_bits(act.to_numpy(), wa), k
    want = oracle.binary("mul", u2, oracle.cast(oracle.unary("silu", oracle.cast(g2, np.float32)), np.float16))
    assert same_bits(act.to_numpy(), want)


def test_replays_do_not_compound_in_place_ops(hdev, oracle):
    rng = np.random.default_rng(902)
    x = rng.standard_normal((8, 512)).astype(np.float32)
    # the only handle on the constant is the graph's edge: resolve() would run gelu in place in its buffer, a replayed
    # launch list must not
    y = T(x, hdev).gelu().tanh()
    exe = y.compile()
    assert exe.launches == 2
    want = oracle.unary("tanh", oracle.unary("gelu", x))
    for _ in range(3):
        exe.dispatch()
        assert same_bits(y.to_numpy(), want)
    # index_write updates its destination (that is its meaning); an op behind it must not work in the destination
    dst = np.zeros((4, 64), np.float32)
    src = rng.standard_normal((2, 64)).astype(np.float32)
    td, ts = T(dst, hdev), T(src, hdev)
    z = td.index_write(ts, (1, 0)).neg()
    ze = z.compile()
    ref = dst.copy()
    ref[1:3] = src
    for _ in range(3):
        ze.dispatch()
        assert same_bits(z.to_numpy(), -ref)
        assert same_bits(td.to_numpy(), ref)
    src2 = rng.standard_normal((2, 64)).astype(np.float32)
    ts.update(src2)
    ze.dispatch()
    ref[1:3] = src2
    assert same_bits(z.to_numpy(), -ref) and same_bits(td.to_numpy(), ref)


def test_compiled_cache_append_and_reindex_chain(hdev, oracle):
    from ratchet_amd import _lib

    rng = np.random.default_rng(903)
    cache_np = rng.standard_normal((1, 4, 24, 80)).astype(np.float16)
    new = rng.standard_normal((1, 4, 3, 80)).astype(np.float16)
    cache, tnew = T(cache_np, hdev), T(new, hdev)
    # the appended cache, heads merged: cache -> permute -> view -> f32
    y = cache.cache(tnew, 2, 5).permute((0, 2, 1, 3)).view((1, 8, 1, 320)).cast(_lib.F32)
    exe = y.compile()
    for k in range(3):
        new2 = rng.standard_normal(new.shape).astype(np.float16)
        tnew.update(new2)
        exe.dispatch()
        cat = np.concatenate([cache_np[:, :, :5], new2], axis=2)
        want = np.ascontiguousarray(cat.transpose(0, 2, 1, 3)).reshape(1, 8, 1, 320).astype(np.float32)
        assert same_bits(y.to_numpy(), want), k
        assert same_bits(cache.to_numpy()[:, :, 5:8], new2) and same_bits(cache.to_numpy()[:, :, 8:], cache_np[:, :, 8:])


def test_dispatch_allocates_nothing_and_holds_what_the_plan_says(hdev):
    from ratchet_amd import _lib

    rng = np.random.default_rng(904)
    x = rng.standard_normal((64, 1024)).astype(np.float16)
    tx = T(x, hdev)
    a = tx.full().sin()                                              # f32, in place chain
    y = a.cast(_lib.F16).add(tx).full().cos().cast(_lib.F16)
    objs, entries = y.memory_plan()
    exe = y.compile()
    # the plan compile() follows differs from resolve()'s only where an input buffer would be reused: not the case here
    # (an op that runs in place is listed with its source's allocation: counted once, at the source)
    own = sum(e["bytes"] for e in entries if e["object"] == -1 and e["source"] == e["id"])
    assert exe.held_bytes == sum(objs) + own
    before = hdev.pool_stats()
    for _ in range(5):
        exe.dispatch()
    after = hdev.pool_stats()
    assert after == before                                           # no request reached the pool, let alone the driver
    want = np.cos((np.sin(x.astype(np.float32)).astype(np.float16) + x).astype(np.float32)).astype(np.float16)
    got = y.to_numpy()
    assert np.max(np.abs(got.astype(np.float32) - want.astype(np.float32))) <= 2e-3
    # a tensor that has its storage already (here a view of an uploaded one; y above as well) has nothing left to record
    from ratchet_amd.host import HostError

    for done in (tx.view((1024, 64)), y):
        with pytest.raises(HostError) as e:
            done.compile()
        assert e.value.kind == "AlreadyResolved"


def test_a_view_the_caller_keeps_still_shows_its_data_after_later_launches_reused_buffers(hdev, oracle):
    # exp(x) is only held by a view; the casts behind the view are the tenants that a shared object would go to next
    rng = np.random.default_rng(905)
    x = rng.standard_normal((64, 1024)).astype(np.float32)
    want_view = oracle.unary("exp", x)
    for mode in ("resolve", "compile"):
        a = T(x, hdev).exp()
        v = a.view((64, 1024))
        del a
        e = v.cast(F16).cast(F32).cast(F16).cast(F32).neg()
        exe = None
        if mode == "resolve":
            e.resolve()
        else:
            exe = e.compile()
            exe.dispatch()
        assert same_bits(v.to_numpy(), want_view), mode
        # a second graph built on the kept view reads exp(x), not the last tenant's data
        got = v.neg().resolve().to_numpy()
        assert same_bits(got, oracle.unary("neg", want_view)), mode
        want = oracle.unary("neg", oracle.cast(oracle.cast(oracle.cast(oracle.cast(want_view, np.float16), np.float32), np.float16), np.float32))
        assert same_bits(e.to_numpy(), want), mode
        if exe:
            exe.close()
