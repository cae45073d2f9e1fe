"""Random lazy graphs through the host mirror of ratchet's Tensor API: ten or twenty random ops (broadcast binaries, unaries, casts,
softmax, permutes, slices, RMSNorm) over three random constants, then
  * resolve() with the caller-pattern fusion off against the CPU oracle's evaluation of the same graph, op by op;
  * resolve() with the fusion on against the unfused result (the one-launch patterns compute in f32 where the op
    sequence rounds to f16 in between: the 16-bit bar of 1e-3, widened for chains of several ops);
  * compile() + two dispatches against the fused resolve(), bit for bit (the Executable replays the same launches).
Earlier nodes stay visible through Python handles, so the in-place rule, the memory plan's pinning and the partial
re-resolve of a graph whose inner nodes are resolved already are all exercised.  Seeds are fixed."""
import numpy as np
import pytest

from gpu_util import same_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hdev():
    from ratchet_amd.host import HostDevice

    d = HostDevice(0)
    yield d
    d.close()

UN = ["tanh", "relu", "neg", "abs", "sigmoid", "silu", "gelu"]


def build(rng, hdev, leaves_np, nops, trace, chain=0.0):
    """the graph's tensors and, for each, the oracle's value; ops the API rejects (shape or dtype rules) are skipped"""
    from ratchet_amd.host import Tensor
    nodes = [Tensor.from_numpy(a, hdev) for a in leaves_np]
    vals = list(leaves_np)
    for _ in range(nops):
        k = int(rng.integers(0, 7))
        i = len(nodes) - 1 if rng.random() < chain else int(rng.integers(0, len(nodes)))   # chain: extend the newest node
        a, av = nodes[i], vals[i]
        try:
            if k == 0:
                j = int(rng.integers(0, len(nodes)))
                b, bv = nodes[j], vals[j]
                if bv.dtype != av.dtype:
                    continue
                try:
                    osh = np.broadcast_shapes(av.shape, bv.shape)
                except ValueError:
                    continue
                op = ("add", "sub", "mul")[int(rng.integers(0, 3))]
                t = getattr(a, op)(b)
                v = ("binary", op, i, j)
            elif k == 1:
                op = UN[int(rng.integers(0, len(UN)))]
                t = a.unary(op)
                v = ("unary", op, i)
            elif k == 2:
                to = np.float32 if av.dtype == np.float16 else np.float16
                t = a.full() if to == np.float32 else a.half()
                v = ("cast", to, i)
            elif k == 3:
                t = a.softmax(av.ndim - 1)
                v = ("softmax", i)
            elif k == 4:
                perm = [int(p) for p in rng.permutation(av.ndim)]
                t = a.permute(perm)
                v = ("permute", perm, i)
            elif k == 5:
                r = []
                for s in av.shape:
                    lo = int(rng.integers(0, s))
                    r.append((lo, int(rng.integers(lo + 1, s + 1))))
                t = a.slice(r)
                v = ("slice", r, i)
            else:
                cols = av.shape[-1]
                w = rng.standard_normal(cols).astype(av.dtype)
                t = a.rms_norm(Tensor.from_numpy(w, hdev), 1e-5)
                v = ("rms", w, i)
        except Exception as e:
            trace.append(("rejected", k, str(e)[:60]))
            continue
        nodes.append(t)
        trace.append(v)
        vals.append(evaluate(v, vals))
    return nodes, vals


def evaluate(v, vals):
    from oracle import cpu_oracle as oracle
    kind = v[0]
    if kind == "binary":
        a, b = vals[v[2]], vals[v[3]]
        osh = np.broadcast_shapes(a.shape, b.shape)
        return oracle.binary(v[1], np.ascontiguousarray(np.broadcast_to(a, osh)), np.ascontiguousarray(np.broadcast_to(b, osh)))
    if kind == "unary":
        return oracle.unary(v[1], np.ascontiguousarray(vals[v[2]]))
    if kind == "cast":
        return oracle.cast(np.ascontiguousarray(vals[v[2]]), v[1])
    if kind == "softmax":
        return oracle.softmax(np.ascontiguousarray(vals[v[1]]))
    if kind == "permute":
        return np.ascontiguousarray(vals[v[2]].transpose(v[1]))
    if kind == "slice":
        return np.ascontiguousarray(vals[v[2]][tuple(slice(a, b) for a, b in v[1])])
    if kind == "rms":
        return oracle.rms_norm(np.ascontiguousarray(vals[v[2]]), v[1], 1e-5, intended=True)
    raise AssertionError(kind)

@pytest.mark.parametrize("seed", range(80))
def test_random_graph(hdev, oracle, seed):
    from ratchet_amd.host import set_pattern_fusion

    rng = np.random.default_rng(9000 + seed)
    rank = int(rng.integers(2, 5))
    shape = tuple(int(rng.choice([1, 2, 3, 4, 8, 16, 24, 64])) for _ in range(rank))
    leaves = []
    for _ in range(3):
        dt = (np.float32, np.float16)[int(rng.integers(0, 2))]
        sh = tuple(s if rng.random() < 0.8 else 1 for s in shape)
        leaves.append(rng.standard_normal(sh).astype(dt))
    results = {}
    max_launches = [0]
    for mode in ("unfused", "fused", "compiled"):
        set_pattern_fusion(mode != "unfused")
        try:
            r2 = np.random.default_rng(9500 + seed)
            trace = []
            # every other seed: longer and mostly a chain, which reaches the launch counts that are recorded into a HIP graph
            nodes, vals = build(r2, hdev, leaves, 10 if seed % 2 else 20, trace, 0.0 if seed % 2 else 0.7)
            # the last node first, then two random earlier ones: handles on earlier nodes stay alive (visible intermediates)
            order = [len(nodes) - 1] + [int(i) for i in r2.integers(3, len(nodes), size=2)] if len(nodes) > 3 else []
            outs = []
            for i in order:
                if mode == "compiled" and nodes[i].resolved():
                    outs.append((i, nodes[i].to_numpy()))            # resolved on the way as a visible intermediate of an earlier one
                elif mode == "compiled":
                    exe = nodes[i].compile()
                    max_launches[0] = max(max_launches[0], exe.launches)
                    first = nodes[i].to_numpy()
                    exe.dispatch()
                    exe.dispatch()
                    assert same_bits(nodes[i].to_numpy(), first), ("replay differs from the first run", seed, i, trace)
                    outs.append((i, first))
                    exe.close()
                else:
                    outs.append((i, nodes[i].resolve().to_numpy()))
            results[mode] = (outs, vals, trace)
        finally:
            set_pattern_fusion(True)
    (o0, vals, trace), (o1, _, _), (o2, _, _) = results["unfused"], results["fused"], results["compiled"]
    for (i, g0), (j, g1), (k, g2) in zip(o0, o1, o2):
        assert i == j == k
        want = vals[i]
        assert g0.shape == want.shape == g1.shape == g2.shape, (seed, i, trace)
        tol = 3e-3 if want.dtype == np.float16 else 2e-4
        bad, mx = oracle.count_not_close(np.ascontiguousarray(g0), np.ascontiguousarray(want), tol, tol)
        assert bad == 0, ("unfused vs oracle", seed, i, mx, trace)
        bad, mx = oracle.count_not_close(np.ascontiguousarray(g1), np.ascontiguousarray(g0), tol, tol)
        assert bad == 0, ("fused vs unfused", seed, i, mx, trace)
        assert same_bits(g2, g1), ("compiled vs resolved", seed, i, trace)
    print("seed", seed, "longest compiled launch list", max_launches[0])
