"""The activation memory plan of the host mirror's resolve(): BufferAllocator::greedy_by_size with in-place leasing
(crates/ratchet-core/src/gpu/buffer_allocator/allocator.rs:141-271), checked on placeholder graphs (CPU only) against
assignments worked out by hand and against a Python restatement of the reference's three functions on random graphs;
on the GPU, the bytes a resolve really holds at its peak are checked against the plan.
"""
import numpy as np
import pytest

from ratchet_amd import _lib
from ratchet_amd.host import Tensor

F32, F16 = _lib.F32, _lib.F16
KB = 1024


def P(n, dt=F32):
    return Tensor.placeholder((n,), dt)


def test_cast_chain_alternates_between_two_objects():
    """x -> a(4 KB) -> b(2 KB) -> c(4 KB) -> d(2 KB) -> e: a lives over launches [0,1], b [1,2], c [2,3], d [3,4].
    Largest first: a opens object 0; c does not overlap a and joins it; b overlaps a (they touch at launch 1) and opens
    object 1; d overlaps c but not b and joins object 1.  8 KB + 4 KB of intermediates fit in 4 KB + 2 KB."""
    x = P(1024)
    e = x.exp().cast(F16).cast(F32).cast(F16).cast(F32)
    objects, entries = e.memory_plan()
    assert objects == [4 * KB, 2 * KB]
    assert [t["object"] for t in entries] == [0, 1, 0, 1, -1]         # the resolved tensor has an allocation of its own
    assert [t["bytes"] for t in entries] == [4 * KB, 2 * KB, 4 * KB, 2 * KB, 4 * KB]


def test_in_place_chain_is_one_allocation_leased_from_its_first_tensor():
    """determine_tensor_source (allocator.rs:141-162): gelu runs in place in the cast's buffer, so both report the cast
    as their source and share its object; neg and add run in place down to the second cast, and because the result of
    the resolve ends that chain the whole chain has an allocation of its own"""
    x = P(1024)
    y = x.exp().cast(F16).gelu().cast(F32).neg().add(x)
    objects, entries = y.memory_plan()
    ids = [t["id"] for t in entries]
    assert objects == [4 * KB, 2 * KB]
    assert [t["object"] for t in entries] == [0, 1, 1, -1, -1, -1]
    assert [t["source"] for t in entries] == [ids[0], ids[1], ids[1], ids[3], ids[3], ids[3]]


def test_first_op_may_run_in_place_in_a_constant_nobody_else_holds():
    """'inplace may be performed on constants' (allocator.rs:206): exp works in the uploaded buffer when the caller has
    dropped its handle, and needs no allocation at all"""
    e = P(1024).exp().cast(F16)
    objects, entries = e.memory_plan()
    assert objects == [] and [t["object"] for t in entries] == [-2, -1]
    x = P(1024)
    e = x.exp().cast(F16)                                              # x still held: exp gets a buffer
    objects, entries = e.memory_plan()
    assert objects == [4 * KB] and [t["object"] for t in entries] == [0, -1]


def test_a_tensor_the_caller_still_holds_is_never_shared():
    x = P(1024)
    kept = x.exp().cast(F16)                                           # visible outside the graph
    e = kept.cast(F32).cast(F16).cast(F32)
    objects, entries = e.memory_plan()
    by_id = {t["id"]: t for t in entries}
    assert by_id[kept.id]["object"] == -1
    assert sorted(objects) == [2 * KB, 4 * KB]


def test_a_kept_view_pins_the_tensor_it_aliases():
    """a view shares its source's buffer: while the caller holds the view, the source must not be housed in an object
    that later launches reuse, although every holder of the source itself is an edge of the graph"""
    x = P(1024)
    a = x.exp()
    v = a.view((1024,))
    aid = a.id
    del a
    e = v.cast(F16).cast(F32).cast(F16).cast(F32)
    objects, entries = e.memory_plan()
    by_id = {t["id"]: t for t in entries}
    assert by_id[aid]["object"] == -1                                  # own allocation: v keeps showing exp(x)
    # dropped, the same view hides nothing: exp's buffer joins the shared objects again
    x = P(1024)
    a = x.exp()
    aid = a.id
    e = a.view((1024,)).cast(F16).cast(F32).cast(F16).cast(F32)
    del a
    objects, entries = e.memory_plan()
    assert {t["id"]: t for t in entries}[aid]["object"] >= 0


def test_a_view_read_by_a_second_unresolved_graph_pins_its_source():
    x = P(1024)
    a = x.exp()
    v = a.view((1024,))
    aid = a.id
    del a
    other = v.neg()                                                    # a second graph, not resolved yet, reads the view
    e = v.cast(F16).cast(F32).cast(F16).cast(F32)
    objects, entries = e.memory_plan()
    assert {t["id"]: t for t in entries}[aid]["object"] == -1
    # a view of a view: the chain is followed down to the buffer's owner
    x = P(1024)
    a = x.exp()
    aid = a.id
    vv = a.view((1024,)).view((1024,))
    del a
    e = vv.cast(F16).cast(F32).cast(F16).cast(F32)
    objects, entries = e.memory_plan()
    assert {t["id"]: t for t in entries}[aid]["object"] == -1
    del other


def test_the_root_being_a_view_pins_its_source():
    x = P(1024)
    a = x.exp().cast(F16).cast(F32)
    aid = a.id
    root = a.view((1024,))
    del a
    objects, entries = root.memory_plan()
    assert {t["id"]: t for t in entries}[aid]["object"] == -1


def test_diamond_keeps_the_shared_operand_alive_to_its_last_reader():
    """a feeds both branches: its interval runs to the add at the end, so nothing else may use its object"""
    x = P(2048)
    a = x.exp()
    left = a.cast(F16).cast(F32)
    right = a.sin().cos()           # sin cannot run in place (a has two consumers); cos runs in place in sin's buffer
    out = left.add(right).cast(F16)
    aid = a.id
    del a, left, right
    objects, entries = out.memory_plan()
    by_obj = {}
    for t in entries:
        by_obj.setdefault(t["object"], []).append(t["id"])
    a_obj = [t for t in entries if t["id"] == aid][0]["object"]
    assert a_obj >= 0 and by_obj[a_obj] == [aid]
    # launches: a 0, cast16 1, cast32 2, sin 3, cos 4, add 5, out 6.  Intervals: a [0,3], cast16 [1,2], cast32 (+ add, in place)
    # [2,6], sin (+ cos, in place) [3,5].  Largest first: a -> object 0; cast32 overlaps a -> object 1; sin overlaps both
    # (it touches a at launch 3) -> object 2; the 4 KB cast16 overlaps a and cast32 (touching at 2) but not sin: it is
    # housed in sin's 8 KB object.
    assert objects == [8 * KB, 8 * KB, 8 * KB]
    assert [t["object"] for t in entries] == [0, 2, 1, 2, 2, 1, -1]


# ---- the reference's algorithm restated in Python from allocator.rs:141-271, for random graphs -------------------------------------

def reference_plan(steps):
    """steps: dicts id / bytes / reads / inplace (index into reads or None) / pinned, in execution order"""
    by_id = {s["id"]: s for s in steps}

    def true_source(i):                                                # determine_tensor_source
        while i in by_id and by_id[i]["inplace"] is not None:
            i = by_id[i]["reads"][by_id[i]["inplace"]]
        return i

    pinned_chains = {true_source(s["id"]) for s in steps if s["pinned"]}
    records = {}                                                       # calculate_usage_records
    for k in range(len(steps) - 1, -1, -1):
        for r in steps[k]["reads"]:
            ts = true_source(r)
            if ts in by_id and ts not in records:
                records[ts] = dict(id=ts, last=k, bytes=by_id[ts]["bytes"], producer=None)
        if steps[k]["id"] in records:
            records[steps[k]["id"]]["producer"] = k
    order = [records[s["id"]] for s in steps if s["id"] in records and s["id"] not in pinned_chains]
    order.sort(key=lambda r: -r["bytes"])                              # stable: ties stay in execution order
    objects, placed = [], []
    for rec in order:                                                  # greedy_by_size
        best = None
        for obj in range(len(objects)):
            if all(not (o["object"] == obj and max(rec["producer"], o["producer"]) <= min(rec["last"], o["last"])) for o in placed):
                best = obj
        if best is None:
            best = len(objects)
            objects.append(rec["bytes"])
        rec["object"] = best
        placed.append(rec)
    obj_of = {r["id"]: r["object"] for r in placed}
    out = {}
    for s in steps:
        ts = true_source(s["id"])
        out[s["id"]] = -2 if ts not in by_id else obj_of.get(ts, -1)
    return objects, out


@pytest.mark.parametrize("seed", range(40))
def test_random_graphs_match_the_python_restatement(seed):
    rng = np.random.default_rng(seed)
    n_elem = 256
    consts = [P(n_elem, F32), P(n_elem, F16)]
    nodes = [dict(t=c, dt=dt, const=True) for c, dt in zip(consts, (F32, F16))]
    made = []
    for _ in range(int(rng.integers(6, 22))):
        kind = rng.choice(["unary", "binary", "cast"])
        a = nodes[int(rng.integers(0, len(nodes)))]
        if kind == "unary":
            node = dict(t=getattr(a["t"], str(rng.choice(["exp", "sin", "neg", "abs"])))(), dt=a["dt"], srcs=[a], inplace_ok=True)
        elif kind == "cast":
            dt = F16 if a["dt"] == F32 else F32
            node = dict(t=a["t"].cast(dt), dt=dt, srcs=[a], inplace_ok=False)
        else:
            same = [m for m in nodes if m["dt"] == a["dt"]]
            b = same[int(rng.integers(0, len(same)))]
            node = dict(t=a["t"].add(b["t"]), dt=a["dt"], srcs=[a, b], inplace_ok=True)
        node["const"] = False
        node["id"] = node["t"].id
        nodes.append(node)
        made.append(node)
    root = made[-1]
    order = root["t"].execution_order()
    for m in made:                                                     # drop every handle but the root's
        if m is not root:
            m["t"] = None
    needed = [m for i in order for m in made if m["id"] == i]
    consumers = {}
    for m in needed:
        for s in m["srcs"]:
            consumers[id(s)] = consumers.get(id(s), 0) + 1
    steps = []
    for m in needed:
        reads = []
        for s in m["srcs"]:
            sid = s.get("id", -1 - nodes.index(s))                     # constants: ids the plan never produces
            if sid not in reads:
                reads.append(sid)
        s0 = m["srcs"][0]
        # tensor.rs:823-824: supports_inplace && strong_count(srcs[0]) == 1; the constants stay held by this test
        inplace = 0 if (m["inplace_ok"] and not s0["const"] and consumers[id(s0)] == 1 and s0["dt"] == m["dt"]) else None
        steps.append(dict(id=m["id"], bytes=n_elem * (4 if m["dt"] == F32 else 2), reads=reads, inplace=inplace, pinned=m is root))
    want_objects, want_of = reference_plan(steps)
    objects, entries = root["t"].memory_plan()
    assert [t["id"] for t in entries] == [s["id"] for s in steps]
    assert objects == want_objects
    assert {t["id"]: t["object"] for t in entries} == want_of
    # the point of the plan: it never needs more than one buffer per intermediate, and on chains far less
    assert sum(objects) <= sum(s["bytes"] for s in steps if not s["pinned"])


@pytest.mark.gpu
def test_resolve_holds_no_more_than_the_plan_at_its_peak():
    """a long chain of casts and in-place unaries on the device: what the pool hands out at the peak of the resolve is the
    inputs, the result and the plan's shared objects, not one buffer per intermediate, and the values are right"""
    from ratchet_amd import host
    from ratchet_amd.host import HostDevice

    host.set_pattern_fusion(False)                                      # cast -> op -> cast would otherwise become one 16-bit launch
    dev = HostDevice(0)
    n = 1 << 20
    x_host = np.linspace(-2, 2, n, dtype=np.float32)
    x = Tensor.from_numpy(x_host, dev)
    t = x
    for k in range(6):
        t = t.cast(F16).neg().cast(F32).abs()
    objects, entries = t.memory_plan()
    assert objects == [4 * n, 2 * n]                                    # 24 launches, 12 allocations' worth of tensors, two objects
    live_before = dev.pool_stats()[0]
    dev.pool_peak(reset=True)
    got = t.resolve().to_numpy()
    peak = dev.pool_peak()
    assert peak - live_before <= sum(objects) + 4 * n + 4096            # + the result's own allocation (pool rounding aside)
    host.set_pattern_fusion(True)
    assert np.array_equal(got, np.abs(x_host.astype(np.float16).astype(np.float32)))
