#!/usr/bin/env python3
"""Benchmark of the MI355X backend for ratchet-core's memory-bound tensor ops.

A "step" is one pass over every op of BASELINE configs[1..4] (Whisper-tiny attention softmax + reindex, the Phi-2 and
Phi-3 prefill elementwise blocks, the broadcast/reindex stress set), each op launched once through the C ABI on the
device's single stream with its inputs already resident in HBM.  A step moves about 5.6 GB, far more than the 256 MB
Infinity Cache, and every op has its own buffers, so each op sees cache-cold inputs on every step.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--ops REGEX] [--no-cpu] [--no-check]

Prints ONE JSON line: whole-step throughput (algorithmic bytes / time over `steps` back-to-back steps between two
synchronisations), per-op microseconds / GB/s / fraction of the 8 TB/s HBM roofline (a separate pass with HIP events around
each launch), the roofline object for the dominant kernel (HIP events around it inside the timed steps) and the CPU baseline
(the C++ restatement of ratchet's CPU executor on one host core, on the same workload).
"""
import argparse
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBPS = 8000.0
# rocprofv3 summaries of this same script (bench.py cannot run the profiler on itself): per launch of the step, in step
# order, the kernel's own duration from a --kernel-trace run and the HBM-side bytes from two --pmc runs (FETCH_SIZE,
# WRITE_SIZE).  Read at run time; a missing file or row gives null, never a stale literal.
PROFILE_KERNEL_TRACE = os.path.join("profiles", "bench_step_kernel_trace.txt")
PROFILE_HBM_TRAFFIC = os.path.join("profiles", "bench_step_hbm_traffic_pmc.txt")
# algorithmic bytes of the 17 ops of the step, in step order (what build_workload's rows carry; checked against them in main)
STEP_ALG_BYTES = [108000000, 4608000, 4608000, 31457280, 20981760, 83886080, 31457280, 31457280, 50337792, 134217728, 201326592,
                  2181038080, 2147483648, 20971520, 6146048, 268570624, 20971520]


def read_step_rows(rel_path):
    """{position in the step (1-based): fields after the position} of the `step_op` lines of a profile summary."""
    rows = {}
    try:
        with open(os.path.join(ROOT, rel_path)) as f:
            for line in f:
                if line.startswith("step_op"):
                    fields = [x.strip() for x in line[len("step_op"):].split("|")]
                    rows[int(fields[0])] = fields[1:]
    except (OSError, ValueError):
        return {}
    return rows


def profile_head(rel_path):
    """the `git_head:` line of a profile summary: the commit whose kernels it describes"""
    try:
        with open(os.path.join(ROOT, rel_path)) as f:
            for line in f:
                if line.startswith("git_head:"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return None


def library_built_from():
    """the commit the loaded library was linked from, as the build recorded it beside the objects"""
    from ratchet_amd import build as hip_build

    return hip_build.built_from()


def git_head():
    """commit of the tree this script runs from, when it is a git checkout (the GPU box receives the tree without .git)"""
    try:
        head = open(os.path.join(ROOT, ".git", "HEAD")).read().strip()
        if head.startswith("ref:"):
            return open(os.path.join(ROOT, ".git", head.split(" ", 1)[1])).read().strip()[:12]
        return head[:12]
    except OSError:
        return None


F32, F16 = 0, 1


def stream_rng(seed, stream):
    """One documented counter-based generator: Philox keyed by RATCHET_SEED, one counter block per tensor."""
    return np.random.Generator(np.random.Philox(key=seed, counter=[0, 0, 0, stream]))


def normal(seed, stream, shape, std, dtype, mean=0.0):
    """N(mean, std) sampled in f32, then rounded once to the storage dtype (as Tensor::randn does, tensor.rs:543-548)."""
    g = stream_rng(seed, stream)
    return (g.standard_normal(shape, dtype=np.float32) * np.float32(std) + np.float32(mean)).astype(dtype)


class Op:
    """One benchmark row: device buffers, a launch closure, algorithmic bytes, and a CPU check/baseline closure.
    `call(ins, out)` enqueues the op on the buffers it is given; `ins` / `out` are the buffers of the step (set 0).
    `rotating` lists which inputs get copies of their own in the sets of the event-free pass (the large operands; scale,
    bias and other small vectors are shared)."""

    def __init__(self, cfg, name, dtype, shapes, alg_bytes, call, ins, out, cpu_sample, kernel, rotating=None):
        self.cfg, self.name, self.dtype, self.shapes = cfg, name, dtype, shapes
        self.alg_bytes = int(alg_bytes)
        self.call, self.ins, self.out = call, list(ins), out
        self.rotating = list(range(len(ins))) if rotating is None else list(rotating)
        self.cpu_sample = cpu_sample        # dict: how to check the output buffer of set 0 and what to time on the CPU
        self.kernel = kernel                # substring of the kernel's name in a rocprofv3 trace
        self.us = []

    def launch(self):
        self.call(self.ins, self.out)


def build_workload(dev, seed):
    from ratchet_amd import _lib

    np16, np32 = np.float16, np.float32
    ops = []
    st = [100]

    def nxt():
        st[0] += 1
        return st[0]

    def up(a):
        return dev.upload(a)

    # ------------------------------------------------------------------ cfg 1: Whisper-tiny attention softmax + reindex
    scores1 = normal(seed, nxt(), (1, 6, 1500, 1500), 3.0, np32)
    d_scores1 = up(scores1)
    d_soft1 = dev.empty(scores1.shape, F32)
    ops.append(Op(1, "softmax", "f32", "[1,6,1500,1500]", 2 * scores1.nbytes, lambda i, o: dev.softmax(i[0], out=o), [d_scores1], d_soft1,
                  dict(kind="softmax", x=scores1, out=d_soft1, rows=9000, tol=1e-5), "softmax_wave_kernel"))
    q1 = normal(seed, nxt(), (1, 1500, 6, 64), 1.0, np32)
    d_q1 = up(q1)
    d_q1p = dev.empty((1, 6, 1500, 64), F32)
    d_q1b = dev.empty((1, 1500, 6, 64), F32)
    q1p = np.ascontiguousarray(q1.transpose(0, 2, 1, 3))
    ops.append(Op(1, "permute[0,2,1,3]", "f32", "[1,1500,6,64]->[1,6,1500,64]", 2 * q1.nbytes,
                  lambda i, o: dev.permute(i[0], (0, 2, 1, 3), out=o), [d_q1], d_q1p,
                  dict(kind="exact", out=d_q1p, run=lambda o: o.permute(q1, (0, 2, 1, 3)), bytes=2 * q1.nbytes), "gather_vec_kernel"))
    ops.append(Op(1, "permute back", "f32", "[1,6,1500,64]->[1,1500,6,64]", 2 * q1.nbytes,
                  lambda i, o: dev.permute(i[0], (0, 2, 1, 3), out=o), [d_q1p], d_q1b,
                  dict(kind="exact", out=d_q1b, run=lambda o: o.permute(q1p, (0, 2, 1, 3)), bytes=2 * q1.nbytes), "gather_vec_kernel"))

    # ------------------------------------------------------------------ cfg 2: Phi-2 prefill elementwise block, f16
    x2 = normal(seed, nxt(), (1, 2048, 2560), 1.0, np16)
    a2 = normal(seed, nxt(), (1, 2048, 2560), 0.5, np16)
    g2 = normal(seed, nxt(), (2560,), 0.02, np16, mean=1.0)
    b2 = normal(seed, nxt(), (2560,), 0.02, np16)
    h2 = normal(seed, nxt(), (1, 2048, 10240), 1.0, np16)
    d_x2, d_a2, d_g2, d_b2, d_h2 = up(x2), up(a2), up(g2), up(b2), up(h2)
    d_res2, d_ln2, d_gelu2 = dev.empty(x2.shape, F16), dev.empty(x2.shape, F16), dev.empty(h2.shape, F16)
    d_x2f32, d_x2f16 = dev.empty(x2.shape, F32), dev.empty(x2.shape, F16)
    x2_f32 = x2.astype(np32)
    ops.append(Op(2, "residual add", "f16", "[1,2048,2560]x2", 3 * x2.nbytes, lambda i, o: dev.binary("add", i[0], i[1], out=o), [d_x2, d_a2], d_res2,
                  dict(kind="exact", out=d_res2, run=lambda o: o.binary("add", x2, a2), bytes=3 * x2.nbytes), "binary_vec_kernel"))
    ops.append(Op(2, "layer_norm", "f16", "2048x2560", 2 * x2.nbytes + g2.nbytes + b2.nbytes,
                  lambda i, o: dev.layer_norm(i[0], i[1], i[2], 1e-5, out=o), [d_x2, d_g2, d_b2], d_ln2,
                  dict(kind="rows", out=d_ln2, x=x2, rows=2048, tol=1e-3, fn=lambda o, xs: o.layer_norm(xs, g2, b2, 1e-5, intended=True)),
                  "norm_pipe16_kernel", rotating=[0]))
    ops.append(Op(2, "gelu", "f16", "[1,2048,10240]", 2 * h2.nbytes, lambda i, o: dev.unary("gelu", i[0], out=o), [d_h2], d_gelu2,
                  dict(kind="rows", out=d_gelu2, x=h2, rows=2048, tol=1e-3, fn=lambda o, xs: o.unary("gelu", xs)), "unary_lut_kernel"))
    ops.append(Op(2, "cast f16->f32", "f16->f32", "[1,2048,2560]", x2.nbytes * 3, lambda i, o: dev.cast(i[0], F32, out=o), [d_x2], d_x2f32,
                  dict(kind="exact", out=d_x2f32, run=lambda o: o.cast(x2, np32), bytes=3 * x2.nbytes), "cast_vec_kernel"))
    ops.append(Op(2, "cast f32->f16", "f32->f16", "[1,2048,2560]", x2.nbytes * 3, lambda i, o: dev.cast(i[0], F16, out=o), [d_x2f32], d_x2f16,
                  dict(kind="exact", out=d_x2f16, run=lambda o: o.cast(x2_f32, np16), bytes=3 * x2.nbytes), "cast_vec_kernel"))

    # ------------------------------------------------------------------ cfg 3: Phi-3-mini prefill, f16
    x3 = normal(seed, nxt(), (1, 4096, 3072), 1.0, np16)
    g3 = normal(seed, nxt(), (3072,), 0.02, np16, mean=1.0)
    gate3 = normal(seed, nxt(), (1, 4096, 8192), 1.0, np16)
    up3 = normal(seed, nxt(), (1, 4096, 8192), 1.0, np16)
    d_x3, d_g3, d_gate3, d_up3 = up(x3), up(g3), up(gate3), up(up3)
    d_rms3, d_silu3, d_swiglu3 = dev.empty(x3.shape, F16), dev.empty(gate3.shape, F16), dev.empty(gate3.shape, F16)
    ops.append(Op(3, "rms_norm", "f16", "4096x3072", 2 * x3.nbytes + g3.nbytes, lambda i, o: dev.rms_norm(i[0], i[1], 1e-5, out=o), [d_x3, d_g3], d_rms3,
                  dict(kind="rows", out=d_rms3, x=x3, rows=4096, tol=1e-3, fn=lambda o, xs: o.rms_norm(xs, g3, 1e-5, intended=True)),
                  "rms16_par_kernel", rotating=[0]))
    ops.append(Op(3, "silu(gate)", "f16", "[1,4096,8192]", 2 * gate3.nbytes, lambda i, o: dev.unary("silu", i[0], out=o), [d_gate3], d_silu3,
                  dict(kind="rows", out=d_silu3, x=gate3, rows=4096, tol=1e-3, fn=lambda o, xs: o.unary("silu", xs)), "unary_lut_kernel"))
    ops.append(Op(3, "mul silu(gate)*up", "f16", "[1,4096,8192]x2", 3 * gate3.nbytes, lambda i, o: dev.binary("mul", i[0], i[1], out=o),
                  [d_up3, d_silu3], d_swiglu3,
                  dict(kind="rows2", out=d_swiglu3, rows=4096,
                       prep=lambda o, n: (up3.reshape(4096, 8192)[:n], o.unary("silu", gate3.reshape(4096, 8192)[:n])),
                       fn=lambda o, inp: o.binary("mul", inp[0], inp[1]),
                       tol=0.0, bytes_per_row=3 * 8192 * 2), "binary_vec_kernel"))
    # scores [1,32,4096,4096]: one head of N(0,2) generated on the host, replicated over the 32 heads on the device
    S, H = 4096, 32
    head = normal(seed, nxt(), (S, S), 2.0, np16)
    mask = np.triu(np.full((S, S), -np.inf, np16), k=1)                      # -inf above the diagonal, 0 elsewhere
    d_head, d_mask = up(head), up(mask)
    d_scores3 = dev.empty((1, H, S, S), F16)
    for h in range(H):
        _lib.check(dev.lib.rt_d2d(dev.handle, d_scores3.ptr.value + h * head.nbytes, d_head.ptr, head.nbytes))
    d_masked3 = dev.empty((1, H, S, S), F16)
    d_soft3 = dev.empty((1, H, S, S), F16)
    nb = H * head.nbytes
    ops.append(Op(3, "scores + causal mask (broadcast fused)", "f16", "[1,32,4096,4096]+[4096,4096]", 2 * nb + mask.nbytes,
                  lambda i, o: dev.binary("add", i[0], i[1], out=o), [d_scores3, d_mask], d_masked3,
                  dict(kind="rows2", out=d_masked3, rows=H * S, tol=0.0, bytes_per_row=2 * S * 2 + S * 2 / H,     # the mask counts once, as in the op's own bytes
                       prep=lambda o, n: (np.tile(head, (n // S, 1)), np.tile(mask, (n // S, 1))),
                       fn=lambda o, inp: o.binary("add", inp[0], inp[1])), "binary_bcast_kernel"))
    ops.append(Op(3, "softmax (causal)", "f16", "131072x4096", 2 * nb, lambda i, o: dev.softmax(i[0], out=o), [d_masked3], d_soft3,
                  dict(kind="rows2", out=d_soft3, rows=H * S, tol=0.0, bytes_per_row=2 * S * 2,
                       prep=lambda o, n: np.tile(o.binary("add", head, mask), (n // S, 1)),
                       fn=lambda o, inp: o.softmax(inp)), "softmax16_stream_kernel"))

    # ------------------------------------------------------------------ cfg 4: broadcast / reindex stress, f16
    kv_a = normal(seed, nxt(), (1, 32, 1984, 80), 1.0, np16)
    kv_b = normal(seed, nxt(), (1, 32, 64, 80), 1.0, np16)
    d_kva, d_kvb = up(kv_a), up(kv_b)
    d_kv = dev.empty((1, 32, 2048, 80), F16)
    ops.append(Op(4, "concat dim 2", "f16", "[1,32,1984,80]+[1,32,64,80]", 2 * (kv_a.nbytes + kv_b.nbytes),
                  lambda i, o: dev.concat([i[0], i[1]], 2, out=o), [d_kva, d_kvb], d_kv,
                  dict(kind="exact", out=d_kv, run=lambda o: o.concat([kv_a, kv_b], 2), bytes=2 * (kv_a.nbytes + kv_b.nbytes)), "concat_kernel"))
    gx = normal(seed, nxt(), (1, 512, 3000), 1.0, np16)
    gw = normal(seed, nxt(), (512,), 0.02, np16, mean=1.0)
    gb = normal(seed, nxt(), (512,), 0.02, np16)
    d_gx, d_gw, d_gb = up(gx), up(gw), up(gb)
    d_gn = dev.empty(gx.shape, F16)
    ops.append(Op(4, "group_norm G=32", "f16", "[1,512,3000]", 2 * gx.nbytes + gw.nbytes + gb.nbytes,
                  lambda i, o: dev.group_norm(i[0], 32, i[1], i[2], 1e-5, out=o), [d_gx, d_gw, d_gb], d_gn,
                  dict(kind="close", out=d_gn, tol=1e-3, run=lambda o: o.group_norm(gx, 32, gw, gb, 1e-5), bytes=2 * gx.nbytes),
                  "gn_reg_kernel", rotating=[0]))
    ma = normal(seed, nxt(), (1, 32, 2048, 1), 1.0, np16)
    mb = normal(seed, nxt(), (1, 1, 1, 2048), 1.0, np16)
    d_ma, d_mb = up(ma), up(mb)
    d_mm = dev.empty((1, 32, 2048, 2048), F16)
    ops.append(Op(4, "mul two-sided broadcast (fused)", "f16", "[1,32,2048,1]x[1,1,1,2048]", ma.nbytes + mb.nbytes + d_mm.nbytes,
                  lambda i, o: dev.binary("mul", i[0], i[1], out=o), [d_ma, d_mb], d_mm,
                  dict(kind="rows2", out=d_mm, rows=65536, tol=0.0, bytes_per_row=2048 * 2,
                       prep=lambda o, n: n,         # the reference's CPU path materialises both broadcasts: that stays inside the timed region
                       fn=lambda o, n: o.binary("mul", np.ascontiguousarray(np.broadcast_to(ma.reshape(-1, 1)[:n], (n, 2048))),
                                                np.ascontiguousarray(np.broadcast_to(mb.reshape(1, 2048), (n, 2048))))),
                  "binary_bcast_kernel"))
    p4 = normal(seed, nxt(), (1, 2048, 32, 80), 1.0, np16)
    d_p4 = up(p4)
    d_p4o = dev.empty((1, 32, 2048, 80), F16)
    ops.append(Op(4, "permute[0,2,1,3]", "f16", "[1,2048,32,80]->[1,32,2048,80]", 2 * p4.nbytes,
                  lambda i, o: dev.permute(i[0], (0, 2, 1, 3), out=o), [d_p4], d_p4o,
                  dict(kind="exact", out=d_p4o, run=lambda o: o.permute(p4, (0, 2, 1, 3)), bytes=2 * p4.nbytes), "gather_vec_kernel"))
    ops_extra["copy_pair"] = (d_scores3, d_masked3)
    ops_extra["attn"] = (d_scores3, d_mask, d_masked3, d_soft3)
    ops_extra["head"] = (head, mask)
    return ops


ops_extra = {}


def copy_ceiling(dev):
    """What a plain copy kernel reaches on this chip on a 1 GiB tensor (1 GiB read + 1 GiB written): the practical HBM
    ceiling for a streaming kernel, quoted beside the 8 TB/s peak."""
    from ratchet_amd import _lib

    src, dst = ops_extra["copy_pair"]
    e0, e1 = dev.event(), dev.event()
    times = []
    for i in range(4):
        e0.record()
        _lib.check(dev.lib.rt_cast(dev.handle, F16, F16, src.ptr, dst.ptr, src.numel))
        e1.record()
        t = e0.elapsed_ms(e1)
        if i:
            times.append(t)
    ms = float(np.mean(times))
    return {"kernel": "copy_vec_kernel", "bytes": 2 * src.nbytes, "us": round(ms * 1e3, 1), "GBps": round(2 * src.nbytes / ms / 1e6, 1),
            "frac_of_peak": round(2 * src.nbytes / ms / 1e6 / PEAK_HBM_GBPS, 4)}


def copy_reference(dev, ops, steps):
    """The floor under every row of the per-op table: the step once more, every op replaced by a plain copy kernel that
    moves the same number of bytes (half read, half written) through fresh regions of two 1 GiB buffers, timed exactly
    like the per-op pass (HIP events around each launch, the launches of a step back to back).  What a row's `us` exceeds
    its copy by is the op's own cost; what the copy itself falls short of the roofline by (a launch and the cache
    write-back and invalidation at a kernel boundary cost about 4 us whatever the kernel does) no kernel design recovers.
    Also times a 16-byte fill launched right after a large kernel: that boundary cost alone."""
    import ctypes

    from ratchet_amd import _lib

    src, dst = ops_extra["copy_pair"]
    ev = [(dev.event(), dev.event()) for _ in ops]
    floor_ev = (dev.event(), dev.event())
    us = [[] for _ in ops]
    floor_us = []
    tiny = dev.empty((4,), F32)
    off = 0
    for _ in range(steps):
        for o, (e0, e1) in zip(ops, ev):
            half = min((o.alg_bytes // 2) & ~15, src.nbytes)       # (the mask add moves 16 MB more per side than the buffers hold)
            if off + half > src.nbytes:
                off = 0
            assert off + half <= src.nbytes and off + half <= dst.nbytes
            e0.record()
            _lib.check(dev.lib.rt_cast(dev.handle, F16, F16, ctypes.c_void_p(src.ptr.value + off), ctypes.c_void_p(dst.ptr.value + off), half // 2))
            e1.record()
            off += half
        floor_ev[0].record()
        tiny.zero_()
        floor_ev[1].record()
        dev.sync()
        for k, (e0, e1) in enumerate(ev):
            us[k].append(e0.elapsed_ms(e1) * 1e3)
        floor_us.append(floor_ev[0].elapsed_ms(floor_ev[1]) * 1e3)
    return [float(np.median(u)) for u in us], float(np.median(floor_us))


def one_pass_patterns(dev, seed, oracle):
    """The models wrap 16-bit norms, softmax and activations in full() ... cast(dt); the library has one-pass entry points
    for those sequences.  Reported beside the step (never part of `value`): time of the one-pass launch and of the op
    sequence it replaces, both with HIP events on the device's stream, at the shapes of BASELINE configs 2 and 3."""
    from ratchet_amd.runtime import BufferView

    np16, np32 = np.float16, np.float32

    def timeit(fn, n=10):
        warm_up(dev, fn)
        e0, e1 = dev.event(), dev.event()
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        return e0.elapsed_ms(e1) / n * 1e3

    out = []

    def row(name, shape, alg_bytes, seq_bytes, launches, fused, seq, got, want, exact):
        us_f, us_s = timeit(fused), timeit(seq)
        ok = None
        if oracle is not None:
            a, b = download_rows(dev, got, 256, shape_cols[0], np16), download_rows(dev, want, 256, shape_cols[0], np16)
            if exact:
                ok = bool(np.all((a.view(np.uint16) == b.view(np.uint16)) | (np.isnan(a) & np.isnan(b))))
            else:
                ok = oracle.count_not_close(a, b, 1e-3, 1e-3)[0] == 0
        out.append({"pattern": name, "shape": shape, "one_pass_us": round(us_f, 1), "sequence_us": round(us_s, 1),
                    "launches_replaced": launches, "alg_MB": round(alg_bytes / 1e6, 1), "sequence_alg_MB": round(seq_bytes / 1e6, 1),
                    "GBps": round(alg_bytes / us_f / 1e3, 1), "frac_hbm": round(alg_bytes / us_f / 1e3 / PEAK_HBM_GBPS, 4),
                    "matches_sequence": ok})

    shape_cols = [0]
    # cfg 2: LayerNorm module on [1,2048,2560] f16 with f32 weights; GELU between full() and cast()
    x = normal(seed, 901, (2048, 2560), 1.0, np16)
    w, b = normal(seed, 902, (2560,), 0.02, np32, mean=1.0), normal(seed, 903, (2560,), 0.02, np32)
    dx, dw, db = dev.upload(x), dev.upload(w), dev.upload(b)
    f32a, f32b = dev.empty(x.shape, F32), dev.empty(x.shape, F32)
    y1, y2 = dev.empty(x.shape, F16), dev.empty(x.shape, F16)
    shape_cols[0] = 2560
    row("full -> layer_norm -> cast", "[1,2048,2560] f16", 2 * x.nbytes, 10 * x.nbytes, 3,
        lambda: dev.norm_via_f32("layer", dx, dw, db, 1e-5, out=y1),
        lambda: (dev.cast(dx, F32, out=f32a), dev.layer_norm(f32a, dw, db, 1e-5, out=f32b), dev.cast(f32b, F16, out=y2)), y1, y2, False)
    del f32a, f32b
    h = normal(seed, 904, (2048, 10240), 1.0, np16)
    dh = dev.upload(h)
    f32a = dev.empty(h.shape, F32)
    y1, y2 = dev.empty(h.shape, F16), dev.empty(h.shape, F16)
    shape_cols[0] = 10240
    row("full -> gelu -> cast", "[1,2048,10240] f16", 2 * h.nbytes, 10 * h.nbytes, 3,
        lambda: dev.unary_via_f32("gelu", dh, out=y1),
        lambda: (dev.cast(dh, F32, out=f32a), dev.unary("gelu", f32a, out=f32a), dev.cast(f32a, F16, out=y2)), y1, y2, True)
    del f32a, dh
    # cfg 3: RMSNorm module on [1,4096,3072]; gated multiply on the [1,4096,16384] gate_up projection; attention softmax
    x = normal(seed, 905, (4096, 3072), 1.0, np16)
    w = normal(seed, 906, (3072,), 0.02, np32, mean=1.0)
    dx, dw = dev.upload(x), dev.upload(w)
    f32a, f32b = dev.empty(x.shape, F32), dev.empty(x.shape, F32)
    y1, y2 = dev.empty(x.shape, F16), dev.empty(x.shape, F16)
    shape_cols[0] = 3072
    row("full -> rms_norm -> cast", "[1,4096,3072] f16", 2 * x.nbytes, 10 * x.nbytes, 3,
        lambda: dev.norm_via_f32("rms", dx, dw, None, 1e-5, out=y1),
        lambda: (dev.cast(dx, F32, out=f32a), dev.rms_norm(f32a, dw, 1e-5, out=f32b), dev.cast(f32b, F16, out=y2)), y1, y2, False)
    del f32a, f32b
    proj = normal(seed, 907, (4096, 16384), 1.0, np16)
    dp = dev.upload(proj)
    half = (4096, 8192)
    g16, u16, act16 = dev.empty(half, F16), dev.empty(half, F16), dev.empty(half, F16)
    g32 = dev.empty(half, F32)
    y1, y2 = dev.empty(half, F16), dev.empty(half, F16)
    gate_v = BufferView(dp, 0, (proj.size - 8192,))
    up_v = BufferView(dp, 8192, (proj.size - 8192,))
    hb = 4096 * 8192 * 2
    shape_cols[0] = 8192
    row("slice x2 -> full -> silu -> cast -> mul", "[1,4096,16384] f16 -> [1,4096,8192]", 3 * hb, 17 * hb, 6,
        lambda: dev.gated_mul_via_f32("silu", gate_v, up_v, 4096, 8192, gate_row_stride=16384, up_row_stride=16384, out=y1),
        lambda: (dev.slice(dp, [(0, 4096), (0, 8192)], out=g16), dev.slice(dp, [(0, 4096), (8192, 16384)], out=u16),
                 dev.cast(g16, F32, out=g32), dev.unary("silu", g32, out=g32), dev.cast(g32, F16, out=act16),
                 dev.binary("mul", u16, act16, out=y2)), y1, y2, True)
    del g16, u16, act16, g32, dp
    S, H = 4096, 32
    scores, mask, masked, _ = ops_extra["attn"]
    s32a = dev.empty((1, H, S, S), F32)
    y1, y2 = dev.empty((1, H, S, S), F16), dev.empty((1, H, S, S), F16)
    nb = H * S * S * 2
    shape_cols[0] = S
    y3 = dev.empty((1, H, S, S), F16)
    row("add(mask) -> softmax (f16 arithmetic, bit-exact)", "[1,32,4096,4096]+[4096,4096] f16", 2 * nb + S * S * 2, 4 * nb + S * S * 2, 2,
        lambda: dev.softmax_masked(scores, mask, out=y3),
        lambda: (dev.binary("add", scores, mask, out=masked), dev.softmax(masked, out=y2)), y3, y2, True)
    del y3
    row("add(mask) -> full -> softmax -> cast", "[1,32,4096,4096]+[4096,4096] f16", 2 * nb + S * S * 2, 12 * nb + S * S * 2, 4,
        lambda: dev.softmax_via_f32(scores, mask, out=y1),
        lambda: (dev.binary("add", scores, mask, out=masked), dev.cast(masked, F32, out=s32a), dev.softmax(s32a, out=s32a),
                 dev.cast(s32a, F16, out=y2)), y1, y2, False)
    return out


def decode_step(dev, seed):
    """A launch-bound sequence, reported beside the step: the memory-bound ops of one Phi-2-sized decode layer (one token,
    2047 tokens already in the KV cache) launched one by one, and the same sequence replayed from a HIP graph."""
    np16, np32 = np.float16, np.float32
    H, D, N, T = 32, 80, 2560, 2047
    table = dev.upload(normal(seed, 951, (4096, N), 1.0, np16))
    ids = dev.upload(np.array([1234], np.int32))
    w32, b32 = dev.upload(normal(seed, 952, (N,), 0.02, np32, mean=1.0)), dev.upload(normal(seed, 953, (N,), 0.02, np32))
    x, h = dev.empty((1, N), F16), dev.empty((1, N), F16)
    q, k, v = (dev.upload(normal(seed, 954 + i, (1, H, 1, D), 1.0, np16)) for i in range(3))
    kc, vc = dev.empty((1, H, 2048, D), F16).zero_(), dev.empty((1, H, 2048, D), F16).zero_()
    kd, vd = dev.empty((1, H, T + 1, D), F16), dev.empty((1, H, T + 1, D), F16)
    scores = dev.upload(normal(seed, 957, (1, H, 1, T + 1), 2.0, np16))
    probs = dev.empty((1, H, 1, T + 1), F16)
    ff = dev.upload(normal(seed, 958, (1, 4 * N), 1.0, np16))
    act, res = dev.empty((1, 4 * N), F16), dev.empty((1, N), F16)

    def seq():
        dev.index_select(table, ids, 0, out=x)                       # embedding row
        dev.norm_via_f32("layer", x, w32, b32, 1e-5, out=h)          # input LayerNorm (full -> layer_norm -> cast)
        dev.rope(q, 32, 10000.0, T, out=q)                           # rotary on q and k, in place
        dev.rope(k, 32, 10000.0, T, out=k)
        dev.cache(kc, k, 2, T, out=kd)                               # KV append
        dev.cache(vc, v, 2, T, out=vd)
        dev.softmax_via_f32(scores, None, out=probs)                 # attention weights over 2048 keys
        dev.unary_via_f32("gelu", ff, out=act)                       # MLP activation
        dev.binary("add", x, h, out=res)                             # residual

    n_ops = 9
    seq()
    dev.sync()

    def timed(fn, n=200):
        dev.sync()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        dev.sync()
        return (time.perf_counter() - t0) / n * 1e6

    eager = timed(seq)
    with dev.capture() as g:
        seq()
    g.launch()
    replay = timed(g.launch)
    return {"sequence": "index_select, layer_norm(via f32), rope x2, cache x2, softmax(via f32), gelu(via f32), add at Phi-2 decode shapes",
            "launches": n_ops, "eager_us": round(eager, 1), "graph_replay_us": round(replay, 1),
            "note": "eager = nine calls through ctypes on the device's stream; replay = one hipGraphLaunch of the captured sequence"}


def host_graph_step(seed):
    """The same decode-layer ops as a lazy graph through the host mirror of the reference's Tensor API: built, planned and
    resolved every step, as the reference's models do, against one dispatch of the graph compiled once (Executable)."""
    from ratchet_amd import host

    np16, np32 = np.float16, np.float32
    H, D, N, T = 32, 80, 2560, 2047
    hd = host.HostDevice(0)
    up = lambda a: host.Tensor.from_numpy(a, hd)
    table, ids = up(normal(seed, 951, (4096, N), 1.0, np16)), up(np.array([1234], np.int32))
    w32, b32 = up(normal(seed, 952, (N,), 0.02, np32, mean=1.0)), up(normal(seed, 953, (N,), 0.02, np32))
    kc, knew = up(np.zeros((1, H, 2048, D), np16)), up(normal(seed, 955, (1, H, 1, D), 1.0, np16))
    scores = up(normal(seed, 957, (1, H, 1, T + 1), 2.0, np16))
    ff = up(normal(seed, 958, (1, 4 * N), 1.0, np16))

    def build():
        x = table.index_select(ids, 0)                                               # embedding row
        h = x.full().layer_norm(w32, b32, 1e-5).cast(F16)                            # one launch (caller pattern)
        k = knew.full().rope(32, 10000.0, T).cast(F16)                               # rotary in f32, as the CPU op has it
        return [x.add(h),                                                            # residual
                kc.cache(k, 2, T),                                                   # KV append
                scores.full().softmax(3).cast(F16),                                  # attention weights, one launch
                ff.full().gelu().cast(F16)]                                          # MLP activation, one launch

    def resolve_all():
        for r in build():
            r.resolve()

    roots = build()
    exes = [r.compile() for r in roots]
    launches = sum(e.launches for e in exes)

    def dispatch_all():
        for e in exes[:-1]:
            e.dispatch(wait=False)
        exes[-1].dispatch()

    def timed(fn, n=100):
        fn()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        return (time.perf_counter() - t0) / n * 1e6

    resolve_us, dispatch_us = timed(resolve_all), timed(dispatch_all)
    held = sum(e.held_bytes for e in exes)
    for e in exes:
        e.close()
    del roots
    hd.close()
    return {"graphs": "index_select + layer_norm(via f32) + add, cache(cast(rope(full))), softmax(via f32), gelu(via f32) at Phi-2 decode shapes",
            "launches": launches, "build_plan_resolve_us": round(resolve_us, 1), "executable_dispatch_us": round(dispatch_us, 1),
            "executable_held_bytes": held,
            "note": "resolve = graph building, pattern matching, memory plan, launches and a wait per graph, through ctypes; "
                    "dispatch = the launch list each compiled graph keeps, on the buffers of its memory plan (one hipGraphLaunch from "
                    "eight launches on, call by call below that), one wait"}


def warm_up(dev, fn, seconds=0.05):
    """Keeps the GPU busy with `fn` for a while before a timing that follows host-side work (a parity check, an upload):
    after tens of milliseconds without work the clocks are down, and the first launches behind such a pause run up to
    15 % slower than the same launches in a busy stream (the rows of the step are timed inside a busy stream)."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(4):
            fn()
        dev.sync()


def rotating_sets(dev, op, min_bytes=768e6, max_sets=192):
    """[(ins, out), ...]: the op's own buffers plus copies of its large operands and outputs, enough of them that going
    round the sets moves more than `min_bytes` (three Infinity Caches) before a buffer comes up again"""
    from ratchet_amd import _lib

    k = int(min(max_sets, max(1, -(-int(min_bytes) // op.alg_bytes))))
    sets = [(op.ins, op.out)]
    for _ in range(k - 1):
        ins = list(op.ins)
        for j in op.rotating:
            b = dev.empty(op.ins[j].shape, op.ins[j].dt)
            _lib.check(dev.lib.rt_d2d(dev.handle, b.ptr, op.ins[j].ptr, b.nbytes))
            ins[j] = b
        sets.append((ins, dev.empty(op.out.shape, op.out.dt)))
    return sets


def time_without_events(dev, op, min_launches=24):
    """us per launch with nothing between the launches: the op issued back to back over its rotating sets (cold operands
    every time), one pair of events around the whole run.  What `us` of the per-op pass has on top of this is the two
    events and the completion signal each of them forces."""
    sets = rotating_sets(dev, op)
    n = max(min_launches, 2 * len(sets)) if op.alg_bytes < 768e6 else 6
    for k in range(min(len(sets), 4)):
        op.call(*sets[k])
    dev.sync()
    best = None
    for _ in range(3):
        e0, e1 = dev.event(), dev.event()
        e0.record()
        for k in range(n):
            op.call(*sets[k % len(sets)])
        e1.record()
        t = e0.elapsed_ms(e1) * 1e3 / n
        best = t if best is None else min(best, t)
    del sets
    return best, n


def extra_rows(dev, seed, oracle):
    """Rows reported beside the step, never part of `value`: inputs the step does not show.  (a) the f16 streaming softmax
    on dense N(0,2) scores [1,32,4096,4096] (no mask, so no run of -inf: the table lookups of a wave fall into different
    LDS banks); (b) BASELINE config 0, the reference's own CPU-runnable case, as three launches on [1,1500,384] f32:
    bias add (broadcast fused), tanh GELU, LayerNorm; (c) the f16 softmax of a decode step's [1,32,1,2048] scores.  Each
    with the copy of the same bytes timed the same way."""
    import ctypes

    from ratchet_amd import _lib

    np16, np32 = np.float16, np.float32
    rows = []
    src, dst = ops_extra["copy_pair"]

    def copy_us(nbytes, n=12):
        half = min((nbytes // 2) & ~15, src.nbytes)
        warm_up(dev, lambda: _lib.check(dev.lib.rt_cast(dev.handle, F16, F16, src.ptr, dst.ptr, half // 2)))
        ts = []
        for k in range(n):
            off = ((k * half) % (src.nbytes - half) & ~255) if half < src.nbytes else 0
            e0, e1 = dev.event(), dev.event()
            e0.record()
            _lib.check(dev.lib.rt_cast(dev.handle, F16, F16, ctypes.c_void_p(src.ptr.value + off), ctypes.c_void_p(dst.ptr.value + off), half // 2))
            e1.record()
            ts.append(e0.elapsed_ms(e1) * 1e3)
        return float(np.median(ts[2:]))

    def timed(fn, n=12):
        warm_up(dev, fn)
        ts = []
        for _ in range(n):
            e0, e1 = dev.event(), dev.event()
            e0.record()
            fn()
            e1.record()
            ts.append(e0.elapsed_ms(e1) * 1e3)
        return float(np.median(ts[2:]))

    def add(name, shape, dtype, alg, us, ok, note=None):
        c = copy_us(alg)
        r = {"row": name, "shape": shape, "dtype": dtype, "alg_MB": round(alg / 1e6, 3), "us": round(us, 2), "GBps": round(alg / us / 1e3, 1),
             "frac_hbm": round(alg / us / 1e3 / PEAK_HBM_GBPS, 4), "copy_us": round(c, 2), "frac_of_copy": round(c / us, 4), "parity_ok": ok}
        if note:
            r["note"] = note
        rows.append(r)

    # (a) dense scores: the score head itself, replicated over the heads, no mask added
    scores, _mask, masked, soft = ops_extra["attn"]
    head, _ = ops_extra["head"]
    us = timed(lambda: dev.softmax(scores, out=soft), n=8)
    ok = None
    if oracle is not None:
        want = oracle.softmax(head[:256])
        got = download_rows(dev, soft, 256, head.shape[1], np16)
        ok = bool(np.all((got.view(np.uint16) == want.view(np.uint16)) | (np.isnan(got) & np.isnan(want))))
    add("softmax, dense scores (no mask)", "131072x4096", "f16", 2 * scores.nbytes, us, ok,
        "launched back to back on a cold input; the causal row of the step reads what the mask add has just written")
    # the causal input in the same position (back to back, input not just written), for comparison with the step's row
    us = timed(lambda: dev.softmax(masked, out=soft), n=8)
    add("softmax, causal scores, launched back to back", "131072x4096", "f16", 2 * scores.nbytes, us, None)

    # (b) config 0
    x = normal(seed, 801, (1, 1500, 384), 1.0, np32)
    bias = normal(seed, 802, (384,), 0.02, np32)
    g = normal(seed, 803, (384,), 0.02, np32, mean=1.0)
    b = normal(seed, 804, (384,), 0.02, np32)
    dx, dbias, dg, db = dev.upload(x), dev.upload(bias), dev.upload(g), dev.upload(b)
    y1, y2, y3 = dev.empty(x.shape, F32), dev.empty(x.shape, F32), dev.empty(x.shape, F32)
    h1 = h2 = h3 = None
    if oracle is not None:
        h1 = oracle.binary("add", x, np.ascontiguousarray(np.broadcast_to(bias, x.shape)))
        h2 = oracle.unary("gelu", h1)
        h3 = oracle.layer_norm(h2, g, b, 1e-5)
    t1 = timed(lambda: dev.binary("add", dx, dbias, out=y1))
    t2 = timed(lambda: dev.unary("gelu", y1, out=y2))
    t3 = timed(lambda: dev.layer_norm(y2, dg, db, 1e-5, out=y3))
    ok1 = ok2 = ok3 = None
    if oracle is not None:
        ok1 = bool(np.array_equal(y1.to_numpy().view(np.uint32), h1.view(np.uint32)))
        ok2 = oracle.count_not_close(y2.to_numpy(), h2, 1e-5, 1e-5)[0] == 0
        ok3 = oracle.count_not_close(y3.to_numpy(), h3, 1e-5, 1e-5)[0] == 0
    note0 = "4.6 MB: the operands stay in the caches between repetitions (cache-warm, unlike the rows of the step)"
    add("cfg0 bias add (broadcast fused)", "[1,1500,384]+[384]", "f32", 2 * x.nbytes + bias.nbytes, t1, ok1, note0)
    add("cfg0 gelu (tanh approx)", "[1,1500,384]", "f32", 2 * x.nbytes, t2, ok2, note0)
    add("cfg0 layer_norm", "1500x384", "f32", 2 * x.nbytes + g.nbytes + b.nbytes, t3, ok3, note0)

    # (c) a decode step's scores in f16: [B * H, T] = [32, 2048], one wave per row (the row sum replayed, not walked)
    sc = normal(seed, 805, (1, 32, 1, 2048), 2.0, np16)
    dsc, ysc = dev.upload(sc), dev.empty(sc.shape, F16)
    t4 = timed(lambda: dev.softmax(dsc, out=ysc))
    ok4 = None
    if oracle is not None:
        want = oracle.softmax(sc)
        got = ysc.to_numpy()
        ok4 = bool(np.all((got.view(np.uint16) == want.view(np.uint16)) | (np.isnan(got) & np.isnan(want))))
    add("softmax, decode scores (32 rows)", "[1,32,1,2048]", "f16", 2 * sc.nbytes, t4, ok4,
        "0.26 MB: bound by the row's sequential f16 sum and the launch, not by memory")
    return rows


def profile_targets(dev, seed, names, reps):
    """For rocprofv3: launches each named target back to back and nothing else, so that a kernel trace or a counter run of
    this script shows those launches alone: a second of them to bring the clocks up, then the `reps` that a summary reads
    (the last `reps` dispatches of the target's kernel).  No events, no checks, no JSON line.
      softmax_masked  rt_softmax_masked on causal [1,32,4096,4096] f16 scores + the [4096,4096] mask (config 3 as written)
      softmax_causal  rt_softmax on the same scores with the mask already added (the step's launch, on its own)
      softmax_dense   rt_softmax on dense N(0,2) scores of that shape (no -inf: the table lookups of a wave differ)
      copy_1gib       the plain copy kernel on 1 GiB (the counters' calibration and the copy ceiling)
      bf16_layer_norm, bf16_rms_norm, f16_rms_norm   the 16-bit reference norms on [4096,3072], cold operands every launch
      decode_softmax_2048, _4096, _8192   rt_softmax on a decode step's f16 scores [1,32,1,T]
      copy_reference  one plain copy per op of the step (half the op's algorithmic bytes read, half written, fresh regions
                      of two 1 GiB buffers), then a 21 MB copy + 16-byte fill and a 2 MB copy + 16-byte fill: per repetition
                      19 copy launches and 2 fills, in that order"""
    from ratchet_amd import _lib

    S, H = 4096, 32
    head = normal(seed, 112, (S, S), 2.0, np.float16)          # stream 112: the score head of build_workload
    mask = np.triu(np.full((S, S), -np.inf, np.float16), k=1)
    d_head, d_mask = dev.upload(head), dev.upload(mask)
    x = dev.empty((1, H, S, S), F16)
    for h in range(H):
        _lib.check(dev.lib.rt_d2d(dev.handle, x.ptr.value + h * head.nbytes, d_head.ptr, head.nbytes))
    y = dev.empty((1, H, S, S), F16)
    masked = None
    for name in names:
        if name == "softmax_masked":
            fn = lambda: dev.softmax_masked(x, d_mask, out=y)
        elif name == "softmax_dense":
            fn = lambda: dev.softmax(x, out=y)
        elif name == "softmax_causal":
            if masked is None:
                masked = dev.empty((1, H, S, S), F16)
                dev.binary("add", x, d_mask, out=masked)
            fn = lambda: dev.softmax(masked, out=y)
        elif name == "copy_1gib":
            fn = lambda: _lib.check(dev.lib.rt_cast(dev.handle, F16, F16, x.ptr, y.ptr, x.numel))
        elif name in ("bf16_layer_norm", "bf16_rms_norm", "f16_rms_norm"):
            # the 16-bit reference norms on [4096,3072], over twelve sets of buffers in turn (cold operands every launch)
            bf = name.startswith("bf16")
            rows_n, cols_n = 4096, 3072
            f32 = normal(seed, 950, (rows_n, cols_n), 1.0, np.float32)
            if bf:                                               # round to nearest even on the bit pattern
                u = f32.view(np.uint32)
                host = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
                g = ((np.float32(1.0) + normal(seed, 951, (cols_n,), 0.02, np.float32)).view(np.uint32) >> 16).astype(np.uint16)
            else:
                host = f32.astype(np.float16)
                g = (np.float32(1.0) + normal(seed, 951, (cols_n,), 0.02, np.float32)).astype(np.float16)
            dt = 2 if bf else F16
            dg = dev.upload(g, bf16=bf)
            sets_n = []
            for _ in range(12):
                a = dev.upload(host, bf16=bf)
                sets_n.append((a, dev.empty((rows_n, cols_n), dt)))
            turn = [0]

            def norm_launch():
                a, o = sets_n[turn[0] % len(sets_n)]
                turn[0] += 1
                if name.endswith("layer_norm"):
                    dev.layer_norm(a, dg, dg, 1e-5, out=o)
                else:
                    dev.rms_norm(a, dg, 1e-5, out=o)

            fn = norm_launch
        elif name.startswith("decode_softmax_"):
            # a decode step's f16 scores [1,32,1,T], T from the name (2048, 4096, 8192): one wave per row
            T = int(name.rsplit("_", 1)[1])
            dsc = dev.upload(normal(seed, 805, (1, H, 1, T), 2.0, np.float16))
            ysc = dev.empty((1, H, 1, T), F16)
            fn = lambda dsc=dsc, ysc=ysc: dev.softmax(dsc, out=ysc)
        elif name == "copy_reference":
            # the copy pass of the bench (one copy per op of the step, same bytes, back to back), without its events; behind
            # it the boundary probes: a 16-byte fill behind a 21 MB copy and behind a 2 MB copy
            import ctypes

            tiny = dev.empty((4,), F32)
            off = [0]

            def copies():
                for k, nbytes in enumerate(STEP_ALG_BYTES + [20971520, 2097152]):
                    half = min((nbytes // 2) & ~15, x.nbytes)
                    if off[0] + half > x.nbytes:
                        off[0] = 0
                    _lib.check(dev.lib.rt_cast(dev.handle, F16, F16, ctypes.c_void_p(x.ptr.value + off[0]), ctypes.c_void_p(y.ptr.value + off[0]), half // 2))
                    off[0] += half
                    if k >= len(STEP_ALG_BYTES):             # the two probes
                        tiny.zero_()

            fn = copies
        else:
            raise SystemExit("bench.py --profile: unknown target %r" % name)
        warm_up(dev, fn, 1.0)                                # clocks up before the launches a summary reads: the last `reps`
        for _ in range(reps):
            fn()
        dev.sync()
        print("profiled", name, reps, flush=True)


def download_rows(dev, buf, nrows, row_elems, np_dtype):
    """first nrows rows (row_elems each) of a device buffer"""
    import ctypes

    from ratchet_amd import _lib

    out = np.empty((nrows, row_elems), dtype=np_dtype)
    _lib.check(dev.lib.rt_d2h(dev.handle, out.ctypes.data_as(ctypes.c_void_p), buf.ptr, out.nbytes))
    return out


def check_and_time_cpu(dev, op, oracle, check=True):
    """Parity of the timed output buffer against the oracle; returns (ok, cpu_seconds, cpu_bytes).  check=False only
    times the oracle (the second, loop-only CPU figure) and leaves the device buffers alone."""
    c = op.cpu_sample
    kind = c["kind"]
    np_dt = {"f32": np.float32, "f16": np.float16, "f16->f32": np.float32, "f32->f16": np.float16}[op.dtype]
    t_cpu, b_cpu = 0.0, 0

    def timed(fn):
        nonlocal t_cpu
        t0 = time.perf_counter()
        r = fn()
        t_cpu += time.perf_counter() - t0
        return r

    if kind == "exact":
        want = timed(lambda: c["run"](oracle))
        b_cpu = c["bytes"]
        if not check:
            return True, t_cpu, b_cpu
        got = c["out"].to_numpy()
        ok = np.array_equal(got.view(np.uint8), np.ascontiguousarray(want).view(np.uint8))
    elif kind == "close":
        want = timed(lambda: c["run"](oracle))
        b_cpu = c["bytes"]
        if not check:
            return True, t_cpu, b_cpu
        bad, _ = oracle.count_not_close(c["out"].to_numpy(), want, c["tol"], c["tol"])
        ok = bad == 0
    elif kind == "softmax":
        x = c["x"].reshape(-1, c["x"].shape[-1])[: c["rows"]]
        want = timed(lambda: oracle.softmax(x))
        b_cpu = 2 * x.nbytes
        if not check:
            return True, t_cpu, b_cpu
        got = download_rows(dev, c["out"], c["rows"], x.shape[-1], np_dt)
        bad, _ = oracle.count_not_close(got, want, c["tol"], c["tol"])
        ok = bad == 0
    elif kind == "rows":
        x = c["x"].reshape(-1, c["x"].shape[-1])[: c["rows"]]
        want = timed(lambda: c["fn"](oracle, x))
        b_cpu = 2 * x.nbytes
        if not check:
            return True, t_cpu, b_cpu
        got = download_rows(dev, c["out"], c["rows"], x.shape[-1], np_dt)
        bad, _ = oracle.count_not_close(got, want, c["tol"], c["tol"])
        ok = bad == 0
    else:  # rows2: the inputs of the first n rows are built outside the timed region, the oracle runs on all of them inside it
        n = c["rows"]
        inp = c["prep"](oracle, n)
        want = timed(lambda: c["fn"](oracle, inp))
        del inp
        want = want.reshape(n, -1)
        b_cpu = int(n * c["bytes_per_row"])
        if not check:
            return True, t_cpu, b_cpu
        got = download_rows(dev, c["out"], n, want.shape[-1], np_dt)
        if c["tol"] == 0.0:
            ok = np.array_equal(got.view(np.uint16), want.view(np.uint16)) or bool(
                np.all((got.view(np.uint16) == want.view(np.uint16)) | (np.isnan(got) & np.isnan(want))))
        else:
            bad, _ = oracle.count_not_close(got, want, c["tol"], c["tol"])
            ok = bad == 0
    return bool(ok), t_cpu, b_cpu


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--ops", type=str, default=None, help="regex selecting ops by 'cfgN name'")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline timing")
    ap.add_argument("--no-check", action="store_true", help="skip the parity check of the timed buffers")
    ap.add_argument("--no-patterns", action="store_true", help="skip the one-pass caller-pattern timings reported beside the step")
    ap.add_argument("--no-decode-graphs", action="store_true",
                    help="skip the two launch-bound decode sequences (they replay HIP graphs, which a kernel trace of the patterns does not need)")
    ap.add_argument("--no-rotate", action="store_true", help="skip the event-free per-op pass over rotating cold buffers (it allocates about 12 GB)")
    ap.add_argument("--profile", type=str, default=None, help="comma-separated targets to launch alone under rocprofv3 (see profile_targets)")
    ap.add_argument("--reps", type=int, default=6, help="launches per --profile target")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (every op is row/element parallel; there is no multi-GPU path). "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    from ratchet_amd import Device

    seed = int(os.environ.get("RATCHET_SEED", "0"))
    dev = Device(0)
    if args.profile:
        profile_targets(dev, seed, args.profile.split(","), args.reps)
        dev.close()
        return
    t_setup = time.perf_counter()
    ops = build_workload(dev, seed)
    if args.ops:
        rx = re.compile(args.ops)
        ops = [o for o in ops if rx.search(f"cfg{o.cfg} {o.name}")]
    elif [o.alg_bytes for o in ops] != STEP_ALG_BYTES:
        raise SystemExit("bench.py: STEP_ALG_BYTES is out of step with build_workload")
    dev.sync()
    t_setup = time.perf_counter() - t_setup

    ev = [(dev.event(), dev.event()) for _ in ops]

    for _ in range(args.warmup):
        for o in ops:
            o.launch()
    dev.sync()

    # per-op pass (not the timed region): HIP events around every launch, one synchronisation per step.  These give the
    # per-op table; the events and the per-step wait cost about 6 us per op, which is why `value` is not taken here.
    # A 16-byte fill goes ahead of the first op of every step, so that it does not start on a queue the wait has drained
    # (the first row would otherwise carry the cost of waking the queue, about 3 us, which no other row has).
    tiny = dev.empty((4,), F32)
    for _ in range(args.steps):
        tiny.zero_()
        for o, (e0, e1) in zip(ops, ev):
            e0.record()
            o.launch()
            e1.record()
        dev.sync()
        for o, (e0, e1) in zip(ops, ev):
            o.us.append(e0.elapsed_ms(e1) * 1e3)
    dom = max(ops, key=lambda o: float(np.mean(o.us)))

    # timed region: exactly `steps` steps of back-to-back launches on the device's stream, a synchronisation on both
    # sides, nothing in between but one pair of HIP events around the dominant kernel of each step (for the roofline)
    dom_ev = [(dev.event(), dev.event()) for _ in range(args.steps)]
    step_start, step_stop = dev.event(), dev.event()
    dev.sync()
    wall0 = time.perf_counter()
    step_start.record()
    for k in range(args.steps):
        for o in ops:
            if o is dom:
                dom_ev[k][0].record()
                o.launch()
                dom_ev[k][1].record()
            else:
                o.launch()
    step_stop.record()
    dev.sync()
    wall = time.perf_counter() - wall0
    gpu_ms = step_start.elapsed_ms(step_stop)
    dom_us = [e0.elapsed_ms(e1) * 1e3 for e0, e1 in dom_ev]

    # the same step recorded once into a HIP graph and replayed (reported beside `value`, which stays on plain launches)
    with dev.capture() as step_graph:
        for o in ops:
            o.launch()
    step_graph.launch()
    dev.sync()
    g0 = time.perf_counter()
    for _ in range(args.steps):
        step_graph.launch()
    dev.sync()
    graph_ms = (time.perf_counter() - g0) * 1e3 / args.steps

    # the step as a graph executor that folds scores.add(mask).softmax() would run it: the two config-3 launches replaced by
    # one rt_softmax_masked (same bits in the same output buffer); reported beside `value`, never part of it
    folded_ms = None
    if not args.ops:
        scores3, mask3, _masked3, soft3 = ops_extra["attn"]
        pair = [o for o in ops if o.cfg == 3 and ("causal" in o.name)]
        rest = [o for o in ops if o not in pair]
        for _ in range(2):
            dev.softmax_masked(scores3, mask3, out=soft3)
        dev.sync()
        f0 = time.perf_counter()
        for _ in range(args.steps):
            for o in rest:
                o.launch()
            dev.softmax_masked(scores3, mask3, out=soft3)
        dev.sync()
        folded_ms = (time.perf_counter() - f0) * 1e3 / args.steps

    total_bytes = sum(o.alg_bytes for o in ops)
    ms_per_step = wall * 1e3 / args.steps                       # host clock between the two synchronisations
    value = total_bytes / (ms_per_step * 1e-3) / 1e9

    oracle = None
    parity_ok, cpu_t, cpu_b, loop_t = True, 0.0, 0, 0.0
    per_op_cpu = {}
    if not (args.no_check and args.no_cpu):
        from oracle import cpu_oracle as oracle          # the checker / CPU baseline only; never on the measured path

        oracle.lib()
        oracle.set_reference_copies(True)
        for o in ops:
            ok, t, b = check_and_time_cpu(dev, o, oracle)
            parity_ok = parity_ok and ok
            if not ok:
                print(f"bench.py: PARITY FAILURE in cfg{o.cfg} {o.name}", file=sys.stderr)
            cpu_t += t
            cpu_b += b
            per_op_cpu[id(o)] = (t, b)
        # second CPU figure: the op's loop alone, without the reference's to_vec / store copies around it
        loop_t = 0.0
        if not args.no_cpu:
            oracle.set_reference_copies(False)
            for o in ops:
                loop_t += check_and_time_cpu(dev, o, oracle, check=False)[1]
            oracle.set_reference_copies(True)

    # the per-op figure that carries no events (after the parity check: the rotating sets are made from the same inputs)
    no_events = {}
    if not args.no_rotate:
        for o in ops:
            no_events[id(o)] = time_without_events(dev, o)
    extras = extra_rows(dev, seed, oracle if not args.no_check else None) if not (args.ops or args.no_patterns) else None
    ceiling = copy_ceiling(dev) if not args.ops else None      # after the parity check: it overwrites an output buffer
    copy_us, boundary_us = copy_reference(dev, ops, args.steps) if not args.ops else ([None] * len(ops), None)
    patterns = one_pass_patterns(dev, seed, oracle if not args.no_check else None) if not (args.ops or args.no_patterns) else None
    decode = decode_step(dev, seed) if not (args.ops or args.no_patterns or args.no_decode_graphs) else None
    host_step = host_graph_step(seed) if not (args.ops or args.no_patterns or args.no_decode_graphs) else None

    # the kernels' own durations and HBM-side bytes, from the committed rocprofv3 summaries (whole step only: rows are by position)
    kt_rows = read_step_rows(PROFILE_KERNEL_TRACE) if not args.ops else {}
    pmc_rows = read_step_rows(PROFILE_HBM_TRAFFIC) if not args.ops else {}

    def kernel_us(pos):
        """the kernel's own average duration at step position `pos` from the committed trace summary; None when the
        summary is missing, when the row's kernel is not the one this op launches, or when the figure exceeds what the
        events measured around the launch in this run by more than 5 % (then the summary describes another build of the kernel)"""
        try:
            name, us = kt_rows[pos][1], float(kt_rows[pos][2])
        except (KeyError, IndexError, ValueError):
            return None
        o = ops[pos - 1]
        if not o.kernel or o.kernel not in name or us > 1.05 * float(np.median(o.us)):
            return None
        return us

    def traffic_bytes(pos):
        """fetch + write of the launch at step position `pos`, from the committed counter summary; None when the summary
        is missing or does not describe this op (its own algorithmic columns disagree with the op's bytes by more than 1 %)"""
        try:
            r = pmc_rows[pos]
            alg_kib = float(r[4]) + float(r[5])
            if abs(alg_kib * 1024 - ops[pos - 1].alg_bytes) > 0.01 * ops[pos - 1].alg_bytes:
                return None
            return int((float(r[2]) + float(r[3])) * 1024)
        except (KeyError, IndexError, ValueError):
            return None

    rows = []
    for pos, o in enumerate(ops, 1):
        med = float(np.median(o.us))
        gbps = o.alg_bytes / (med * 1e-6) / 1e9
        t, b = per_op_cpu.get(id(o), (0.0, 0))
        rows.append({"cfg": o.cfg, "op": o.name, "dtype": o.dtype, "shape": o.shapes, "alg_MB": round(o.alg_bytes / 1e6, 3),
                     "us": round(med, 2), "us_mean": round(float(np.mean(o.us)), 2), "GBps": round(gbps, 1),
                     "frac_hbm": round(gbps / PEAK_HBM_GBPS, 4),
                     # a plain copy kernel moving the same bytes, timed the same way in the same place of the step
                     # launched back to back over rotating cold buffers, no events in between (one pair around `launches` of them)
                     "us_no_events": None if id(o) not in no_events else round(no_events[id(o)][0], 2),
                     "frac_hbm_no_events": None if id(o) not in no_events else round(o.alg_bytes / no_events[id(o)][0] / 1e3 / PEAK_HBM_GBPS, 4),
                     "copy_us": None if copy_us[pos - 1] is None else round(copy_us[pos - 1], 2),
                     "frac_of_copy": None if copy_us[pos - 1] is None else round(copy_us[pos - 1] / med, 4),
                     # the kernel alone (rocprofv3 --kernel-trace of this script, profiles/): `us` adds the two events and the launch gap
                     "kernel_us": kernel_us(pos),
                     "kernel_frac_hbm": None if not kernel_us(pos) else round(o.alg_bytes / (kernel_us(pos) * 1e-6) / 1e9 / PEAK_HBM_GBPS, 4),
                     "cpu_GBps": round(b / t / 1e9, 4) if t > 0 else None})

    dom_avg_us = float(np.mean(dom_us))
    dom_gbps = dom.alg_bytes / (dom_avg_us * 1e-6) / 1e9
    result = {
        "metric": "HBM GB/s over one pass of every op in BASELINE configs[1..4] (per-op us / GB/s / % of 8 TB/s in 'ops')",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "ms_per_step_gpu_timeline": round(gpu_ms / args.steps, 4),
        "ms_per_step_graph_replay": round(graph_ms, 4),
        "ms_per_step_masked_softmax_folded": None if folded_ms is None else round(folded_ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic (Philox, RATCHET_SEED=%d; the [4096,4096] score head is replicated over 32 heads)" % seed,
        "config": {"workload": "all ops of BASELINE configs[1..4]: Whisper-tiny softmax+permute (f32), Phi-2 prefill block (f16), "
                               "Phi-3-mini prefill block incl. [1,32,4096,4096] causal softmax (f16), broadcast/reindex stress (f16)",
                   "ops": len(ops), "algorithmic_GB_per_step": round(total_bytes / 1e9, 3), "cache": "cold (5.6 GB/step >> 256 MB)"},
        "roofline": {"bound": "hbm", "kernel": dom.kernel or dom.name, "op": f"cfg{dom.cfg} {dom.name}",
                     "achieved": round(dom_gbps, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": round(dom_gbps / PEAK_HBM_GBPS, 4),
                     "avg_launch_us": round(dom_avg_us, 2), "algorithmic_bytes": dom.alg_bytes,
                     # FETCH_SIZE + WRITE_SIZE per launch, scaled by a 1 GiB copy kernel; null when the summary lacks the row
                     "traffic": traffic_bytes(ops.index(dom) + 1), "traffic_source": PROFILE_HBM_TRAFFIC,
                     "kernel_us_source": PROFILE_KERNEL_TRACE,
                     # the commit the two summaries were taken at (their `git_head:` line) and the commit of this run
                     "profiles_git_head": {"kernel_trace": profile_head(PROFILE_KERNEL_TRACE), "hbm_traffic": profile_head(PROFILE_HBM_TRAFFIC)},
                     "git_head": git_head(), "library_built_from": library_built_from()},
        "cpu_baseline": None if args.no_cpu or cpu_t == 0 else {
            "value": round(cpu_b / cpu_t / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "every op of the step on one host core with the reference's to_vec/store copies, whole tensors "
                      "(%.1f MB algorithmic, %.1f s)" % (cpu_b / 1e6, cpu_t),
            # the same ops timed without those copies: what the reference's loops alone cost
            "loop_only": None if loop_t == 0 else {"value": round(cpu_b / loop_t / 1e9, 4), "unit": "GB/s", "seconds": round(loop_t, 2)},
            "host_cpus": os.cpu_count()},
        "hbm_copy_ceiling": ceiling,
        # a 16-byte fill launched right behind a 21 MB permute, HIP events around it: what one more kernel boundary costs
        "kernel_boundary_us": None if boundary_us is None else round(boundary_us, 2),
        "extra_rows": extras,
        "one_pass_patterns": patterns,
        "decode_step": decode,
        "host_graph_step": host_step,
        "parity_ok": bool(parity_ok) if not args.no_check else None,
        "ops": rows,
        "wall_s": round(wall, 3), "setup_s": round(t_setup, 2),
    }
    print(json.dumps(result))
    dev.close()
    if not args.no_check and not parity_ok:
        sys.exit(1)


if __name__ == "__main__":
    main()
