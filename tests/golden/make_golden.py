#!/usr/bin/env python3
"""Writes tests/golden/vectors.npz: small input/output vectors for every op of the path, produced by the CPU oracle
(oracle/, the restatement of ratchet-core's CPU executor) in the build container.

The reference ships no golden vectors for these ops (its tests compute torch ground truth at run time), so these pin the
oracle itself: a later change to the oracle, or a host libm that rounds tanh/exp differently, shows up as a diff against
this file, and the GPU tests compare the HIP kernels with the same vectors.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import cpu_oracle as orc  # noqa: E402


def edge_values(dtype):
    v = [0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.0, -3.0, 10.0, -10.0, 11.0, 12.0, -17.0, -18.0, 88.0, -88.0, 1e-3, -1e-3, 6e-8, 6.1e-5,
         65504.0, -65504.0, np.inf, -np.inf, np.nan, 0.3465, 1.04, 22.0, 3.14159, 0.7853982, 1e-5]
    with np.errstate(over="ignore"):
        return np.array(v, dtype=np.float32).astype(dtype)


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    for dtype, tag in ((np.float32, "f32"), (np.float16, "f16")):
        x = np.concatenate([edge_values(dtype), (rng.standard_normal(97) * 3).astype(dtype)])
        y = np.concatenate([(rng.standard_normal(len(edge_values(dtype))) * 2).astype(dtype), edge_values(dtype)[:97]])
        y = np.resize(y, x.shape).astype(dtype)
        out[f"ew_x_{tag}"], out[f"ew_y_{tag}"] = x, y
        for op in orc.BINARY_OPS:
            out[f"binary_{op}_{tag}"] = orc.binary(op, x, y)
        for op in orc.UNARY_OPS:
            out[f"unary_{op}_{tag}"] = orc.unary(op, x)
        rows = (rng.standard_normal((6, 40)) * 2).astype(dtype)
        rows[1, 20:] = -np.inf                       # causal-style mask
        rows[2, 3] = 12.0 if dtype == np.float16 else 100.0   # exp overflow: NaN at that element, 0 elsewhere
        rows[3, :] = -np.inf                         # fully masked row
        out[f"softmax_x_{tag}"], out[f"softmax_y_{tag}"] = rows, orc.softmax(rows)
        nx = rng.standard_normal((5, 48)).astype(dtype)
        w = (1 + 0.02 * rng.standard_normal(48)).astype(dtype)
        b = (0.02 * rng.standard_normal(48)).astype(dtype)
        out[f"norm_x_{tag}"], out[f"norm_w_{tag}"], out[f"norm_b_{tag}"] = nx, w, b
        out[f"layer_norm_{tag}"] = orc.layer_norm(nx, w, b, 1e-5)
        out[f"layer_norm_nobias_{tag}"] = orc.layer_norm(nx, w, None, 1e-5)
        out[f"rms_norm_{tag}"] = orc.rms_norm(nx, w, 1e-5)
        gx = rng.standard_normal((2, 8, 6)).astype(dtype)
        gw, gb = rng.standard_normal(8).astype(dtype), rng.standard_normal(8).astype(dtype)
        out[f"gn_x_{tag}"], out[f"gn_w_{tag}"], out[f"gn_b_{tag}"] = gx, gw, gb
        out[f"group_norm_{tag}"] = orc.group_norm(gx, 4, gw, gb, 1e-5)
    c32 = np.concatenate([edge_values(np.float32), np.array([65519.99, 65520.0, 2.9802322e-8, 3e-8, 1e-8, 1.0009765625, 1.00048828125],
                                                            np.float32)])
    out["cast_x_f32"] = c32
    out["cast_f32_to_f16"] = orc.cast(c32, np.float16)
    out["cast_f16_to_f32"] = orc.cast(out["cast_f32_to_f16"], np.float32)
    out["cast_f32_to_bf16"] = orc.cast(c32, np.uint16, dst_bf16=True)
    r = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5)
    out["reindex_x"] = r
    out["permute_0213"] = orc.permute(r, (0, 2, 1, 3))
    out["permute_3102"] = orc.permute(r, (3, 1, 0, 2))
    out["slice_mid"] = orc.slice_(r, [(1, 2), (0, 3), (1, 3), (2, 5)])
    bsrc = np.arange(3 * 5, dtype=np.float32).reshape(1, 3, 1, 5)
    out["broadcast_x"] = bsrc
    out["broadcast_y"] = orc.broadcast(bsrc, (2, 3, 4, 5))
    out["concat_y"] = orc.concat([r, r[:, :, :2] * -1, r[:, :, 1:2] + 0.5], 2)
    # ---- KV-cache append, index ops, RoPE (appended after the vectors above so that those keep their values)
    kv = rng.standard_normal((1, 2, 6, 16)).astype(np.float32)
    kv[:, :, 2:] = 0
    src = rng.standard_normal((1, 2, 1, 16)).astype(np.float32)
    out["cache_in"], out["cache_src"] = kv.copy(), src
    out["cache_dst"] = orc.cache(kv, src, 2, 2)                 # the reference test's layout (ops/cache.rs:162-217)
    out["cache_after"] = kv
    table = rng.standard_normal((50, 12)).astype(np.float16)
    ids = np.array([7, 0, 49, 7, 23], np.int32)
    out["select_table"], out["select_ids"] = table, ids
    out["select_rows"] = orc.index_select(table, ids, 0)
    out["select_cols"] = orc.index_select(table, np.array([11, 0, 5], np.int32), 1)
    iw = np.array([1, 2, 3, 4, 5, 6], np.float32).reshape(3, 2)
    out["index_write_y"] = orc.index_write(iw, np.array([[7, 8]], np.float32), [2, 0])    # ops/index_write.rs:203-224
    q = rng.standard_normal((1, 2, 5, 24)).astype(np.float32)
    out["rope_x"] = q
    out["rope_dim16_off3"] = orc.rope(q, 16, 10000.0, 3)
    out["rope_dim24_off0"] = orc.rope(q, 24, 10000.0, 0)
    # ---- the models' full() -> op -> cast(dt) sequences on f16 tensors, as the oracle's op sequence gives them
    h = np.concatenate([edge_values(np.float16), (rng.standard_normal(33) * 3).astype(np.float16)])
    out["via32_x"] = h
    for op in ("gelu", "silu", "exp", "tanh", "sigmoid"):
        out[f"via32_{op}"] = orc.cast(orc.unary(op, orc.cast(h, np.float32)), np.float16)
    nx16 = rng.standard_normal((4, 64)).astype(np.float16)
    w32, b32 = (1 + 0.02 * rng.standard_normal(64)).astype(np.float32), (0.02 * rng.standard_normal(64)).astype(np.float32)
    out["via32_norm_x"], out["via32_norm_w"], out["via32_norm_b"] = nx16, w32, b32
    out["via32_layer_norm"] = orc.cast(orc.layer_norm(orc.cast(nx16, np.float32), w32, b32, 1e-5, intended=True), np.float16)
    out["via32_rms_norm"] = orc.cast(orc.rms_norm(orc.cast(nx16, np.float32), w32, 1e-5, intended=True), np.float16)
    sc = (rng.standard_normal((1, 2, 8, 16)) * 2).astype(np.float16)
    mask = np.triu(np.full((8, 16), -np.inf, np.float16), k=9)
    out["via32_scores"], out["via32_mask"] = sc, mask
    masked = orc.binary("add", sc, np.ascontiguousarray(np.broadcast_to(mask, sc.shape)))
    out["via32_softmax"] = orc.cast(orc.softmax(orc.cast(masked, np.float32)), np.float16)
    proj = rng.standard_normal((3, 32)).astype(np.float16)
    out["via32_proj"] = proj
    act = orc.cast(orc.unary("silu", orc.cast(np.ascontiguousarray(proj[:, :16]), np.float32)), np.float16)
    out["via32_gated"] = orc.binary("mul", np.ascontiguousarray(proj[:, 16:]), act)
    path = os.path.join(HERE, "vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
