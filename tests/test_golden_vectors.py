"""The committed vectors in tests/golden/vectors.npz against (a) the CPU oracle (CPU test: the oracle, and the host libm
under it, still give what was recorded) and (b) the HIP kernels through the C ABI (GPU test)."""
import os

import numpy as np
import pytest

from gpu_util import mismatch_count

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz"), allow_pickle=False)
UNARY = ["gelu", "tanh", "exp", "log", "sin", "cos", "abs", "sqrt", "relu", "floor", "ceil", "neg", "silu", "sigmoid"]


def same(a, b):
    return mismatch_count(np.asarray(a), np.asarray(b)) == 0


def test_oracle_reproduces_the_recorded_vectors(oracle):
    for tag in ("f32", "f16"):
        x, y = GOLD[f"ew_x_{tag}"], GOLD[f"ew_y_{tag}"]
        for op in ("add", "sub", "mul", "div"):
            assert same(oracle.binary(op, x, y), GOLD[f"binary_{op}_{tag}"]), (op, tag)
        for op in UNARY:
            assert same(oracle.unary(op, x), GOLD[f"unary_{op}_{tag}"]), (op, tag)
        assert same(oracle.softmax(GOLD[f"softmax_x_{tag}"]), GOLD[f"softmax_y_{tag}"])
        nx, w, b = GOLD[f"norm_x_{tag}"], GOLD[f"norm_w_{tag}"], GOLD[f"norm_b_{tag}"]
        assert same(oracle.layer_norm(nx, w, b, 1e-5), GOLD[f"layer_norm_{tag}"])
        assert same(oracle.layer_norm(nx, w, None, 1e-5), GOLD[f"layer_norm_nobias_{tag}"])
        assert same(oracle.rms_norm(nx, w, 1e-5), GOLD[f"rms_norm_{tag}"])
        assert same(oracle.group_norm(GOLD[f"gn_x_{tag}"], 4, GOLD[f"gn_w_{tag}"], GOLD[f"gn_b_{tag}"], 1e-5), GOLD[f"group_norm_{tag}"])
    assert same(oracle.cast(GOLD["cast_x_f32"], np.float16), GOLD["cast_f32_to_f16"])
    assert np.array_equal(oracle.cast(GOLD["cast_x_f32"], np.uint16, dst_bf16=True), GOLD["cast_f32_to_bf16"])
    r = GOLD["reindex_x"]
    assert np.array_equal(oracle.permute(r, (0, 2, 1, 3)), GOLD["permute_0213"])
    assert np.array_equal(oracle.permute(r, (3, 1, 0, 2)), GOLD["permute_3102"])
    assert np.array_equal(GOLD["permute_0213"], r.transpose(0, 2, 1, 3))
    assert np.array_equal(oracle.slice_(r, [(1, 2), (0, 3), (1, 3), (2, 5)]), GOLD["slice_mid"])
    assert np.array_equal(GOLD["broadcast_y"], np.broadcast_to(GOLD["broadcast_x"], (2, 3, 4, 5)))
    kv = GOLD["cache_in"].copy()
    assert np.array_equal(oracle.cache(kv, GOLD["cache_src"], 2, 2), GOLD["cache_dst"]) and np.array_equal(kv, GOLD["cache_after"])
    assert np.array_equal(GOLD["cache_dst"], np.concatenate([GOLD["cache_in"][:, :, :2], GOLD["cache_src"]], axis=2))
    assert np.array_equal(oracle.index_select(GOLD["select_table"], GOLD["select_ids"], 0), GOLD["select_rows"])
    assert np.array_equal(GOLD["select_rows"], GOLD["select_table"][GOLD["select_ids"]])
    assert np.array_equal(GOLD["index_write_y"], np.array([[1, 2], [3, 4], [7, 8]], np.float32))
    assert same(oracle.rope(GOLD["rope_x"], 16, 10000.0, 3), GOLD["rope_dim16_off3"])
    assert same(oracle.rope(GOLD["rope_x"], 24, 10000.0, 0), GOLD["rope_dim24_off0"])
    h32 = oracle.cast(GOLD["via32_x"], np.float32)
    for op in ("gelu", "silu", "exp", "tanh", "sigmoid"):
        assert same(oracle.cast(oracle.unary(op, h32), np.float16), GOLD[f"via32_{op}"]), op


@pytest.mark.gpu
def test_kernels_reproduce_the_recorded_vectors(oracle):
    from ratchet_amd import Device, _lib

    dev = Device(0)
    try:
        for tag, tol in (("f32", 1e-5), ("f16", 1e-3)):
            x, y = GOLD[f"ew_x_{tag}"], GOLD[f"ew_y_{tag}"]
            dx, dy = dev.upload(x), dev.upload(y)
            for op in ("add", "sub", "mul", "div"):
                assert same(dev.binary(op, dx, dy).to_numpy(), GOLD[f"binary_{op}_{tag}"]), (op, tag)
            for op in UNARY:
                got, want = dev.unary(op, dx).to_numpy(), GOLD[f"unary_{op}_{tag}"]
                if op in ("log", "sin", "cos"):
                    bad, mx = oracle.count_not_close(got, want, 1e-6 if tag == "f32" else 1e-3, 1e-6 if tag == "f32" else 1e-3)
                    assert bad == 0, (op, tag, mx)
                else:
                    zeros = (got == 0) & (want == 0)                  # the sign of relu(-0.0) is not part of the contract
                    assert same(np.where(zeros, 0, got), np.where(zeros, 0, want)), (op, tag)
            got = dev.softmax(dev.upload(GOLD[f"softmax_x_{tag}"])).to_numpy()
            if tag == "f16":
                assert same(got, GOLD[f"softmax_y_{tag}"])
            else:
                bad, mx = oracle.count_not_close(got, GOLD[f"softmax_y_{tag}"], tol, tol)
                assert bad == 0, mx
            nx, w, b = (dev.upload(GOLD[f"norm_{k}_{tag}"]) for k in ("x", "w", "b"))
            for got, key in ((dev.layer_norm(nx, w, b, 1e-5), "layer_norm"), (dev.layer_norm(nx, w, None, 1e-5), "layer_norm_nobias"),
                             (dev.rms_norm(nx, w, 1e-5), "rms_norm")):
                bad, mx = oracle.count_not_close(got.to_numpy(), GOLD[f"{key}_{tag}"], tol, tol)
                assert bad == 0, (key, tag, mx)
            got = dev.group_norm(dev.upload(GOLD[f"gn_x_{tag}"]), 4, dev.upload(GOLD[f"gn_w_{tag}"]), dev.upload(GOLD[f"gn_b_{tag}"]), 1e-5)
            bad, mx = oracle.count_not_close(got.to_numpy(), GOLD[f"group_norm_{tag}"], tol, tol)
            assert bad == 0, ("group_norm", tag, mx)
        c = dev.upload(GOLD["cast_x_f32"])
        assert same(dev.cast(c, _lib.F16).to_numpy(), GOLD["cast_f32_to_f16"])
        assert np.array_equal(dev.cast(c, _lib.BF16).to_numpy(), GOLD["cast_f32_to_bf16"])
        assert same(dev.cast(dev.upload(GOLD["cast_f32_to_f16"]), _lib.F32).to_numpy(), GOLD["cast_f16_to_f32"])
        r = dev.upload(GOLD["reindex_x"])
        assert np.array_equal(dev.permute(r, (0, 2, 1, 3)).to_numpy(), GOLD["permute_0213"])
        assert np.array_equal(dev.permute(r, (3, 1, 0, 2)).to_numpy(), GOLD["permute_3102"])
        assert np.array_equal(dev.slice(r, [(1, 2), (0, 3), (1, 3), (2, 5)]).to_numpy(), GOLD["slice_mid"])
        assert np.array_equal(dev.broadcast_to(dev.upload(GOLD["broadcast_x"]), (2, 3, 4, 5)).to_numpy(), GOLD["broadcast_y"])
        rr = GOLD["reindex_x"]
        parts = [rr, np.ascontiguousarray(rr[:, :, :2] * -1), np.ascontiguousarray(rr[:, :, 1:2] + 0.5)]
        assert np.array_equal(dev.concat([dev.upload(p) for p in parts], 2).to_numpy(), GOLD["concat_y"])
        kv = dev.upload(GOLD["cache_in"])
        assert np.array_equal(dev.cache(kv, dev.upload(GOLD["cache_src"]), 2, 2).to_numpy(), GOLD["cache_dst"])
        assert np.array_equal(kv.to_numpy(), GOLD["cache_after"])
        t = dev.upload(GOLD["select_table"])
        assert np.array_equal(dev.index_select(t, dev.upload(GOLD["select_ids"]), 0).to_numpy(), GOLD["select_rows"])
        assert np.array_equal(dev.index_select(t, dev.upload(np.array([11, 0, 5], np.int32)), 1).to_numpy(), GOLD["select_cols"])
        iw = dev.upload(np.array([1, 2, 3, 4, 5, 6], np.float32).reshape(3, 2))
        assert np.array_equal(dev.index_write(iw, dev.upload(np.array([[7, 8]], np.float32)), [2, 0]).to_numpy(), GOLD["index_write_y"])
        q = dev.upload(GOLD["rope_x"])
        for dim, off, key in ((16, 3, "rope_dim16_off3"), (24, 0, "rope_dim24_off0")):
            bad, mx = oracle.count_not_close(dev.rope(q, dim, 10000.0, off).to_numpy(), GOLD[key], 1e-6, 1e-6)
            assert bad == 0, (key, mx)
        h = dev.upload(GOLD["via32_x"])
        for op in ("gelu", "silu", "exp", "tanh", "sigmoid"):
            assert same(dev.unary_via_f32(op, h).to_numpy(), GOLD[f"via32_{op}"]), op
        nx, w, b = dev.upload(GOLD["via32_norm_x"]), dev.upload(GOLD["via32_norm_w"]), dev.upload(GOLD["via32_norm_b"])
        for got, key in ((dev.norm_via_f32("layer", nx, w, b, 1e-5), "via32_layer_norm"), (dev.norm_via_f32("rms", nx, w, None, 1e-5), "via32_rms_norm")):
            bad, mx = oracle.count_not_close(got.to_numpy(), GOLD[key], 1e-3, 1e-3)
            assert bad == 0, (key, mx)
        got = dev.softmax_via_f32(dev.upload(GOLD["via32_scores"]), dev.upload(GOLD["via32_mask"])).to_numpy()
        bad, mx = oracle.count_not_close(got, GOLD["via32_softmax"], 1e-3, 1e-3)
        assert bad == 0, mx
        from ratchet_amd.runtime import BufferView
        proj = dev.upload(GOLD["via32_proj"])
        got = dev.gated_mul_via_f32("silu", BufferView(proj, 0, (80,)), BufferView(proj, 16, (80,)), 3, 16, gate_row_stride=32, up_row_stride=32)
        assert same(got.to_numpy(), GOLD["via32_gated"])
    finally:
        dev.close()
