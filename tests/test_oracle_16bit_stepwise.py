"""CPU-only, bit-exact pins of the oracle's 16-bit softmax, layer_norm, rms_norm and gelu paths.

Every test rebuilds the reference's sequence of operations (crates/ratchet-core/src/cpu/softmax.rs:28-36,
cpu/norm.rs:72-147 and :185-213, cpu/unary.rs:46-51) from independent parts and demands zero bit mismatches:

* f16 arithmetic is numpy's float16 (each operator widens to float32, operates, rounds to nearest even: what the
  `half` crate does);
* bf16 arithmetic is float32 arithmetic followed by a round-to-nearest-even on the bit pattern, written here in
  numpy (not the oracle's converter);
* sums are explicit left-to-right float32 loops (numpy's own `sum` is pairwise and would differ in the last bit);
* exp / tanh are this machine's libm `expf` / `tanhf`, called through ctypes, because Rust's `f32::exp` / `f32::tanh`
  lower to the same symbols.

Each model is also run with one rounding point removed or one step re-ordered, and with the oracle switched to
f16-sequential row sums: those variants must disagree with the oracle, which shows that the comparison notices
such a mistake.
"""
import ctypes
import ctypes.util

import numpy as np
import pytest

_LIBM = ctypes.CDLL(ctypes.util.find_library("m") or "libm.so.6")
for _name in ("expf", "tanhf"):
    getattr(_LIBM, _name).restype = ctypes.c_float
    getattr(_LIBM, _name).argtypes = [ctypes.c_float]

f32 = np.float32
h = np.float16


def _libm(name, v):
    """libm's float routine applied to every element of a float32 array"""
    fn = getattr(_LIBM, name)
    flat = np.ascontiguousarray(v, dtype=f32).ravel()
    return np.array([fn(float(t)) for t in flat], dtype=f32).reshape(np.shape(v))


def _seq_sum(v):
    """left-to-right float32 sum, starting from 0, of an array that is widened to float32 first"""
    s = f32(0.0)
    for t in np.asarray(v, dtype=f32):
        s = f32(s + t)
    return s


def _bits16(a):
    return np.ascontiguousarray(a).view(np.uint16)


# ------------------------------------------------------------------------------------------------ bf16 in numpy
def rb(v):
    """float32 -> nearest bfloat16 (ties to even), returned as the float32 that holds exactly that value"""
    v = np.asarray(v, dtype=f32)
    u = v.view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    nan = np.isnan(v)
    rounded = np.where(nan, (u | 0x00400000) & 0xFFFF0000, rounded)
    return rounded.astype(np.uint32).view(f32).reshape(v.shape)


def bf16_bits(v):
    """bit patterns (uint16) of float32 values that are exactly representable in bfloat16"""
    u = np.asarray(v, dtype=f32).view(np.uint32)
    assert np.all((u & 0xFFFF) == 0)
    return (u >> 16).astype(np.uint16)


def bf16_from_bits(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(f32)


def test_bf16_rounding_helper_on_known_cases():
    # 1 + 2^-8 is a tie between 1 and 1 + 2^-7: goes to the even mantissa (1); 1 + 3*2^-8 ties up to 1 + 2^-6
    cases = [(1.0, 0x3F80), (1.0 + 2.0 ** -8, 0x3F80), (1.0 + 2.0 ** -8 + 2.0 ** -20, 0x3F81),
             (1.0 + 3 * 2.0 ** -8, 0x3F82), (-2.5, 0xC020), (3.3895314e38, 0x7F7F), (3.4e38, 0x7F80), (0.0, 0x0000)]
    for value, bits in cases:
        assert int(bf16_bits(rb(f32(value)))) == bits, value
    assert np.isnan(rb(f32(np.nan)))


def test_bf16_rounding_helper_agrees_with_torch():
    import torch

    rng = np.random.default_rng(30)
    u = rng.integers(0, 2 ** 32, 200_000, dtype=np.uint64).astype(np.uint32)
    v = u.view(f32)
    v = v[np.isfinite(v)]
    want = torch.from_numpy(v).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(bf16_bits(rb(v)), want)


# ------------------------------------------------------------------------------------------------ softmax
def _softmax_f16_model(row):
    with np.errstate(all="ignore"):
        e = _libm("expf", row.astype(f32)).astype(h)              # x.exp(): f16::from_f32(f32::exp(x.to_f32()))
    s = h(0)
    for t in e:
        s = h(f32(s) + f32(t))                                    # sum += e_j in f16
    with np.errstate(all="ignore"):
        return (e.astype(f32) / f32(s)).astype(h)


def _softmax_bf16_model(row32, sum_in_f32=False):
    e = rb(_libm("expf", row32))
    s = f32(0)
    for t in e:
        s = f32(s + t) if sum_in_f32 else rb(f32(s + t))
    with np.errstate(all="ignore"):
        return rb(e / rb(s))


def test_softmax_f16_bit_exact_stepwise(oracle):
    rng = np.random.default_rng(31)
    x = (rng.standard_normal((6, 301)) * 2).astype(h)
    x[1, 200:] = -np.inf                                          # masked tail: exactly zero
    x[2, 5] = 12.0                                                # exp overflows f16 -> inf / inf = NaN there
    got = oracle.softmax(x)
    for r in range(x.shape[0]):
        want = _softmax_f16_model(x[r])
        ok = (_bits16(want) == _bits16(got[r])) | (np.isnan(want) & np.isnan(got[r]))
        assert ok.all(), (r, np.flatnonzero(~ok)[:5])
    assert np.isnan(got[2, 5]) and np.all(got[2, :5] == 0)


def test_softmax_bf16_bit_exact_stepwise(oracle):
    rng = np.random.default_rng(32)
    x32 = rb((rng.standard_normal((5, 257)) * 2).astype(f32))
    x32[3, 100:] = -np.inf
    got = oracle.softmax(bf16_bits(x32), bf16=True)
    differs_with_f32_sum = False
    for r in range(x32.shape[0]):
        want = _softmax_bf16_model(x32[r])
        assert np.array_equal(bf16_bits(want), got[r]), r
        differs_with_f32_sum |= not np.array_equal(bf16_bits(_softmax_bf16_model(x32[r], sum_in_f32=True)), got[r])
    # 257 terms of order 1 against bf16's 8 bits: a float32 running sum gives another denominator
    assert differs_with_f32_sum


# ------------------------------------------------------------------------------------------------ f16 norms
def _layer_norm_f16_model(xr, w, b, eps, drop_rounding=False, two_pass=False):
    n = h(f32(xr.size))                                           # T::from(step as f32)
    mu = h(_seq_sum(xr)) / n                                      # Sum for f16: f32 fold, one rounding; then f16 divide
    mu2 = mu * mu
    sq = xr * xr
    x2 = h(_seq_sum(sq)) / n
    var = x2 - mu2
    xc = xr - mu
    if two_pass:
        d = xc * xc
        var = h(_seq_sum(d)) / n
    r = h(1.0) / np.sqrt(var + h(f32(eps)))
    if drop_rounding:                                             # (xc * r) not rounded before the scale multiply
        y = ((xc.astype(f32) * f32(r)) * w.astype(f32)).astype(h)
    else:
        y = (xc * r) * w
    return y + b if b is not None else y


def _rms_norm_f16_model(xr, w, eps, scale_first=False):
    n = h(f32(xr.size))
    sq = xr * xr
    x2 = h(_seq_sum(sq)) / n
    r = h(1.0) / np.sqrt(x2 + h(f32(eps)))
    if scale_first:
        return xr * (r * w)
    return (xr * r) * w


@pytest.mark.parametrize("cols", [96, 513])
def test_layer_norm_f16_bit_exact_stepwise(oracle, cols):
    rng = np.random.default_rng(18)
    x = (rng.standard_normal((6, cols)) + 0.25).astype(h)
    w = (1 + 0.02 * rng.standard_normal(cols)).astype(h)
    b = (0.02 * rng.standard_normal(cols)).astype(h)
    got = oracle.layer_norm(x, w, b, 1e-5, intended=True)
    got_nb = oracle.layer_norm(x, w, None, 1e-5, intended=True)
    dropped = two_pass = 0
    for r in range(x.shape[0]):
        assert np.array_equal(_bits16(_layer_norm_f16_model(x[r], w, b, 1e-5)), _bits16(got[r])), r
        assert np.array_equal(_bits16(_layer_norm_f16_model(x[r], w, None, 1e-5)), _bits16(got_nb[r])), r
        dropped += np.count_nonzero(_bits16(_layer_norm_f16_model(x[r], w, b, 1e-5, drop_rounding=True)) != _bits16(got[r]))
        two_pass += np.count_nonzero(_bits16(_layer_norm_f16_model(x[r], w, b, 1e-5, two_pass=True)) != _bits16(got[r]))
    assert dropped > 0 and two_pass > 0                           # the comparison sees a missing rounding point / another variance


@pytest.mark.parametrize("cols", [96, 513])
def test_rms_norm_f16_bit_exact_stepwise(oracle, cols):
    rng = np.random.default_rng(33)
    x = rng.standard_normal((6, cols)).astype(h)
    w = (1 + 0.02 * rng.standard_normal(cols)).astype(h)
    got = oracle.rms_norm(x, w, 1e-5, intended=True)
    reordered = 0
    for r in range(x.shape[0]):
        assert np.array_equal(_bits16(_rms_norm_f16_model(x[r], w, 1e-5)), _bits16(got[r])), r
        reordered += np.count_nonzero(_bits16(_rms_norm_f16_model(x[r], w, 1e-5, scale_first=True)) != _bits16(got[r]))
    assert reordered > 0


def test_f16_sum_mode_switch_is_visible_to_the_stepwise_models(oracle):
    """With the row sums accumulated in f16 (the other reading of `Sum for f16`) the oracle must leave the models."""
    rng = np.random.default_rng(34)
    cols = 1024
    x = (rng.standard_normal((4, cols)) + 0.5).astype(h)
    w = (1 + 0.02 * rng.standard_normal(cols)).astype(h)
    b = (0.02 * rng.standard_normal(cols)).astype(h)
    want_ln = np.stack([_layer_norm_f16_model(x[r], w, b, 1e-5) for r in range(4)])
    want_rms = np.stack([_rms_norm_f16_model(x[r], w, 1e-5) for r in range(4)])
    assert np.array_equal(_bits16(oracle.layer_norm(x, w, b, 1e-5, intended=True)), _bits16(want_ln))
    assert np.array_equal(_bits16(oracle.rms_norm(x, w, 1e-5, intended=True)), _bits16(want_rms))
    oracle.set_f16_sum_mode(True)
    try:
        ln_seq = oracle.layer_norm(x, w, b, 1e-5, intended=True)
        rms_seq = oracle.rms_norm(x, w, 1e-5, intended=True)
    finally:
        oracle.set_f16_sum_mode(False)
    assert not np.array_equal(_bits16(ln_seq), _bits16(want_ln))
    assert not np.array_equal(_bits16(rms_seq), _bits16(want_rms))
    # and back: the default reading again matches bit for bit
    assert np.array_equal(_bits16(oracle.rms_norm(x, w, 1e-5, intended=True)), _bits16(want_rms))


# ------------------------------------------------------------------------------------------------ bf16 norms
def _layer_norm_bf16_model(xr, w, b, eps, drop_rounding=False):
    n = rb(f32(xr.size))
    mu = rb(rb(_seq_sum(xr)) / n)
    mu2 = rb(mu * mu)
    sq = rb(xr * xr)
    x2 = rb(rb(_seq_sum(sq)) / n)
    var = rb(x2 - mu2)
    xc = rb(xr - mu)
    with np.errstate(all="ignore"):
        r = rb(f32(1.0) / rb(np.sqrt(rb(var + rb(f32(eps))))))
    if drop_rounding:
        y = rb((xc * r) * w)
    else:
        y = rb(rb(xc * r) * w)
    return rb(y + b) if b is not None else y


def _rms_norm_bf16_model(xr, w, eps, drop_rounding=False):
    n = rb(f32(xr.size))
    sq = rb(xr * xr)
    x2 = rb(rb(_seq_sum(sq)) / n)
    r = rb(f32(1.0) / rb(np.sqrt(rb(x2 + rb(f32(eps))))))
    if drop_rounding:
        return rb((xr * r) * w)
    return rb(rb(xr * r) * w)


@pytest.mark.parametrize("cols", [80, 515])
def test_layer_norm_bf16_bit_exact_stepwise(oracle, cols):
    rng = np.random.default_rng(35)
    x = rb((rng.standard_normal((5, cols)) * 1.5 + 1.0).astype(f32))     # a mean away from zero keeps var >= 0 meaningful
    w = rb((1 + 0.02 * rng.standard_normal(cols)).astype(f32))
    b = rb((0.02 * rng.standard_normal(cols)).astype(f32))
    got = oracle.layer_norm(bf16_bits(x), bf16_bits(w), bf16_bits(b), 1e-5, bf16=True, intended=True)
    got_nb = oracle.layer_norm(bf16_bits(x), bf16_bits(w), None, 1e-5, bf16=True, intended=True)
    dropped = 0
    for r in range(x.shape[0]):
        want = _layer_norm_bf16_model(x[r], w, b, 1e-5)
        ok = (bf16_bits(want) == got[r]) | np.isnan(want)
        assert ok.all() and np.array_equal(np.isnan(want), np.isnan(bf16_from_bits(got[r]))), r
        want_nb = _layer_norm_bf16_model(x[r], w, None, 1e-5)
        assert ((bf16_bits(want_nb) == got_nb[r]) | np.isnan(want_nb)).all(), r
        dropped += np.count_nonzero(bf16_bits(_layer_norm_bf16_model(x[r], w, b, 1e-5, drop_rounding=True)) != got[r])
    assert dropped > 0


@pytest.mark.parametrize("cols", [80, 515])
def test_rms_norm_bf16_bit_exact_stepwise(oracle, cols):
    rng = np.random.default_rng(36)
    x = rb(rng.standard_normal((5, cols)).astype(f32))
    w = rb((1 + 0.02 * rng.standard_normal(cols)).astype(f32))
    got = oracle.rms_norm(bf16_bits(x), bf16_bits(w), 1e-5, bf16=True, intended=True)
    dropped = 0
    for r in range(x.shape[0]):
        assert np.array_equal(bf16_bits(_rms_norm_bf16_model(x[r], w, 1e-5)), got[r]), r
        dropped += np.count_nonzero(bf16_bits(_rms_norm_bf16_model(x[r], w, 1e-5, drop_rounding=True)) != got[r])
    assert dropped > 0


# ------------------------------------------------------------------------------------------------ bf16 unary
def test_gelu_bf16_bit_exact_over_all_inputs(oracle):
    """cpu/unary.rs:46-51 in bf16: 0.5 * x * (1 + tanh(0.7978846 * x * (1 + 0.044715 * x * x))), every operator and
    the tanh rounded to bf16, constants converted with bf16::from_f32."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = bf16_from_bits(bits)
    with np.errstate(all="ignore"):
        c0, c1, c2, one = rb(f32(0.5)), rb(f32(0.7978846)), rb(f32(0.044715)), f32(1.0)
        inner = rb(one + rb(rb(c2 * x) * x))
        arg = rb(rb(c1 * x) * inner)
        t = rb(_libm("tanhf", arg))
        want = rb(rb(c0 * x) * rb(one + t))
        unrounded_inner = rb(rb(c0 * x) * rb(one + rb(_libm("tanhf", rb(rb(c1 * x) * (one + (c2 * x) * x))))))
    got = oracle.unary("gelu", bits, bf16=True)
    nan = np.isnan(want)
    assert np.array_equal(nan, np.isnan(bf16_from_bits(got)))
    assert np.array_equal(bf16_bits(want)[~nan], got[~nan])
    assert np.count_nonzero(bf16_bits(unrounded_inner)[~nan] != got[~nan]) > 0


@pytest.mark.parametrize("op", ["silu", "sigmoid", "exp", "tanh"])
def test_unary_bf16_bit_exact_over_all_inputs(oracle, op):
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = bf16_from_bits(bits)
    with np.errstate(all="ignore"):
        if op == "silu":
            want = rb(x / rb(f32(1.0) + rb(_libm("expf", -x))))
        elif op == "sigmoid":
            want = rb(f32(1.0) / rb(f32(1.0) + rb(_libm("expf", -x))))
        else:
            want = rb(_libm(op + "f", x))
    got = oracle.unary(op, bits, bf16=True)
    nan = np.isnan(want)
    assert np.array_equal(nan, np.isnan(bf16_from_bits(got)))
    assert np.array_equal(bf16_bits(want)[~nan], got[~nan])


def test_gelu_f16_bit_exact_over_all_inputs_with_libm_tanhf(oracle):
    """the f16 model with the machine's own tanhf in place of a float64 tanh: no mismatch allowance is needed"""
    x = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(h)
    with np.errstate(all="ignore"):
        inner = h(1.0) + (h(0.044715) * x) * x
        arg = (h(0.7978846) * x) * inner
        t = _libm("tanhf", arg.astype(f32)).astype(h)
        want = (h(0.5) * x) * (h(1.0) + t)
    got = oracle.unary("gelu", x)
    nan = np.isnan(want)
    assert np.array_equal(nan, np.isnan(got))
    assert np.array_equal(_bits16(want)[~nan], _bits16(got)[~nan])
