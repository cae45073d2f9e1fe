"""CPU-only checks that pin the oracle's scalar arithmetic: conversions, binary ops, casts.

Referees: numpy's float16/float32 (an independent IEEE-754 implementation) and closed forms.
"""
import numpy as np
import pytest

ALL_F16 = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16)


def _bits(a):
    return a.view({2: np.uint16, 4: np.uint32}[a.dtype.itemsize])


def _same_bits_or_nan(a, b):
    """bit equality, except that any NaN matches any NaN (payloads are not part of the contract)"""
    a, b = np.asarray(a), np.asarray(b)
    both_nan = np.isnan(a) & np.isnan(b)
    return np.all((_bits(a) == _bits(b)) | both_nan)


def test_f16_to_f32_exhaustive(oracle):
    got = oracle.cast(ALL_F16, np.float32)
    assert _same_bits_or_nan(got, ALL_F16.astype(np.float32))


@pytest.mark.parametrize("hw", [0, 1])
def test_f32_to_f16_matches_numpy(oracle, hw):
    oracle.set_hw_f16(hw)
    try:
        rng = np.random.default_rng(1)
        # random bit patterns cover every exponent; plus values straddling every f16 rounding boundary
        rand = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
        mid = ALL_F16.astype(np.float32)
        finite = mid[np.isfinite(mid)]
        ties = (finite[:-1].astype(np.float64) + np.roll(finite, -1)[:-1].astype(np.float64)) / 2
        ties = ties[np.isfinite(ties)].astype(np.float32)
        edge = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e-8, 2.98e-8, 2.9802322e-8, 3e-8, 5.96e-8,
                         6.1e-5, 6.0975552e-05, np.inf, -np.inf, np.nan, 1e-5, 1e38, -1e38], dtype=np.float32)
        near = np.concatenate([np.nextafter(ties, np.float32(np.inf)), np.nextafter(ties, np.float32(-np.inf))])
        x = np.concatenate([rand, finite, ties, near, edge])
        with np.errstate(over="ignore", invalid="ignore"):
            want = x.astype(np.float16)
        got = oracle.cast(x, np.float16)
        assert _same_bits_or_nan(got, want)
    finally:
        oracle.set_hw_f16(1)


def test_hw_and_soft_conversions_agree_on_nan_payloads(oracle):
    x = np.array([0x7fc00001, 0x7f800001, 0xffc12345, 0x7fffe000], dtype=np.uint32).view(np.float32)
    oracle.set_hw_f16(0)
    soft = oracle.cast(x, np.float16)
    oracle.set_hw_f16(1)
    hw = oracle.cast(x, np.float16)
    assert np.array_equal(_bits(soft), _bits(hw))
    assert np.all(np.isnan(soft))


def test_bf16_round_trip_and_rounding(oracle):
    rng = np.random.default_rng(2)
    x = rng.standard_normal(100000).astype(np.float32)
    got = oracle.cast(x, np.uint16, dst_bf16=True)
    # independent model: round-to-nearest-even on the upper 16 bits
    u = x.view(np.uint32).astype(np.uint64)
    want = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(got, want)
    back = oracle.cast(got, np.float32, src_bf16=True)
    assert np.array_equal(back.view(np.uint32), want.astype(np.uint32) << 16)


def test_cast_f32_int_is_a_bit_reinterpretation(oracle):
    # crates/ratchet-core/src/cpu/mod.rs:116-125: bytemuck::try_cast_slice, not a numeric conversion
    x = np.array([1.0, -2.5, 0.0, 3e9], dtype=np.float32)
    assert np.array_equal(oracle.cast(x, np.int32), x.view(np.int32))
    assert np.array_equal(oracle.cast(x, np.uint32), x.view(np.uint32))
    i = np.array([0x3f800000, 0x40490fdb], dtype=np.uint32)
    assert np.array_equal(oracle.cast(i, np.float32).view(np.uint32), i)


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_binary_bit_exact_vs_numpy(oracle, op, dtype):
    rng = np.random.default_rng(3)
    n = 300_000
    a = (rng.standard_normal(n) * 10 ** rng.uniform(-6, 4, n)).astype(dtype)
    b = (rng.standard_normal(n) * 10 ** rng.uniform(-6, 4, n)).astype(dtype)
    specials = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504, 6e-8, -6e-8, 1, -1], dtype=dtype)
    a = np.concatenate([a, np.repeat(specials, len(specials))])
    b = np.concatenate([b, np.tile(specials, len(specials))])
    with np.errstate(all="ignore"):
        want = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}[op](a, b)
    got = oracle.binary(op, a, b)
    assert want.dtype == got.dtype
    assert _same_bits_or_nan(got, want)


def test_binary_f16_all_pairs_subsample_against_float64(oracle):
    # f16 (op) f16 computed exactly in float64 then rounded once is the IEEE answer for + - * (exact in f64)
    rng = np.random.default_rng(4)
    a = ALL_F16[rng.integers(0, 65536, 500_000)]
    b = ALL_F16[rng.integers(0, 65536, 500_000)]
    with np.errstate(all="ignore"):
        for op, f in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply)):
            want = f(a.astype(np.float64), b.astype(np.float64)).astype(np.float16)
            assert _same_bits_or_nan(oracle.binary(op, a, b), want), op


def test_binary_reference_copies_do_not_change_results(oracle):
    rng = np.random.default_rng(5)
    a = rng.standard_normal(1000).astype(np.float16)
    b = rng.standard_normal(1000).astype(np.float16)
    with_copies = oracle.binary("div", a, b)
    oracle.set_reference_copies(False)
    try:
        assert np.array_equal(_bits(oracle.binary("div", a, b)), _bits(with_copies))
    finally:
        oracle.set_reference_copies(True)


def test_all_close_rule(oracle):
    # crates/ratchet-core/src/tensor.rs:1039-1043
    a = np.array([1.0, np.nan, np.inf, -np.inf, np.inf, 1.0, 0.0], dtype=np.float32)
    b = np.array([1.00001, np.nan, np.inf, -np.inf, -np.inf, 1.1, 1e-6], dtype=np.float32)
    bad, mx = oracle.count_not_close(a, b, 1e-4, 1e-4)
    # 1.0 vs 1.1 fails; inf vs -inf passes the third clause (inf <= atol + rtol*inf), as it does in the reference
    assert bad == 1
    bad, _ = oracle.count_not_close(a[:4], b[:4], 1e-4, 1e-4)
    assert bad == 0
