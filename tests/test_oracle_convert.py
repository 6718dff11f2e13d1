"""Pins the oracle's storage conversions against closed forms, numpy and torch.

Reference contract: src/AiDotNet.Tensors/NumericOperations/BFloat16.cs:64-90 and the
cases of tests/AiDotNet.Tensors.Tests/NumericOperations/BFloat16Tests.cs:17-35, 52-69.
"""
import numpy as np
import torch

import oracle


def _bits(x):
    return np.array(x, np.float32).view(np.uint32)


def test_bf16_known_bit_patterns():
    L = oracle.lib()
    assert L.orc_bf16_from_float(1.0) == 0x3F80          # BFloat16.One.RawValue
    assert L.orc_bf16_from_float(-1.0) == 0xBF80
    assert L.orc_bf16_from_float(0.0) == 0x0000
    assert L.orc_bf16_from_float(float("inf")) == 0x7F80
    assert L.orc_bf16_from_float(float("-inf")) == 0xFF80
    # ties: 1 + 2^-8 is exactly half way between 0x3F80 and 0x3F81 -> even (0x3F80)
    assert L.orc_bf16_from_float(1.0 + 2.0 ** -8) == 0x3F80
    # 1 + 3*2^-8 is half way between 0x3F81 and 0x3F82 -> even (0x3F82)
    assert L.orc_bf16_from_float(1.0 + 3 * 2.0 ** -8) == 0x3F82
    # just above the tie rounds up
    assert L.orc_bf16_from_float(np.float32(1.0 + 2.0 ** -8 + 2.0 ** -20)) == 0x3F81
    # largest finite float rounds to +Inf in bf16 (mantissa carry into the exponent)
    assert L.orc_bf16_from_float(np.finfo(np.float32).max) == 0x7F80


def test_bf16_nan_keeps_quiet_bit():
    out = oracle.f32_to_bf16(np.array([0x7F800001, 0xFF800001, 0x7FC00000, 0x7FFFFFFF], np.uint32).view(np.float32))
    assert list(out) == [0x7FC0, 0xFFC0, 0x7FC0, 0x7FFF]
    assert np.isnan(oracle.bf16_to_f32(out)).all()


def test_bf16_lossless_round_trip_values():
    vals = np.array([0, 1, -1, 2, 0.5, 1024, -1024, np.inf, -np.inf], np.float32)
    assert np.array_equal(oracle.bf16_to_f32(oracle.f32_to_bf16(vals)), vals)


def test_bf16_matches_torch_rne_on_random_and_special_bits():
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2 ** 32, size=400_000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    finite = ~np.isnan(x)
    got = oracle.f32_to_bf16(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got[finite], want[finite])
    # closed form on everything that is not NaN
    b = bits[finite].astype(np.uint64)
    cf = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(got[finite], cf)
    # random round trip relative error < 2^-8 (BFloat16Tests.cs:52-69 asserts < 5e-3)
    y = rng.standard_normal(10000).astype(np.float32)
    back = oracle.bf16_to_f32(oracle.f32_to_bf16(y))
    assert np.max(np.abs(back - y) / np.abs(y)) <= 2.0 ** -8


def test_f16_widen_exhaustive_against_numpy():
    allbits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32(allbits)
    want = allbits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(got[nan]).all()


def test_f16_narrow_matches_numpy_rne():
    rng = np.random.default_rng(2)
    xs = [rng.standard_normal(200_000).astype(np.float32) * s for s in (1.0, 1e-3, 1e-6, 1e-8, 300.0, 7e4)]
    # every half value, the midpoints between neighbours and their float neighbours
    allh = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mid = (allh[:-1].astype(np.float64) + allh[1:].astype(np.float64)) / 2
    mid32 = mid.astype(np.float32)
    xs += [allh, -allh, mid32, -mid32, np.nextafter(mid32, np.float32(np.inf)), np.nextafter(mid32, np.float32(-np.inf))]
    xs += [np.array([65504, 65519.99, 65520, 65536, 1e9, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25,
                     np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -26, 0.0, -0.0], np.float32)]
    x = np.concatenate(xs)
    got = oracle.f32_to_f16(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    assert np.isnan(oracle.f16_to_f32(oracle.f32_to_f16(np.array([np.nan], np.float32)))).all()


def test_hash_generator_matches_python_restatement():
    # GpuCpuConsistencyTests.cs:100-109 in plain Python integer arithmetic
    def ref(v):
        x = (v * 747796405 + 2891336453) & 0xFFFFFFFF
        x = ((((x >> ((x >> 28) + 4)) ^ x) * 277803737)) & 0xFFFFFFFF
        x = ((x >> 22) ^ x) & 0xFFFFFFFF
        return np.float32(np.float32(x & 0xFFFF) / np.float32(65535.0)) - np.float32(0.5)
    got = oracle.hash_uniform(2000, seed=12345)
    want = np.array([ref((i + 12345) & 0xFFFFFFFF) for i in range(2000)], np.float32)
    assert np.array_equal(got, want)
    assert got.min() >= -0.5 and got.max() <= 0.5 and abs(got.mean()) < 0.05
