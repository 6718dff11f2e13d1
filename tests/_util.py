"""Shared helpers for the parity tests (metrics follow the reference's own test precedents)."""
import numpy as np
import torch

import oracle


def mixed_err(actual, expected):
    """max |a - e| / (1 + |e|): the gate of TransformerMatmulPerfTests.cs:52-54 (tests/AiDotNet.Tensors.Tests)."""
    a = np.asarray(actual, np.float64); e = np.asarray(expected, np.float64)
    return float(np.max(np.abs(a - e) / (1.0 + np.abs(e)))) if a.size else 0.0


def rel_frobenius(actual, expected):
    """Relative Frobenius error (Fp16TensorCoreGemmTests.cs:81-90)."""
    a = np.asarray(actual, np.float64); e = np.asarray(expected, np.float64)
    return float(np.linalg.norm(a - e) / max(np.linalg.norm(e), 1e-30))


def dyadic(rng, shape, hi=8, div=8.0):
    """Small integers / div: partial sums are exact in fp32, every summation order gives the same bits."""
    return (rng.integers(-hi, hi + 1, size=shape).astype(np.float32)) / np.float32(div)


def dev(x, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(x))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def bits16(t: torch.Tensor) -> np.ndarray:
    """fp16 / bf16 device tensor -> uint16 bit patterns on the host."""
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def from_bits16(bits: np.ndarray, dtype) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(dtype).cuda()


def round_to(x: np.ndarray, kind: str):
    """Round fp32 host data to the storage type with the ORACLE's conversion; returns (bits, widened fp32)."""
    if kind == "f16":
        b = oracle.f32_to_f16(x); return b, oracle.f16_to_f32(b)
    b = oracle.f32_to_bf16(x); return b, oracle.bf16_to_f32(b)


TORCH16 = {"f16": torch.float16, "bf16": torch.bfloat16}
