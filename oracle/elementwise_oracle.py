"""CPU restatement (numpy) of the element-wise fp16 steps of the reference's extension module.

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg; the
product never imports it.

  rms_norm              longserve_cuda_kernels/src/rms_norm.cu:19-47
  silu_and_mul_inplace  longserve_cuda_kernels/src/silu_and_mul.cu:14-17, :26-35
  rotary_emb            longserve_cuda_kernels/src/rotary_emb.cu:23-35

How each is pinned (tests/test_oracle_pins.py): rms_norm and silu against torch's float64 formulas
(x * w / sqrt(mean(x^2) + eps), x * sigmoid(x) * up) within one fp16 rounding; rotary against the rotation identity
(complex multiplication by cos + i sin, norm preservation for cos^2 + sin^2 = 1) and, for the roundings, against
exact rational arithmetic (fractions.Fraction) on small inputs.  The reference holds no golden vectors for these
functions (there is no test of them in the reference tree); parity with its fast-math `__expf`/`rsqrtf` bit patterns
is unpinned and below the fp16 rounding the tests allow.
"""
from __future__ import annotations

import numpy as np


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """x [T, H] float16, w [H] float16 -> float16; sum of squares in float64, the product in float32 in the reference's
    order (a * b * inv_rms, rms_norm.cu:42-45), one rounding to half."""
    xf = x.astype(np.float32)
    ss = (x.astype(np.float64) ** 2).sum(axis=1)
    inv = (1.0 / np.sqrt(ss / x.shape[1] + np.float64(eps))).astype(np.float32)
    return ((xf * w.astype(np.float32)[None, :]) * inv[:, None]).astype(np.float16)


def silu_and_mul_inplace(io: np.ndarray) -> None:
    """io [T, 2I] float16: io[:, :I] = half(silu(gate)) * up with a half multiply (silu_and_mul.cu:30-33)."""
    inter = io.shape[1] // 2
    g = io[:, :inter].astype(np.float64)
    s = (g / (1.0 + np.exp(-g))).astype(np.float16)          # one rounding float64 -> half
    io[:, :inter] = (s.astype(np.float32) * io[:, inter:].astype(np.float32)).astype(np.float16)  # exact product, one rounding


def rotary_emb(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> None:
    """x [T, H, D] float16 in place, cos/sin [T, D/2] float16 (rotary_emb.cu:26-35): x1 = x[..., :D/2], x2 = x[..., D/2:],
    x1' = fma(x1, cos, -(x2*sin)), x2' = fma(x1, sin, x2*cos); the inner products are rounded to half, the fma once.
    A product of two halves is exact in float32 and the fused sums here are exact in float64 for operands within
    2^-14 .. 2^15, so float64 -> half conversion performs the single rounding."""
    half = x.shape[2] // 2
    x1, x2 = x[..., :half].copy(), x[..., half:].copy()
    c, s = cos[:, None, :], sin[:, None, :]
    t1 = (x2.astype(np.float32) * s.astype(np.float32)).astype(np.float16)
    t2 = (x2.astype(np.float32) * c.astype(np.float32)).astype(np.float16)
    x[..., :half] = (x1.astype(np.float64) * c.astype(np.float64) - t1.astype(np.float64)).astype(np.float16)
    x[..., half:] = (x1.astype(np.float64) * s.astype(np.float64) + t2.astype(np.float64)).astype(np.float16)
