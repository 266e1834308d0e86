"""Shared test helpers: seeded synthetic data and error measures."""
from __future__ import annotations

import numpy as np

import oracle


def rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def normal_bf16(seed: int, shape, std: float = 1.0, mean: float = 0.0) -> np.ndarray:
    return oracle.f32_to_bf16((rng(seed).standard_normal(shape, dtype=np.float32) * std + mean).astype(np.float32))


def make_qweight(seed: int, n: int, k: int, bits: int = 4, group: int = 64, std: float = 0.02) -> oracle.QWeight:
    """W ~ N(0, std^2) in fp32 from PCG64(seed), MLX-affine quantised (bits 4/8) or rounded to bf16 (bits 16)."""
    w = (rng(seed).standard_normal((n, k), dtype=np.float32) * std).astype(np.float32)
    if bits == 16:
        return oracle.dense(oracle.f32_to_bf16(w))
    return oracle.quantize(w, bits, group)


def rel_l2(got_bf16: np.ndarray, ref_f32: np.ndarray) -> float:
    g = oracle.bf16_to_f32(got_bf16).astype(np.float64).ravel()
    r = np.asarray(ref_f32, dtype=np.float64).ravel()
    return float(np.linalg.norm(g - r) / max(np.linalg.norm(r), 1e-30))


def bf16_mismatch(a: np.ndarray, b: np.ndarray):
    """(fraction of elements whose bf16 bits differ, max difference in bf16 ulps of the larger magnitude)."""
    a = np.asarray(a, dtype=np.uint16).ravel()
    b = np.asarray(b, dtype=np.uint16).ravel()
    diff = a != b
    if not diff.any():
        return 0.0, 0.0
    fa, fb = oracle.bf16_to_f32(a).astype(np.float64), oracle.bf16_to_f32(b).astype(np.float64)
    mag = np.maximum(np.abs(fa), np.abs(fb))
    ulp = np.where(mag > 0, 2.0 ** (np.floor(np.log2(np.maximum(mag, 1e-38))) - 7), 1e-38)
    return float(diff.mean()), float((np.abs(fa - fb) / ulp).max())


def to_device(fk, W: oracle.QWeight):
    return fk.DeviceWeight(W.w, W.scales, W.biases, W.n, W.k, W.bits, W.group)
