"""Seeded synthetic tensors with the statistics the benchmark configurations name.

All generators return raw bf16 bit patterns (uint16) so that the same array can be
fed to the packer, uploaded to the GPU and compared bit for bit.
"""
from __future__ import annotations

import numpy as np


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bits, round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def weights_llm(M: int, K: int, seed: int, sigma: float = 0.02, p_outlier: float = 3e-4,
                sigma_outlier: float = 8.0) -> np.ndarray:
    """N(0, sigma) with each entry independently replaced, with probability
    p_outlier, by N(0, sigma_outlier): the LLM-like law (~0.03-0.05 % escapes)."""
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((M, K), dtype=np.float32) * np.float32(sigma)
    if p_outlier > 0:
        n_out = rng.binomial(M * K, p_outlier)
        idx = rng.integers(0, M * K, size=n_out)
        w.reshape(-1)[idx] = rng.standard_normal(n_out, dtype=np.float32) * np.float32(sigma_outlier)
    return f32_to_bf16_bits(w)


def weights_diffusion(M: int, K: int, seed: int, sigma_a: float = 0.05, sigma_b: float = 1.0,
                      p_b: float = 0.02) -> np.ndarray:
    """Mixture (1-p_b) N(0, sigma_a) + p_b N(0, sigma_b): the escape-heavy law
    (~0.2-1 % escapes, every row holding several)."""
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((M, K), dtype=np.float32) * np.float32(sigma_a)
    mask = rng.random((M, K), dtype=np.float32) < np.float32(p_b)
    w[mask] = rng.standard_normal(int(mask.sum()), dtype=np.float32) * np.float32(sigma_b)
    return f32_to_bf16_bits(w)


def activations(B: int, K: int, seed: int, sigma: float = 1.0) -> np.ndarray:
    """bf16 activations ~ N(0, sigma), shape [B, K]."""
    rng = np.random.default_rng(seed)
    return f32_to_bf16_bits(rng.standard_normal((B, K), dtype=np.float32) * np.float32(sigma))
