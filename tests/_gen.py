"""Seeded synthetic inputs shared by the tests (numpy default_rng, fp32 -> bf16 RNE)."""
from __future__ import annotations

import numpy as np

from oracle import pf8_oracle as O


def bf16_normal(shape, seed, std=1.0, outlier_frac=0.0, outlier_scale=1.0):
    """N(0, std) with a Bernoulli(outlier_frac) mask multiplied by outlier_scale -> bf16 bits."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(shape, dtype=np.float32) * np.float32(std)
    if outlier_frac > 0:
        mask = rng.random(shape, dtype=np.float32) < outlier_frac
        x = np.where(mask, x * np.float32(outlier_scale), x).astype(np.float32)
    return O.f32_to_bf16_bits(x)


def zipf_counts(total, E, s, seed, n_empty=2, pad=128):
    """Expert token counts: p_r ~ r^-s assigned to experts by a seeded permutation, the n_empty
    least likely experts forced to zero, multinomial draw; returns (counts, padded_counts)."""
    rng = np.random.default_rng(seed)
    ranks = np.arange(1, E + 1, dtype=np.float64)
    p = ranks ** (-s)
    if n_empty:
        p[-n_empty:] = 0.0
    p /= p.sum()
    perm = rng.permutation(E)
    pe = np.empty(E)
    pe[perm] = p
    counts = rng.multinomial(total, pe)
    padded = ((counts + pad - 1) // pad) * pad
    return counts.astype(np.int64), padded.astype(np.int64)


def to_torch_bf16(bits, device="cuda"):
    import torch

    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16).to(device)


def from_torch_bf16(t):
    import torch

    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def to_torch_fp8(codes, device="cuda"):
    import torch

    return torch.from_numpy(np.ascontiguousarray(codes)).view(torch.float8_e4m3fn).to(device)


def from_torch_fp8(t):
    import torch

    return t.detach().contiguous().view(torch.uint8).cpu().numpy()


def rel_fro(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def mismatch_report(got, exp, what):
    got, exp = np.asarray(got), np.asarray(exp)
    assert got.shape == exp.shape, f"{what}: shape {got.shape} vs {exp.shape}"
    bad = np.argwhere(got != exp)
    if bad.size == 0:
        return ""
    i = tuple(bad[0])
    return f"{what}: {len(bad)} of {got.size} differ; first at {i}: got {got[i]!r} expected {exp[i]!r}"
