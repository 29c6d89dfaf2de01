"""Shared helpers for the parity tests."""
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# Tolerances of the benchmark definition: rel-L2 <= 1e-4 for fp32 inputs, <= 2e-2 for bf16/fp16 inputs against the
# fp32/fp64 oracle evaluated on the same rounded inputs; fp64 is held to 1e-12.
TOL = {torch.float32: 1e-4, torch.float64: 1e-12, torch.float16: 2e-2, torch.bfloat16: 2e-2}


def rel_l2(x, ref):
    x = x.detach().double().cpu().numpy() if hasattr(x, "detach") else np.asarray(x, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.linalg.norm(x - ref) / max(np.linalg.norm(ref), 1e-300))


def worst_block(x, ref, rows=64):
    """Largest rel-L2 over blocks of `rows` consecutive positions of any head; x, ref: (..., N, D)."""
    x = x.detach().double().cpu().numpy() if hasattr(x, "detach") else np.asarray(x, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    n, d = ref.shape[-2:]
    pad = (-n) % rows
    if pad:
        widths = [(0, 0)] * (ref.ndim - 2) + [(0, pad), (0, 0)]
        x, ref = np.pad(x, widths), np.pad(ref, widths)
    shape = ref.shape[:-2] + ((n + pad) // rows, rows * d)
    num = np.linalg.norm((x - ref).reshape(shape), axis=-1)
    den = np.linalg.norm(ref.reshape(shape), axis=-1)
    return float(np.max(num / np.maximum(den, 1e-300)))


def inputs(b, h, n, dk, dv, dtype, seed=0):
    """Seeded Q,K,V,dO ~ N(0,1); Q,K L2-normalised along D (GPTCosAttention.py:229-230); cast to dtype."""
    g = torch.Generator().manual_seed(seed)
    q = torch.nn.functional.normalize(torch.randn(b, h, n, dk, generator=g), p=2, dim=-1).to(dtype)
    k = torch.nn.functional.normalize(torch.randn(b, h, n, dk, generator=g), p=2, dim=-1).to(dtype)
    v = torch.randn(b, h, n, dv, generator=g).to(dtype)
    do = torch.randn(b, h, n, dv, generator=g).to(dtype)
    return q, k, v, do


def load_golden(name):
    return dict(np.load(os.path.join(GOLDEN, name)))
