"""Writes the golden fixtures (inputs + expected outputs) used by the CPU and GPU test suites.

The reference ships no golden vectors for this path and its extension cannot be built or imported
here, so the expected values come from this repository's CPU oracle (oracle/cottention_oracle.c),
which tests/test_oracle_pinning.py pins against brute force, the reference's three closed forms,
autograd and finite differences.  Run from the repository root:

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle, torch_forms as tf  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def causal_case(name, shape, dv, seed):
    q, k, v, g = tf.synthetic_inputs(shape, dv=dv, seed=seed, dtype=torch.float32)
    o = oracle.causal(q, k, v)
    o_rev = oracle.causal(q, k, v, True)
    dq, dk, dv_ = oracle.causal_bwd(q, k, v, g)
    np.savez_compressed(os.path.join(HERE, name), q=q.numpy(), k=k.numpy(), v=v.numpy(), g=g.numpy(),
                        o=o, o_rev=o_rev, dq=dq, dk=dk, dv=dv_)


def noncausal_case(name, shape, dv, seed):
    q, k, v, g = tf.synthetic_inputs(shape, dv=dv, seed=seed, dtype=torch.float32)
    o = oracle.noncausal(q, k, v)
    dq, dk, dv_ = oracle.noncausal_bwd(q, k, v, g)
    np.savez_compressed(os.path.join(HERE, name), q=q.numpy(), k=k.numpy(), v=v.numpy(), g=g.numpy(),
                        o=o, dq=dq, dk=dk, dv=dv_)


def decode_case(name, b, h, dk, dv, steps, seed):
    gen = torch.Generator().manual_seed(seed)
    s0 = (0.01 * torch.randn(b, h, dk, dv, generator=gen)).numpy()
    q = torch.nn.functional.normalize(torch.randn(steps, b, h, dk, generator=gen), dim=-1).numpy()
    k = torch.nn.functional.normalize(torch.randn(steps, b, h, dk, generator=gen), dim=-1).numpy()
    v = torch.randn(steps, b, h, dv, generator=gen).numpy()
    state = s0.astype(np.float64).copy()
    outs = np.stack([oracle.decode_step(state, q[t], k[t], v[t]) for t in range(steps)])
    np.savez_compressed(os.path.join(HERE, name), s0=s0, q=q, k=k, v=v, o=outs, s_final=state)


if __name__ == "__main__":
    causal_case("causal_cfg1_1x2x128x64.npz", (1, 2, 128, 64), 64, seed=0)    # the reference CPU-runnable benchmark case: fp32 (1,2,128,64)
    causal_case("causal_odd_1x2x63x32_dv48.npz", (1, 2, 63, 32), 48, seed=1)   # odd S (Custom_Kernel.py:157), Dk != Dv
    noncausal_case("noncausal_2x2x50x32.npz", (2, 2, 50, 32), 32, seed=2)
    decode_case("decode_2x2x32x48_4steps.npz", 2, 2, 32, 48, 4, seed=3)
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
