"""The reference's own PyTorch formulations of the hot path, restated -- TEST INFRASTRUCTURE ONLY.

These are the closed forms the reference writes out as text; they run on the host CPU and serve
(a) as independent cross-checks of the C oracle and (b) as the timed `cpu_baseline` (the path a
user of the reference gets without its CUDA extension).  Never imported by the shipped GPU path.
"""
import torch


def causal_cumsum(q, k, v):
    """Cumsum form, GPT_Trainer/GPTCosAttention.py:319 (also Cuda_Kernel/speeds.py:74-75):
    O = ((V[...,None] * K[...,None,:]).cumsum(-3) * Q[...,None,:]).sum(-1)."""
    vk = (v.unsqueeze(-1) * k.unsqueeze(-2)).cumsum(-3)          # (..., N, Dv, Dk)
    return (vk * q.unsqueeze(-2)).sum(-1)


def causal_masked(q, k, v, reversed=False):
    """Masked quadratic form, Cuda_Kernel/speed_test.py:15-20: ((Q K^T) o tril) V."""
    n = q.shape[-2]
    qk = q @ k.transpose(-1, -2)
    mask = torch.ones(n, n, dtype=torch.bool, device=q.device)
    mask = torch.triu(mask) if reversed else torch.tril(mask)
    return qk.masked_fill(~mask, 0) @ v


def causal_recurrent(q, k, v):
    """Token-by-token recurrence of the decode branch, GPT_Trainer/GPTCosAttention.py:262-267,
    with the reference's (Dv, Dk) state orientation."""
    state = torch.zeros(q.shape[:-2] + (v.shape[-1], k.shape[-1]), dtype=q.dtype)
    out = torch.zeros_like(v)
    for s in range(q.shape[-2]):
        state = state + v[..., s, :].unsqueeze(-1) * k[..., s, :].unsqueeze(-2)
        out[..., s, :] = (q[..., s, :].unsqueeze(-2) * state).sum(-1)
    return out


def causal_grads_closed_form(q, k, v, g):
    """Cuda_Kernel/Custom_Kernel.py:63,68,72 -- cumsum closed forms of (dQ, dK, dV)."""
    dq = ((v.unsqueeze(-1) * k.unsqueeze(-2)).cumsum(-3) * g.unsqueeze(-1)).sum(-2)
    suffix = (g.unsqueeze(-1) * q.unsqueeze(-2)).flip(-3).cumsum(-3).flip(-3)   # (..., N, Dv, Dk)
    dk = (suffix * v.unsqueeze(-1)).sum(-2)
    dv = (suffix * k.unsqueeze(-2)).sum(-1)
    return dq, dk, dv


def noncausal_einsum(q, k, v):
    """BERT_Trainer/BertCosAttention.py:249 (D <= S branch)."""
    return torch.einsum("nhsw,nhwe->nhse", q, torch.einsum("nhse,nhsw->nhew", k, v))


def noncausal_quadratic(q, k, v):
    """BERT_Trainer/BertCosAttention.py:222 (D > S branch): (Q K^T) V."""
    return torch.einsum("nhsq,nhqw->nhsw", torch.einsum("nhse,nhqe->nhsq", q, k), v)


def synthetic_inputs(shape_qk, dv=None, seed=0, dtype=torch.float32, with_grad_out=True):
    """Seeded benchmark/parity inputs: Q,K,V,dO ~ N(0,1) in fp32, Q and K L2-normalised along D
    (GPT_Trainer/GPTCosAttention.py:229-230), then cast to `dtype`."""
    gen = torch.Generator().manual_seed(seed)
    b, h, n, dk = shape_qk
    dv = dk if dv is None else dv
    q = torch.nn.functional.normalize(torch.randn(b, h, n, dk, generator=gen), p=2, dim=-1)
    k = torch.nn.functional.normalize(torch.randn(b, h, n, dk, generator=gen), p=2, dim=-1)
    v = torch.randn(b, h, n, dv, generator=gen)
    out = [q.to(dtype), k.to(dtype), v.to(dtype)]
    if with_grad_out:
        out.append(torch.randn(b, h, n, dv, generator=gen).to(dtype))
    return out


def input_prep_gpt(q, k, v, keep=None, sig=None):
    """CPU statement of the module-side preparation in front of the causal op, in the reference's order
    (GPT_Trainer/GPTCosAttention.py:216-235): L2-normalise q and k (:216-217); divide v by
    clamp(cnt ** sig, min=1) with cnt[b,s] = number of kept keys at positions <= s (:228, causal mask times
    padding mask, summed over keys); multiply q, k, v by the keep mask (:232-235).
    q,k: (B,H,N,Dk), v: (B,H,N,Dv), keep: (B,N) bool (True = real token) or None, sig: (H,) or None.
    Returns (q_hat, k_hat, v_scaled, cnt)."""
    b, h, n, _ = q.shape
    km = torch.ones(b, n, dtype=torch.bool) if keep is None else keep.bool()
    qh = torch.nn.functional.normalize(q, dim=-1, p=2)
    kh = torch.nn.functional.normalize(k, dim=-1, p=2)
    causal = torch.tril(torch.ones(n, n, dtype=q.dtype))                       # [s, t] = 1 for t <= s
    cnt = (causal[None, None] * km[:, None, None, :].to(q.dtype)).sum(-1, keepdim=True)   # (B,1,N,1)
    vs = v
    if sig is not None:
        vs = v / (cnt ** sig.reshape(1, h, 1, 1)).clamp(min=1)
    m = km[:, None, :, None].to(q.dtype)
    return qh * m, kh * m, vs * m, cnt.reshape(b, n)


def input_prep_bert(q, k, v, keep=None, sig=None):
    """Same for the non-causal module, in ITS order (BERT_Trainer/BertCosAttention.py:162-178): mask first
    (:164-167), normalise (:171-172), divide v by clamp(total_kept ** sig, min=1) (:178)."""
    b, h, n, _ = q.shape
    km = torch.ones(b, n, dtype=torch.bool) if keep is None else keep.bool()
    m = km[:, None, :, None].to(q.dtype)
    qh = torch.nn.functional.normalize(q * m, dim=-1, p=2)
    kh = torch.nn.functional.normalize(k * m, dim=-1, p=2)
    cnt = km.sum(-1).to(q.dtype).reshape(b, 1, 1, 1)
    vs = v * m
    if sig is not None:
        vs = vs / (cnt ** sig.reshape(1, h, 1, 1)).clamp(min=1)
    return qh, kh, vs, cnt.reshape(b, 1).expand(b, n).contiguous()
