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
    (GPT_Trainer/GPTCosAttention.py:229-248): L2-normalise q and k (:229-230); divide v by
    clamp(cnt ** sig, min=1) with cnt[b,s] = number of kept keys at positions <= s (:241, causal mask times
    padding mask, summed over keys); multiply q, k, v by the keep mask (:243-248).
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


# ---- module level: the attention blocks around the op, as the reference writes them, in plain torch -------------

def gptj_sinusoid_table(num_pos, dim):
    """GPT-J rotary table (transformers.models.gptj.modeling_gptj.create_sinusoidal_positions, imported by the
    reference at GPT_Trainer/GPTCosAttention.py:7): columns [sin(p f_0..f_{dim/2-1}) | cos(...)], f_i = 10000^(-2i/dim)."""
    freqs = torch.tensor([10000.0 ** (-(2 * i) / dim) for i in range(dim // 2)], dtype=torch.float32)
    ang = torch.outer(torch.arange(num_pos, dtype=torch.float32), freqs)
    return torch.cat((ang.sin(), ang.cos()), dim=1)


def gptj_rotate(x, sin, cos):
    """apply_rotary_pos_emb of GPT-J: x*cos + rotate_every_two(x)*sin with sin/cos repeated pairwise.
    x: (B,S,H,R); sin, cos: (B,S,R/2)."""
    sin = torch.repeat_interleave(sin[:, :, None, :], 2, 3)
    cos = torch.repeat_interleave(cos[:, :, None, :], 2, 3)
    rot = torch.stack((-x[..., 1::2], x[..., ::2]), dim=-1).flatten(-2)
    return x * cos + rot * sin


def _gpt_qkv(hidden, wq, wk, wv, num_heads, rotary_dim, max_pos, position_ids):
    b, s, e = hidden.shape
    d = e // num_heads
    q = (hidden @ wq.T).view(b, s, num_heads, d)
    k = (hidden @ wk.T).view(b, s, num_heads, d)
    v = (hidden @ wv.T).view(b, s, num_heads, d).permute(0, 2, 1, 3)
    table = gptj_sinusoid_table(max_pos, rotary_dim or e).to(hidden.dtype)
    sincos = table[position_ids]
    sin, cos = torch.split(sincos, sincos.shape[-1] // 2, dim=-1)
    if rotary_dim is not None:
        k = torch.cat([gptj_rotate(k[..., :rotary_dim], sin, cos), k[..., rotary_dim:]], dim=-1)
        q = torch.cat([gptj_rotate(q[..., :rotary_dim], sin, cos), q[..., rotary_dim:]], dim=-1)
    else:
        k, q = gptj_rotate(k, sin, cos), gptj_rotate(q, sin, cos)
    return q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v


def gpt_attention_block(hidden, wq, wk, wv, wo, norm_const, num_heads, rotary_dim, max_pos, keep=None, position_ids=None):
    """Training/evaluation path of the GPT block (GPT_Trainer/GPTCosAttention.py:430-506 with _cos_attn :200-282):
    projections, rotary, input preparation, causal cosine attention, merge heads, output projection.
    hidden: (B,S,E); weights as nn.Linear stores them; norm_const: (H,); keep: (B,S) bool."""
    b, s, e = hidden.shape
    if position_ids is None:
        position_ids = torch.arange(s)[None, :].expand(b, s)
    q, k, v = _gpt_qkv(hidden, wq, wk, wv, num_heads, rotary_dim, max_pos, position_ids)
    qh, kh, vs, _ = input_prep_gpt(q, k, v, keep, torch.sigmoid(norm_const))
    out = causal_cumsum(qh, kh, vs)
    return out.permute(0, 2, 1, 3).reshape(b, s, e) @ wo.T


def gpt_attention_block_recurrent(hidden, wq, wk, wv, wo, norm_const, num_heads, rotary_dim, max_pos, state, cur_s,
                                  keep=None, position_ids=None):
    """Recurrent-inference path (:222-223 value scaling by absolute position, :253-272 per-token loop).
    state: (B,H,Dv,Dk) as the reference keeps it (sum of v (x) k); returns (output, state, cur_s)."""
    b, s, e = hidden.shape
    if position_ids is None:
        position_ids = torch.arange(cur_s - 1, cur_s - 1 + s)[None, :].expand(b, s)
    q, k, v = _gpt_qkv(hidden, wq, wk, wv, num_heads, rotary_dim, max_pos, position_ids)
    q = torch.nn.functional.normalize(q, dim=-1, p=2)
    k = torch.nn.functional.normalize(k, dim=-1, p=2)
    pos = (cur_s + torch.arange(s)).reshape(1, 1, -1, 1).to(hidden.dtype)
    v = v / (pos ** torch.sigmoid(norm_const).reshape(1, num_heads, 1, 1)).clamp(min=1)
    if keep is not None:
        m = keep[:, None, :, None].to(hidden.dtype)
        q, k, v = q * m, k * m, v * m
    out = torch.zeros_like(v)
    for t in range(s):
        state = state + v[:, :, t].unsqueeze(-1) * k[:, :, t].unsqueeze(-2)
        out[:, :, t] = (q[:, :, t].unsqueeze(-2) * state).sum(-1)
        cur_s += 1
    return out.permute(0, 2, 1, 3).reshape(b, s, e) @ wo.T, state, cur_s


def bert_attention_block(hidden, wq, bq, wk, bk, wv, bv, norm_const, num_heads, keep=None):
    """BERT self-attention block (BERT_Trainer/BertCosAttention.py:111-334): projections with bias, mask, normalise,
    value scaling by the number of real tokens, Q (K^T V), merge heads."""
    b, s, e = hidden.shape
    d = e // num_heads

    def heads(x):
        return x.view(b, s, num_heads, d).permute(0, 2, 1, 3)
    q, k, v = heads(hidden @ wq.T + bq), heads(hidden @ wk.T + bk), heads(hidden @ wv.T + bv)
    qh, kh, vs, _ = input_prep_bert(q, k, v, keep, torch.sigmoid(norm_const))
    return noncausal_einsum(qh, kh, vs).permute(0, 2, 1, 3).reshape(b, s, e)
