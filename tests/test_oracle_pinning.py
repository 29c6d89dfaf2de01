"""Pins the CPU oracle (oracle/cottention_oracle.c) before anything is compared against it.

The reference holds no golden vectors for this path, so every oracle routine is pinned by
(1) a brute-force evaluation of the defining sum written independently here, (2) agreement of the
three formulations the reference writes down (cumsum, masked quadratic, recurrence), (3) automatic
and numerical differentiation, and (4) special cases with a hand-computable answer.  A dropped
term, a wrong sign, a transposed operand or an off-by-one on the diagonal fails at least one.
"""
import itertools

import numpy as np
import pytest
import torch

from oracle import torch_forms as tf


def rnd(*shape, seed=0):
    return np.random.default_rng(seed).standard_normal(shape)


def brute_causal(A, B, C, reversed=False):
    """Defining sum, four nested Python loops: out[s,j] = sum_i A[s,i] sum_{s'} B[s',i] C[s',j]."""
    N, Di = A.shape
    Dj = C.shape[1]
    out = np.zeros((N, Dj))
    for s in range(N):
        rng_ = range(s, N) if reversed else range(0, s + 1)
        for j in range(Dj):
            for i in range(Di):
                for t in rng_:
                    out[s, j] += A[s, i] * B[t, i] * C[t, j]
    return out


@pytest.mark.parametrize("reversed_", [False, True])
def test_causal_loop_vs_brute_force(oracle, reversed_):
    A, B, C = rnd(6, 3, seed=1), rnd(6, 3, seed=2), rnd(6, 2, seed=3)
    want = brute_causal(A, B, C, reversed_)
    assert np.allclose(oracle.causal(A, B, C, reversed_), want, atol=1e-12)
    assert np.allclose(oracle.causal_masked(A, B, C, reversed_), want, atol=1e-12)


def test_causal_diagonal_included_and_first_row(oracle):
    # N=1: O = (q.k) v ; the reference updates the state before the dot product
    # (combined_kernel_general.cu:143-149), so s'=s is part of the sum.
    q, k, v = rnd(1, 4, seed=4), rnd(1, 4, seed=5), rnd(1, 3, seed=6)
    assert np.allclose(oracle.causal(q, k, v), (q @ k.T) * v)
    # one-hot keys/queries pick out running sums of V: q_s = k_s = e_0 -> O_s = sum_{t<=s} v_t
    N = 7
    e0 = np.zeros((N, 4)); e0[:, 0] = 1.0
    v = rnd(N, 3, seed=7)
    assert np.allclose(oracle.causal(e0, e0, v), np.cumsum(v, axis=0))
    assert np.allclose(oracle.causal(e0, e0, v, True), np.cumsum(v[::-1], axis=0)[::-1])


@pytest.mark.parametrize("shape", [(1, 2, 128, 64, 64), (2, 3, 63, 32, 48), (1, 1, 33, 64, 32)])
def test_three_reference_forms_agree(oracle, shape):
    b, h, n, dk, dv = shape
    q, k, v = (torch.from_numpy(rnd(b, h, n, d, seed=i)) for i, d in enumerate((dk, dk, dv)))
    o_loop = oracle.causal(q, k, v)
    assert np.allclose(o_loop, tf.causal_cumsum(q, k, v).numpy(), atol=1e-10)       # GPTCosAttention.py:319
    assert np.allclose(o_loop, tf.causal_masked(q, k, v).numpy(), atol=1e-10)       # speed_test.py:15-20
    assert np.allclose(o_loop, tf.causal_recurrent(q, k, v).numpy(), atol=1e-10)    # GPTCosAttention.py:262-267
    assert np.allclose(o_loop, oracle.causal_masked(q, k, v), atol=1e-10)


def test_reversed_is_flip_of_forward(oracle):
    # combined_kernel_general.cu:126-130: s = S - s_ - 1
    A, B, C = rnd(2, 19, 8, seed=1), rnd(2, 19, 8, seed=2), rnd(2, 19, 5, seed=3)
    f = lambda x: x[:, ::-1].copy()
    assert np.allclose(oracle.causal(A, B, C, True), f(oracle.causal(f(A), f(B), f(C), False)))
    q, k, v = (torch.from_numpy(x) for x in (A, B, C))
    assert np.allclose(oracle.causal(A, B, C, True), tf.causal_masked(q, k, v, reversed=True).numpy())


@pytest.mark.parametrize("shape", [(1, 2, 63, 16, 16), (2, 2, 20, 8, 12)])
def test_causal_bwd_vs_autograd_and_closed_forms(oracle, shape):
    b, h, n, dk, dv = shape
    q, k, v, g = (torch.from_numpy(rnd(b, h, n, d, seed=10 + i)) for i, d in enumerate((dk, dk, dv, dv)))
    dq, dk_, dv_ = oracle.causal_bwd(q, k, v, g)
    # autograd through the cumsum closed form (independent of the hand-written gradient formulas)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    tf.causal_cumsum(qa, ka, va).backward(g)
    for got, want in ((dq, qa.grad), (dk_, ka.grad), (dv_, va.grad)):
        assert np.allclose(got, want.numpy(), atol=1e-10)
    # Custom_Kernel.py:63,68,72
    for got, want in zip((dq, dk_, dv_), tf.causal_grads_closed_form(q, k, v, g)):
        assert np.allclose(got, want.numpy(), atol=1e-10)
    # Custom_Kernel.py:106-108: the three gradients are the generic op with permuted operands
    assert np.allclose(dq, oracle.causal(g, v, k, False), atol=1e-10)
    assert np.allclose(dk_, oracle.causal(v, g, q, True), atol=1e-10)
    assert np.allclose(dv_, oracle.causal(k, q, g, True), atol=1e-10)


def _fd_check(fwd, bwd, inputs, g, eps=1e-6, n_probe=40, seed=0):
    """Central differences of <fwd(inputs), g> against the analytic gradient at random entries."""
    grads = bwd(*inputs, g)
    rng = np.random.default_rng(seed)
    for which, x in enumerate(inputs):
        for _ in range(n_probe):
            idx = tuple(rng.integers(0, s) for s in x.shape)
            xp = [a.copy() for a in inputs]; xm = [a.copy() for a in inputs]
            xp[which][idx] += eps; xm[which][idx] -= eps
            num = ((fwd(*xp) - fwd(*xm)) * g).sum() / (2 * eps)
            assert abs(num - grads[which][idx]) <= 1e-6 * max(1.0, abs(num)), (which, idx, num, grads[which][idx])


def test_causal_bwd_finite_differences(oracle):
    # the reference's own invariant is gradcheck(eps=1e-4) at (1,2,63,128), Custom_Kernel.py:157,188
    q, k, v, g = rnd(1, 2, 15, 8, seed=1), rnd(1, 2, 15, 8, seed=2), rnd(1, 2, 15, 6, seed=3), rnd(1, 2, 15, 6, seed=4)
    _fd_check(oracle.causal, oracle.causal_bwd, [q, k, v], g)


def test_gradcheck_of_closed_forms_fp64():
    # torch.autograd.gradcheck on an autograd.Function whose backward is the closed form the oracle
    # restates -- the invariant the reference checks on its kernel (Custom_Kernel.py:188).
    class F(torch.autograd.Function):
        @staticmethod
        def forward(ctx, q, k, v):
            ctx.save_for_backward(q, k, v)
            return tf.causal_masked(q, k, v)

        @staticmethod
        def backward(ctx, g):
            return tf.causal_grads_closed_form(*ctx.saved_tensors, g)

    gen = torch.Generator().manual_seed(0)
    q, k, v = (torch.rand(1, 2, 9, 8, generator=gen, dtype=torch.float64, requires_grad=True) for _ in range(3))
    assert torch.autograd.gradcheck(F.apply, (q, k, v), eps=1e-4, atol=1e-6)


def test_noncausal_forms_and_grads(oracle):
    b, h, n, dk, dv = 2, 2, 21, 8, 12
    q, k, v, g = (torch.from_numpy(rnd(b, h, n, d, seed=20 + i)) for i, d in enumerate((dk, dk, dv, dv)))
    o = oracle.noncausal(q, k, v)
    assert np.allclose(o, tf.noncausal_einsum(q, k, v).numpy(), atol=1e-10)          # BertCosAttention.py:249
    assert np.allclose(o, tf.noncausal_quadratic(q, k, v).numpy(), atol=1e-10)       # BertCosAttention.py:222
    # the last causal row sees every key: equals the non-causal row
    assert np.allclose(oracle.causal(q, k, v)[..., -1, :], o[..., -1, :], atol=1e-10)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    tf.noncausal_einsum(qa, ka, va).backward(g)
    dq, dk_, dv_ = oracle.noncausal_bwd(q, k, v, g)
    for got, want in ((dq, qa.grad), (dk_, ka.grad), (dv_, va.grad)):
        assert np.allclose(got, want.numpy(), atol=1e-10)
    # GPTCosAttention.py:34-35 (grad_Q, grad_K as written there)
    assert np.allclose(dq, (g @ (v.transpose(-1, -2) @ k)).numpy(), atol=1e-10)
    assert np.allclose(dk_, (v @ (g.transpose(-1, -2) @ q)).numpy(), atol=1e-10)
    # :36 as written, Q (dO^T K), is NOT the derivative; K (Q^T dO) is.  (needs dk == dv to even typecheck)
    assert np.allclose(dv_, (k @ (q.transpose(-1, -2) @ g)).numpy(), atol=1e-10)
    # permutation identities used by the shipped backward
    assert np.allclose(dq, oracle.noncausal(g, v, k), atol=1e-10)
    assert np.allclose(dk_, oracle.noncausal(v, g, q), atol=1e-10)
    assert np.allclose(dv_, oracle.noncausal(k, q, g), atol=1e-10)
    _fd_check(oracle.noncausal, oracle.noncausal_bwd, [x.numpy() for x in (q, k, v)], g.numpy(), n_probe=15)


def test_decode_steps_reproduce_causal_rows(oracle):
    b, h, n, dk, dv = 2, 3, 11, 8, 6
    q, k, v = rnd(b, h, n, dk, seed=1), rnd(b, h, n, dk, seed=2), rnd(b, h, n, dv, seed=3)
    want = oracle.causal(q, k, v)
    S = np.zeros((b, h, dk, dv))
    for s in range(n):
        o = oracle.decode_step(S, q[:, :, s], k[:, :, s], v[:, :, s])
        assert np.allclose(o, want[:, :, s], atol=1e-12)
    assert np.allclose(S, np.einsum("bhnd,bhne->bhde", k, v))
    # reference orientation (Dv, Dk): GPTCosAttention.py:264 accumulates v (x) k
    ref_state = np.einsum("bhne,bhnd->bhed", v, k)
    assert np.allclose(S.transpose(0, 1, 3, 2), ref_state)


def test_padded_rows_contribute_nothing(oracle):
    # GPTCosAttention.py:245-248 zeroes q,k,v at padded positions
    q, k, v = rnd(1, 1, 12, 8, seed=1), rnd(1, 1, 12, 8, seed=2), rnd(1, 1, 12, 8, seed=3)
    keep = np.ones(12, bool); keep[[3, 4, 9]] = False
    qm, km, vm = (x * keep[None, None, :, None] for x in (q, k, v))
    o = oracle.causal(qm, km, vm)
    assert np.all(o[0, 0, ~keep] == 0)
    assert np.allclose(o[0, 0, keep], oracle.causal(q[:, :, keep], k[:, :, keep], v[:, :, keep])[0, 0])


def test_linearity_in_each_operand(oracle):
    A, B, C, A2 = rnd(1, 9, 4, seed=1), rnd(1, 9, 4, seed=2), rnd(1, 9, 5, seed=3), rnd(1, 9, 4, seed=4)
    assert np.allclose(oracle.causal(A + 2 * A2, B, C), oracle.causal(A, B, C) + 2 * oracle.causal(A2, B, C))
    assert np.allclose(oracle.causal(A, B + 2 * A2, C), oracle.causal(A, B, C) + 2 * oracle.causal(A, A2, C))


def test_input_prep_forms_against_hand_written_loops():
    # The CPU statement of the module-side preparation (oracle/torch_forms.py) against plain loops written here,
    # on an input with padded positions, a zero row (norm clamp) and counts on both sides of the clamp at 1.
    b, h, n, dk, dv = 2, 3, 7, 4, 5
    g = torch.Generator().manual_seed(5)
    q, k = torch.randn(b, h, n, dk, generator=g, dtype=torch.float64), torch.randn(b, h, n, dk, generator=g, dtype=torch.float64)
    v = torch.randn(b, h, n, dv, generator=g, dtype=torch.float64)
    q[0, 1, 2] = 0.0
    keep = torch.tensor([[1, 1, 0, 1, 1, 0, 1], [0, 1, 1, 1, 1, 1, 1]], dtype=torch.bool)
    sig = torch.tensor([0.3, 0.5, 0.9], dtype=torch.float64)
    qh, kh, vs, cnt = tf.input_prep_gpt(q, k, v, keep, sig)
    for bi in range(b):
        run = 0
        for s in range(n):
            run += int(keep[bi, s])
            assert cnt[bi, s] == run
            for hi in range(h):
                for x, xh in ((q, qh), (k, kh)):
                    nrm = float(np.sqrt(sum(float(e) ** 2 for e in x[bi, hi, s])))
                    want = [float(e) / max(nrm, 1e-12) * int(keep[bi, s]) for e in x[bi, hi, s]]
                    assert np.allclose(xh[bi, hi, s].numpy(), want, rtol=1e-13, atol=0)
                scale = max(run ** float(sig[hi]), 1.0)
                want = [float(e) / scale * int(keep[bi, s]) for e in v[bi, hi, s]]
                assert np.allclose(vs[bi, hi, s].numpy(), want, rtol=1e-13, atol=0)
    # the non-causal module masks first and uses the total count; for 0/1 masks only the count differs
    qb, kb, vb, cntb = tf.input_prep_bert(q, k, v, keep, sig)
    assert torch.equal(qb, qh) and torch.equal(kb, kh)
    assert torch.equal(cntb, keep.sum(-1, keepdim=True).expand(b, n).to(torch.float64))
    tot = keep.sum(-1).to(torch.float64).reshape(b, 1, 1, 1)
    assert torch.allclose(vb, v * keep[:, None, :, None] / (tot ** sig.reshape(1, h, 1, 1)).clamp(min=1), rtol=1e-13, atol=0)
