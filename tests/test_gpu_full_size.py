"""GPU parity at the FULL size of every benchmark configuration, through the C ABI, against the CPU oracle.

The whole-tensor rel-L2 of a long sequence would hide one bad chunk (its share of the norm is 1/sqrt(chunks)), so
every comparison here also bounds the worst 64-row block of every head.  Bars: rel-L2 <= 2e-2 for bf16 tensors
(oracle in fp64 on the same rounded inputs), per block as well as overall; the fp32 decode state <= 1e-5."""
import os

import numpy as np
import pytest
import torch

from util import TOL, inputs, rel_l2, worst_block

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16


@pytest.fixture(scope="module")
def ct():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import cottention_transformer_amd as ct_
    from cottention_transformer_amd import _loader
    assert os.path.exists(_loader.lib_path()), "libcottention_hip.so must be prebuilt in-tree"
    _loader.lib()
    return ct_


def say(*a):
    print(*a, flush=True)


def check(name, got, ref, tol):
    whole, block = rel_l2(got, ref), worst_block(got, ref)
    say(f"  {name}: rel-L2 {whole:.2e}, worst 64-row block {block:.2e}")
    assert whole <= tol, name
    assert block <= tol, name + " (one block)"


LONG_CASES = [
    # b, h, n, dk, dv, dtype                       launch plan the shape takes
    (1, 16, 65536, 128, 128, BF),   # long-context benchmark configuration: 16 groups of 64 chunks, 128 x 128 tiles
    (2, 4, 19217, 64, 64, BF),      # dQ + (dK, dV) pair workgroups with several groups of several chunks, ragged tail
    (1, 4, 8192, 128, 128, HF),     # fp16, few chunks per group
    (1, 3, 20000, 64, 128, BF),     # Dk != Dv: three separate gradient problems in groups
]


@pytest.mark.parametrize("case", LONG_CASES, ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_long_sequences_forward_and_backward(ct, oracle, case):
    b, h, n, dk, dv, dt = case
    say("long sequence", case)
    q, k, v, do = inputs(b, h, n, dk, dv, dt, seed=n)
    qd, kd, vd, gd = (x.to(DEV) for x in (q, k, v, do))
    check("O", ct.causal_dot_product(qd, kd, vd), oracle.causal(q, k, v), TOL[dt])
    check("O reversed", ct.causal_dot_product(qd, kd, vd, True), oracle.causal(q, k, v, True), TOL[dt])
    for name, got, ref in zip(("dQ", "dK", "dV"), ct.causal_backward(qd, kd, vd, gd), oracle.causal_bwd(q, k, v, do)):
        check(name, got, ref, TOL[dt])


FUSED_NONCAUSAL_CASES = [
    # shapes whose heads alone fill the chip: one workgroup per head runs both passes over several chunks
    (32, 12, 512, 64, 64, BF),      # BERT benchmark configuration
    (16, 16, 300, 64, 32, BF),      # ragged tail, Dk != Dv
    (32, 8, 300, 128, 128, HF),     # 128-wide heads
    (16, 16, 1000, 48, 80, BF),     # padded head dims
]


@pytest.mark.parametrize("case", FUSED_NONCAUSAL_CASES,
                         ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_noncausal_many_heads_forward_and_backward(ct, oracle, case):
    b, h, n, dk, dv, dt = case
    say("non-causal, one workgroup per head", case)
    q, k, v, do = inputs(b, h, n, dk, dv, dt, seed=n + 5)
    qd, kd, vd, gd = (x.to(DEV) for x in (q, k, v, do))
    check("O", ct.noncausal_dot_product(qd, kd, vd), oracle.noncausal(q, k, v), TOL[dt])
    for name, got, ref in zip(("dQ", "dK", "dV"), ct.noncausal_backward(qd, kd, vd, gd), oracle.noncausal_bwd(q, k, v, do)):
        check(name, got, ref, TOL[dt])


def test_decode_512_steps_at_benchmark_size(ct, oracle):
    """Decode benchmark configuration: fp32 state (256,16,128,128) ~ N(0, 0.01), bf16 q, k, v, 512 consecutive steps
    (GPT_Trainer/GPTCosAttention.py:262-269).  The oracle follows every 8th batch element step by step in fp64
    (outputs compared at steps 1, 256 and 512, its state at the end); the final state of ALL batch elements is
    compared with s0 + sum_t k_t v_t^T accumulated in fp64."""
    b, h, d, steps = 256, 16, 128, 512
    sub = slice(0, b, 8)
    g = torch.Generator(device=DEV).manual_seed(4)
    s0 = 0.01 * torch.randn(b, h, d, d, generator=g, device=DEV)
    qs = torch.nn.functional.normalize(torch.randn(steps, b, h, d, generator=g, device=DEV), dim=-1).to(BF)
    ks = torch.nn.functional.normalize(torch.randn(steps, b, h, d, generator=g, device=DEV), dim=-1).to(BF)
    vs = torch.randn(steps, b, h, d, generator=g, device=DEV).to(BF)
    state = s0.clone()
    ref_state = s0[sub].double().cpu().numpy().copy()
    qc, kc, vc = (x[:, sub].cpu() for x in (qs, ks, vs))
    out = torch.empty(b, h, d, dtype=BF, device=DEV)
    for t in range(steps):
        ct.decode_step(state, qs[t], ks[t], vs[t], out=out)
        ref = oracle.decode_step(ref_state, qc[t], kc[t], vc[t])
        if t + 1 in (1, 256, 512):
            err = rel_l2(out[sub], ref)
            say(f"  step {t + 1}: output rel-L2 {err:.2e}")
            assert err <= 2e-2, t + 1
    err = rel_l2(state[sub], ref_state)
    say(f"  state after {steps} steps vs oracle: {err:.2e}")
    assert err <= 1e-5
    total = s0.double()
    for t0 in range(0, steps, 64):
        total += torch.einsum("tbhi,tbhj->bhij", ks[t0:t0 + 64].double(), vs[t0:t0 + 64].double())
    err = float((state.double() - total).norm() / total.norm())
    say(f"  state of all batch elements vs fp64 sum: {err:.2e}")
    assert err <= 1e-5


def test_decode_on_a_state_beyond_the_last_level_cache(ct, oracle):
    """A state of 400 MiB (B=400, H=16, D=128) takes the decode kernel's streaming variant (non-temporal state
    accesses): three steps, outputs of every 16th batch element against the oracle and the final state of all of
    them against s0 + sum_t k_t v_t^T in fp64."""
    b, h, d, steps = 400, 16, 128, 3
    sub = slice(0, b, 16)
    g = torch.Generator(device=DEV).manual_seed(9)
    s0 = 0.01 * torch.randn(b, h, d, d, generator=g, device=DEV)
    qs = torch.nn.functional.normalize(torch.randn(steps, b, h, d, generator=g, device=DEV), dim=-1).to(BF)
    ks = torch.nn.functional.normalize(torch.randn(steps, b, h, d, generator=g, device=DEV), dim=-1).to(BF)
    vs = torch.randn(steps, b, h, d, generator=g, device=DEV).to(BF)
    state = s0.clone()
    ref_state = s0[sub].double().cpu().numpy().copy()
    for t in range(steps):
        out = ct.decode_step(state, qs[t], ks[t], vs[t])
        ref = oracle.decode_step(ref_state, qs[t, sub].cpu(), ks[t, sub].cpu(), vs[t, sub].cpu())
        assert rel_l2(out[sub], ref) <= 2e-2, t
    assert rel_l2(state[sub], ref_state) <= 1e-6
    total = s0.double() + torch.einsum("tbhi,tbhj->bhij", ks.double(), vs.double())
    assert float((state.double() - total).norm() / total.norm()) <= 1e-6


@pytest.mark.parametrize("case", [(8, 16, 2048, 64, 64, BF, 64), (1, 16, 65536, 128, 128, BF, 32)],
                         ids=["8x16x2048x64", "1x16x65536x128"])
def test_one_launch_forward_with_preparation_at_benchmark_sizes(ct, oracle, case):
    """cott_causal_fwd_prep at the two shapes the benchmark times it on (the headline shape: column halves, one group;
    the long-context shape: whole 128 x 128 problems in 16 groups, the group sums by the kernel with loader and
    compute wavefronts), on the projections' (B,N,H,D) tensors with a mask, value scaling and the rotation by position
    ids: the prepared tensors against the CPU statement of GPT_Trainer/GPTCosAttention.py:229-248, 462-476 (elementwise,
    the counts as a running sum of the mask) and the outputs against the causal oracle on those, per 64-row block."""
    from oracle import torch_forms as tf
    b, h, n, dk, dv, dt, rdim = case
    say("one-launch forward with preparation", case)
    g = torch.Generator().manual_seed(n + dk)
    q, k, v = (torch.randn(b, n, h, d, generator=g).to(dt) for d in (dk, dk, dv))
    keep = torch.rand(b, n, generator=g) > 0.1
    sig = torch.sigmoid(torch.randn(h, generator=g))
    table = tf.gptj_sinusoid_table(n, rdim).float()
    ids = torch.arange(n)[None, :].expand(b, n)
    cnt = keep.double().cumsum(-1)                                                # kept keys at positions <= s (:241)
    sin, cos = torch.split(table.double()[ids], rdim // 2, dim=-1)
    rot = lambda x: torch.cat([tf.gptj_rotate(x[..., :rdim], sin, cos), x[..., rdim:]], -1)   # (B,N,H,D) layout
    m = keep[:, :, None, None].double()
    rq = (torch.nn.functional.normalize(rot(q.double()), dim=-1, p=2) * m).permute(0, 2, 1, 3)
    rk = (torch.nn.functional.normalize(rot(k.double()), dim=-1, p=2) * m).permute(0, 2, 1, 3)
    scale = (cnt[:, :, None, None] ** sig.double().reshape(1, 1, h, 1)).clamp(min=1)
    rv = (v.double() / scale * m).permute(0, 2, 1, 3)
    o, prepared = ct.causal_dot_product_prepared(q.to(DEV), k.to(DEV), v.to(DEV), keep=keep.to(DEV), cnt=cnt.float().to(DEV),
                                                 sig=sig.to(DEV), rotary=(table.to(DEV), ids.contiguous().to(DEV)), bnhd=True)
    for name, got, ref in zip(("q_hat", "k_hat", "v_hat"), prepared, (rq, rk, rv)):
        check(name, got, ref.numpy(), TOL[dt])
    check("O", o, oracle.causal(rq.contiguous(), rk.contiguous(), rv.contiguous()), TOL[dt])
