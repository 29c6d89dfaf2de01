"""GPU parity of the forward pass that saves states for the backward pass (cott_causal_fwd_save /
cott_causal_bwd_saved) against the plain entry points and the CPU oracle."""
import os

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


SAVED_CASES = [
    # a head is one group: the one slot is the sum over the whole sequence
    (8, 16, 2048, 64, 64, BF),      # headline shape: dQ in complement form beside the (dK, dV) pair workgroups
    (3, 43, 1000, 48, 48, HF),      # the same with a ragged tail and padded head dims
    (8, 16, 2048, 32, 32, BF),
    # pair workgroups in sequence groups
    (2, 16, 8192, 64, 64, BF),
    (1, 16, 10000, 64, 64, HF),
    (1, 16, 6000, 96, 96, BF),      # padded head dims (the forward pass runs column halves of 48)
    # shapes whose backward pass is cut into groups with dQ in complement form
    (1, 16, 4096, 128, 128, BF),    # forward in column halves (two workgroups write each slot)
    (2, 8, 10000, 128, 128, HF),    # ragged tail, fp16
    (1, 16, 7777, 128, 64, BF),     # Dk != Dv: dQ and dK form the set, dV runs apart
    (1, 16, 30000, 64, 128, BF),
    (1, 5, 30000, 128, 128, BF),    # 16 cuts; forward and backward cut the sequence differently
    (1, 16, 65536, 128, 128, BF),   # the long-context benchmark configuration at its full size, as the benchmark runs it
]


@pytest.mark.parametrize("case", SAVED_CASES, ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_states_saved_by_the_forward_pass_feed_the_backward_pass(ct, oracle, case):
    b, h, n, dk, dv, dt = case
    say("saved states", case)
    plan = ct.saved_states_plan(dt, b, h, n, dk, dv)
    assert plan is not None, "the case is meant to have cuts"
    cpc, cuts, slot, _ = plan
    q, k, v, do = inputs(b, h, n, dk, dv, dt, seed=n + 1)
    qd, kd, vd, gd = (x.to(DEV) for x in (q, k, v, do))
    o, saved = ct.causal_dot_product_saving(qd, kd, vd)
    assert torch.equal(o, ct.causal_dot_product(qd, kd, vd)), "the saving forward must not change o"
    assert saved.shape == (b, h, cuts, slot) and saved.dtype == torch.float32
    # a slot is the padded state in 16 x 16 tiles: [tile row][tile column][g][m][c] holds element [16it+4g+c][16jt+m]
    pk, pv = (32 if d <= 32 else 64 if d <= 64 else 128 for d in (dk, dv))
    assert slot == pk * pv
    states = saved.view(b, h, cuts, pk // 16, pv // 16, 4, 16, 4).permute(0, 1, 2, 3, 5, 7, 4, 6).reshape(b, h, cuts, pk, pv)
    states = states[..., :dk, :dv]
    # slot g = sum over the positions before 64 * (nchunks - g * cpc) of k^T v, in fp64 from the same rounded inputs
    nchunks = (n + 63) // 64
    for g_ in range(cuts):
        end = min(n, 64 * (nchunks - g_ * cpc))
        ref = torch.einsum("bhsi,bhsj->bhij", kd[:, :, :end].double(), vd[:, :, :end].double())
        err = float((states[:, :, g_].double() - ref).norm() / ref.norm())
        assert err <= 1e-5, (g_, err)
    got = ct.causal_backward(qd, kd, vd, gd, saved=saved)
    plain = ct.causal_backward(qd, kd, vd, gd)
    for name, a, p_, r in zip(("dQ", "dK", "dV"), got, plain, oracle.causal_bwd(q, k, v, do)):
        e_ref, e_plain = rel_l2(a, r), rel_l2(a, p_.double().cpu().numpy())
        e_blk = worst_block(a, r)  # (dQ in complement form: no stretch of the sequence may carry the error of the rest)
        say(f"  {name}: vs oracle {e_ref:.2e} (worst 64-row block {e_blk:.2e}), vs the plain backward {e_plain:.2e}")
        assert e_ref <= TOL[dt] and e_blk <= TOL[dt], name
        assert e_plain <= 5e-3, name


def test_saved_states_are_refused_where_the_backward_pass_takes_none(ct):
    # problems split into column halves: no plan, the saving forward returns None and the backward refuses
    b, h, n, dk, dv = 4, 16, 2048, 128, 64
    assert ct.saved_states_plan(BF, b, h, n, dk, dv) is None
    q, k, v, do = (x.to(DEV) for x in inputs(b, h, n, dk, dv, BF, seed=3))
    o, saved = ct.causal_dot_product_saving(q, k, v)
    assert saved is None and torch.equal(o, ct.causal_dot_product(q, k, v))
    with pytest.raises(RuntimeError, match="takes no saved states"):
        ct.causal_backward(q, k, v, do, saved=torch.zeros(b, h, 1, 128 * 64, device=DEV))
    # a plan exists, but the states were cut differently
    b, h, n, d = 1, 16, 4096, 128
    q, k, v, do = (x.to(DEV) for x in inputs(b, h, n, d, d, BF, seed=4))
    _, saved = ct.causal_dot_product_saving(q, k, v)
    with pytest.raises(RuntimeError, match="saved must be"):
        ct.causal_backward(q, k, v, do, saved=saved[:, :, :-1].contiguous())


def test_custom_attention_saves_the_states_on_long_16_bit_sequences(ct, oracle):
    """CustomAttention.apply on bf16 tensors long enough to be cut into groups: the forward pass keeps the states and
    the backward pass uses them (spied on); gradients against the oracle."""
    from unittest import mock
    from cottention_transformer_amd import ops
    from cottention_transformer_amd.autograd import CustomAttention
    b, h, n, d = 1, 16, 4096, 128
    q, k, v, do = inputs(b, h, n, d, d, BF, seed=11)
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    with mock.patch.object(ops, "causal_backward", wraps=ops.causal_backward) as spy:
        out = CustomAttention.apply(qd, kd, vd)
        out.backward(do.to(DEV))
        assert spy.call_count == 1 and spy.call_args.kwargs.get("saved") is not None
    assert rel_l2(out, oracle.causal(q, k, v)) <= TOL[BF]
    for name, a, r in zip(("dQ", "dK", "dV"), (qd.grad, kd.grad, vd.grad), oracle.causal_bwd(q, k, v, do)):
        assert rel_l2(a, r) <= TOL[BF], name
    # fp32 tensors under autocast compute the forward in bf16 and the backward in fp32: nothing is saved
    q32, k32, v32 = (x.float().to(DEV).requires_grad_(True) for x in (q, k, v))
    with mock.patch.object(ops, "causal_backward", wraps=ops.causal_backward) as spy:
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = CustomAttention.apply(q32, k32, v32)
        out.backward(do.to(DEV))
        assert spy.call_count == 1 and spy.call_args.kwargs.get("saved") is None
    assert out.dtype == BF and q32.grad.dtype == torch.float32


@pytest.mark.parametrize("case", [(8, 16, 2048, 64, 64, BF), (2, 16, 8192, 64, 64, HF), (1, 16, 6000, 128, 128, BF)],
                         ids=lambda c: "x".join(map(str, c[:5])))
def test_saved_states_with_merged_heads(ct, oracle, case):
    """cott_causal_fwd_save_bnhd / cott_causal_bwd_saved_bnhd: o written and d_o read as (B,N,H,Dv); same numbers as the
    (B,H,N,D) pair, bit for bit."""
    b, h, n, dk, dv, dt = case
    q, k, v, do = (x.to(DEV) for x in inputs(b, h, n, dk, dv, dt, seed=n + 3))
    o, saved = ct.causal_dot_product_saving(q, k, v)
    om, saved_m = ct.causal_dot_product_saving(q, k, v, merged_heads=True)
    assert saved is not None and torch.equal(saved, saved_m)
    assert om.shape == (b, n, h, dv) and torch.equal(om.permute(0, 2, 1, 3), o)
    plain = ct.causal_backward(q, k, v, do, saved=saved)
    merged = ct.causal_backward(q, k, v, do.permute(0, 2, 1, 3).contiguous(), merged_heads=True, saved=saved_m)
    for name, a, p_ in zip(("dQ", "dK", "dV"), merged, plain):
        assert torch.equal(a, p_), name


def test_block_level_functions_hand_the_states_to_their_backward(ct):
    """CustomAttentionMergedHeads and PreparedCausalAttention (what modules.GPTCosAttention runs) keep the states of
    their forward pass and their backward takes them; gradients equal to those of the plain composition within the
    16-bit bar (the blocks' own parity tests are in test_gpu_modules.py)."""
    from unittest import mock
    from cottention_transformer_amd import ops
    from cottention_transformer_amd.autograd import CustomAttention, CustomAttentionMergedHeads, PreparedCausalAttention
    b, h, n, d = 8, 16, 1024, 64
    q, k, v, do = (x.to(DEV) for x in inputs(b, h, n, d, d, BF, seed=21))
    ref = ct.causal_backward(q, k, v, do)
    qg, kg, vg = (x.clone().requires_grad_(True) for x in (q, k, v))
    with mock.patch.object(ops, "causal_backward", wraps=ops.causal_backward) as spy:
        CustomAttentionMergedHeads.apply(qg, kg, vg).backward(do.permute(0, 2, 1, 3).contiguous())
        assert spy.call_count == 1 and spy.call_args.kwargs.get("saved") is not None
    for a, r in zip((qg.grad, kg.grad, vg.grad), ref):
        assert rel_l2(a, r.double().cpu().numpy()) <= 5e-3
    # the preparation inside the forward kernel: raw projections in (B,N,H,D), no mask, no value scaling, no rotation
    raw = [torch.randn(b, n, h, d, generator=torch.Generator().manual_seed(s)).to(BF).to(DEV).requires_grad_(True)
           for s in (1, 2, 3)]
    if not ct.fused_preparation_supported(BF, b, h, n, d, d, 0):
        pytest.skip("the fused preparation is not built for this shape")
    with mock.patch.object(ops, "causal_backward", wraps=ops.causal_backward) as spy:
        out = PreparedCausalAttention.apply(*raw, None, None, None, None, 0, True, True)
        out.backward(do.permute(0, 2, 1, 3).contiguous())
        assert spy.call_count == 1 and spy.call_args.kwargs.get("saved") is not None
    # the same through the separate pieces: prepare, then the plain attention function
    raw2 = [x.detach().clone().requires_grad_(True) for x in raw]
    qh, kh, vh = ct.PrepareInputs.apply(*raw2, None, None, None, BF, None, None, True)
    out2 = CustomAttention.apply(qh, kh, vh)
    out2.backward(do)
    assert rel_l2(out.permute(0, 2, 1, 3), out2.detach().double().cpu().numpy()) <= 5e-3
    for a, r in zip(raw, raw2):
        assert rel_l2(a.grad, r.grad.double().cpu().numpy()) <= 2e-2


def test_random_shapes_every_16_bit_path_against_the_fp32_kernels(ct):
    """30 seeded random shapes (head dims 32..128, 2..300 heads, 1..65536 positions, bf16 / fp16): the plain, the
    saved-state and the merged-heads backward, the saving forward and the forward written over V, all against the
    fp32 kernels of this library (themselves checked against the oracle in test_gpu_parity.py) on the same rounded
    inputs: whole tensor and worst 64-row block within the 16-bit bar.  Launch plans differ from shape to shape
    (column halves, sequence groups, pair workgroups, two launches, saved states or none)."""
    import random
    rnd = random.Random(5)

    def err(a, r):
        return max(rel_l2(a, r.double().cpu().numpy()), worst_block(a, r.double().cpu().numpy()))

    worst = 0.0
    for it in range(30):
        dk = rnd.choice([32, 48, 64, 64, 64, 96, 128, 128])
        dv = rnd.choice([dk, dk, dk, 32, 64, 128, 80])
        h = rnd.choice([1, 2, 4, 8, 16])
        b = max(1, rnd.choice([2, 8, 16, 40, 48, 90, 96, 128, 129, 200, 300]) // h)
        n = min(rnd.choice([1, 63, 64, 65, 300, 1000, 2048, 4096, 10000, 30000, 65536]),
                max(64, (1 << 26) // (b * h * max(dk, dv))))
        dt = rnd.choice([BF, BF, HF])
        q, k, v, do = (x.to(DEV) for x in inputs(b, h, n, dk, dv, dt, seed=it))
        say(f"random case {it}: B{b} H{h} N{n} Dk{dk} Dv{dv} {dt} plan {ct.saved_states_plan(dt, b, h, n, dk, dv)}")
        ref_o = ct.causal_dot_product(q.float(), k.float(), v.float())
        ref = ct.causal_backward(q.float(), k.float(), v.float(), do.float())
        o = ct.causal_dot_product(q, k, v)
        o2, saved = ct.causal_dot_product_saving(q, k, v)
        assert torch.equal(o, o2)
        v2 = v.clone()
        assert ct.causal_dot_product(q, k, v2, into_v=True) is v2 and torch.equal(v2, o)
        errs = [err(o, ref_o)]
        outs = [ct.causal_backward(q, k, v, do)]
        if saved is not None:
            outs.append(ct.causal_backward(q, k, v, do, saved=saved))
        if ct.merged_heads_supported(dt, n, h, dk, dv):
            assert torch.equal(ct.causal_dot_product(q, k, v, merged_heads=True).permute(0, 2, 1, 3), o)
            outs.append(ct.causal_backward(q, k, v, do.permute(0, 2, 1, 3).contiguous(), merged_heads=True))
        for grads in outs:
            errs += [err(a, r) for a, r in zip(grads, ref)]
        assert max(errs) <= TOL[dt], (it, errs)
        worst = max(worst, max(errs))
    say(f"worst error over all cases and paths: {worst:.2e}")


# Shapes on either side of the launch planner's measured thresholds (column halves of one group against whole problems
# in groups, by heads, tile size and group length; pair workgroups for few small heads on long sequences; the
# non-causal column halves): every plan the rules choose between runs at a size where the rule applies.
PLANNER_CASES = [
    (9, 8, 1024, 128, 128, BF),    # forward of 72 wide heads, short groups: column halves of one group
    (9, 8, 4096, 128, 128, BF),    # ... groups of 22 chunks: whole problems in three groups
    (11, 8, 8192, 128, 128, HF),   # 88 wide heads, two groups of 64 chunks
    (8, 8, 4096, 64, 64, BF),      # 64 small heads: column halves in two groups (whole problems would get 16 chunks)
    (8, 8, 8192, 64, 64, BF),      # ... whole problems in four groups of 32 chunks
    (3, 8, 4096, 128, 128, BF),    # gradients of 24 wide heads: groups of 22 chunks with saved states, halves without
    (4, 8, 8192, 128, 128, BF),    # gradients of 32 wide heads: groups of 64 chunks with saved states
    (4, 8, 4096, 128, 128, HF),    # ... column halves of one group
    (6, 8, 16384, 64, 64, BF),     # 48 small heads, 256 chunks: pair workgroups once the forward has left its states
    (5, 16, 2048, 96, 96, BF),     # 80 heads of padded width
]


@pytest.mark.parametrize("case", PLANNER_CASES, ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_shapes_around_the_planner_thresholds_against_the_fp32_kernels(ct, case):
    b, h, n, dk, dv, dt = case
    say("planner case", case, "plan", ct.saved_states_plan(dt, b, h, n, dk, dv))
    q, k, v, do = (x.to(DEV) for x in inputs(b, h, n, dk, dv, dt, seed=11))

    def err(a, r):
        return max(rel_l2(a, r.double().cpu().numpy()), worst_block(a, r.double().cpu().numpy()))

    ref_o = ct.causal_dot_product(q.float(), k.float(), v.float())
    ref_r = ct.causal_dot_product(q.float(), k.float(), v.float(), reversed=True)
    ref = ct.causal_backward(q.float(), k.float(), v.float(), do.float())
    o, saved = ct.causal_dot_product_saving(q, k, v)
    assert torch.equal(o, ct.causal_dot_product(q, k, v))
    errs = [err(o, ref_o), err(ct.causal_dot_product(q, k, v, reversed=True), ref_r)]
    outs = [ct.causal_backward(q, k, v, do)]
    if saved is not None:
        outs.append(ct.causal_backward(q, k, v, do, saved=saved))
    for grads in outs:
        errs += [err(a, r) for a, r in zip(grads, ref)]
    assert max(errs) <= TOL[dt], errs


@pytest.mark.parametrize("case", [(48, 8, 512, 64, 64, BF), (24, 8, 512, 64, 64, HF), (96, 8, 512, 64, 64, BF),
                                  (40, 12, 384, 128, 128, BF), (48, 8, 300, 64, 32, BF)],
                         ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_non_causal_shapes_around_the_planner_thresholds_against_the_fp32_kernels(ct, case):
    """One workgroup per head with and without column halves (257..384 small heads take halves), four to eight chunks
    (the A rows of the first chunks are requested before the first pass)."""
    from cottention_transformer_amd import ops
    b, h, n, dk, dv, dt = case
    say("non-causal planner case", case)
    q, k, v, do = (x.to(DEV) for x in inputs(b, h, n, dk, dv, dt, seed=12))
    ref_o = ops.noncausal_dot_product(q.float(), k.float(), v.float())
    ref = ops.noncausal_backward(q.float(), k.float(), v.float(), do.float())
    errs = [max(rel_l2(ops.noncausal_dot_product(q, k, v), ref_o.double().cpu().numpy()),
                worst_block(ops.noncausal_dot_product(q, k, v), ref_o.double().cpu().numpy()))]
    for a, r in zip(ops.noncausal_backward(q, k, v, do), ref):
        errs += [rel_l2(a, r.double().cpu().numpy()), worst_block(a, r.double().cpu().numpy())]
    assert max(errs) <= TOL[dt], errs
