"""GPU parity: the HIP path, called through the C ABI (ctypes) from the host layer, against the CPU
oracle on identical seeded inputs.  Tolerances of the benchmark definition: rel-L2 <= 1e-4 for fp32 inputs,
<= 2e-2 for bf16/fp16 inputs (oracle evaluated in fp64 on the same rounded inputs); fp64 <= 1e-12."""
import os
import sys

import numpy as np
import pytest
import torch

from util import TOL, inputs, load_golden, rel_l2

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"


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


BF, HF, F32, F64 = torch.bfloat16, torch.float16, torch.float32, torch.float64

CAUSAL_CASES = [
    # b, h, n, dk, dv, dtype                      what it exercises
    (1, 2, 128, 64, 64, F32),     # the reference CPU-runnable benchmark case: fp32 (1,2,128,64)
    (1, 2, 128, 64, 64, BF),      # two chunks -> two groups
    (1, 2, 63, 128, 128, F64),    # the reference's gradcheck shape (Custom_Kernel.py:157)
    (1, 2, 63, 64, 64, BF),       # odd S, single partial chunk
    (2, 3, 200, 64, 32, BF),      # Dk != Dv (speeds.py:137)
    (1, 2, 130, 32, 128, HF),     # D=32 (combined_kernel_general.cu:273-277), fp16
    (1, 1, 130, 128, 128, BF),    # D=128 (kernel_mod_4 range, :281-284)
    (2, 2, 257, 48, 80, BF),      # head dims that are multiples of 16 but not of 32
    (1, 2, 1023, 64, 64, BF),     # speeds.py:5 length; one chunk per group
    (2, 4, 19217, 64, 64, BF),    # several chunks per group and several groups per head
    (6, 16, 300, 128, 128, BF),   # 96 heads of one group each, widest tiles: gradients as two launches (dK, dV | dQ in halves)
    (7, 16, 200, 96, 80, HF),     # ... with padded head dims (all three problems share padded dims 128 x 128)
    (1, 2, 100, 64, 32, F32),
    (1, 1, 70, 256, 48, F32),     # D beyond the MFMA range -> generic path
    (1, 2, 77, 256, 256, BF),     # 16-bit storage on the generic path
    (1, 1, 64, 64, 24, F32),      # D_value not a multiple of 16 (only D_attn is checked, :372-374)
    (1, 2, 1023, 64, 64, F32),    # fp32 MFMA kernels: ragged tail, one chunk per group
    (2, 2, 257, 48, 80, F32),     # ... head dims padded to 64 / 128, steps of 32 positions
    (1, 1, 130, 128, 128, F32),   # ... D=128
    (1, 2, 130, 32, 128, F32),    # ... D=32 against a wide value head
    (2, 3, 200, 64, 32, F32),     # ... two column tiles only (half the wavefronts own state)
    (1, 3, 2500, 64, 64, F32),    # ... several chunks per group
]


@pytest.mark.parametrize("case", CAUSAL_CASES, ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
@pytest.mark.parametrize("rev", [False, True], ids=["fwd", "reversed"])
def test_causal_forward(ct, oracle, case, rev):
    b, h, n, dk, dv, dt = case
    say("causal fwd", case, "reversed" if rev else "")
    q, k, v, _ = inputs(b, h, n, dk, dv, dt, seed=n)
    ref = oracle.causal(q, k, v, rev)
    out = ct.causal_dot_product(q.to(DEV), k.to(DEV), v.to(DEV), rev)
    assert out.shape == (b, h, n, dv) and out.dtype == dt
    assert rel_l2(out, ref) <= TOL[dt]


@pytest.mark.parametrize("case", [c for c in CAUSAL_CASES if c[4] % 16 == 0 and c[2] < 5000],
                         ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_causal_backward(ct, oracle, case):
    b, h, n, dk, dv, dt = case
    say("causal bwd", case)
    q, k, v, do = inputs(b, h, n, dk, dv, dt, seed=n + 1)
    refs = oracle.causal_bwd(q, k, v, do)
    outs = ct.causal_backward(q.to(DEV), k.to(DEV), v.to(DEV), do.to(DEV))
    for name, got, ref in zip(("dQ", "dK", "dV"), outs, refs):
        assert rel_l2(got, ref) <= TOL[dt], name


@pytest.mark.parametrize("seed", range(16))
def test_random_shapes_all_forms(ct, oracle, seed):
    """Shapes drawn at random (ragged lengths, unequal head dims, every launch form the planner can pick for small
    problems): causal forward in both directions, causal and non-causal gradients, against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    b, h = int(rng.integers(1, 4)), int(rng.integers(1, 6))
    n = int(rng.choice([1, 17, 64, 65, 127, 200, 333, 640, 1000]))
    dk = int(rng.choice([32, 48, 64, 80, 96, 128]))
    dv = int(rng.choice([32, 48, 64, 80, 96, 128]))
    dt = [BF, HF, F32][int(rng.integers(0, 3))]
    say("random shape", seed, (b, h, n, dk, dv, dt))
    q, k, v, do = inputs(b, h, n, dk, dv, dt, seed=seed)
    qd, kd, vd, dod = q.to(DEV), k.to(DEV), v.to(DEV), do.to(DEV)
    for rev in (False, True):
        assert rel_l2(ct.causal_dot_product(qd, kd, vd, rev), oracle.causal(q, k, v, rev)) <= TOL[dt], ("causal", rev)
    for name, got, ref in zip(("dQ", "dK", "dV"), ct.causal_backward(qd, kd, vd, dod), oracle.causal_bwd(q, k, v, do)):
        assert rel_l2(got, ref) <= TOL[dt], name
    assert rel_l2(ct.noncausal_dot_product(qd, kd, vd), oracle.noncausal(q, k, v)) <= TOL[dt]
    for name, got, ref in zip(("dQ", "dK", "dV"), ct.noncausal_backward(qd, kd, vd, dod), oracle.noncausal_bwd(q, k, v, do)):
        assert rel_l2(got, ref) <= TOL[dt], "non-causal " + name


MERGED_CASES = [
    # b, h, n, dk, dv, dtype                   launch form the shape takes
    (2, 16, 2048, 64, 64, BF),    # forward: two column halves per head; gradients: dQ + (dK, dV) pair workgroups
    (2, 3, 1000, 64, 32, HF),     # Dk != Dv: three separate gradient problems, ragged tail
    (1, 4, 8192, 128, 128, BF),   # sequence groups, 128-wide heads
    (3, 5, 63, 32, 128, BF),      # a single partial chunk
    (2, 12, 300, 48, 80, HF),     # head dims padded to 64 / 128
]


@pytest.mark.parametrize("case", MERGED_CASES, ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_merged_heads_layout(ct, oracle, case):
    """o written as (B,N,H,Dv) and d_o read as (B,N,H,Dv) (cott_causal_fwd_bnhd / cott_causal_bwd_bnhd): the same
    numbers as the (B,H,N,D) entry points, bit for bit, and within tolerance of the oracle."""
    b, h, n, dk, dv, dt = case
    say("merged heads", case)
    q, k, v, do = inputs(b, h, n, dk, dv, dt, seed=n + 7)
    qd, kd, vd, dod = q.to(DEV), k.to(DEV), v.to(DEV), do.to(DEV)
    assert ct.merged_heads_supported(dt, n, h, dk, dv)
    om = ct.causal_dot_product(qd, kd, vd, merged_heads=True)
    assert om.shape == (b, n, h, dv) and om.is_contiguous()
    assert torch.equal(om.permute(0, 2, 1, 3), ct.causal_dot_product(qd, kd, vd))
    assert rel_l2(om.permute(0, 2, 1, 3), oracle.causal(q, k, v, False)) <= TOL[dt]
    plain = ct.causal_backward(qd, kd, vd, dod)
    merged = ct.causal_backward(qd, kd, vd, dod.permute(0, 2, 1, 3).contiguous(), merged_heads=True)
    for name, got, want, ref in zip(("dQ", "dK", "dV"), merged, plain, oracle.causal_bwd(q, k, v, do)):
        assert torch.equal(got, want), name
        assert rel_l2(got, ref) <= TOL[dt], name


@pytest.mark.parametrize("case", [(2, 12, 512, 64, 64, BF), (1, 3, 63, 64, 32, HF), (1, 2, 9000, 128, 128, BF), (2, 5, 300, 48, 80, BF)],
                         ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_merged_heads_layout_noncausal(ct, oracle, case):
    """cott_noncausal_fwd_bnhd / cott_noncausal_bwd_bnhd against the (B,H,N,D) entry points (bit for bit) and the
    oracle; the third shape is cut into sequence groups (group-state, prefix and apply kernels)."""
    b, h, n, dk, dv, dt = case
    say("merged heads, non-causal", case)
    q, k, v, do = inputs(b, h, n, dk, dv, dt, seed=n + 11)
    qd, kd, vd, dod = q.to(DEV), k.to(DEV), v.to(DEV), do.to(DEV)
    om = ct.noncausal_dot_product(qd, kd, vd, merged_heads=True)
    assert om.shape == (b, n, h, dv)
    assert torch.equal(om.permute(0, 2, 1, 3), ct.noncausal_dot_product(qd, kd, vd))
    assert rel_l2(om.permute(0, 2, 1, 3), oracle.noncausal(q, k, v)) <= TOL[dt]
    plain = ct.noncausal_backward(qd, kd, vd, dod)
    merged = ct.noncausal_backward(qd, kd, vd, dod.permute(0, 2, 1, 3).contiguous(), merged_heads=True)
    for name, got, want in zip(("dQ", "dK", "dV"), merged, plain):
        assert torch.equal(got, want), name


def test_merged_heads_layout_is_refused_where_not_built(ct):
    q, k, v, _ = inputs(1, 2, 64, 64, 64, F32, seed=3)
    assert not ct.merged_heads_supported(F32, 64, 2, 64, 64)
    with pytest.raises(RuntimeError, match="bf16 / fp16"):
        ct.causal_dot_product(q.to(DEV), k.to(DEV), v.to(DEV), merged_heads=True)
    q, k, v, _ = inputs(1, 2, 64, 256, 256, BF, seed=3)  # beyond the MFMA head dims
    with pytest.raises(RuntimeError, match="head dims"):
        ct.causal_dot_product(q.to(DEV), k.to(DEV), v.to(DEV), merged_heads=True)
    with pytest.raises(RuntimeError, match="forward direction"):
        ct.causal_dot_product(q.to(DEV), k.to(DEV), v.to(DEV), True, merged_heads=True)


def test_golden_fixtures(ct):
    for name in ("causal_cfg1_1x2x128x64.npz", "causal_odd_1x2x63x32_dv48.npz"):
        say("golden", name)
        g = load_golden(name)
        q, k, v, do = (torch.from_numpy(g[x]).to(DEV) for x in ("q", "k", "v", "g"))
        assert rel_l2(ct.causal_dot_product(q, k, v), g["o"]) <= 1e-4
        assert rel_l2(ct.causal_dot_product(q, k, v, True), g["o_rev"]) <= 1e-4
        for got, key in zip(ct.causal_backward(q, k, v, do), ("dq", "dk", "dv")):
            assert rel_l2(got, g[key]) <= 1e-4
        # same fixture through the bf16 MFMA path (inputs rounded first, so only kernel error counts loosely)
        ob = ct.causal_dot_product(q.bfloat16(), k.bfloat16(), v.bfloat16())
        assert rel_l2(ob, g["o"]) <= 2e-2
    g = load_golden("noncausal_2x2x50x32.npz")
    q, k, v, do = (torch.from_numpy(g[x]).to(DEV) for x in ("q", "k", "v", "g"))
    assert rel_l2(ct.noncausal_dot_product(q, k, v), g["o"]) <= 1e-4
    for got, key in zip(ct.noncausal_backward(q, k, v, do), ("dq", "dk", "dv")):
        assert rel_l2(got, g[key]) <= 1e-4
    d = load_golden("decode_2x2x32x48_4steps.npz")
    state = torch.from_numpy(d["s0"]).to(DEV)
    for t in range(d["q"].shape[0]):
        o = ct.decode_step(state, *(torch.from_numpy(d[x][t]).to(DEV) for x in ("q", "k", "v")))
        assert rel_l2(o, d["o"][t]) <= 1e-4
    assert rel_l2(state, d["s_final"]) <= 1e-4


@pytest.mark.parametrize("case", [(2, 3, 512, 64, 64, BF), (1, 2, 63, 64, 32, HF), (2, 2, 1000, 128, 128, BF),
                                  (1, 2, 100, 64, 32, F32), (1, 2, 50, 32, 32, F64), (1, 1, 40, 256, 64, F32),
                                  (2, 3, 512, 64, 64, F32), (1, 2, 1000, 128, 128, F32), (3, 2, 77, 48, 80, F32)],
                         ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_noncausal_forward_backward(ct, oracle, case):
    b, h, n, dk, dv, dt = case
    say("noncausal", case)
    q, k, v, do = inputs(b, h, n, dk, dv, dt, seed=7)
    out = ct.noncausal_dot_product(q.to(DEV), k.to(DEV), v.to(DEV))
    assert rel_l2(out, oracle.noncausal(q, k, v)) <= TOL[dt]
    for name, got, ref in zip(("dQ", "dK", "dV"), ct.noncausal_backward(q.to(DEV), k.to(DEV), v.to(DEV), do.to(DEV)),
                              oracle.noncausal_bwd(q, k, v, do)):
        assert rel_l2(got, ref) <= TOL[dt], name


@pytest.mark.parametrize("case", [(2, 3, 128, 128, BF), (1, 2, 64, 32, HF), (2, 2, 64, 64, F32), (1, 2, 32, 48, F64),
                                  (1, 1, 128, 2048, F32), (1, 2, 8192, 8, F32), (1, 1, 4096, 12, F64)], ids=lambda c: "x".join(map(str, c[:4])) + "-" + str(c[4]).split(".")[-1])
def test_decode_steps(ct, oracle, case):
    b, h, dk, dv, dt = case
    say("decode", case)
    g = torch.Generator().manual_seed(3)
    sdt = F64 if dt == F64 else F32
    s0 = (0.01 * torch.randn(b, h, dk, dv, generator=g)).to(sdt)
    state, ref_state = s0.clone().to(DEV), s0.double().numpy().copy()
    for _ in range(6):
        q = torch.nn.functional.normalize(torch.randn(b, h, dk, generator=g), dim=-1).to(dt)
        k = torch.nn.functional.normalize(torch.randn(b, h, dk, generator=g), dim=-1).to(dt)
        v = torch.randn(b, h, dv, generator=g).to(dt)
        ref = oracle.decode_step(ref_state, q, k, v)
        out = ct.decode_step(state, q.to(DEV), k.to(DEV), v.to(DEV))
        assert rel_l2(out, ref) <= TOL[dt]
    assert rel_l2(state, ref_state) <= (1e-12 if dt == F64 else 1e-6)


@pytest.mark.parametrize("case", [(2, 3, 64, 64, BF, 64), (3, 2, 128, 128, F32, 32), (1, 4, 48, 32, HF, 16), (2, 2, 32, 64, F64, 0)],
                         ids=lambda c: "x".join(map(str, c[:4])) + "-" + str(c[4]).split(".")[-1] + "-rot" + str(c[5]))
def test_decode_step_on_raw_projections(ct, case):
    """cott_decode_step_prep (rotation, normalisation and value scaling inside the decode kernel) over several
    tokens against the CPU statements of those steps (oracle/torch_forms.py) followed by the plain recurrence."""
    from oracle import torch_forms as tf
    b, h, dk, dv, dt, rdim = case
    say("decode on raw projections", case)
    g = torch.Generator().manual_seed(dk + dv)
    steps, npos = 5, 40
    q, k = (torch.randn(steps, b, 1, h, dk, generator=g).to(dt) for _ in range(2))
    v = torch.randn(steps, b, 1, h, dv, generator=g).to(dt)
    sig = torch.sigmoid(torch.randn(h, generator=g))
    table = tf.gptj_sinusoid_table(npos, rdim).float() if rdim else None
    sdt = torch.float64 if dt == F64 else torch.float32
    state = torch.zeros(b, h, dk, dv, dtype=sdt, device=DEV)
    ref_state = torch.zeros(b, h, dk, dv, dtype=torch.float64)
    for t in range(steps):
        cnt, pos = float(t + 1), t + 3
        out = ct.decode_step_prepared(state, q[t].to(DEV), k[t].to(DEV), v[t].to(DEV), sig=sig.to(DEV), cnt=cnt,
                                      rotary=(table.to(DEV), pos) if rdim else None)
        q64, k64, v64 = (x[t][:, 0].double() for x in (q, k, v))          # (B,H,D)
        if rdim:
            sn, cs = (x.reshape(1, 1, -1).expand(b, 1, -1) for x in torch.split(table[pos].double(), rdim // 2, dim=-1))
            rot = lambda x: torch.cat([tf.gptj_rotate(x[..., :rdim].unsqueeze(1), sn, cs).squeeze(1), x[..., rdim:]], -1)
            q64, k64 = rot(q64), rot(k64)
        qn = q64 / q64.norm(dim=-1, keepdim=True).clamp(min=1e-12)
        kn = k64 / k64.norm(dim=-1, keepdim=True).clamp(min=1e-12)
        vs = v64 / (cnt ** sig.double()).clamp(min=1.0).reshape(1, h, 1)
        ref_state += kn.unsqueeze(-1) * vs.unsqueeze(-2)
        want = torch.einsum("bhi,bhij->bhj", qn, ref_state)
        assert out.shape == (b, h, dv) and out.dtype == dt
        assert rel_l2(out, want.numpy()) <= TOL[dt], t
    assert rel_l2(state, ref_state.numpy()) <= (1e-12 if dt == F64 else 2e-6)


def test_decode_after_prompt_equals_causal_forward(ct, oracle):
    # GPTCosAttention.py:253-272 vs :282: token-by-token decode reproduces the causal rows
    b, h, n, d = 2, 2, 48, 64
    q, k, v, _ = inputs(b, h, n, d, d, F32, seed=11)
    want = ct.causal_dot_product(q.to(DEV), k.to(DEV), v.to(DEV))
    state = torch.zeros(b, h, d, d, device=DEV)
    rows = [ct.decode_step(state, q[:, :, s].to(DEV), k[:, :, s].to(DEV), v[:, :, s].to(DEV)) for s in range(n)]
    assert rel_l2(torch.stack(rows, 2), want.double().cpu().numpy()) <= 1e-5
    assert rel_l2(torch.stack(rows, 2), oracle.causal(q, k, v)) <= 1e-4
    # the reference's past_KV is the transposed state: (B,H,Dv,Dk) = sum v (x) k   (:264)
    assert rel_l2(state.transpose(-1, -2), np.einsum("bhne,bhnd->bhed", v.double().numpy(), k.double().numpy())) <= 1e-5

PREFILL_CASES = [
    (2, 3, 200, 64, 64, BF),      # one group, column halves
    (1, 2, 1023, 64, 64, BF),     # several groups per head: every group starts from prefix + handed-over state
    (8, 16, 256, 64, 64, BF),     # many heads
    (1, 2, 130, 128, 128, HF),
    (2, 2, 257, 48, 80, BF),      # padded head dims: state rows/columns beyond (Dk,Dv) must not be touched
    (2, 2, 257, 48, 80, F32),
    (1, 3, 2500, 64, 64, F32),
    (1, 2, 63, 128, 128, F64),    # plain-FMA path, fp64 state
    (1, 1, 70, 256, 48, F32),     # plain-FMA path, state slices
]


@pytest.mark.parametrize("case", PREFILL_CASES, ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_prefill_hands_state_to_next_piece_and_to_decode(ct, oracle, case):
    # GPTCosAttention.py:253-272 builds the decode state token by token; here one call over the prompt returns it.
    # Ground truth is the pinned causal oracle on the WHOLE sequence: feeding the sequence in two pieces with
    # the state handed over, then three decode steps, must reproduce its rows.
    b, h, n, dk, dv, dt = case
    say("prefill", case)
    extra = 3
    q, k, v, _ = inputs(b, h, n + extra, dk, dv, dt, seed=n + 2)
    ref = oracle.causal(q, k, v)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    n1 = n // 3 + 1
    o1, s1 = ct.causal_prefill(qd[:, :, :n1], kd[:, :, :n1], vd[:, :, :n1])
    s1_copy = s1.clone()
    o2, s2 = ct.causal_prefill(qd[:, :, n1:n], kd[:, :, n1:n], vd[:, :, n1:n], state=s1)
    assert torch.equal(s1, s1_copy), "input state must not be modified"
    assert s2.dtype == (F64 if dt == F64 else F32) and s2.shape == (b, h, dk, dv)
    assert rel_l2(torch.cat([o1, o2], 2), ref[:, :, :n]) <= TOL[dt]
    kv = np.einsum("bhni,bhnj->bhij", k[:, :, :n].double().numpy(), v[:, :, :n].double().numpy())
    # fp32 state from 16-bit inputs: the products are exact, only the fp32 sums round (2e-6).  fp32 inputs of 33..64
    # columns are multiplied as split bf16 operands, 16 of their 24 significant bits (about 6e-6 per product, the
    # arithmetic of every fp32 result of those shapes, bounded well inside the 1e-4 of fp32 inputs)
    state_tol = 1e-12 if dt == F64 else (2e-5 if dt == F32 else 2e-6)
    assert rel_l2(s2, kv) <= state_tol
    # one call over the whole prompt gives the same state
    o, s = ct.causal_prefill(qd[:, :, :n], kd[:, :, :n], vd[:, :, :n])
    assert rel_l2(o, ref[:, :, :n]) <= TOL[dt] and rel_l2(s, kv) <= state_tol
    if dv % 4 == 0:
        rows = [ct.decode_step(s2, qd[:, :, t], kd[:, :, t], vd[:, :, t]) for t in range(n, n + extra)]
        assert rel_l2(torch.stack(rows, 2), ref[:, :, n:]) <= TOL[dt]
    # return_state=False / empty piece
    o3, none = ct.causal_prefill(qd[:, :, :n1], kd[:, :, :n1], vd[:, :, :n1], return_state=False)
    assert none is None and torch.equal(o3, o1)
    oe, se = ct.causal_prefill(qd[:, :, :0], kd[:, :, :0], vd[:, :, :0], state=s1)
    assert oe.shape == (b, h, 0, dv) and torch.equal(se, s1)
    oe, se = ct.causal_prefill(qd[:, :, :0], kd[:, :, :0], vd[:, :, :0])       # no state in: the state out is zero
    assert se.shape == (b, h, dk, dv) and not se.any()


def test_padded_rows_and_noncontiguous_inputs(ct, oracle):
    b, h, n, d = 2, 4, 150, 64
    q, k, v, _ = inputs(b, h, n, d, d, BF, seed=5)
    keep = torch.ones(n, dtype=torch.bool); keep[[0, 17, 64, 65, 149]] = False
    qm, km, vm = (x * keep[None, None, :, None] for x in (q, k, v))      # GPTCosAttention.py:245-248
    out = ct.causal_dot_product(qm.to(DEV), km.to(DEV), vm.to(DEV))
    assert torch.all(out[:, :, ~keep] == 0)
    assert rel_l2(out, oracle.causal(qm, km, vm)) <= 2e-2
    # permuted-head layout (B,N,H,D) viewed as (B,H,N,D) is accepted and made contiguous (Custom_Kernel.py:11-13)
    qp, kp, vp = (x.to(DEV).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3) for x in (q, k, v))
    assert not qp.is_contiguous()
    assert rel_l2(ct.causal_dot_product(qp, kp, vp), oracle.causal(q, k, v)) <= 2e-2


def test_custom_attention_autograd_and_dropin_names(ct, oracle):
    sys.path.insert(0, os.path.join(ROOT, "cottention_transformer_amd", "Cuda_Kernel"))
    try:
        import FastAttention
        from Custom_Kernel import CustomAttention
        from FastAttention2 import kernel
    finally:
        sys.path.pop(0)
    b, h, n, d = 1, 2, 200, 64
    q, k, v, do = inputs(b, h, n, d, d, F32, seed=2)
    qg, kg, vg = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    out = CustomAttention.apply(qg, kg, vg)                               # GPTCosAttention.py:282
    out.backward(do.to(DEV))
    assert rel_l2(out, oracle.causal(q, k, v)) <= 1e-4
    for got, ref in zip((qg.grad, kg.grad, vg.grad), oracle.causal_bwd(q, k, v, do)):
        assert rel_l2(got, ref) <= 1e-4
    # positional call of Custom_Kernel.py:24,106-108 and the three-launch backward built from it
    qd, kd, vd, gd = (x.to(DEV) for x in (q, k, v, do))
    assert rel_l2(kernel.float32(qd, kd, vd, 1, False, False), oracle.causal(q, k, v)) <= 1e-4
    refs = oracle.causal_bwd(q, k, v, do)
    assert rel_l2(kernel.float32(gd, vd, kd, 1, False, False), refs[0]) <= 1e-4
    assert rel_l2(kernel.float32(vd, gd, qd, 1, False, True), refs[1]) <= 1e-4
    assert rel_l2(kernel.float32(kd, qd, gd, 1, False, True), refs[2]) <= 1e-4
    for got, ref in zip(FastAttention.backward.float32(qd, kd, vd, gd, 1), refs):
        assert rel_l2(got, ref) <= 1e-4
    assert rel_l2(FastAttention.forward_bfloat16(qd.bfloat16(), kd.bfloat16(), vd.bfloat16(), 1), oracle.causal(
        q.bfloat16(), k.bfloat16(), v.bfloat16())) <= 2e-2
    # inplace=True leaves the output in V (combined_kernel_general.cu:403-404)
    v2 = vd.clone()
    r = kernel.float32(qd, kd, v2, 1, True, False)
    assert r.data_ptr() == v2.data_ptr() and rel_l2(v2, oracle.causal(q, k, v)) <= 1e-4
    # rejections of combined_kernel_general.cu:365-374
    with pytest.raises(RuntimeError, match="same dimension"):
        kernel.float32(qd, kd[..., :32], vd, 1, False, False)
    with pytest.raises(RuntimeError, match="divisible by 16"):
        kernel.float32(qd[..., :40].contiguous(), kd[..., :40].contiguous(), vd, 1, False, False)
    with pytest.raises(RuntimeError, match="16\\*2"):
        kernel.float32(qd[..., :16].contiguous(), kd[..., :16].contiguous(), vd, 1, False, False)


def test_autocast_backward_in_the_forward_type_is_an_option(ct, oracle):
    """CustomAttention.backward_in_forward_dtype: fp32 tensors under autocast, forward AND backward in bf16, gradients
    handed back in fp32; off by default (the reference's fp32 backward on the saved fp32 tensors, test_autocast_rule)."""
    from unittest import mock
    from cottention_transformer_amd import ops
    from cottention_transformer_amd.autograd import CustomAttention
    assert CustomAttention.backward_in_forward_dtype is False
    b, h, n, d = 2, 3, 700, 64
    q, k, v, do = inputs(b, h, n, d, d, F32, seed=6)
    qg, kg, vg = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    try:
        CustomAttention.backward_in_forward_dtype = True
        with mock.patch.object(ops, "causal_backward", wraps=ops.causal_backward) as spy:
            with torch.autocast("cuda", dtype=torch.bfloat16):
                out = CustomAttention.apply(qg, kg, vg)
            out.backward(do.to(DEV).bfloat16())
            assert spy.call_count == 1 and all(t.dtype == BF for t in spy.call_args.args[:4])
    finally:
        CustomAttention.backward_in_forward_dtype = False
    assert out.dtype == BF and all(t.grad.dtype == F32 for t in (qg, kg, vg))
    qb, kb, vb, gb = (x.bfloat16() for x in (q, k, v, do))
    assert rel_l2(out, oracle.causal(qb, kb, vb)) <= 2e-2
    for got, ref in zip((qg.grad, kg.grad, vg.grad), oracle.causal_bwd(qb, kb, vb, gb)):
        assert rel_l2(got, ref) <= 2e-2


INPLACE_CASES = [
    # (b, h, n, dk, dv, dtype, reversed): what each case runs through
    (8, 16, 512, 64, 64, BF, False),     # two column halves per head: both workgroups of a head write rows the other reads
    (1, 2, 5000, 64, 64, BF, False),     # sequence groups: the group-state pass reads v before the scan overwrites it
    (1, 2, 5000, 128, 128, HF, True),    # reversed, widest tiles (outputs staged per wavefront)
    (2, 3, 1000, 48, 80, BF, False),     # padded head dims
    (1, 2, 3000, 64, 64, F32, False),    # fp32 MFMA kernels
    (1, 2, 300, 64, 64, F64, False),     # plain-FMA kernels: no alias allowed, computed beside v and copied
    (1, 2, 300, 64, 20, F32, True),      # output dim outside the MFMA kernels' range: likewise
]


@pytest.mark.parametrize("case", INPLACE_CASES, ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_output_written_over_v(ct, oracle, case):
    """inplace=True of forward_<T> (combined_kernel_general.cu:403-404): V holds the output afterwards, bit for bit what
    the out-of-place call returns, and where the library allows the alias no second tensor of V's size is allocated."""
    from cottention_transformer_amd import _loader, ops
    b, h, n, dk, dv, dt, rev = case
    say("inplace", case)
    q, k, v, _ = inputs(b, h, n, dk, dv, dt, seed=n + dv)
    qd, kd, vd = (x.to(DEV) for x in (q, k, v))
    ref = ct.causal_dot_product(qd, kd, vd, rev)
    assert rel_l2(ref, oracle.causal(q, k, v, rev)) <= TOL[dt]
    v2 = vd.clone()
    alias = bool(_loader.lib().cott_causal_fwd_may_alias_v(b, h, n, dk, dv, ops._DTYPES[dt]))
    assert alias == (dt != F64 and dv % 16 == 0 and 32 <= dv <= 128)
    ct.causal_dot_product(qd, kd, vd.clone(), rev, into_v=True)  # (warm-up: workspace and caches allocated)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    r = ct.causal_dot_product(qd, kd, v2, rev, into_v=True)
    torch.cuda.synchronize()
    grown = torch.cuda.max_memory_allocated() - before
    assert r.data_ptr() == v2.data_ptr()
    assert torch.equal(v2, ref), "the in-place result must equal the out-of-place one bit for bit"
    if alias:  # nothing but the call's workspace (group-state slots) is allocated
        ws = _loader.lib().cott_causal_workspace_bytes(b, h, n, dk, dv, ops._DTYPES[dt])
        ws_alloc = -(-ws // (2 << 20)) * (2 << 20)  # (the caching allocator hands out large blocks in 2 MiB steps)
        assert grown <= ws_alloc + 4096, "an aliased call must not allocate a second output"
    if dk == dv:
        with pytest.raises(RuntimeError, match="must not share memory"):
            ct.causal_dot_product(v2, kd, v2, rev, into_v=True)


def test_autocast_rule(ct, oracle):
    # fp32 inputs under autocast run the forward in bf16 (combined_kernel_general.cu:377-389); backward
    # runs outside autocast on the saved fp32 tensors (Custom_Kernel.py:16,38)
    b, h, n, d = 1, 2, 96, 64
    q, k, v, do = inputs(b, h, n, d, d, F32, seed=4)
    qg, kg, vg = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = ct.CustomAttention.apply(qg, kg, vg)
    assert out.dtype == torch.bfloat16
    assert rel_l2(out, oracle.causal(q.bfloat16(), k.bfloat16(), v.bfloat16())) <= 2e-2
    out.backward(do.to(DEV).bfloat16())
    assert qg.grad.dtype == torch.float32
    for got, ref in zip((qg.grad, kg.grad, vg.grad), oracle.causal_bwd(q, k, v, do.bfloat16())):
        assert rel_l2(got, ref) <= 1e-4


def test_gradcheck_fp64(ct):
    # the reference's own invariant: gradcheck(CustomAttention.apply, fp64, eps=1e-4) (Custom_Kernel.py:188),
    # full check at a reduced size and the fast (random-projection) mode at the reference's (1,2,63,128)
    g = torch.Generator().manual_seed(0)
    small = [torch.rand(1, 2, 9, 32, generator=g, dtype=F64).to(DEV).requires_grad_(True) for _ in range(3)]
    assert torch.autograd.gradcheck(ct.CustomAttention.apply, small, eps=1e-4, atol=1e-6)
    assert torch.autograd.gradcheck(ct.NonCausalAttention.apply, small, eps=1e-4, atol=1e-6)
    big = [torch.rand(1, 2, 63, 128, generator=g, dtype=F64).to(DEV).requires_grad_(True) for _ in range(3)]
    assert torch.autograd.gradcheck(ct.CustomAttention.apply, big, eps=1e-4, atol=1e-5, fast_mode=True)


def test_headline_shape_properties(ct, oracle):
    """Full headline benchmark size (B8 H16 N2048 D64 bf16): oracle on a head subset plus size-independent
    properties -- linearity in V, `reversed` == flip(forward(flip)), last causal row == non-causal row."""
    b, h, n, d = 8, 16, 2048, 64
    say("headline shape")
    q, k, v, do = inputs(b, h, n, d, d, BF, seed=0)
    qd, kd, vd, gd = (x.to(DEV) for x in (q, k, v, do))
    out = ct.causal_dot_product(qd, kd, vd)
    dq, dk, dv = ct.causal_backward(qd, kd, vd, gd)
    sel = [(0, 0), (3, 7), (7, 15)]
    for bi, hi in sel:
        s = (slice(bi, bi + 1), slice(hi, hi + 1))
        assert rel_l2(out[s], oracle.causal(q[s], k[s], v[s])) <= 2e-2
        for got, ref in zip((dq[s], dk[s], dv[s]), oracle.causal_bwd(q[s], k[s], v[s], do[s])):
            assert rel_l2(got, ref) <= 2e-2
    # reversed == flip o forward o flip (combined_kernel_general.cu:126-130), bit-for-bit not required
    rev = ct.causal_dot_product(qd, kd, vd, True)
    via_flip = ct.causal_dot_product(qd.flip(2), kd.flip(2), vd.flip(2)).flip(2)
    assert rel_l2(rev, via_flip.double().cpu().numpy()) <= 1e-2
    # last causal row sees every key
    nc = ct.noncausal_dot_product(qd, kd, vd)
    assert rel_l2(out[:, :, -1], nc[:, :, -1].double().cpu().numpy()) <= 1e-2
    # linearity in V (exact in exact arithmetic; bf16 output rounding bounds the defect)
    out2 = ct.causal_dot_product(qd, kd, (2 * vd))
    assert rel_l2(out2, (2 * out).double().cpu().numpy()) <= 1e-2


PREP_CASES = [
    # b, h, n, dk, dv, in dtype, out dtype, masked
    (2, 3, 200, 64, 64, F32, BF, True),     # the autocast module: fp32 projections in, bf16 operands out
    (2, 3, 200, 64, 64, F32, F32, True),
    (1, 2, 63, 128, 128, F64, F64, True),
    (2, 2, 257, 48, 80, BF, BF, True),      # rows that do not fill a power-of-two lane group
    (1, 2, 130, 32, 128, HF, HF, False),
    (1, 1, 70, 256, 40, F32, HF, True),
    (1, 2, 33, 1024, 512, F32, F32, True),  # several element groups per lane
    (8, 16, 256, 64, 64, F32, BF, False),
]


@pytest.mark.parametrize("case", PREP_CASES,
                         ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1] + "-" + str(c[6]).split(".")[-1])
def test_fused_input_preparation_forward_and_backward(ct, case):
    # GPT_Trainer/GPTCosAttention.py:229-248 and BERT_Trainer/BertCosAttention.py:162-178 against their CPU statement
    # (oracle/torch_forms.py, pinned by loops in tests/test_oracle_pinning.py), gradients by torch.autograd in fp64.
    from oracle import torch_forms as tf
    b, h, n, dk, dv, dt_in, dt_out, masked = case
    say("prep", case)
    g = torch.Generator().manual_seed(n + dk)
    q, k = (torch.randn(b, h, n, dk, generator=g).to(dt_in) for _ in range(2))
    v = torch.randn(b, h, n, dv, generator=g).to(dt_in)
    q[0, 0, 1] = 0                                             # a zero row: norm clamp, gradient passes as g / eps
    keep = (torch.rand(b, n, generator=g) > 0.2) if masked else None
    sig = torch.sigmoid(torch.randn(h, generator=g)).double()
    q64, k64, v64 = (t.clone().double().requires_grad_(True) for t in (q, k, v))
    sig64 = sig.clone().requires_grad_(True)
    for form in (tf.input_prep_gpt, tf.input_prep_bert):
        rq, rk, rv, cnt = form(q64, k64, v64, keep, sig64)
        oq, ok, ov = ct.prepare_inputs(q.to(DEV), k.to(DEV), v.to(DEV), None if keep is None else keep.to(DEV),
                                       cnt.float().to(DEV), sig.float().to(DEV), out_dtype=dt_out)
        assert oq.dtype == dt_out and ov.shape == v.shape
        for got, ref in ((oq, rq), (ok, rk), (ov, rv)):
            assert rel_l2(got, ref.detach().numpy()) <= TOL[dt_out]
        if keep is not None:
            assert torch.all(oq[~keep.to(DEV)[:, None, :].expand(b, h, n)] == 0)
        # backward: upstream gradients in the output dtype
        gq, gk = (torch.randn(b, h, n, dk, generator=g).to(dt_out) for _ in range(2))
        gv = torch.randn(b, h, n, dv, generator=g).to(dt_out)
        gq[0, 0, 1] = 0                                        # keeps the g / eps term of the zero row finite
        grads = torch.autograd.grad([rq, rk, rv], [q64, k64, v64, sig64], [gq.double(), gk.double(), gv.double()])
        dq, dk_, dv_, dsig = ct.prepare_inputs_backward(q.to(DEV), k.to(DEV), v.to(DEV), gq.to(DEV), gk.to(DEV), gv.to(DEV),
                                                        None if keep is None else keep.to(DEV), cnt.float().to(DEV),
                                                        sig.float().to(DEV), want_dsig=True)
        assert dq.dtype == dt_in
        tol_in = max(TOL[dt_in], TOL[dt_out])
        for got, ref in ((dq, grads[0]), (dk_, grads[1]), (dv_, grads[2])):
            assert rel_l2(got, ref.numpy()) <= tol_in
        assert rel_l2(dsig, grads[3].numpy()) <= max(tol_in, 1e-4)
    # no value scaling: cnt and sig omitted
    oq, ok, ov = ct.prepare_inputs(q.to(DEV), k.to(DEV), v.to(DEV), out_dtype=dt_out)
    assert rel_l2(ov, v.double().numpy()) <= TOL[dt_out]


def test_prepare_inputs_autograd_function_feeds_attention(ct, oracle):
    # module-shaped use: fp32 projections -> fused prep (bf16 out) -> causal op, gradients back to q, k, v, norm_const
    from oracle import torch_forms as tf
    b, h, n, d = 2, 4, 192, 64
    g = torch.Generator().manual_seed(9)
    q, k, v = (torch.randn(b, h, n, d, generator=g) for _ in range(3))
    keep = torch.rand(b, n, generator=g) > 0.1
    norm_const = torch.randn(h, generator=g)
    go = torch.randn(b, h, n, d, generator=g)
    # CPU reference in fp64
    q64, k64, v64, c64 = (t.double().requires_grad_(True) for t in (q, k, v, norm_const))
    rq, rk, rv, cnt = tf.input_prep_gpt(q64, k64, v64, keep, torch.sigmoid(c64))
    ro = tf.causal_cumsum(rq, rk, rv)
    ref_grads = torch.autograd.grad(ro, [q64, k64, v64, c64], go.double())
    # HIP path
    qd, kd, vd, cd = (t.to(DEV).requires_grad_(True) for t in (q, k, v, norm_const))
    oq, ok, ov = ct.PrepareInputs.apply(qd, kd, vd, keep.to(DEV), cnt.float().to(DEV), torch.sigmoid(cd), torch.bfloat16)
    out = ct.CustomAttention.apply(oq, ok, ov)
    assert rel_l2(out, ro.detach().numpy()) <= 2e-2
    out.backward(go.to(DEV).to(out.dtype))
    for got, ref in zip((qd.grad, kd.grad, vd.grad, cd.grad), ref_grads):
        assert got.dtype == torch.float32
        assert rel_l2(got, ref.numpy()) <= 2e-2


@pytest.mark.parametrize("case", [(2, 3, 150, 64, 64, F32, BF, 32), (2, 2, 97, 48, 80, BF, BF, 48), (1, 2, 63, 128, 128, F64, F64, 64),
                                  (1, 4, 130, 256, 64, HF, F32, 64), (2, 2, 40, 512, 512, F32, F32, 256)],
                         ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1] + "-rot" + str(c[7]))
def test_input_preparation_with_rotary_and_projection_layout(ct, case):
    # GPTCosAttention.py:444-479: split heads (B,S,H,D), rotary on the first R columns of q and k, permute to
    # (B,H,S,D), then the preparation steps -- against the same sequence written with the CPU forms.
    from oracle import torch_forms as tf
    b, h, n, dk, dv, dt_in, dt_out, rdim = case
    say("prep+rotary", case)
    g = torch.Generator().manual_seed(n + rdim)
    q, k = (torch.randn(b, n, h, dk, generator=g).to(dt_in) for _ in range(2))
    v = torch.randn(b, n, h, dv, generator=g).to(dt_in)
    keep = torch.rand(b, n, generator=g) > 0.2
    sig = torch.sigmoid(torch.randn(h, generator=g)).double()
    table = tf.gptj_sinusoid_table(300, rdim)
    pos = torch.randint(0, 300, (b, n), generator=g)
    q64, k64, v64 = (t.clone().double().requires_grad_(True) for t in (q, k, v))
    sig64 = sig.clone().requires_grad_(True)
    sin, cos = torch.split(table.double()[pos], rdim // 2, dim=-1)
    qr = torch.cat([tf.gptj_rotate(q64[..., :rdim], sin, cos), q64[..., rdim:]], -1).permute(0, 2, 1, 3)
    kr = torch.cat([tf.gptj_rotate(k64[..., :rdim], sin, cos), k64[..., rdim:]], -1).permute(0, 2, 1, 3)
    rq, rk, rv, cnt = tf.input_prep_gpt(qr, kr, v64.permute(0, 2, 1, 3), keep, sig64)
    args = dict(keep=keep.to(DEV), cnt=cnt.float().to(DEV), sig=sig.float().to(DEV), rotary=(table.to(DEV), pos.to(DEV)),
                bnhd=True)
    oq, ok, ov = ct.prepare_inputs(q.to(DEV), k.to(DEV), v.to(DEV), out_dtype=dt_out, **args)
    assert oq.shape == (b, h, n, dk) and ov.shape == (b, h, n, dv) and oq.is_contiguous()
    for got, ref in ((oq, rq), (ok, rk), (ov, rv)):
        assert rel_l2(got, ref.detach().numpy()) <= TOL[dt_out]
    gq, gk = (torch.randn(b, h, n, dk, generator=g).to(dt_out) for _ in range(2))
    gv = torch.randn(b, h, n, dv, generator=g).to(dt_out)
    grads = torch.autograd.grad([rq, rk, rv], [q64, k64, v64, sig64], [gq.double(), gk.double(), gv.double()])
    dq, dk_, dv_, dsig = ct.prepare_inputs_backward(q.to(DEV), k.to(DEV), v.to(DEV), gq.to(DEV), gk.to(DEV), gv.to(DEV),
                                                    want_dsig=True, **args)
    assert dq.shape == q.shape and dq.dtype == dt_in
    tol = max(TOL[dt_in], TOL[dt_out])
    for got, ref in ((dq, grads[0]), (dk_, grads[1]), (dv_, grads[2])):
        assert rel_l2(got, ref.numpy()) <= tol
    assert rel_l2(dsig, grads[3].numpy()) <= max(tol, 1e-4)
    with pytest.raises(RuntimeError):
        ct.prepare_inputs(q.to(DEV), k.to(DEV), v.to(DEV), rotary=(table.to(DEV), (pos + 300).to(DEV)), bnhd=True)
    # without the host-side check a stray position is clamped to the table by the kernel, never read out of bounds
    far = pos.clone(); far[0, 0] = 10 ** 9; far[0, 1] = -5
    clamped = far.clamp(0, 299)
    a1 = ct.prepare_inputs(q.to(DEV), k.to(DEV), v.to(DEV), rotary=(table.to(DEV), far.to(DEV)), bnhd=True, check_positions=False)
    a2 = ct.prepare_inputs(q.to(DEV), k.to(DEV), v.to(DEV), rotary=(table.to(DEV), clamped.to(DEV)), bnhd=True)
    assert all(torch.equal(x, y) for x, y in zip(a1, a2))


def test_calls_can_be_captured_in_a_hip_graph_and_replayed(ct, oracle):
    # The library allocates nothing and never synchronises, so its launches can be recorded into a graph: a decode
    # step (state updated in place by every replay) and a forward+backward pair with fixed buffers.  Replays are
    # interleaved with eager work and synchronisation, and every replay is checked against the eager result.
    from cottention_transformer_amd import _loader
    L = _loader.lib()
    b, h, d = 4, 4, 64
    g = torch.Generator().manual_seed(21)
    steps = 5
    qs = torch.nn.functional.normalize(torch.randn(steps, b, h, d, generator=g), dim=-1).to(BF).to(DEV)
    ks = torch.nn.functional.normalize(torch.randn(steps, b, h, d, generator=g), dim=-1).to(BF).to(DEV)
    vs = torch.randn(steps, b, h, d, generator=g).to(BF).to(DEV)
    q1, k1, v1 = (torch.empty(b, h, d, dtype=BF, device=DEV) for _ in range(3))
    out = torch.empty(b, h, d, dtype=BF, device=DEV)
    state = torch.zeros(b, h, d, d, device=DEV)
    eager_state = torch.zeros(b, h, d, d, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                         # warm-up on the capture stream
        q1.copy_(qs[0]); k1.copy_(ks[0]); v1.copy_(vs[0])
        ct.decode_step(torch.zeros_like(state), q1, k1, v1, out=out)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        rc = L.cott_decode_step(state.data_ptr(), q1.data_ptr(), k1.data_ptr(), v1.data_ptr(), out.data_ptr(), b, h, d, d,
                                _loader.BF16, torch.cuda.current_stream().cuda_stream)
        assert rc == 0
    for t in range(steps):
        q1.copy_(qs[t]); k1.copy_(ks[t]); v1.copy_(vs[t])
        graph.replay()
        want = ct.decode_step(eager_state, qs[t], ks[t], vs[t])          # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {t}"
    assert torch.equal(state, eager_state)

    # forward + backward of a multi-group shape (workspace in use) in one graph
    bb, hh, n = 1, 2, 1023
    q, k, v, do = (x.to(DEV) for x in inputs(bb, hh, n, 64, 64, BF, seed=33))
    o = torch.empty_like(v); dq = torch.empty_like(q); dk = torch.empty_like(k); dv = torch.empty_like(v)
    nf = L.cott_causal_workspace_bytes(bb, hh, n, 64, 64, _loader.BF16)
    nb = L.cott_causal_bwd_workspace_bytes(bb, hh, n, 64, 64, _loader.BF16)
    assert nf > 0 and nb > 0
    wsf = torch.empty(nf, dtype=torch.uint8, device=DEV); wsb = torch.empty(nb, dtype=torch.uint8, device=DEV)
    graph2 = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph2, stream=side):
        st = torch.cuda.current_stream().cuda_stream
        assert L.cott_causal_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), bb, hh, n, 64, 64, _loader.BF16, 0,
                                 wsf.data_ptr(), nf, st) == 0
        assert L.cott_causal_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                                 dv.data_ptr(), bb, hh, n, 64, 64, _loader.BF16, wsb.data_ptr(), nb, st) == 0
    for rep in range(3):
        new = [x.to(DEV) for x in inputs(bb, hh, n, 64, 64, BF, seed=40 + rep)]
        for dst, src in zip((q, k, v, do), new):
            dst.copy_(src)
        graph2.replay()
        want_o = ct.causal_dot_product(*new[:3])
        want_g = ct.causal_backward(*new)
        torch.cuda.synchronize()
        assert torch.equal(o, want_o), f"replay {rep}"
        for got, want in zip((dq, dk, dv), want_g):
            assert torch.equal(got, want), f"replay {rep}"

    # the same pair as a training step runs it: the forward leaves its states, the backward takes them (both a shape
    # cut into groups and one with pair workgroups of one group each)
    import ctypes
    for bb, hh, n in ((1, 2, 1023), (8, 16, 1024)):
        q, k, v, do = (x.to(DEV) for x in inputs(bb, hh, n, 64, 64, BF, seed=50))
        plan = ct.saved_states_plan(BF, bb, hh, n, 64, 64)
        assert plan is not None
        cpc, cuts, slot, nb = plan
        o = torch.empty_like(v); dq = torch.empty_like(q); dk = torch.empty_like(k); dv = torch.empty_like(v)
        saved = torch.empty(bb, hh, cuts, slot, device=DEV)
        nf = L.cott_causal_workspace_bytes(bb, hh, n, 64, 64, _loader.BF16)
        wsf = torch.empty(max(nf, 16), dtype=torch.uint8, device=DEV); wsb = torch.empty(max(nb, 16), dtype=torch.uint8, device=DEV)
        sp = ctypes.cast(saved.data_ptr(), ctypes.c_void_p)
        graph3 = torch.cuda.CUDAGraph()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.graph(graph3, stream=side):
            st = torch.cuda.current_stream().cuda_stream
            assert L.cott_causal_fwd_save(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), sp, cpc, cuts, bb, hh, n,
                                          64, 64, _loader.BF16, wsf.data_ptr() if nf else None, nf, st) == 0
            assert L.cott_causal_bwd_saved(q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), dq.data_ptr(),
                                           dk.data_ptr(), dv.data_ptr(), sp, cpc, cuts, bb, hh, n, 64, 64, _loader.BF16,
                                           wsb.data_ptr() if nb else None, nb, st) == 0
        for rep in range(3):
            new = [x.to(DEV) for x in inputs(bb, hh, n, 64, 64, BF, seed=60 + rep)]
            for dst, src in zip((q, k, v, do), new):
                dst.copy_(src)
            graph3.replay()
            want_o, want_s = ct.causal_dot_product_saving(*new[:3])
            want_g = ct.causal_backward(*new, saved=want_s)
            torch.cuda.synchronize()
            assert torch.equal(o, want_o) and torch.equal(saved, want_s), f"replay {rep}"
            for got, want in zip((dq, dk, dv), want_g):
                assert torch.equal(got, want), f"replay {rep}"


FUSED_PREP_CASES = [
    # b, h, n, dk, dv, dtype, rotary_dim, projections' layout, masked   launch form
    (8, 16, 256, 64, 64, BF, 64, True, True),      # two column halves per head, outputs staged through LDS
    (8, 16, 130, 64, 128, BF, 32, True, True),     # wide values in column halves, rotation of half of the columns
    (32, 16, 200, 48, 80, HF, 32, False, True),    # padded head dims, two workgroups per CU
    (16, 16, 63, 32, 64, BF, 0, False, False),     # no rotation, no mask, a single partial chunk
    (8, 32, 1000, 64, 64, HF, 16, True, True),     # several chunks, ragged tail
    # 128-wide q / k rows: the kernel whose loader wavefronts stage all three tiles
    (8, 16, 300, 128, 128, BF, 64, True, True),    # two column halves per head (value tiles of 64 columns)
    (40, 8, 200, 128, 128, HF, 128, False, True),  # whole 128 x 128 tiles, every column rotated
    (8, 16, 130, 96, 80, BF, 32, True, False),     # padded head dims, no mask
    # sequences cut into groups: the group sums are formed from rows prepared the same way
    (1, 4, 3000, 64, 64, BF, 64, True, True),      # 64-wide heads in groups
    (2, 2, 2500, 48, 80, HF, 16, False, True),     # padded, per-head layout
    (1, 16, 4100, 128, 128, BF, 64, True, True),   # 128-wide: column halves in groups, ragged tail
    (1, 3, 6000, 128, 128, BF, 32, False, True),   # 128-wide: whole tiles in many groups
    # whole problems in groups (the plans of many heads on long sequences): the group sums come from the kernel with
    # loader and compute wavefronts
    (1, 64, 4100, 128, 128, BF, 64, True, True),   # 128 x 128 tiles, four groups, ragged tail
    (4, 16, 8200, 64, 64, HF, 32, False, True),    # 64 x 64 tiles
    (2, 32, 4096, 64, 128, BF, 16, True, False),   # 64-wide rows, 128-wide values
]


@pytest.mark.parametrize("case", FUSED_PREP_CASES,
                         ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1] + f"-rot{c[6]}")
def test_input_preparation_inside_the_forward_kernel(ct, oracle, case):
    """cott_causal_fwd_prep: rotary, normalisation, value scaling and mask inside the causal forward kernel
    (GPT_Trainer/GPTCosAttention.py:229-248, 462-476, 282 as one launch) against the CPU statements of those steps
    (oracle/torch_forms.py) followed by the causal oracle; the prepared tensors it leaves for the backward pass
    against the same statements; and the autograd function built on it against autograd through the CPU forms."""
    from oracle import torch_forms as tf
    b, h, n, dk, dv, dt, rdim, bnhd, masked = case
    say("fused preparation", case)
    assert ct.fused_preparation_supported(dt, b, h, n, dk, dv, rdim)
    g = torch.Generator().manual_seed(n + dk + rdim)
    shape = (lambda d: (b, n, h, d)) if bnhd else (lambda d: (b, h, n, d))
    q, k, v = (torch.randn(shape(d), generator=g).to(dt) for d in (dk, dk, dv))
    keep = (torch.rand(b, n, generator=g) > 0.2) if masked else None
    sig = torch.sigmoid(torch.randn(h, generator=g))
    go = torch.randn(b, h, n, dv, generator=g).to(dt)
    pos0 = 5
    table = tf.gptj_sinusoid_table(n + 40, rdim).float() if rdim else None
    # CPU reference in fp64, (B,H,N,D)
    q64, k64, v64, s64 = (t.double().requires_grad_(True) for t in (q, k, v, sig))
    qh, kh, vh = ((t.permute(0, 2, 1, 3) if bnhd else t) for t in (q64, k64, v64))
    if rdim:
        sin, cos = torch.split(table.double()[pos0:pos0 + n][None].expand(b, n, rdim), rdim // 2, dim=-1)
        rot = lambda x: torch.cat([tf.gptj_rotate(x.permute(0, 2, 1, 3)[..., :rdim], sin, cos).permute(0, 2, 1, 3),
                                   x[..., rdim:]], -1)
        qh, kh = rot(qh), rot(kh)
    rq, rk, rv, cnt = tf.input_prep_gpt(qh, kh, vh, keep, s64)
    ref_o = oracle.causal(rq.detach(), rk.detach(), rv.detach())
    # the kernel
    args = dict(keep=None if keep is None else keep.to(DEV), cnt=cnt.float().to(DEV), sig=sig.to(DEV),
                rotary=(table.to(DEV), pos0) if rdim else None, bnhd=bnhd)
    for merged in (False, True):
        o, prepared = ct.causal_dot_product_prepared(q.to(DEV), k.to(DEV), v.to(DEV), merged_heads=merged, **args)
        assert o.shape == ((b, n, h, dv) if merged else (b, h, n, dv)) and o.dtype == dt
        assert rel_l2(o.permute(0, 2, 1, 3) if merged else o, ref_o) <= TOL[dt], merged
        for name, got, ref in zip("qkv", prepared, (rq, rk, rv)):
            assert got.shape == ref.shape and rel_l2(got, ref.detach().numpy()) <= TOL[dt], name
        if keep is not None:
            assert torch.all(prepared[0][~keep.to(DEV)[:, None, :].expand(b, h, n)] == 0)
    # the same numbers as the two-kernel path on the same prepared operands (the products are the same code)
    o2 = ct.causal_dot_product(*prepared)
    assert rel_l2(o2, o.permute(0, 2, 1, 3).double().cpu().numpy()) <= 1e-2
    o_np, none = ct.causal_dot_product_prepared(q.to(DEV), k.to(DEV), v.to(DEV), want_prepared=False, **args)
    assert none is None and rel_l2(o_np, ref_o) <= TOL[dt]
    # Gradients through the autograd function, at every length: the oracle's closed forms (Custom_Kernel.py:63,68,72)
    # give the gradients with respect to the prepared tensors, and autograd carries those through the CPU statement of
    # the preparation; no O(N D^2) cumsum tensor is needed.  Short sequences also go through the cumsum form, whose
    # gradients autograd derives on its own.
    d_prepared = [torch.from_numpy(x) for x in oracle.causal_bwd(rq.detach(), rk.detach(), rv.detach(), go)]
    ref_grads = torch.autograd.grad([rq, rk, rv], [q64, k64, v64, s64], d_prepared, retain_graph=n <= 300)
    if n <= 300:
        by_cumsum = torch.autograd.grad(tf.causal_cumsum(rq, rk, rv), [q64, k64, v64, s64], go.double())
        for a, r in zip(ref_grads, by_cumsum):
            assert rel_l2(a, r.numpy()) <= 1e-9
    qd, kd, vd, sd = (t.to(DEV).requires_grad_(True) for t in (q, k, v, sig))
    out = ct.PreparedCausalAttention.apply(qd, kd, vd, args["keep"], args["cnt"], sd, table.to(DEV) if rdim else None, pos0,
                                           bnhd, False)
    assert rel_l2(out, ref_o) <= TOL[dt]
    out.backward(go.to(DEV))
    for name, got, ref in zip(("dq", "dk", "dv", "dsig"), (qd.grad, kd.grad, vd.grad, sd.grad), ref_grads):
        assert got.shape == ref.shape and rel_l2(got, ref.numpy()) <= 2e-2, name


@pytest.mark.parametrize("case", [(8, 16, 256, 64, 64, BF, 64, True), (4, 32, 1000, 64, 128, HF, 16, False),
                                  (10, 16, 300, 128, 128, BF, 32, True),      # 128-wide rows: the column-owner scan
                                  (2, 8, 700, 128, 128, HF, 128, False),      # ... cut into groups (preparing group-state pass)
                                  (1, 4, 3000, 64, 64, BF, 64, True)],        # 64-wide rows in groups
                         ids=["8x16x256-bf16-bnhd", "4x32x1000-fp16", "10x16x300x128-bf16-bnhd", "2x8x700x128-fp16-groups",
                              "1x4x3000-bf16-bnhd-groups"])
def test_fused_preparation_with_position_ids(ct, oracle, case):
    """cott_causal_fwd_prep with the block's own position_ids tensor (GPT_Trainer/GPTCosAttention.py:458): ids that are
    neither consecutive nor equal across the batch, one row repeated for the whole batch as GPT-J's model passes them,
    and ids outside the table (clamped on the device), forward and gradients, against the CPU statements."""
    from oracle import torch_forms as tf
    b, h, n, dk, dv, dt, rdim, bnhd = case
    say("fused preparation, position ids", case)
    g = torch.Generator().manual_seed(n + rdim)
    shape = (lambda d: (b, n, h, d)) if bnhd else (lambda d: (b, h, n, d))
    q, k, v = (torch.randn(shape(d), generator=g).to(dt) for d in (dk, dk, dv))
    keep = torch.rand(b, n, generator=g) > 0.2
    sig = torch.sigmoid(torch.randn(h, generator=g))
    go = torch.randn(b, h, n, dv, generator=g).to(dt)
    rows = n + 40
    table = tf.gptj_sinusoid_table(rows, rdim).float()
    for kind in ("scattered", "one row", "outside the table"):
        if kind == "scattered":
            ids = torch.randint(0, rows, (b, n), generator=g)
        elif kind == "one row":
            ids = torch.arange(7, 7 + n)[None, :]
        else:
            ids = torch.randint(-5, rows + 9, (b, n), generator=g)
        ref_ids = ids.clamp(0, rows - 1).expand(b, n)
        q64, k64, v64, s64 = (t.double().requires_grad_(True) for t in (q, k, v, sig))
        qh, kh, vh = ((t.permute(0, 2, 1, 3) if bnhd else t) for t in (q64, k64, v64))
        sin, cos = torch.split(table.double()[ref_ids], rdim // 2, dim=-1)
        rot = lambda x: torch.cat([tf.gptj_rotate(x.permute(0, 2, 1, 3)[..., :rdim], sin, cos).permute(0, 2, 1, 3),
                                   x[..., rdim:]], -1)
        rq, rk, rv, cnt = tf.input_prep_gpt(rot(qh), rot(kh), vh, keep, s64)
        ref_o = oracle.causal(rq.detach(), rk.detach(), rv.detach())
        d_prepared = [torch.from_numpy(x) for x in oracle.causal_bwd(rq.detach(), rk.detach(), rv.detach(), go)]
        ref_grads = torch.autograd.grad([rq, rk, rv], [q64, k64, v64, s64], d_prepared)
        o, prepared = ct.causal_dot_product_prepared(q.to(DEV), k.to(DEV), v.to(DEV), keep=keep.to(DEV), cnt=cnt.float().to(DEV),
                                                     sig=sig.to(DEV), rotary=(table.to(DEV), ids.to(DEV)), bnhd=bnhd)
        assert rel_l2(o, ref_o) <= TOL[dt], kind
        for name, got, ref in zip("qkv", prepared, (rq, rk, rv)):
            assert rel_l2(got, ref.detach().numpy()) <= TOL[dt], (kind, name)
        if kind == "outside the table":
            continue  # (the separate backward of the preparation clamps the same way; covered by its own test)
        qd, kd, vd, sd = (t.to(DEV).requires_grad_(True) for t in (q, k, v, sig))
        out = ct.PreparedCausalAttention.apply(qd, kd, vd, keep.to(DEV), cnt.float().to(DEV), sd, table.to(DEV), ids.to(DEV),
                                               bnhd, False)
        assert rel_l2(out, ref_o) <= TOL[dt], kind
        out.backward(go.to(DEV))
        for name, got, ref in zip(("dq", "dk", "dv", "dsig"), (qd.grad, kd.grad, vd.grad, sd.grad), ref_grads):
            assert got.shape == ref.shape and rel_l2(got, ref.numpy()) <= 2e-2, (kind, name)


NC_FUSED_PREP_CASES = [
    # b, h, n, dk, dv, dtype, projections' layout, masked      launch form
    (32, 12, 512, 64, 64, BF, True, True),     # the BERT-base shape: two column halves per head, eight chunks
    (40, 8, 300, 64, 64, HF, True, True),      # ragged tail
    (16, 16, 130, 64, 32, BF, True, True),     # one workgroup per head, narrower values
    (64, 8, 63, 32, 64, BF, False, False),     # no mask, a single partial chunk, per-head layout
    (48, 8, 200, 48, 48, HF, False, True),     # padded head dims
    (16, 16, 300, 128, 128, BF, True, True),   # 128-wide heads
    (20, 16, 200, 128, 64, HF, False, True),   # wide q / k rows, narrower values
    (24, 12, 130, 80, 112, BF, True, False),   # padded to 128 on both sides
]


@pytest.mark.parametrize("case", NC_FUSED_PREP_CASES,
                         ids=lambda c: "x".join(map(str, c[:5])) + "-" + str(c[5]).split(".")[-1])
def test_input_preparation_inside_the_non_causal_kernel(ct, oracle, case):
    """cott_noncausal_fwd_prep: mask, normalisation and value scaling inside the non-causal kernel
    (BERT_Trainer/BertCosAttention.py:162-178, 249 as one launch) against the CPU statement of those steps
    (oracle/torch_forms.py) followed by the non-causal oracle; the prepared tensors it leaves for the backward pass;
    the two-kernel path on the same inputs; and the autograd function against autograd through the CPU forms."""
    from oracle import torch_forms as tf
    b, h, n, dk, dv, dt, bnhd, masked = case
    say("fused preparation, non-causal", case)
    assert ct.noncausal_fused_preparation_supported(dt, b, h, n, dk, dv)
    g = torch.Generator().manual_seed(n + dk)
    shape = (lambda d: (b, n, h, d)) if bnhd else (lambda d: (b, h, n, d))
    q, k, v = (torch.randn(shape(d), generator=g).to(dt) for d in (dk, dk, dv))
    keep = None
    if masked:  # padding at the end of every sequence, as a BERT batch has it
        keep = torch.arange(n)[None, :] < torch.randint(1, n + 1, (b, 1), generator=g)
    sig = torch.sigmoid(torch.randn(h, generator=g))
    go = torch.randn(b, h, n, dv, generator=g).to(dt)
    q64, k64, v64, s64 = (t.double().requires_grad_(True) for t in (q, k, v, sig))
    qh, kh, vh = ((t.permute(0, 2, 1, 3) if bnhd else t) for t in (q64, k64, v64))
    rq, rk, rv, cnt = tf.input_prep_bert(qh, kh, vh, keep, s64)
    ref_o = oracle.noncausal(rq.detach(), rk.detach(), rv.detach())
    args = dict(keep=None if keep is None else keep.to(DEV), cnt=cnt.float().to(DEV), sig=sig.to(DEV), bnhd=bnhd)
    for merged in (False, True):
        o, prepared = ct.noncausal_dot_product_prepared(q.to(DEV), k.to(DEV), v.to(DEV), merged_heads=merged, **args)
        assert o.shape == ((b, n, h, dv) if merged else (b, h, n, dv)) and o.dtype == dt
        assert rel_l2(o.permute(0, 2, 1, 3) if merged else o, ref_o) <= TOL[dt], merged
        for name, got, ref in zip("qkv", prepared, (rq, rk, rv)):
            assert got.shape == ref.shape and rel_l2(got, ref.detach().numpy()) <= TOL[dt], name
        if keep is not None:
            dropped = ~keep.to(DEV)[:, None, :].expand(b, h, n)
            assert all(torch.all(t[dropped] == 0) for t in prepared)
    # the separate preparation pass followed by the plain op gives the same numbers to 16-bit rounding
    p2 = ct.prepare_inputs(q.to(DEV), k.to(DEV), v.to(DEV), args["keep"], args["cnt"], args["sig"], out_dtype=dt, bnhd=bnhd)
    for a, r in zip(prepared, p2):
        assert rel_l2(a, r.double().cpu().numpy()) <= 1e-2
    o2 = ct.noncausal_dot_product(*p2)
    assert rel_l2(o2, o.permute(0, 2, 1, 3).double().cpu().numpy()) <= 1e-2
    # gradients through the autograd function
    ro = tf.noncausal_einsum(rq, rk, rv)
    ref_grads = torch.autograd.grad(ro, [q64, k64, v64, s64], go.double())
    qd, kd, vd, sd = (t.to(DEV).requires_grad_(True) for t in (q, k, v, sig))
    out = ct.PreparedNonCausalAttention.apply(qd, kd, vd, args["keep"], args["cnt"], sd, bnhd, False)
    assert rel_l2(out, ref_o) <= TOL[dt]
    out.backward(go.to(DEV))
    for name, got, ref in zip(("dq", "dk", "dv", "dsig"), (qd.grad, kd.grad, vd.grad, sd.grad), ref_grads):
        assert got.shape == ref.shape and rel_l2(got, ref.numpy()) <= 2e-2, name


def test_non_causal_fused_preparation_is_refused_where_not_built(ct):
    assert not ct.noncausal_fused_preparation_supported(F32, 32, 12, 512, 64, 64)
    assert not ct.noncausal_fused_preparation_supported(BF, 1, 2, 4096, 64, 64)      # few heads: sequence groups
    q = torch.randn(1, 2, 4096, 64, device=DEV, dtype=BF)
    assert ct.noncausal_fused_preparation_supported(BF, 16, 16, 512, 128, 128)       # wide heads
    with pytest.raises(RuntimeError, match="one workgroup"):
        ct.noncausal_dot_product_prepared(q, q, q)


def test_fused_preparation_is_refused_where_not_built(ct):
    assert not ct.fused_preparation_supported(F32, 8, 16, 256, 64, 64)
    assert not ct.fused_preparation_supported(BF, 8, 16, 256, 64, 64, 12)    # rotary width not a multiple of 8
    assert not ct.fused_preparation_supported(BF, 8, 16, 256, 128, 32, 64)   # 128-wide q / k rows with narrow value tiles
    assert ct.fused_preparation_supported(BF, 1, 2, 4096, 64, 64)            # few heads: sequence groups
    assert ct.fused_preparation_supported(BF, 8, 16, 256, 128, 128, 64)      # wide q / k rows
    q, k, v, _ = inputs(8, 16, 64, 128, 32, BF, seed=1)
    with pytest.raises(RuntimeError, match="not built for these head dims"):
        ct.causal_dot_product_prepared(q.to(DEV), k.to(DEV), v.to(DEV))
    q, k, v, _ = inputs(8, 16, 64, 64, 64, F32, seed=1)
    with pytest.raises(RuntimeError, match="bf16 / fp16"):
        ct.causal_dot_product_prepared(q.to(DEV), k.to(DEV), v.to(DEV))
