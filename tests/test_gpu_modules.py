"""GPU parity of the module-level drop-ins (cottention_transformer_amd/modules.py) against the CPU statements of the
reference's attention blocks (oracle/torch_forms.py) with identical weights and inputs."""
import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from util import rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def mods():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from cottention_transformer_amd import _loader, modules
    assert os.path.exists(_loader.lib_path()), "libcottention_hip.so must be prebuilt in-tree"
    _loader.lib()
    return modules


def gpt_cfg(e=256, heads=4, rot=32, max_pos=512, fast=False):
    return SimpleNamespace(max_position_embeddings=max_pos, attn_pdrop=0.0, resid_pdrop=0.0, hidden_size=e,
                           num_attention_heads=heads, rotary_dim=rot, fast_inference=fast)


def additive_mask(keep):
    # what the surrounding HF model hands to the block: 0 at real tokens, a large negative number at padding
    return ((~keep).float() * torch.finfo(torch.float32).min)[:, None, None, :]


def gpt_reference(tf, m, hidden, keep, **kw):
    w = [getattr(m, n).weight.detach().double().cpu() for n in ("q_proj", "k_proj", "v_proj", "out_proj")]
    nc = m.norm_const.detach().double().cpu().reshape(-1)
    return w, nc


@pytest.mark.parametrize("autocast", [False, True], ids=["fp32", "autocast-bf16"])
def test_gpt_block_forward_backward(mods, autocast):
    from oracle import torch_forms as tf
    say("gpt block", autocast)
    torch.manual_seed(0)
    cfg = gpt_cfg()
    m = mods.GPTCosAttention(cfg).to(DEV)
    with torch.no_grad():
        m.norm_const.copy_(torch.tensor([0.2, 0.5, -0.4, 1.0]).reshape(1, 4, 1, 1))
    b, s = 2, 200
    g = torch.Generator().manual_seed(1)
    hidden = torch.randn(b, s, cfg.hidden_size, generator=g)
    keep = torch.rand(b, s, generator=g) > 0.15
    gout = torch.randn(b, s, cfg.hidden_size, generator=g)
    # CPU reference in fp64 with the same weights
    w = [getattr(m, n).weight.detach().double().cpu().requires_grad_(True) for n in ("q_proj", "k_proj", "v_proj", "out_proj")]
    nc = m.norm_const.detach().double().cpu().reshape(-1).requires_grad_(True)
    h64 = hidden.double().requires_grad_(True)
    ref = tf.gpt_attention_block(h64, *w, nc, cfg.num_attention_heads, cfg.rotary_dim, cfg.max_position_embeddings, keep)
    ref_grads = torch.autograd.grad(ref, [h64, *w, nc], gout.double())
    # HIP path
    hd = hidden.to(DEV).requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
        out, present = m(hd, attention_mask=additive_mask(keep).to(DEV))
    assert present is None and out.shape == hidden.shape
    tol = 3e-2 if autocast else 1e-4
    assert rel_l2(out.float(), ref.detach().numpy()) <= tol
    out.backward(gout.to(DEV).to(out.dtype))
    got = [hd.grad, m.q_proj.weight.grad, m.k_proj.weight.grad, m.v_proj.weight.grad, m.out_proj.weight.grad,
           m.norm_const.grad.reshape(-1)]
    for name, a, r in zip(("hidden", "wq", "wk", "wv", "wo", "norm_const"), got, ref_grads):
        assert rel_l2(a.float(), r.numpy()) <= tol, name


@pytest.mark.parametrize("positions", ["none", "model", "custom"])
@pytest.mark.parametrize("masked", [False, True], ids=["no-mask", "masked"])
def test_gpt_block_with_the_preparation_inside_the_attention_kernel(mods, masked, positions):
    """Enough heads that no head is cut into sequence groups, bf16 autocast: the forward of the block then runs rotation,
    normalisation, value scaling, mask and attention as one launch (PreparedCausalAttention), whether the block makes
    the positions itself (position_ids=None), receives them the way GPT-J's model passes them (one arange row for the
    whole batch, GPT_Trainer/GPTCosAttention.py:458) or receives other ids per batch element.  Same check as above,
    against the fp64 CPU statement of the block."""
    from unittest import mock
    from oracle import torch_forms as tf
    from cottention_transformer_amd import ops
    say("gpt block, fused preparation", masked)
    torch.manual_seed(0)
    cfg = gpt_cfg(e=1024, heads=16, rot=32, max_pos=256)
    m = mods.GPTCosAttention(cfg).to(DEV)
    with torch.no_grad():
        m.norm_const.copy_(torch.linspace(-1.0, 1.0, 16).reshape(1, 16, 1, 1))
    b, s = 16, 136
    g = torch.Generator().manual_seed(2)
    hidden = torch.randn(b, s, cfg.hidden_size, generator=g)
    keep = (torch.rand(b, s, generator=g) > 0.15) if masked else torch.ones(b, s, dtype=torch.bool)
    gout = torch.randn(b, s, cfg.hidden_size, generator=g)
    w = [getattr(m, n).weight.detach().double().cpu().requires_grad_(True) for n in ("q_proj", "k_proj", "v_proj", "out_proj")]
    nc = m.norm_const.detach().double().cpu().reshape(-1).requires_grad_(True)
    h64 = hidden.double().requires_grad_(True)
    ids = {"none": None, "model": torch.arange(0, s)[None, :],
           "custom": torch.randint(0, cfg.max_position_embeddings, (b, s), generator=g)}[positions]
    ref = tf.gpt_attention_block(h64, *w, nc, cfg.num_attention_heads, cfg.rotary_dim, cfg.max_position_embeddings, keep,
                                 position_ids=None if ids is None else ids.expand(b, s))
    ref_grads = torch.autograd.grad(ref, [h64, *w, nc], gout.double())
    hd = hidden.to(DEV).requires_grad_(True)
    with mock.patch.object(ops, "causal_dot_product_prepared", wraps=ops.causal_dot_product_prepared) as spy:
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out, present = m(hd, attention_mask=additive_mask(keep).to(DEV) if masked else None,
                             position_ids=None if ids is None else ids.to(DEV))
        assert spy.call_count == 1, "the fused forward was not taken"
    assert rel_l2(out.float(), ref.detach().numpy()) <= 3e-2
    out.backward(gout.to(DEV).to(out.dtype))
    got = [hd.grad, m.q_proj.weight.grad, m.k_proj.weight.grad, m.v_proj.weight.grad, m.out_proj.weight.grad,
           m.norm_const.grad.reshape(-1)]
    for name, a, r in zip(("hidden", "wq", "wk", "wv", "wo", "norm_const"), got, ref_grads):
        assert rel_l2(a.float(), r.numpy()) <= 3e-2, name


def test_gpt_block_recurrent_inference(mods):
    # GPTCosAttention.py:77-87,234-236,253-272: a prompt, then single tokens, against the per-token loop on the CPU
    from oracle import torch_forms as tf
    say("gpt recurrent")
    torch.manual_seed(0)
    cfg = gpt_cfg(fast=True)
    m = mods.GPTCosAttention(cfg).to(DEV).eval()
    b, s, extra = 2, 70, 3
    g = torch.Generator().manual_seed(4)
    hidden = torch.randn(b, s + extra, cfg.hidden_size, generator=g)
    w = [getattr(m, n).weight.detach().double().cpu() for n in ("q_proj", "k_proj", "v_proj", "out_proj")]
    nc = m.norm_const.detach().double().cpu().reshape(-1)
    d = cfg.hidden_size // cfg.num_attention_heads
    state = torch.zeros(b, cfg.num_attention_heads, d, d, dtype=torch.float64)
    ref, state, cur = tf.gpt_attention_block_recurrent(hidden.double(), *w, nc, cfg.num_attention_heads, cfg.rotary_dim,
                                                       cfg.max_position_embeddings, state, 1)
    with torch.no_grad():
        outs = [m(hidden[:, :s].to(DEV))[0]]
        for t in range(s, s + extra):
            outs.append(m(hidden[:, t:t + 1].to(DEV))[0])
    assert m.cur_s == cur
    assert rel_l2(torch.cat(outs, 1), ref.numpy()) <= 1e-4
    assert rel_l2(m.state.transpose(-1, -2), state.numpy()) <= 1e-5     # the reference keeps v (x) k
    m.reset_state()
    assert m.state is None and m.cur_s == 1


@pytest.mark.parametrize("autocast", [False, True], ids=["fp32", "autocast-bf16"])
def test_bert_block_forward_backward(mods, autocast):
    from oracle import torch_forms as tf
    say("bert block", autocast)
    torch.manual_seed(0)
    cfg = SimpleNamespace(hidden_size=256, num_attention_heads=4, attention_probs_dropout_prob=0.0, is_decoder=False)
    m = mods.BertCosAttention(cfg).to(DEV)
    b, s = 3, 128
    g = torch.Generator().manual_seed(2)
    hidden = torch.randn(b, s, cfg.hidden_size, generator=g)
    keep = torch.arange(s)[None, :] < torch.tensor([128, 90, 17])[:, None]
    gout = torch.randn(b, s, cfg.hidden_size, generator=g)
    names = ("query", "key", "value")
    w = [getattr(m, n).weight.detach().double().cpu().requires_grad_(True) for n in names]
    bias = [getattr(m, n).bias.detach().double().cpu().requires_grad_(True) for n in names]
    nc = m.norm_const.detach().double().cpu().reshape(-1).requires_grad_(True)
    h64 = hidden.double().requires_grad_(True)
    ref = tf.bert_attention_block(h64, w[0], bias[0], w[1], bias[1], w[2], bias[2], nc, cfg.num_attention_heads, keep)
    ref_grads = torch.autograd.grad(ref, [h64, *w, nc], gout.double())
    hd = hidden.to(DEV).requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
        (out,) = m(hd, attention_mask=additive_mask(keep).to(DEV))
    tol = 3e-2 if autocast else 1e-4
    assert rel_l2(out.float(), ref.detach().numpy()) <= tol
    out.backward(gout.to(DEV).to(out.dtype))
    got = [hd.grad, m.query.weight.grad, m.key.weight.grad, m.value.weight.grad, m.norm_const.grad.reshape(-1)]
    for name, a, r in zip(("hidden", "wq", "wk", "wv", "norm_const"), got, ref_grads):
        assert rel_l2(a.float(), r.numpy()) <= tol, name


@pytest.mark.parametrize("autocast", [False, True], ids=["bf16-input", "autocast-bf16"])
def test_input_projections_with_the_row_split_weight_gradient(mods, autocast):
    """`InputProjections` at a row count where the weight gradient is multiplied in pieces (8192 rows: four pieces),
    with and without biases, against fp64 linear layers on the CPU."""
    from cottention_transformer_amd.autograd import _weight_gradient, project
    say("input projections", autocast)
    torch.manual_seed(5)
    rows, e = 8192, 128
    lins = [torch.nn.Linear(e, 64 * (i + 1), bias=(i != 1)).to(DEV) for i in range(3)]
    x = torch.randn(4, rows // 4, e)
    gs = [torch.randn(4, rows // 4, 64 * (i + 1)) for i in range(3)]
    x64 = x.double().requires_grad_(True)
    ref_par = [[p.detach().double().cpu().requires_grad_(True) for p in lin.parameters()] for lin in lins]
    ref_ys = [torch.nn.functional.linear(x64, *ps) for ps in ref_par]
    ref_grads = torch.autograd.grad(ref_ys, [x64] + [p for ps in ref_par for p in ps], [g.double() for g in gs])
    xd = x.to(DEV)
    if not autocast:
        xd = xd.bfloat16()
        lins = [lin.bfloat16() for lin in lins]
    xd.requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
        ys = project(xd, *lins)
    assert all(y.dtype == torch.bfloat16 for y in ys)
    for y, r in zip(ys, ref_ys):
        assert rel_l2(y.float(), r.detach().numpy()) <= 1e-2
    torch.autograd.backward(ys, [g.to(DEV).bfloat16() for g in gs])
    got = [xd.grad] + [p.grad for lin in lins for p in lin.parameters()]
    assert xd.grad.dtype == xd.dtype and all(p.grad.dtype == p.dtype for lin in lins for p in lin.parameters())
    for a, r in zip(got, ref_grads):
        assert rel_l2(a.float(), r.numpy()) <= 1e-2
    # the pieces are what ran: the same product as one GEMM differs in the last bits only
    gy, x2 = gs[0].reshape(rows, -1).to(DEV).bfloat16(), x.reshape(rows, e).to(DEV).bfloat16()
    pieces = _weight_gradient(gy, x2)
    assert pieces.dtype == torch.float32
    assert rel_l2(pieces, (gy.double().t() @ x2.double()).cpu().numpy()) <= 1e-2


def test_blocks_without_a_mask_reuse_their_constant_side_inputs(mods):
    """No attention mask: the keep mask, the counts and the position ids are constants the blocks make once per
    shape.  Two calls in a row (the second on the cached tensors) and a call at another shape, against the CPU
    statements with an all-true mask."""
    from oracle import torch_forms as tf
    torch.manual_seed(0)
    cfg = gpt_cfg()
    gpt = mods.GPTCosAttention(cfg).to(DEV)
    bcfg = SimpleNamespace(hidden_size=256, num_attention_heads=4, attention_probs_dropout_prob=0.0, is_decoder=False)
    bert = mods.BertCosAttention(bcfg).to(DEV)
    g = torch.Generator().manual_seed(3)
    for b, s in ((2, 96), (2, 96), (3, 40)):
        say("blocks without a mask", b, s)
        hidden = torch.randn(b, s, 256, generator=g)
        keep = torch.ones(b, s, dtype=torch.bool)
        w = [getattr(gpt, n).weight.detach().double().cpu() for n in ("q_proj", "k_proj", "v_proj", "out_proj")]
        ref = tf.gpt_attention_block(hidden.double(), *w, gpt.norm_const.detach().double().cpu().reshape(-1),
                                     cfg.num_attention_heads, cfg.rotary_dim, cfg.max_position_embeddings, keep)
        out = gpt(hidden.to(DEV))[0]
        assert rel_l2(out.float(), ref.numpy()) <= 1e-4
        wb = [getattr(bert, n).weight.detach().double().cpu() for n in ("query", "key", "value")]
        bb = [getattr(bert, n).bias.detach().double().cpu() for n in ("query", "key", "value")]
        ref = tf.bert_attention_block(hidden.double(), wb[0], bb[0], wb[1], bb[1], wb[2], bb[2],
                                      bert.norm_const.detach().double().cpu().reshape(-1), 4, keep)
        (out,) = bert(hidden.to(DEV))
        assert rel_l2(out.float(), ref.numpy()) <= 1e-4


@pytest.mark.parametrize("masked", [False, True], ids=["no-mask", "masked"])
def test_bert_block_with_the_preparation_inside_the_attention_kernel(mods, masked):
    """Enough heads that a head is handled by one workgroup, bf16 autocast: the forward of the block then runs mask,
    normalisation, value scaling and Q (K^T V) as one launch (PreparedNonCausalAttention).  Against the fp64 CPU
    statement of the block, outputs and all gradients."""
    from unittest import mock
    from oracle import torch_forms as tf
    from cottention_transformer_amd import ops
    say("bert block, fused preparation", masked)
    torch.manual_seed(0)
    cfg = SimpleNamespace(hidden_size=768, num_attention_heads=12, attention_probs_dropout_prob=0.0, is_decoder=False)
    m = mods.BertCosAttention(cfg).to(DEV)
    with torch.no_grad():
        m.norm_const.copy_(torch.linspace(-1.0, 1.0, 12).reshape(1, 12, 1, 1))
    b, s = 24, 136
    g = torch.Generator().manual_seed(4)
    hidden = torch.randn(b, s, cfg.hidden_size, generator=g)
    keep = (torch.arange(s)[None, :] < torch.randint(1, s + 1, (b, 1), generator=g)) if masked \
        else torch.ones(b, s, dtype=torch.bool)
    gout = torch.randn(b, s, cfg.hidden_size, generator=g)
    names = ("query", "key", "value")
    w = [getattr(m, n).weight.detach().double().cpu().requires_grad_(True) for n in names]
    bias = [getattr(m, n).bias.detach().double().cpu().requires_grad_(True) for n in names]
    nc = m.norm_const.detach().double().cpu().reshape(-1).requires_grad_(True)
    h64 = hidden.double().requires_grad_(True)
    ref = tf.bert_attention_block(h64, w[0], bias[0], w[1], bias[1], w[2], bias[2], nc, cfg.num_attention_heads, keep)
    ref_grads = torch.autograd.grad(ref, [h64, *w, *bias, nc], gout.double())
    hd = hidden.to(DEV).requires_grad_(True)
    with mock.patch.object(ops, "noncausal_dot_product_prepared", wraps=ops.noncausal_dot_product_prepared) as spy:
        with torch.autocast("cuda", dtype=torch.bfloat16):
            (out,) = m(hd, attention_mask=additive_mask(keep).to(DEV) if masked else None)
        assert spy.call_count == 1, "the fused forward was not taken"
    assert rel_l2(out.float(), ref.detach().numpy()) <= 3e-2
    out.backward(gout.to(DEV).to(out.dtype))
    got = [hd.grad] + [getattr(m, n).weight.grad for n in names] + [getattr(m, n).bias.grad for n in names] \
        + [m.norm_const.grad.reshape(-1)]
    labels = ("hidden", "wq", "wk", "wv", "bq", "bk", "bv", "norm_const")
    for name, a, r in zip(labels, got, ref_grads):
        # (the value bias only reaches the output through masked, scaled rows; its gradient is small against the others)
        assert rel_l2(a.float(), r.numpy()) <= 3e-2, name


def test_module_options_of_the_reference_signatures(mods):
    """The forward options the blocks keep from the reference's signatures: `use_cache` / `output_attentions` of the GPT
    block (GPT_Trainer/GPTCosAttention.py:481-508: rotated keys and values handed back, the attention output repeated
    in place of the weights) and `output_attentions` / `is_decoder` of the BERT block
    (BERT_Trainer/BertCosAttention.py:319-334).  These paths rotate and permute with torch ops; their outputs must
    equal the default path's."""
    torch.manual_seed(1)
    cfg = gpt_cfg()
    m = mods.GPTCosAttention(cfg).to(DEV)
    for p_ in m.parameters():
        p_.requires_grad_(False)
    g = torch.Generator().manual_seed(5)
    b, s = 2, 150
    hidden = torch.randn(b, s, cfg.hidden_size, generator=g).to(DEV)
    keep = torch.rand(b, s, generator=g) > 0.2
    mask = additive_mask(keep).to(DEV)
    base = m(hidden, attention_mask=mask)
    assert len(base) == 2 and base[1] is None
    out_c, present = m(hidden, attention_mask=mask, use_cache=True)
    h, d = cfg.num_attention_heads, cfg.hidden_size // cfg.num_attention_heads
    assert present[0].shape == (b, h, s, d) and present[1].shape == (b, h, s, d)
    assert rel_l2(out_c, base[0].double().cpu().numpy()) <= 1e-5
    # the values come back as projected, the keys rotated (their norms are those of the projections)
    v_proj = m.v_proj(hidden).view(b, s, h, d).permute(0, 2, 1, 3)
    k_proj = m.k_proj(hidden).view(b, s, h, d).permute(0, 2, 1, 3)
    assert rel_l2(present[1], v_proj.double().cpu().numpy()) <= 1e-6
    assert torch.allclose(present[0].norm(dim=-1), k_proj.norm(dim=-1), rtol=1e-4, atol=1e-5)
    assert not torch.allclose(present[0], k_proj)
    out_a = m(hidden, attention_mask=mask, output_attentions=True)
    assert len(out_a) == 3 and out_a[2].shape == (b, h, s, d)
    assert rel_l2(out_a[0], base[0].double().cpu().numpy()) <= 1e-5

    bcfg = SimpleNamespace(hidden_size=256, num_attention_heads=4, attention_probs_dropout_prob=0.0, is_decoder=True)
    bert = mods.BertCosAttention(bcfg).to(DEV)
    for p_ in bert.parameters():
        p_.requires_grad_(False)
    plain = bert(hidden, attention_mask=mask)
    assert len(plain) == 2 and plain[1][0].shape == (b, 4, s, 64) and plain[1][1].shape == (b, 4, s, 64)
    # is_decoder: the tuple handed back is (key_layer, value_layer) as projected and split into heads, BEFORE the mask
    # and the normalisation touch them -- a literal restatement of BERT_Trainer/BertCosAttention.py:143-144,158,332-333
    lit_k = bert.key(hidden).view(b, s, 4, 64).permute(0, 2, 1, 3)
    lit_v = bert.value(hidden).view(b, s, 4, 64).permute(0, 2, 1, 3)
    assert rel_l2(plain[1][0], lit_k.double().cpu().numpy()) <= 1e-6 and rel_l2(plain[1][1], lit_v.double().cpu().numpy()) <= 1e-6
    # output_attentions: the reference's active path never assigns attention_probs (every assignment is commented out,
    # :198-268), so its `(context_layer, attention_probs)` at :330 would raise; here None stands in for the weights
    with_attn = bert(hidden, attention_mask=mask, output_attentions=True)
    assert len(with_attn) == 3 and with_attn[1] is None
    assert torch.equal(with_attn[0], plain[0])
    with pytest.raises(NotImplementedError):
        bert(hidden, encoder_hidden_states=hidden)
