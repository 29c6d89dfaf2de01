"""CPU checks of the module-level pieces: the rotary helpers (against the GPT-J implementation of the installed
`transformers`, which is what the reference imports at GPT_Trainer/GPTCosAttention.py:7, and against hand-written
rotations), and the two CPU statements of the GPT block against each other (cumsum path vs per-token recurrence)."""
import math
from types import SimpleNamespace

import pytest
import torch

from oracle import torch_forms as tf


def test_rotary_helpers_match_gptj_and_hand_rotation():
    from cottention_transformer_amd import modules
    dim, npos = 16, 50
    table = modules.rotary_table(npos, dim)
    assert table.shape == (npos, dim)
    # hand check: row p = [sin(p f_i) | cos(p f_i)], f_i = 10000^(-2i/dim)
    for p in (0, 1, 7, 49):
        for i in range(dim // 2):
            f = 10000.0 ** (-(2 * i) / dim)
            assert abs(float(table[p, i]) - math.sin(p * f)) < 1e-5
            assert abs(float(table[p, dim // 2 + i]) - math.cos(p * f)) < 1e-5
    assert torch.allclose(tf.gptj_sinusoid_table(npos, dim), table, atol=1e-5)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 5, 3, dim, generator=g)
    pos = torch.tensor([[0, 1, 2, 3, 4], [10, 11, 12, 13, 49]])
    sin, cos = torch.split(table[pos], dim // 2, dim=-1)
    got, got_tf = modules.apply_rotary(x, sin, cos), tf.gptj_rotate(x, sin, cos)
    assert torch.allclose(got, got_tf, atol=1e-6)
    # hand rotation of pair i of one row by angle p f_i
    b, s, h = 1, 4, 2
    p = int(pos[b, s])
    for i in range(dim // 2):
        a = p * 10000.0 ** (-(2 * i) / dim)
        x0, x1 = float(x[b, s, h, 2 * i]), float(x[b, s, h, 2 * i + 1])
        assert abs(float(got[b, s, h, 2 * i]) - (x0 * math.cos(a) - x1 * math.sin(a))) < 1e-4
        assert abs(float(got[b, s, h, 2 * i + 1]) - (x1 * math.cos(a) + x0 * math.sin(a))) < 1e-4
    assert torch.allclose(got.norm(dim=-1), x.norm(dim=-1), atol=1e-5)      # rotations keep lengths
    gptj = pytest.importorskip("transformers.models.gptj.modeling_gptj")
    assert torch.allclose(gptj.create_sinusoidal_positions(npos, dim), table, atol=1e-6)
    assert torch.allclose(gptj.apply_rotary_pos_emb(x, sin, cos), got, atol=1e-6)


def _weights(e, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(e, e, generator=g, dtype=torch.float64) / math.sqrt(e) for _ in range(4)]


def test_gpt_block_training_path_equals_recurrent_path():
    # With no padding the running count of kept keys at position s is s+1 = cur_s + s for cur_s = 1, so the
    # training path (cumsum form, GPTCosAttention.py:241,282) and the recurrent path (:223,253-272) must agree.
    b, s, heads, e, rot = 2, 19, 2, 64, 16
    wq, wk, wv, wo = _weights(e, 1)
    g = torch.Generator().manual_seed(2)
    hidden = torch.randn(b, s, e, generator=g, dtype=torch.float64)
    nc = torch.tensor([0.3, -0.7], dtype=torch.float64)
    full = tf.gpt_attention_block(hidden, wq, wk, wv, wo, nc, heads, rot, 64)
    state = torch.zeros(b, heads, e // heads, e // heads, dtype=torch.float64)
    rec, state, cur = tf.gpt_attention_block_recurrent(hidden, wq, wk, wv, wo, nc, heads, rot, 64, state, 1)
    assert cur == 1 + s
    assert torch.allclose(full, rec, rtol=1e-10, atol=1e-12)
    # feeding the sequence in two pieces continues from the state
    st = torch.zeros_like(state)
    a, st, c = tf.gpt_attention_block_recurrent(hidden[:, :11], wq, wk, wv, wo, nc, heads, rot, 64, st, 1)
    bb, st, c = tf.gpt_attention_block_recurrent(hidden[:, 11:], wq, wk, wv, wo, nc, heads, rot, 64, st, c)
    assert torch.allclose(torch.cat([a, bb], 1), full, rtol=1e-10, atol=1e-12) and torch.allclose(st, state)


def test_module_parameter_names_match_the_reference_checkpoints():
    from cottention_transformer_amd import modules
    cfg = SimpleNamespace(max_position_embeddings=32, attn_pdrop=0.0, resid_pdrop=0.0, hidden_size=64,
                          num_attention_heads=2, rotary_dim=16)
    m = modules.GPTCosAttention(cfg)
    # GPT_Trainer/GPTCosAttention.py:67-70,89 (its mask buffers are non-persistent, :43-51)
    assert sorted(m.state_dict()) == ["k_proj.weight", "norm_const", "out_proj.weight", "q_proj.weight", "v_proj.weight"]
    assert m.norm_const.shape == (1, 2, 1, 1) and float(m.norm_const.flatten()[0]) == 0.5
    cfg = SimpleNamespace(hidden_size=64, num_attention_heads=2, attention_probs_dropout_prob=0.0, is_decoder=False)
    m = modules.BertCosAttention(cfg)
    # BERT_Trainer/BertCosAttention.py:73-75,81
    assert sorted(m.state_dict()) == ["key.bias", "key.weight", "norm_const", "query.bias", "query.weight",
                                      "value.bias", "value.weight"]
    with pytest.raises(RuntimeError):                                    # no CPU fallback behind the modules
        m(torch.randn(1, 4, 64))


def test_dropin_module_files_resolve_like_the_reference_imports():
    import importlib
    import os
    import sys
    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cottention_transformer_amd")
    from cottention_transformer_amd import modules
    for sub, name in (("GPT_Trainer", "GPTCosAttention"), ("BERT_Trainer", "BertCosAttention")):
        sys.path.insert(0, os.path.join(root, sub))        # `from GPTCosAttention import GPTCosAttention`
        try:
            mod = importlib.import_module(name)
        finally:
            sys.path.pop(0)
        assert getattr(mod, name) is getattr(modules, name)
        pkg = importlib.import_module(f"cottention_transformer_amd.{sub}.{name}")
        assert getattr(pkg, name) is getattr(modules, name)


@pytest.mark.parametrize("bias", [False, True])
def test_input_projections_equal_separate_linear_layers(bias):
    """`InputProjections` (one operator for the q / k / v projections) against three nn.Linear calls: same outputs,
    same gradients for the input, the weights and the biases."""
    from cottention_transformer_amd.autograd import project
    torch.manual_seed(3)
    lins = [torch.nn.Linear(24, 16 + 8 * i, bias=bias).double() for i in range(3)]
    x = torch.randn(2, 5, 24, dtype=torch.float64, requires_grad=True)
    gs = [torch.randn(2, 5, 16 + 8 * i, dtype=torch.float64) for i in range(3)]
    ys = project(x, *lins)
    torch.autograd.backward(ys, gs)
    got = [x.grad.clone()] + [p.grad.clone() for lin in lins for p in lin.parameters()]
    x.grad = None
    for lin in lins:
        lin.zero_grad()
    ref_ys = [lin(x) for lin in lins]
    torch.autograd.backward(ref_ys, gs)
    ref = [x.grad.clone()] + [p.grad.clone() for lin in lins for p in lin.parameters()]
    for a, b in zip(ys, ref_ys):
        assert torch.allclose(a, b, rtol=1e-12, atol=1e-12)
    assert len(got) == len(ref)
    for a, b in zip(got, ref):
        assert torch.allclose(a, b, rtol=1e-12, atol=1e-12)


def test_projections_call_layers_that_are_not_plain_linears():
    """`project` reads weight and bias of plain nn.Linear layers; a layer with a forward hook, a parametrization or a
    subclass (adapters, quantised linears) is CALLED, as the reference calls its projections
    (GPT_Trainer/GPTCosAttention.py:443-445), so what those add is not skipped."""
    from cottention_transformer_amd.autograd import project, _is_plain_linear
    torch.manual_seed(0)
    x = torch.randn(2, 3, 8, dtype=torch.float64)
    plain = torch.nn.Linear(8, 4).double()
    assert _is_plain_linear(plain)
    hooked = torch.nn.Linear(8, 4).double()
    hooked.register_forward_hook(lambda mod, inp, out: out + 1.0)

    class Scaled(torch.nn.Linear):
        def forward(self, inp):
            return 2.0 * super().forward(inp)

    sub = Scaled(8, 4).double()
    par = torch.nn.Linear(8, 4).double()

    class Double(torch.nn.Module):
        def forward(self, w):
            return 2.0 * w

    torch.nn.utils.parametrize.register_parametrization(par, "weight", Double())
    for lin in (hooked, sub, par):
        assert not _is_plain_linear(lin)
        (got,) = project(x, lin)
        assert torch.allclose(got, lin(x), rtol=1e-12, atol=1e-12)
    a, b2 = project(x, plain, hooked)          # one odd layer sends the whole group through the modules
    assert torch.allclose(a, plain(x)) and torch.allclose(b2, hooked(x))
