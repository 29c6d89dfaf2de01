"""Attention modules with the reference's constructor, parameter names and forward signatures, running the
cosine-attention core on the HIP path.

    GPTCosAttention   <- GPT_Trainer/GPTCosAttention.py:40-508 (GPT-J attention block: q/k/v projections, rotary
                         embedding, causal cosine attention, output projection; optional recurrent inference)
    BertCosAttention  <- BERT_Trainer/BertCosAttention.py:60-334 (BERT self-attention block, non-causal form)

Parameter / buffer names match (q_proj, k_proj, v_proj, out_proj, norm_const; query, key, value, norm_const), so a
state_dict of the reference modules loads unchanged.  What differs is inside: the normalise / value-scale / mask
steps run as one fused pass (`PrepareInputs`), the attention core is `CustomAttention` / `NonCausalAttention`, and
recurrent inference keeps an fp32 state per batch element that a whole prompt fills in one call (`causal_prefill`)
before single tokens continue from it (`decode_step`).
"""
import torch
from torch import nn

from . import ops
from .autograd import (CustomAttention, CustomAttentionMergedHeads, NonCausalAttention,
                       NonCausalAttentionMergedHeads, PreparedCausalAttention, PreparedNonCausalAttention, PrepareInputs,
                       _autocast_target, project)


def _autocast_on():
    try:
        return torch.is_autocast_enabled("cuda")
    except TypeError:  # older signature
        return torch.is_autocast_enabled()


def _common_dtype(q, k, v):
    """Under autocast the projections are bf16 but the rotary table is fp32, so q and k arrive as fp32 and v as
    bf16; the reference's normalize / divide promote everything to fp32 as well (GPTCosAttention.py:229-241)."""
    dt = torch.promote_types(torch.promote_types(q.dtype, k.dtype), v.dtype)
    return q.to(dt), k.to(dt), v.to(dt)


def rotary_table(num_pos, dim):
    """[num_pos, dim] table of the GPT-J rotary embedding: sin of pos * 10000^(-2i/dim) in the first half of the
    columns, cos in the second (what `create_sinusoidal_positions` returns, GPTCosAttention.py:7,73)."""
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.int64).float() / dim))
    angle = torch.arange(num_pos, dtype=torch.int64).float()[:, None] * inv_freq[None, :]
    return torch.cat([torch.sin(angle), torch.cos(angle)], dim=1)


def apply_rotary(x, sin, cos):
    """Rotates consecutive pairs (x[2i], x[2i+1]) by the angle of column i.  x: (B,S,H,R); sin, cos: (B,S,R/2)
    (`apply_rotary_pos_emb` of GPT-J, used at GPTCosAttention.py:462-476)."""
    s, c = sin[:, :, None, :], cos[:, :, None, :]
    even, odd = x[..., 0::2], x[..., 1::2]
    return torch.stack([even * c - odd * s, odd * c + even * s], dim=-1).flatten(-2)


def _keep_from_additive_mask(attention_mask, batch, length, device):
    """The modules receive the additive mask of the surrounding model, (B,1,1,S) with 0 at real tokens; both turn
    it into a boolean keep mask with `attention_mask == 0` (GPTCosAttention.py:232, BertCosAttention.py:163)."""
    if attention_mask is None:
        return torch.ones(batch, length, dtype=torch.bool, device=device)
    return (attention_mask == 0).reshape(batch, length)


class GPTCosAttention(nn.Module):
    def __init__(self, config):
        super().__init__()
        max_positions = config.max_position_embeddings
        self.attn_dropout = nn.Dropout(config.attn_pdrop)
        self.resid_dropout = nn.Dropout(config.resid_pdrop)
        self.embed_dim = config.hidden_size
        self.num_attention_heads = config.num_attention_heads
        self.head_dim = self.embed_dim // self.num_attention_heads
        if self.head_dim * self.num_attention_heads != self.embed_dim:
            raise ValueError(
                f"embed_dim must be divisible by num_attention_heads (got `embed_dim`: {self.embed_dim} and"
                f" `num_attention_heads`: {self.num_attention_heads}).")
        self.k_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=False)
        self.v_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=False)
        self.q_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=False)
        self.out_proj = nn.Linear(self.embed_dim, self.embed_dim, bias=False)
        self.rotary_dim = config.rotary_dim
        self.embed_positions = rotary_table(max_positions, self.rotary_dim or self.embed_dim)
        # learnable exponent of the value scaling, one per head (GPTCosAttention.py:89)
        self.norm_const = nn.Parameter(0.5 * torch.ones(1, self.num_attention_heads, 1, 1))
        # recurrent inference (GPTCosAttention.py:77-87): state is created on first use, per batch element
        self.fast_inference = bool(getattr(config, "fast_inference", False))
        self.state = None   # (B,H,D,D) fp32, sum of k v^T; the reference's past_KV is its transpose in fp64
        self.cur_s = 1

    def reset_state(self):
        self.state = None
        self.cur_s = 1

    def _decode_one(self, query, key, value):
        """One new token in recurrent inference, from the raw projections (B,1,H,D): rotation by position
        cur_s - 1, normalisation, value scaling by cur_s ** sigmoid(norm_const) and the state update / read-out
        (GPTCosAttention.py:229-248, 253-272, 462-476) as one kernel launch.  Returns (B,1,H*D)."""
        b, _, h, d = query.shape
        query, key, value = _common_dtype(query, key, value)
        if self.state is None:
            self.state = torch.zeros(b, h, d, value.shape[-1], device=query.device,
                                     dtype=torch.float64 if query.dtype == torch.float64 else torch.float32)
        cached = getattr(self, "_sig_cache", None)
        if cached is None or cached[0] != self.norm_const._version or cached[1].device != query.device:
            cached = (self.norm_const._version, self.norm_const.detach().sigmoid().reshape(h).float().to(query.device))
            self._sig_cache = cached
        table = self.embed_positions
        if table.device != query.device:
            table = self.embed_positions = table.to(query.device)
        out = ops.decode_step_prepared(self.state, query, key, value, sig=cached[1], cnt=float(self.cur_s),
                                       rotary=(table, self.cur_s - 1))
        self.cur_s += 1
        return out.reshape(b, 1, h * value.shape[-1])

    def _unmasked_side_inputs(self, b, s, device):
        """Keep mask (all true) and running count of kept keys (1, 2, ..., s) of a batch without padding: constants,
        made once per shape instead of with a fill and a cumulative sum in every forward."""
        cached = getattr(self, "_unmasked_cache", None)
        if cached is None or cached[0] != (b, s, device):
            keep = torch.ones(b, s, dtype=torch.bool, device=device)
            cnt = torch.arange(1, s + 1, device=device, dtype=torch.float32)[None, :].expand(b, s).contiguous()
            cached = self._unmasked_cache = ((b, s, device), keep, cnt)
        return cached[1], cached[2]

    def _split_heads(self, tensor):
        return tensor.view(tensor.size()[:-1] + (self.num_attention_heads, self.head_dim))  # (B,S,H,D)

    def _rotate(self, query, key, position_ids):
        table = self.embed_positions
        if table.device != position_ids.device:
            table = table.to(position_ids.device)
            self.embed_positions = table
        sincos = table[position_ids]                                   # (B,S,R)
        sin, cos = torch.split(sincos, sincos.shape[-1] // 2, dim=-1)
        if self.rotary_dim is not None:
            r = self.rotary_dim
            key = torch.cat([apply_rotary(key[..., :r], sin, cos), key[..., r:]], dim=-1)
            query = torch.cat([apply_rotary(query[..., :r], sin, cos), query[..., r:]], dim=-1)
        else:
            key, query = apply_rotary(key, sin, cos), apply_rotary(query, sin, cos)
        return query, key

    def _cos_attn(self, query, key, value, attention_mask=None, head_mask=None, rotary=None, bnhd=False,
                  merge_heads=False, first_position=None):
        """GPTCosAttention.py:161-282.  query, key, value: (B,H,S,D), already rotated -- or, with `bnhd`, (B,S,H,D)
        as the projections produce them, with rotary=(table, position_ids) still to be applied; in that case the
        rotation, the head permute and the preparation steps are one fused pass.
        merge_heads: the caller wants the output as (B,S,H,D) (:500); returned that way, with None in place of
        the second value, when the training path can write it directly, else (B,H,S,D) as usual.
        first_position: an int when the positions are first_position, first_position + 1, ... (the block made them
        itself), else None; the preparation runs inside the attention kernel where that is built, with the consecutive
        positions or with the caller's position_ids as they are."""
        if bnhd:
            b, s, h, _ = query.shape
        else:
            b, h, s, _ = query.shape
        query, key, value = _common_dtype(query, key, value)
        if attention_mask is None:
            keep, cnt_all = self._unmasked_side_inputs(b, s, query.device)
        else:
            keep, cnt_all = _keep_from_additive_mask(attention_mask, b, s, query.device), None
        sig = self.norm_const.sigmoid().reshape(h)
        table, pos = rotary if rotary is not None else (None, None)
        if self.fast_inference:
            # value scaling by absolute position (:236), then the recurrence (:253-272) from the stored state
            cnt = (self.cur_s + torch.arange(s, device=query.device, dtype=torch.float32)).expand(b, s)
            dt = query.dtype
            q, k, v = ops.prepare_inputs(query, key, value, keep, cnt, sig, out_dtype=dt, rotary=rotary, bnhd=bnhd,
                                         check_positions=False)
            if self.state is None:
                self.state = torch.zeros(b, h, q.shape[-1], v.shape[-1], device=q.device,
                                         dtype=torch.float64 if dt == torch.float64 else torch.float32)
            if s == 1:
                out = ops.decode_step(self.state, q[:, :, 0], k[:, :, 0], v[:, :, 0]).unsqueeze(2)
            else:
                out, self.state = ops.causal_prefill(q, k, v, state=self.state)
            self.cur_s += s
            return out, out
        # kept keys at positions <= s (:241)
        cnt = cnt_all if cnt_all is not None else keep.to(torch.float32).cumsum(-1)
        dt = _autocast_target(query)
        if (bnhd and merge_heads and query.dtype == dt and (table is None or first_position is not None or pos is not None)
                and ops.fused_preparation_preferred(dt, b, h, s, query.shape[-1], value.shape[-1],
                                                    0 if table is None else table.shape[-1])
                and ops.merged_heads_supported(dt, s, h, query.shape[-1], value.shape[-1])):
            # one forward launch: rotation, normalisation, value scaling, mask and the attention op
            return PreparedCausalAttention.apply(query, key, value, None if attention_mask is None else keep, cnt, sig,
                                                 table, first_position if first_position is not None else pos, True,
                                                 True), None
        q, k, v = PrepareInputs.apply(query, key, value, keep, cnt, sig, dt, table, pos, bnhd)
        if merge_heads and ops.merged_heads_supported(q.dtype, s, h, q.shape[-1], v.shape[-1]):
            return CustomAttentionMergedHeads.apply(q, k, v), None
        out = CustomAttention.apply(q, k, v)
        return out, out

    def forward(self, hidden_states, layer_past=None, attention_mask=None, position_ids=None, head_mask=None,
                use_cache=False, output_attentions=False):
        query, key, value = (self._split_heads(t)                       # (B,S,H,D)
                             for t in project(hidden_states, self.q_proj, self.k_proj, self.v_proj))
        if (self.fast_inference and hidden_states.shape[1] == 1 and position_ids is None and layer_past is None
                and use_cache is not True and not output_attentions and attention_mask is None
                and self.head_dim in (32, 64, 128, 256) and self.rotary_dim is not None
                and self.rotary_dim % 2 == 0 and self.rotary_dim <= self.head_dim):
            attn_output = self._decode_one(query, key, value)
            if not _autocast_on():
                attn_output = attn_output.to(hidden_states.dtype)
            return (self.resid_dropout(project(attn_output, self.out_proj)[0]), None)
        first_position = None
        if position_ids is None:
            start = self.cur_s - 1 if self.fast_inference else 0
            key_ = (start, hidden_states.shape[0], hidden_states.shape[1], hidden_states.device)
            cached = getattr(self, "_position_cache", None)
            if cached is None or cached[0] != key_:  # the same ids every training step: made once
                ids = torch.arange(start, start + hidden_states.shape[1], device=hidden_states.device)
                cached = self._position_cache = (key_, ids[None, :].expand(hidden_states.shape[0], -1))
            position_ids = cached[1]
            first_position = start
        if layer_past is None and use_cache is not True and self.rotary_dim is not None and self.rotary_dim % 4 == 0:
            # nobody needs the rotated keys themselves: rotation, head permute and preparation in one pass
            table = self.embed_positions
            if table.device != hidden_states.device:
                table = self.embed_positions = table.to(hidden_states.device)
            present = None
            attn_output, attn_weights = self._cos_attn(query, key, value, attention_mask, head_mask,
                                                       rotary=(table, position_ids), bnhd=True,
                                                       merge_heads=not output_attentions, first_position=first_position)
        else:
            query, key = self._rotate(query, key, position_ids)
            key, query, value = key.permute(0, 2, 1, 3), query.permute(0, 2, 1, 3), value.permute(0, 2, 1, 3)
            if layer_past is not None:
                key = torch.cat((layer_past[0], key), dim=-2)
                value = torch.cat((layer_past[1], value), dim=-2)
            present = (key.to(hidden_states.dtype), value) if use_cache is True else None
            attn_output, attn_weights = self._cos_attn(query, key, value, attention_mask, head_mask)
        if not _autocast_on():
            attn_output = attn_output.to(hidden_states.dtype)
        if attn_weights is not None:  # came back (B,H,S,D): merge the heads here (:500)
            attn_output = attn_output.permute(0, 2, 1, 3).contiguous()
        attn_output = attn_output.view(attn_output.size()[:-2] + (self.embed_dim,))
        attn_output = self.resid_dropout(project(attn_output, self.out_proj)[0])
        outputs = (attn_output, present)
        if output_attentions:
            outputs += (attn_weights,)
        return outputs


class BertCosAttention(nn.Module):
    def __init__(self, config, position_embedding_type=None):
        super().__init__()
        if config.hidden_size % config.num_attention_heads != 0 and not hasattr(config, "embedding_size"):
            raise ValueError(f"The hidden size ({config.hidden_size}) is not a multiple of the number of attention "
                             f"heads ({config.num_attention_heads})")
        self.num_attention_heads = config.num_attention_heads
        self.attention_head_size = int(config.hidden_size / config.num_attention_heads)
        self.all_head_size = self.num_attention_heads * self.attention_head_size
        self.query = nn.Linear(config.hidden_size, self.all_head_size)
        self.key = nn.Linear(config.hidden_size, self.all_head_size)
        self.value = nn.Linear(config.hidden_size, self.all_head_size)
        self.norm_const = nn.Parameter(0.5 * torch.ones(1, self.num_attention_heads, 1, 1))
        self.dropout = nn.Dropout(config.attention_probs_dropout_prob)
        self.position_embedding_type = position_embedding_type or getattr(config, "position_embedding_type", "absolute")
        if self.position_embedding_type in ("relative_key", "relative_key_query"):
            raise NotImplementedError("relative position embeddings are not implemented for cosine attention")
        self.is_decoder = getattr(config, "is_decoder", False)

    def transpose_for_scores(self, x):
        return x.view(x.size()[:-1] + (self.num_attention_heads, self.attention_head_size)).permute(0, 2, 1, 3)

    def forward(self, hidden_states, attention_mask=None, head_mask=None, encoder_hidden_states=None,
                encoder_attention_mask=None, past_key_value=None, output_attentions=False):
        if encoder_hidden_states is not None or past_key_value is not None:
            raise NotImplementedError("cross-attention and cached keys are not implemented for cosine attention")
        if head_mask is not None:
            raise NotImplementedError
        split = hidden_states.shape[:-1] + (self.num_attention_heads, self.attention_head_size)
        # (B,S,H,D); the head permute of transpose_for_scores happens inside the preparation pass
        query_layer, key_layer, value_layer = (t.view(split) for t in
                                               project(hidden_states, self.query, self.key, self.value))
        b, s, h, _ = query_layer.shape
        # mask, normalise, divide the values by (number of real tokens) ** sigmoid(norm_const)  (:162-178)
        if attention_mask is None:  # no padding: constants, made once per shape
            cached = getattr(self, "_unmasked_cache", None)
            if cached is None or cached[0] != (b, s, query_layer.device):
                cached = self._unmasked_cache = ((b, s, query_layer.device),
                                                 torch.ones(b, s, dtype=torch.bool, device=query_layer.device),
                                                 torch.full((b, s), float(s), device=query_layer.device))
            keep, cnt = cached[1], cached[2]
        else:
            keep = _keep_from_additive_mask(attention_mask, b, s, query_layer.device)
            # (made contiguous here, once, rather than by the forward and again by the backward of the preparation)
            cnt = keep.sum(-1, keepdim=True).to(torch.float32).expand(b, s).contiguous()
        dt = _autocast_target(query_layer)
        d = self.attention_head_size
        if (query_layer.dtype == dt and ops.noncausal_fused_preparation_supported(dt, b, h, s, d, d)
                and ops.merged_heads_supported(dt, s, h, d, d)):
            # one forward launch: normalisation, value scaling, mask and the attention op
            context_layer = PreparedNonCausalAttention.apply(query_layer, key_layer, value_layer, keep, cnt,
                                                             self.norm_const.sigmoid().reshape(h), True, True)
            if not _autocast_on():
                context_layer = context_layer.to(hidden_states.dtype)
            context_layer = context_layer.view(context_layer.size()[:-2] + (self.all_head_size,))
            outputs = (context_layer, None) if output_attentions else (context_layer,)
            if self.is_decoder:
                outputs = outputs + ((key_layer.permute(0, 2, 1, 3), value_layer.permute(0, 2, 1, 3)),)
            return outputs
        q, k, v = PrepareInputs.apply(query_layer, key_layer, value_layer, keep, cnt, self.norm_const.sigmoid().reshape(h),
                                      dt, None, None, True)
        # Q (K^T V)  (:249); (QK^T)V at :222 is the same product
        if ops.merged_heads_supported(q.dtype, s, h, q.shape[-1], v.shape[-1]):
            context_layer = NonCausalAttentionMergedHeads.apply(q, k, v)  # already (B,S,H,D) (:317)
            if not _autocast_on():
                context_layer = context_layer.to(hidden_states.dtype)
        else:
            context_layer = NonCausalAttention.apply(q, k, v)
            if not _autocast_on():
                context_layer = context_layer.to(hidden_states.dtype)
            context_layer = context_layer.permute(0, 2, 1, 3).contiguous()
        context_layer = context_layer.view(context_layer.size()[:-2] + (self.all_head_size,))
        outputs = (context_layer, None) if output_attentions else (context_layer,)
        if self.is_decoder:
            outputs = outputs + ((key_layer.permute(0, 2, 1, 3), value_layer.permute(0, 2, 1, 3)),)
        return outputs
