"""torch.autograd boundary: `CustomAttention` with the reference's signature, plus the
non-causal counterpart.  Reference: Cuda_Kernel/Custom_Kernel.py:7-141."""
import torch
import torch.nn.utils.parametrize

from . import ops

_SUPPORTED = (torch.float32, torch.float64, torch.float16, torch.bfloat16)


def _autocast_target(q, half_entry=False):
    """Forward-time dtype rule of forward_<T>, Cuda_Kernel/combined_kernel_general.cu:377-389:
    under autocast an fp32 Q is computed in the autocast type (fp16 only for the `float16` entry),
    otherwise in Q's own type; K and V are converted to match."""
    try:
        enabled = torch.is_autocast_enabled("cuda")
    except TypeError:  # older signature
        enabled = torch.is_autocast_enabled()
    if enabled and q.dtype == torch.float32:
        return torch.float16 if half_entry else torch.bfloat16
    return q.dtype


class CustomAttention(torch.autograd.Function):
    """O = causal cosine-attention core of (Q, K, V), tensors (N, H, S, D); apply(Q, K, V) -> O.

    backward_in_forward_dtype (class attribute, default False = the reference's behaviour): under autocast the
    reference computes the forward in bf16 but saves the fp32 tensors (Custom_Kernel.py:16) and runs the backward on
    them in fp32 (:38, :106-108).  Set to True, the tensors are saved as the forward pass rounded them and the
    backward runs in that 16-bit type too (gradients returned in the inputs' types): the gradients of the function
    that was actually evaluated, from the 16-bit kernels (several times faster than the fp32 ones) and from half
    the saved bytes."""

    backward_in_forward_dtype = False

    @staticmethod
    def forward(ctx, Q, K, V):
        if Q.dtype not in _SUPPORTED:
            raise ValueError("Only float32, float64, float16, and bfloat16 are supported")
        Q, K, V = Q.contiguous(), K.contiguous(), V.contiguous()
        dt = _autocast_target(Q, half_entry=(Q.dtype == torch.float16))
        ctx.grad_dtypes = None
        if dt in (torch.float16, torch.bfloat16) and CustomAttention.backward_in_forward_dtype:
            ctx.grad_dtypes = (Q.dtype, K.dtype, V.dtype)
            Q, K, V = Q.to(dt), K.to(dt), V.to(dt)
        if dt == Q.dtype == K.dtype == V.dtype and dt in (torch.float16, torch.bfloat16):
            # 16-bit tensors, forward and backward in the same type: on sequences long enough to be cut into groups
            # the forward pass also leaves the states the backward pass starts dQ from (None otherwise)
            out, states = ops.causal_dot_product_saving(Q, K, V)
            ctx.save_for_backward(Q, K, V, *(() if states is None else (states,)))
            return out
        ctx.save_for_backward(Q, K, V)  # saved before any autocast conversion (Custom_Kernel.py:16)
        return ops.causal_dot_product(Q.to(dt), K.to(dt), V.to(dt), False)

    @staticmethod
    def backward(ctx, grad_output):
        Q, K, V, *states = ctx.saved_tensors
        if Q.dtype not in _SUPPORTED:
            raise ValueError("Only float32, float64, float16, and bfloat16 are supported")
        # One fused call in the saved tensors' dtype replaces the three launches of
        # Custom_Kernel.py:106-108 (same operand permutations inside the library).
        g = grad_output.contiguous().to(Q.dtype)
        grads = ops.causal_backward(Q, K.to(Q.dtype), V.to(Q.dtype), g, saved=states[0] if states else None)
        if ctx.grad_dtypes is not None:
            grads = tuple(x.to(t) for x, t in zip(grads, ctx.grad_dtypes))
        return grads


class CustomAttentionMergedHeads(torch.autograd.Function):
    """CustomAttention with the head merge folded in: apply(Q, K, V) -> O of shape (N, S, H, Dv), i.e. the rows
    of the (N, S, H*Dv) input of the output projection (GPT_Trainer/GPTCosAttention.py:106-113, called at :500), and a backward
    that reads the gradient in that layout.  Only where ops.merged_heads_supported() holds for the dtype the
    forward computes in; callers fall back to CustomAttention + permute otherwise."""

    @staticmethod
    def forward(ctx, Q, K, V):
        if Q.dtype not in _SUPPORTED:
            raise ValueError("Only float32, float64, float16, and bfloat16 are supported")
        dt = _autocast_target(Q, half_entry=(Q.dtype == torch.float16))
        Q, K, V = Q.contiguous().to(dt), K.contiguous().to(dt), V.contiguous().to(dt)
        # in the computed (16-bit) type: the backward reads the merged layout too; with the states for its dQ
        out, states = ops.causal_dot_product_saving(Q, K, V, merged_heads=True)
        ctx.save_for_backward(Q, K, V, *(() if states is None else (states,)))
        return out

    @staticmethod
    def backward(ctx, grad_output):
        Q, K, V, *states = ctx.saved_tensors
        return ops.causal_backward(Q, K, V, grad_output.contiguous().to(Q.dtype), merged_heads=True,
                                   saved=states[0] if states else None)


class NonCausalAttention(torch.autograd.Function):
    """O = Q (K^T V): the BERT form (BERT_Trainer/BertCosAttention.py:249) as one fused operator."""

    @staticmethod
    def forward(ctx, Q, K, V):
        if Q.dtype not in _SUPPORTED:
            raise ValueError("Only float32, float64, float16, and bfloat16 are supported")
        Q, K, V = Q.contiguous(), K.contiguous(), V.contiguous()
        ctx.save_for_backward(Q, K, V)
        dt = _autocast_target(Q)
        return ops.noncausal_dot_product(Q.to(dt), K.to(dt), V.to(dt))

    @staticmethod
    def backward(ctx, grad_output):
        Q, K, V = ctx.saved_tensors
        g = grad_output.contiguous().to(Q.dtype)
        return ops.noncausal_backward(Q, K.to(Q.dtype), V.to(Q.dtype), g)


class NonCausalAttentionMergedHeads(torch.autograd.Function):
    """NonCausalAttention returning O as (N, S, H, Dv) and reading its gradient in that layout
    (BERT_Trainer/BertCosAttention.py:317); same conditions as CustomAttentionMergedHeads."""

    @staticmethod
    def forward(ctx, Q, K, V):
        if Q.dtype not in _SUPPORTED:
            raise ValueError("Only float32, float64, float16, and bfloat16 are supported")
        dt = _autocast_target(Q)
        Q, K, V = Q.contiguous().to(dt), K.contiguous().to(dt), V.contiguous().to(dt)
        ctx.save_for_backward(Q, K, V)
        return ops.noncausal_dot_product(Q, K, V, merged_heads=True)

    @staticmethod
    def backward(ctx, grad_output):
        Q, K, V = ctx.saved_tensors
        return ops.noncausal_backward(Q, K, V, grad_output.contiguous().to(Q.dtype), merged_heads=True)


class PrepareInputs(torch.autograd.Function):
    """(q, k, v, keep, cnt, sig, out_dtype[, rot_table, position_ids, bnhd]) -> (q_hat, k_hat, v_scaled), (B,H,N,D):
    the normalise / value-scale / mask steps in front of the attention op (GPT_Trainer/GPTCosAttention.py:229-248),
    optionally with the rotary embedding and the head permute before them (:462-476), as one fused operator with a
    fused backward.  `sig` = sigmoid(norm_const) per head, differentiable; the other side inputs are constants."""

    @staticmethod
    def forward(ctx, q, k, v, keep, cnt, sig, out_dtype, rot_table=None, position_ids=None, bnhd=False):
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        ctx.save_for_backward(q, k, v, keep, cnt, sig, rot_table, position_ids)
        ctx.bnhd = bool(bnhd)
        rotary = (rot_table, position_ids) if rot_table is not None else None
        # positions are not read back here (that would stall the launch queue): the kernel clamps them to the table
        return ops.prepare_inputs(q, k, v, keep, cnt, sig, out_dtype, rotary=rotary, bnhd=bnhd, check_positions=False)

    @staticmethod
    def backward(ctx, gq, gk, gv):
        q, k, v, keep, cnt, sig, rot_table, position_ids = ctx.saved_tensors
        want = sig is not None and ctx.needs_input_grad[5]
        rotary = (rot_table, position_ids) if rot_table is not None else None
        dq, dk, dv, dsig = ops.prepare_inputs_backward(q, k, v, gq.contiguous(), gk.contiguous(), gv.contiguous(), keep,
                                                       cnt, sig, want_dsig=want, rotary=rotary, bnhd=ctx.bnhd,
                                                       check_positions=False)
        if dsig is not None:
            dsig = dsig.to(sig.dtype)
        return dq, dk, dv, None, None, dsig, None, None, None, None


class PreparedCausalAttention(torch.autograd.Function):
    """(q, k, v, keep, cnt, sig, rot_table, first_position, bnhd, merged_heads) -> O: the preparation steps of
    PrepareInputs and the causal attention op as ONE forward launch on the raw projections
    (ops.causal_dot_product_prepared).  The kernel also leaves the prepared q, k, v for the backward pass, which is
    the attention gradient on them followed by the fused backward of the preparation.  first_position: an int (the
    table row of position s is first_position + s) or the block's (B,N) position_ids tensor, any values, which is never
    read back to the host.  Only where ops.fused_preparation_supported() holds."""

    @staticmethod
    def forward(ctx, q, k, v, keep, cnt, sig, rot_table=None, first_position=0, bnhd=False, merged_heads=False):
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        ids = first_position if torch.is_tensor(first_position) else None
        rotary = (rot_table, ids if ids is not None else int(first_position)) if rot_table is not None else None
        out, prepared, states = ops.causal_dot_product_prepared(q, k, v, keep, cnt, sig, rotary=rotary, bnhd=bnhd,
                                                                merged_heads=merged_heads, want_prepared=True,
                                                                save_states=True)
        ctx.save_for_backward(q, k, v, keep, cnt, sig, rot_table, ids, *prepared, *(() if states is None else (states,)))
        ctx.first_position = 0 if ids is not None else int(first_position)
        ctx.bnhd, ctx.merged = bool(bnhd), bool(merged_heads)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        q, k, v, keep, cnt, sig, rot_table, ids, qh, kh, vh, *states = ctx.saved_tensors
        gq, gk, gv = ops.causal_backward(qh, kh, vh, grad_output.contiguous().to(qh.dtype), merged_heads=ctx.merged,
                                         saved=states[0] if states else None)
        rotary = None
        if rot_table is not None:
            b, n = (q.shape[0], q.shape[1]) if ctx.bnhd else (q.shape[0], q.shape[2])
            if ids is not None:
                pos = (ids if ids.dim() == 2 else ids[None, :]).expand(b, n)
            else:
                pos = torch.arange(ctx.first_position, ctx.first_position + n, device=q.device).expand(b, n)
            rotary = (rot_table, pos)
        want = sig is not None and ctx.needs_input_grad[5]
        dq, dk, dv, dsig = ops.prepare_inputs_backward(q, k, v, gq, gk, gv, keep, cnt, sig, want_dsig=want, rotary=rotary,
                                                       bnhd=ctx.bnhd, check_positions=False)
        if dsig is not None:
            dsig = dsig.to(sig.dtype)
        return dq, dk, dv, None, None, dsig, None, None, None, None


class PreparedNonCausalAttention(torch.autograd.Function):
    """(q, k, v, keep, cnt, sig, bnhd, merged_heads) -> O: the preparation steps of PrepareInputs (no rotation) and
    the non-causal op Q (K^T V) as ONE forward launch on the raw projections (ops.noncausal_dot_product_prepared;
    BERT_Trainer/BertCosAttention.py:162-178 in front of :249).  The kernel leaves the prepared q, k, v for the
    backward pass: the attention gradients on them, then the fused backward of the preparation.  Only where
    ops.noncausal_fused_preparation_supported() holds."""

    @staticmethod
    def forward(ctx, q, k, v, keep, cnt, sig, bnhd=False, merged_heads=False):
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        out, prepared = ops.noncausal_dot_product_prepared(q, k, v, keep, cnt, sig, bnhd=bnhd, merged_heads=merged_heads)
        ctx.save_for_backward(q, k, v, keep, cnt, sig, *prepared)
        ctx.bnhd, ctx.merged = bool(bnhd), bool(merged_heads)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        q, k, v, keep, cnt, sig, qh, kh, vh = ctx.saved_tensors
        gq, gk, gv = ops.noncausal_backward(qh, kh, vh, grad_output.contiguous().to(qh.dtype), merged_heads=ctx.merged)
        want = sig is not None and ctx.needs_input_grad[5]
        dq, dk, dv, dsig = ops.prepare_inputs_backward(q, k, v, gq, gk, gv, keep, cnt, sig, want_dsig=want, bnhd=ctx.bnhd,
                                                       check_positions=False)
        if dsig is not None:
            dsig = dsig.to(sig.dtype)
        return dq, dk, dv, None, None, dsig, None, None


def _weight_gradient(gy, x):
    """gy^T x for gy (R, out), x (R, in).  With many rows and a small weight the library's single GEMM fills the
    chip with too few tiles over a long reduction (out = in = 1024, R = 16384, bf16: 109 us); the rows are cut into
    pieces multiplied as one batched GEMM and summed in fp32 instead (8 pieces: 47 us)."""
    r = x.shape[0]
    pieces = 1
    if x.is_cuda and x.dtype in (torch.float16, torch.bfloat16) and gy.shape[1] * x.shape[1] <= 1 << 20:
        while pieces < 16 and r % (2 * pieces) == 0 and r // (2 * pieces) >= 2048:
            pieces *= 2
    if pieces == 1:
        return gy.t() @ x
    parts = torch.bmm(gy.view(pieces, r // pieces, -1).transpose(1, 2), x.view(pieces, r // pieces, -1))
    return parts.sum(0, dtype=torch.float32)


class InputProjections(torch.autograd.Function):
    """(x, w_0, b_0, w_1, b_1, ...) -> (x w_0^T + b_0, x w_1^T + b_1, ...): the q / k / v projections of an attention
    block (GPT_Trainer/GPTCosAttention.py:443-445, BERT_Trainer/BertCosAttention.py:121,143-144 with biases) as one
    operator.  Under autocast x is converted once for all of them, the gradient of x is accumulated by the GEMMs
    themselves and converted back once, and the weight gradients take `_weight_gradient`.  b_i may be None."""

    @staticmethod
    def forward(ctx, x, *wb):
        # the type nn.Linear would compute in: the autocast type for 16- and 32-bit inputs on the GPU, else x's own
        cd = x.dtype
        if x.is_cuda and x.dtype != torch.float64 and torch.is_autocast_enabled("cuda"):
            cd = torch.get_autocast_dtype("cuda")
        x2 = x.reshape(-1, x.shape[-1]).to(cd)
        ws = [w.to(cd) for w in wb[0::2]]
        ctx.save_for_backward(x2, *ws)
        ctx.x_meta = (x.shape, x.dtype)
        ctx.wb_dtypes = [None if t is None else t.dtype for t in wb]
        outs = []
        for w, b in zip(ws, wb[1::2]):
            y = torch.nn.functional.linear(x2, w, None if b is None else b.to(cd))
            outs.append(y.view(x.shape[:-1] + (w.shape[0],)))
        return tuple(outs)

    @staticmethod
    def backward(ctx, *gys):
        x2, *ws = ctx.saved_tensors
        shape, xdt = ctx.x_meta
        gys = [g.reshape(-1, g.shape[-1]).to(x2.dtype) for g in gys]
        gx = None
        if ctx.needs_input_grad[0]:
            gx = gys[0] @ ws[0]
            for g, w in zip(gys[1:], ws[1:]):
                gx.addmm_(g, w)
            gx = gx.view(shape).to(xdt)
        grads = [gx]
        for i, g in enumerate(gys):
            wdt, bdt = ctx.wb_dtypes[2 * i], ctx.wb_dtypes[2 * i + 1]
            grads.append(_weight_gradient(g, x2).to(wdt) if ctx.needs_input_grad[1 + 2 * i] else None)
            grads.append(g.sum(0, dtype=torch.promote_types(g.dtype, torch.float32)).to(bdt)
                         if bdt is not None and ctx.needs_input_grad[2 + 2 * i] else None)
        return tuple(grads)


def _is_plain_linear(lin):
    """Whether calling the layer is nothing but x w^T + b with the parameters it holds: exactly torch.nn.Linear, no
    forward (pre-)hooks and no parametrization.  Adapters, quantised linears and hooked layers must be CALLED."""
    if type(lin) is not torch.nn.Linear:
        return False
    if lin._forward_hooks or lin._forward_pre_hooks or getattr(lin, "_forward_hooks_with_kwargs", None):
        return False
    if getattr(torch.nn.modules.module, "_global_forward_hooks", None) or getattr(
            torch.nn.modules.module, "_global_forward_pre_hooks", None):
        return False
    return not torch.nn.utils.parametrize.is_parametrized(lin)


def project(x, *linears):
    """The outputs of the given nn.Linear layers on x: through `InputProjections` when every layer is a plain
    nn.Linear, else by calling the layers as the reference does (GPT_Trainer/GPTCosAttention.py:443-445), so that hooks,
    parametrizations and subclasses (LoRA adapters, quantised linears) keep their effect."""
    if not all(_is_plain_linear(lin) for lin in linears):
        return tuple(lin(x) for lin in linears)
    args = []
    for lin in linears:
        args += [lin.weight, lin.bias]
    return InputProjections.apply(x, *args)
