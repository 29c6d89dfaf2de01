"""Host-side operators over torch tensors: thin wrappers that validate, allocate outputs and
workspace with torch, and enqueue the HIP kernels on torch's current stream through the C ABI.

Tensor contract is the reference's: (B, H, N, D) for q/k/v/o (Cuda_Kernel/combined_kernel_general.cu
:360-369), state (B, H, Dk, Dv) for decode.  Nothing here computes on the CPU.
"""
import ctypes

import torch

from . import _loader

_DTYPES = {torch.float32: _loader.F32, torch.float64: _loader.F64, torch.float16: _loader.F16,
           torch.bfloat16: _loader.BF16}


def _check(rc, what):
    if rc == _loader.OK:
        return
    msg = _loader.last_error() or f"{what} failed with status {rc}"
    raise RuntimeError(msg)


def _dtype_code(t):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise ValueError("Only float32, float64, float16, and bfloat16 are supported") from None


def _require_gpu(**tensors):
    dev = None
    for name, t in tensors.items():
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be a CUDA tensor")  # wording of combined_kernel_general.cu:355-357
        if dev is None:
            dev = t.device
        elif t.device != dev:
            devs = sorted({str(x.device) for x in tensors.values()})
            raise RuntimeError(f"all tensors must be on the same device, got {devs}")


def _shapes(q, k, v):
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise RuntimeError("Q, K and V must have shape (N, H, S, D)")
    if q.size(3) != k.size(3):
        raise RuntimeError("Q and K must have the same dimension")  # combined_kernel_general.cu:365
    if q.shape[:3] != k.shape[:3] or q.shape[:3] != v.shape[:3]:
        raise RuntimeError(f"Q, K and V must agree in (N, H, S): {tuple(q.shape)} {tuple(k.shape)} {tuple(v.shape)}")
    b, h, n, dk = q.shape
    return b, h, n, dk, v.size(3)


def _workspace(nbytes, device):
    if nbytes == 0:
        return None, 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    return ws, ws.data_ptr()


# The host side of a call costs about as much as the kernels of a small problem run, so the fixed parts are kept
# short: workspace sizes are remembered per shape, the device is only switched when it is not the current one, and
# the stream handle comes from torch's raw accessor.
_CACHE_LIMIT = 4096  # shapes remembered per cache; a caller that sweeps sequence lengths starts over, it does not grow


def _remember(cache, key, value):
    if len(cache) >= _CACHE_LIMIT:
        cache.clear()
    cache[key] = value
    return value


_ws_bytes_cache = {}


def _ws_bytes(query, *key):
    k = (query, key)
    n = _ws_bytes_cache.get(k)
    if n is None:
        n = _remember(_ws_bytes_cache, k, getattr(_loader.lib(), query)(*key))
    return n


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on(device):
    """Context that makes `device` current for the launch (a no-op when it already is)."""
    return _NO_SWITCH if torch.cuda.current_device() == device.index else torch.cuda.device(device)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device=None):
    if _raw_stream is not None and device is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _overlaps(a, b):
    """Whether the storage ranges spanned by two tensors intersect."""
    if a.numel() == 0 or b.numel() == 0 or a.untyped_storage().data_ptr() != b.untyped_storage().data_ptr():
        return False
    span = lambda t: (t.data_ptr(), t.data_ptr() + (sum((s - 1) * st for s, st in zip(t.shape, t.stride())) + 1) * t.element_size())
    (a0, a1), (b0, b1) = span(a), span(b)
    return a0 < b1 and b0 < a1


def merged_heads_supported(dtype, n, h, dk, dv):
    """Whether the causal ops can write o / read grad_out as (B,N,H,Dv) (see causal_dot_product)."""
    ok = lambda d: 32 <= d <= 128 and d % 16 == 0
    return dtype in (torch.bfloat16, torch.float16) and ok(dk) and ok(dv) and n * h * max(dk, dv) <= 1 << 30


def causal_dot_product(q, k, v, reversed=False, merged_heads=False, into_v=False):
    """o[s,j] = sum_i q[s,i] sum_{s'<=s (>=s if reversed)} k[s',i] v[s',j]; all of one dtype.

    merged_heads: return o as (B,N,H,Dv), the rows of the (B,N,H*Dv) tensor an output projection reads, instead
    of (B,H,N,Dv): the head merge of GPT_Trainer/GPTCosAttention.py:500 without its copy (bf16 / fp16 only, see
    merged_heads_supported).
    into_v: the result overwrites v and v is returned (inplace=True of Cuda_Kernel/combined_kernel_general.cu
    :403-404).  Where the library allows it (cott_causal_fwd_may_alias_v: the MFMA kernels) the kernels write
    straight into v's memory; otherwise the result is computed beside it and copied.  v must be contiguous."""
    _require_gpu(Q=q, K=k, V=v)
    b, h, n, dk, dv = _shapes(q, k, v)
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError("Q, K and V must have the same dtype")
    code = _dtype_code(q)
    if into_v:
        if merged_heads or not v.is_contiguous():
            raise RuntimeError("into_v needs a contiguous (B,H,N,Dv) v")
        if _overlaps(q, v) or _overlaps(k, v):
            raise RuntimeError("into_v: Q and K must not share memory with V")
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    L = _loader.lib()
    if into_v and not L.cott_causal_fwd_may_alias_v(b, h, n, dk, dv, code):
        v.copy_(causal_dot_product(q, k, v, reversed))
        return v
    if merged_heads:
        if reversed:
            raise RuntimeError("merged_heads is only available for the forward direction")
        o = torch.empty((b, n, h, dv), dtype=q.dtype, device=q.device)
        with _on(q.device):
            ws, ws_ptr = _workspace(_ws_bytes("cott_causal_workspace_bytes", b, h, n, dk, dv, code), q.device)
            rc = L.cott_causal_fwd_bnhd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), b, h, n, dk, dv, code,
                                        ws_ptr, ws.numel() if ws is not None else 0, _stream(q.device))
        _check(rc, "cott_causal_fwd_bnhd")
        return o
    o = v if into_v else torch.empty((b, h, n, dv), dtype=q.dtype, device=q.device)
    with _on(q.device):
        ws, ws_ptr = _workspace(_ws_bytes("cott_causal_workspace_bytes", b, h, n, dk, dv, code), q.device)
        rc = L.cott_causal_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), b, h, n, dk, dv, code,
                               int(bool(reversed)), ws_ptr, ws.numel() if ws is not None else 0, _stream(q.device))
    _check(rc, "cott_causal_fwd")
    return o


_saved_plan_cache = {}


def saved_states_plan(dtype, b, h, n, dk, dv):
    """(chunks_per_cut, ncuts, floats per slot, backward workspace bytes) of the states the forward pass can leave for the backward
    pass of this shape, or None when that backward pass takes none (it only does on sequences long enough, for the
    number of heads, to be cut into groups; bf16 / fp16).  cott_causal_saved_plan, remembered per shape."""
    if dtype not in (torch.bfloat16, torch.float16):
        return None
    key = (dtype, b, h, n, dk, dv)
    plan = _saved_plan_cache.get(key, False)
    if plan is False:
        cpc, cuts, slot, ws = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0), ctypes.c_size_t(0)
        rc = _loader.lib().cott_causal_saved_plan(b, h, n, dk, dv, _DTYPES[dtype], ctypes.byref(cpc),
                                                  ctypes.byref(cuts), ctypes.byref(slot), ctypes.byref(ws))
        _check(rc, "cott_causal_saved_plan")
        plan = _remember(_saved_plan_cache, key, (cpc.value, cuts.value, slot.value, ws.value) if cuts.value > 0 else None)
    return plan


def causal_dot_product_saving(q, k, v, merged_heads=False):
    """(o, saved): causal_dot_product(q, k, v) that also leaves, where saved_states_plan() has cuts for the shape,
    the (B,H,ncuts,slot) fp32 states (in the kernels' tile layout, see include/cottention.h) that causal_backward(..., saved=saved) starts dQ from instead of passing over
    k and v once more (what CustomAttention.forward keeps for backward, Cuda_Kernel/Custom_Kernel.py:16, plus this
    one small tensor).  saved is None where the plan has no cuts.  merged_heads: o as (B,N,H,Dv), see causal_dot_product."""
    _require_gpu(Q=q, K=k, V=v)
    b, h, n, dk, dv = _shapes(q, k, v)
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError("Q, K and V must have the same dtype")
    plan = saved_states_plan(q.dtype, b, h, n, dk, dv)
    if plan is None:
        return causal_dot_product(q, k, v, merged_heads=merged_heads), None
    cpc, cuts, slot, _ = plan
    code = _dtype_code(q)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    o = torch.empty((b, n, h, dv) if merged_heads else (b, h, n, dv), dtype=q.dtype, device=q.device)
    saved = torch.empty((b, h, cuts, slot), dtype=torch.float32, device=q.device)
    L = _loader.lib()
    fn = L.cott_causal_fwd_save_bnhd if merged_heads else L.cott_causal_fwd_save
    with _on(q.device):
        ws, ws_ptr = _workspace(_ws_bytes("cott_causal_workspace_bytes", b, h, n, dk, dv, code), q.device)
        rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), saved.data_ptr(), cpc, cuts,
                b, h, n, dk, dv, code, ws_ptr, ws.numel() if ws is not None else 0, _stream(q.device))
    _check(rc, "cott_causal_fwd_save")
    return o, saved


_prep_supported_cache = {}


def fused_preparation_supported(dtype, b, h, n, dk, dv, rotary_dim=0):
    """Whether causal_dot_product_prepared has a kernel for the shape: bf16 / fp16, head dims 32..128 in steps of 16
    (128-wide q / k rows with value tiles of at least 64 columns), a rotary width that is a multiple of 8
    (cott_causal_fwd_prep_supported)."""
    if dtype not in (torch.bfloat16, torch.float16):
        return False
    key = (dtype, b, h, n, dk, dv, rotary_dim)
    ok = _prep_supported_cache.get(key)
    if ok is None:
        ok = _remember(_prep_supported_cache, key, bool(
            _loader.lib().cott_causal_fwd_prep_supported(b, h, n, dk, dv, _DTYPES[dtype], rotary_dim)))
    return ok


def fused_preparation_preferred(dtype, b, h, n, dk, dv, rotary_dim=0):
    """Whether the one launch of causal_dot_product_prepared is also the faster form for the shape (all but those planned
    as column halves in sequence groups: cott_causal_fwd_prep_preferred); the modules take prepare_inputs +
    causal_dot_product elsewhere."""
    if dtype not in (torch.bfloat16, torch.float16):
        return False
    key = ("preferred", dtype, b, h, n, dk, dv, rotary_dim)
    ok = _prep_supported_cache.get(key)
    if ok is None:
        ok = _remember(_prep_supported_cache, key, bool(
            _loader.lib().cott_causal_fwd_prep_preferred(b, h, n, dk, dv, _DTYPES[dtype], rotary_dim)))
    return ok


def causal_dot_product_prepared(q, k, v, keep=None, cnt=None, sig=None, rotary=None, bnhd=False, merged_heads=False,
                                want_prepared=True, save_states=False):
    """Causal forward on the RAW projections q, k, v: rotation, normalisation, value scaling and masking
    (prepare_inputs) happen inside the attention kernel (GPT_Trainer/GPTCosAttention.py:229-248, 462-476 in front
    of :282 as one launch).  rotary = (table (P,R) fp32, positions): positions is either an int, the table row of
    position s then being that int + s, or the (B,N) integer position_ids tensor of the block (:458), any values
    (rows outside the table are clamped to it on the device; nothing is read back).  bnhd: q, k, v are (B,N,H,D);
    merged_heads: o is returned as (B,N,H,Dv).
    Returns (o, (q_hat, k_hat, v_hat)) with the prepared tensors (B,H,N,D) that the backward pass needs, or
    (o, None) when want_prepared is false.  Raises where fused_preparation_supported() is false.
    save_states: returns (o, prepared, saved) with the states causal_backward(q_hat, k_hat, v_hat, ..., saved=saved)
    takes (None where saved_states_plan() has none for the shape)."""
    _require_gpu(Q=q, K=k, V=v)
    b, h, n, dk, dv = _prep_shapes(q, k, v, bnhd)
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError("Q, K and V must have the same dtype")
    code = _dtype_code(q)
    keep, cnt, sig = _prep_side_inputs(b, h, n, keep, cnt, sig, q.device)
    table, pos0, rdim, rows, pos_ids = None, 0, 0, 0, None
    if rotary is not None:
        table, pos0 = rotary
        if table.dim() != 2 or table.size(1) % 8 != 0 or table.size(1) > dk:
            raise RuntimeError("rotary table must be (positions, rotary_dim), rotary_dim a multiple of 8 and <= Dk")
        table = table.to(device=q.device, dtype=torch.float32).contiguous()
        rows, rdim = table.shape
        if torch.is_tensor(pos0):
            if pos0.dim() == 1:
                pos0 = pos0[None, :]
            if pos0.shape[-1] != n or pos0.shape[0] not in (1, b) or pos0.dim() != 2:
                raise RuntimeError(f"position ids must be (B,N) = {(b, n)}, got {tuple(pos0.shape)}")
            pos_ids = pos0.to(device=q.device, dtype=torch.int64).expand(b, n).contiguous()
            pos0 = 0
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    o = torch.empty((b, n, h, dv) if merged_heads else (b, h, n, dv), dtype=q.dtype, device=q.device)
    prepared = None
    if want_prepared:
        prepared = (torch.empty((b, h, n, dk), dtype=q.dtype, device=q.device),
                    torch.empty((b, h, n, dk), dtype=q.dtype, device=q.device),
                    torch.empty((b, h, n, dv), dtype=q.dtype, device=q.device))
    L = _loader.lib()
    plan = saved_states_plan(q.dtype, b, h, n, dk, dv) if save_states else None
    saved = None
    with _on(q.device):
        head = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                *((t.data_ptr() for t in prepared) if prepared else (None, None, None)),
                _ptr(keep), _ptr(cnt), _ptr(sig), _ptr(table), _ptr(pos_ids), int(pos0), rdim, rows, int(bool(bnhd)),
                int(bool(merged_heads)))
        ws, ws_ptr = _workspace(_ws_bytes("cott_causal_workspace_bytes", b, h, n, dk, dv, code), q.device)
        tail = (b, h, n, dk, dv, code, ws_ptr, ws.numel() if ws is not None else 0, _stream(q.device))
        if plan is not None:
            cpc, cuts, slot, _ = plan
            saved = torch.empty((b, h, cuts, slot), dtype=torch.float32, device=q.device)
            rc = L.cott_causal_fwd_prep_save(*head, saved.data_ptr(), cpc, cuts, *tail)
        else:
            rc = L.cott_causal_fwd_prep(*head, *tail)
    _check(rc, "cott_causal_fwd_prep")
    return (o, prepared, saved) if save_states else (o, prepared)


def noncausal_fused_preparation_supported(dtype, b, h, n, dk, dv):
    """Whether noncausal_dot_product_prepared has a kernel for the shape: bf16 / fp16, head dims 32..128 in steps of
    16, enough heads that a head is handled by one workgroup (cott_noncausal_fwd_prep_supported)."""
    if dtype not in (torch.bfloat16, torch.float16):
        return False
    key = ("nc", dtype, b, h, n, dk, dv)
    ok = _prep_supported_cache.get(key)
    if ok is None:
        ok = _remember(_prep_supported_cache, key, bool(
            _loader.lib().cott_noncausal_fwd_prep_supported(b, h, n, dk, dv, _DTYPES[dtype])))
    return ok


def noncausal_dot_product_prepared(q, k, v, keep=None, cnt=None, sig=None, bnhd=False, merged_heads=False):
    """Non-causal Q (K^T V) on the RAW projections: normalisation, value scaling and masking (prepare_inputs without a
    rotation) happen inside the attention kernel (BERT_Trainer/BertCosAttention.py:162-178 in front of :249 as one
    launch).  bnhd: q, k, v are (B,N,H,D); merged_heads: o is returned as (B,N,H,Dv).  Returns
    (o, (q_hat, k_hat, v_hat)) with the prepared tensors (B,H,N,D) that the backward pass needs.  Raises where
    noncausal_fused_preparation_supported() is false."""
    _require_gpu(Q=q, K=k, V=v)
    b, h, n, dk, dv = _prep_shapes(q, k, v, bnhd)
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError("Q, K and V must have the same dtype")
    code = _dtype_code(q)
    keep, cnt, sig = _prep_side_inputs(b, h, n, keep, cnt, sig, q.device)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    o = torch.empty((b, n, h, dv) if merged_heads else (b, h, n, dv), dtype=q.dtype, device=q.device)
    prepared = (torch.empty((b, h, n, dk), dtype=q.dtype, device=q.device),
                torch.empty((b, h, n, dk), dtype=q.dtype, device=q.device),
                torch.empty((b, h, n, dv), dtype=q.dtype, device=q.device))
    with _on(q.device):
        rc = _loader.lib().cott_noncausal_fwd_prep(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                                   *(t.data_ptr() for t in prepared), _ptr(keep), _ptr(cnt), _ptr(sig),
                                                   int(bool(bnhd)), int(bool(merged_heads)), b, h, n, dk, dv, code,
                                                   _stream(q.device))
    _check(rc, "cott_noncausal_fwd_prep")
    return o, prepared


def causal_prefill(q, k, v, state=None, return_state=True):
    """Causal forward over a whole prompt (or one piece of a sequence) with the recurrence state handed over:
    returns (o, state_out) with o[s] = q[s] (state + sum_{s'<=s} k[s'] v[s']^T) and
    state_out = state + sum_{s'} k[s'] v[s']^T, the tensor `decode_step` continues from.  Replaces the
    per-token loop over the prompt of GPT_Trainer/GPTCosAttention.py:253-272.
    state: None (zero) or (B,H,Dk,Dv) fp32 (fp64 for fp64 inputs); it is not modified."""
    _require_gpu(Q=q, K=k, V=v)
    b, h, n, dk, dv = _shapes(q, k, v)
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError("Q, K and V must have the same dtype")
    code = _dtype_code(q)
    sdt = torch.float64 if q.dtype == torch.float64 else torch.float32
    if state is not None:
        _require_gpu(state=state)
        if state.shape != (b, h, dk, dv) or state.dtype != sdt or not state.is_contiguous():
            raise RuntimeError(f"causal_prefill: state must be a contiguous {sdt} tensor of shape {(b, h, dk, dv)}")
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    o = torch.empty((b, h, n, dv), dtype=q.dtype, device=q.device)
    s_out = torch.empty((b, h, dk, dv), dtype=sdt, device=q.device) if return_state else None
    L = _loader.lib()
    with _on(q.device):
        ws, ws_ptr = _workspace(_ws_bytes("cott_causal_workspace_bytes", b, h, n, dk, dv, code), q.device)
        rc = L.cott_causal_fwd_state(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                     state.data_ptr() if state is not None else None,
                                     s_out.data_ptr() if s_out is not None else None, b, h, n, dk, dv, code, ws_ptr,
                                     ws.numel() if ws is not None else 0, _stream(q.device))
    _check(rc, "cott_causal_fwd_state")
    return o, s_out


def causal_backward(q, k, v, grad_out, merged_heads=False, saved=None):
    """(dQ, dK, dV) of causal_dot_product(q, k, v) for upstream gradient grad_out ((B,N,H,Dv) with merged_heads).
    saved: the states causal_dot_product_saving() (or causal_dot_product_prepared(save_states=True)) returned for
    the same q, k, v."""
    _require_gpu(Q=q, K=k, V=v, prev_grad=grad_out)
    b, h, n, dk, dv = _shapes(q, k, v)
    want = (b, n, h, dv) if merged_heads else tuple(v.shape)
    if tuple(grad_out.shape) != want:
        raise RuntimeError(f"prev_grad must have shape {want}, got {tuple(grad_out.shape)}")
    if not (q.dtype == k.dtype == v.dtype == grad_out.dtype):
        raise RuntimeError("Q, K, V and prev_grad must have the same dtype")
    code = _dtype_code(q)
    q, k, v, g = q.contiguous(), k.contiguous(), v.contiguous(), grad_out.contiguous()
    dq, dk_, dv_ = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    L = _loader.lib()
    if saved is not None:
        plan = saved_states_plan(q.dtype, b, h, n, dk, dv)
        if plan is None:
            raise RuntimeError("causal_backward: this call takes no saved states")
        cpc, cuts, slot, ws_bytes = plan
        _require_gpu(saved=saved)
        if tuple(saved.shape) != (b, h, cuts, slot) or saved.dtype != torch.float32 or not saved.is_contiguous():
            raise RuntimeError(f"causal_backward: saved must be a contiguous fp32 tensor of shape {(b, h, cuts, slot)}")
        with _on(q.device):
            ws, ws_ptr = _workspace(ws_bytes, q.device)
            fn = L.cott_causal_bwd_saved_bnhd if merged_heads else L.cott_causal_bwd_saved
            rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), dq.data_ptr(),
                    dk_.data_ptr(), dv_.data_ptr(), saved.data_ptr(), cpc, cuts, b, h, n, dk, dv, code,
                    ws_ptr, ws.numel() if ws is not None else 0, _stream(q.device))
        _check(rc, "cott_causal_bwd_saved")
        return dq, dk_, dv_
    with _on(q.device):
        ws, ws_ptr = _workspace(_ws_bytes("cott_causal_bwd_workspace_bytes", b, h, n, dk, dv, code), q.device)
        fn = L.cott_causal_bwd_bnhd if merged_heads else L.cott_causal_bwd
        rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), dq.data_ptr(), dk_.data_ptr(), dv_.data_ptr(), b, h,
                n, dk, dv, code, ws_ptr, ws.numel() if ws is not None else 0, _stream(q.device))
    _check(rc, "cott_causal_bwd_bnhd" if merged_heads else "cott_causal_bwd")
    return dq, dk_, dv_


def noncausal_dot_product(q, k, v, merged_heads=False):
    """o = q (k^T v) per (batch, head): BERT_Trainer/BertCosAttention.py:249.  merged_heads: o as (B,N,H,Dv)
    (the context-layer permute of :317 without its copy; see merged_heads_supported)."""
    _require_gpu(Q=q, K=k, V=v)
    b, h, n, dk, dv = _shapes(q, k, v)
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError("Q, K and V must have the same dtype")
    code = _dtype_code(q)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    o = torch.empty((b, n, h, dv) if merged_heads else (b, h, n, dv), dtype=q.dtype, device=q.device)
    L = _loader.lib()
    with _on(q.device):
        ws, ws_ptr = _workspace(_ws_bytes("cott_noncausal_workspace_bytes", b, h, n, dk, dv, code), q.device)
        fn = L.cott_noncausal_fwd_bnhd if merged_heads else L.cott_noncausal_fwd
        rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), b, h, n, dk, dv, code, ws_ptr,
                ws.numel() if ws is not None else 0, _stream(q.device))
    _check(rc, "cott_noncausal_fwd_bnhd" if merged_heads else "cott_noncausal_fwd")
    return o


def noncausal_backward(q, k, v, grad_out, merged_heads=False):
    """(dQ, dK, dV) of noncausal_dot_product (grad_out (B,N,H,Dv) with merged_heads)."""
    _require_gpu(Q=q, K=k, V=v, prev_grad=grad_out)
    b, h, n, dk, dv = _shapes(q, k, v)
    want = (b, n, h, dv) if merged_heads else tuple(v.shape)
    if tuple(grad_out.shape) != want:
        raise RuntimeError(f"prev_grad must have shape {want}, got {tuple(grad_out.shape)}")
    if not (q.dtype == k.dtype == v.dtype == grad_out.dtype):
        raise RuntimeError("Q, K, V and prev_grad must have the same dtype")
    code = _dtype_code(q)
    q, k, v, g = q.contiguous(), k.contiguous(), v.contiguous(), grad_out.contiguous()
    dq, dk_, dv_ = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    L = _loader.lib()
    with _on(q.device):
        ws, ws_ptr = _workspace(_ws_bytes("cott_noncausal_workspace_bytes", b, h, n, dk, dv, code), q.device)
        fn = L.cott_noncausal_bwd_bnhd if merged_heads else L.cott_noncausal_bwd
        rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), dq.data_ptr(), dk_.data_ptr(), dv_.data_ptr(), b, h,
                n, dk, dv, code, ws_ptr, ws.numel() if ws is not None else 0, _stream(q.device))
    _check(rc, "cott_noncausal_bwd_bnhd" if merged_heads else "cott_noncausal_bwd")
    return dq, dk_, dv_


def decode_step(state, q, k, v, out=None):
    """One recurrent step, in place on `state` (B,H,Dk,Dv; fp32, or fp64 for fp64 inputs):
    state += k v^T ; returns o = q state  (GPT_Trainer/GPTCosAttention.py:264,267).
    q,k: (B,H,Dk); v: (B,H,Dv).  The reference's `past_KV` is `state.transpose(-1,-2)`."""
    _require_gpu(state=state, q=q, k=k, v=v)
    if state.dim() != 4 or q.dim() != 3 or k.dim() != 3 or v.dim() != 3:
        raise RuntimeError("decode_step: state (B,H,Dk,Dv), q/k (B,H,Dk), v (B,H,Dv)")
    b, h, dk, dv = state.shape
    if q.shape != (b, h, dk) or k.shape != (b, h, dk) or v.shape != (b, h, dv):
        raise RuntimeError("decode_step: q/k/v do not match the state shape")
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError("q, k and v must have the same dtype")
    code = _dtype_code(q)
    want = torch.float64 if q.dtype == torch.float64 else torch.float32
    if state.dtype != want or not state.is_contiguous():
        raise RuntimeError(f"decode_step: state must be a contiguous {want} tensor (it is updated in place)")
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    if out is None:
        out = torch.empty((b, h, dv), dtype=q.dtype, device=q.device)
    elif out.shape != (b, h, dv) or out.dtype != q.dtype or not out.is_contiguous() or out.device != q.device:
        raise RuntimeError("decode_step: bad `out` tensor")
    L = _loader.lib()
    with _on(q.device):
        rc = L.cott_decode_step(state.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), b, h, dk,
                                dv, code, _stream(q.device))
    _check(rc, "cott_decode_step")
    return out


def decode_step_prepared(state, q, k, v, sig=None, cnt=0.0, rotary=None, out=None):
    """decode_step on the RAW projections of the new token: rotation (rotary = (table (P,R) fp32, position int)),
    L2 normalisation of q and k and v / max(cnt^sig[h], 1) run inside the kernel (one launch instead of
    prepare_inputs + decode_step).  q, k: (B,H,Dk) or the (B,1,H,Dk) projection output; v likewise; sig: (H) or
    None; cnt: number of tokens so far including this one."""
    if q.dim() == 4 and q.shape[1] == 1:
        q, k, v = q[:, 0], k[:, 0], v[:, 0]
    _require_gpu(state=state, q=q, k=k, v=v)
    if state.dim() != 4 or q.dim() != 3 or k.dim() != 3 or v.dim() != 3:
        raise RuntimeError("decode_step_prepared: state (B,H,Dk,Dv), q/k (B,H,Dk), v (B,H,Dv)")
    b, h, dk, dv = state.shape
    if q.shape != (b, h, dk) or k.shape != (b, h, dk) or v.shape != (b, h, dv):
        raise RuntimeError("decode_step_prepared: q/k/v do not match the state shape")
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError("q, k and v must have the same dtype")
    code = _dtype_code(q)
    want = torch.float64 if q.dtype == torch.float64 else torch.float32
    if state.dtype != want or not state.is_contiguous():
        raise RuntimeError(f"decode_step_prepared: state must be a contiguous {want} tensor")
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    if out is None:
        out = torch.empty((b, h, dv), dtype=q.dtype, device=q.device)
    elif out.shape != (b, h, dv) or out.dtype != q.dtype or not out.is_contiguous() or out.device != q.device:
        raise RuntimeError("decode_step_prepared: bad `out` tensor")
    if sig is not None:
        if sig.shape != (h,):
            raise RuntimeError(f"sig must have shape {(h,)}")
        sig = sig.detach().to(device=q.device, dtype=torch.float32).contiguous()
    table, pos, rdim, rows = None, 0, 0, 0
    if rotary is not None:
        table, pos = rotary
        if table.dim() != 2 or table.dtype != torch.float32 or table.device != q.device or not table.is_contiguous():
            raise RuntimeError("rotary table must be a contiguous float32 (positions, rotary_dim) tensor on the inputs' device")
        rows, rdim = table.shape
        pos = int(pos)
    L = _loader.lib()
    with _on(q.device):
        rc = L.cott_decode_step_prep(state.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                     sig.data_ptr() if sig is not None else None, float(cnt),
                                     table.data_ptr() if table is not None else None, pos, rdim, rows, b, h, dk, dv, code,
                                     _stream(q.device))
    _check(rc, "cott_decode_step_prep")
    return out


def _prep_side_inputs(b, h, n, keep, cnt, sig, device):
    if keep is not None:
        if keep.shape != (b, n):
            raise RuntimeError(f"keep must have shape {(b, n)}, got {tuple(keep.shape)}")
        if keep.dtype == torch.bool and keep.device == device and keep.is_contiguous():
            keep = keep.view(torch.uint8)  # a bool tensor already holds one 0 / 1 byte per element: no copy
        else:
            keep = keep.to(device=device, dtype=torch.uint8).contiguous()
    if (cnt is None) != (sig is None):
        raise RuntimeError("cnt and sig are given together (or neither)")
    if cnt is not None:
        if cnt.shape != (b, n) or sig.shape != (h,):
            raise RuntimeError(f"cnt must have shape {(b, n)} and sig {(h,)}")
        cnt = cnt.to(device=device, dtype=torch.float32).contiguous()
        sig = sig.detach().to(device=device, dtype=torch.float32).contiguous()
    return keep, cnt, sig


def _ptr(t):
    return t.data_ptr() if t is not None else None


def _prep_shapes(q, k, v, bnhd):
    """(b, h, n, dk, dv) of q, k, v given as (B,H,N,D), or as (B,N,H,D) when `bnhd`."""
    if bnhd:
        if q.dim() != 4 or k.dim() != 4 or v.dim() != 4 or q.shape != k.shape or q.shape[:3] != v.shape[:3]:
            raise RuntimeError("Q, K and V must have shape (N, S, H, D) and agree in (N, S, H)")
        b, n, h, dk = q.shape
        return b, h, n, dk, v.size(3)
    return _shapes(q, k, v)


def _rotary_args(rotary, b, n, dk, device, check=True):
    if rotary is None:
        return None, None, 0, 0
    table, pos = rotary
    if table.dim() != 2 or table.size(1) % 4 != 0 or table.size(1) > dk:
        raise RuntimeError("rotary table must be (positions, rotary_dim), rotary_dim a multiple of 4 and <= Dk")
    if pos.dim() == 2 and pos.shape == (1, n):  # one row for the whole batch, as GPT-J's model makes them
        pos = pos.expand(b, n)
    if pos.shape != (b, n):
        raise RuntimeError(f"position ids must have shape {(b, n)}")
    # (this check reads the positions back and so waits for the device; callers in a hot loop pass check=False,
    # the kernel then clamps stray positions to the table)
    if check and pos.numel() and (int(pos.max()) >= table.size(0) or int(pos.min()) < 0):
        raise RuntimeError("position id outside the rotary table")
    table = table.to(device=device, dtype=torch.float32).contiguous()
    pos = pos.to(device=device, dtype=torch.int64).contiguous()
    return table, pos, table.size(1), table.size(0)


def prepare_inputs(q, k, v, keep=None, cnt=None, sig=None, out_dtype=None, rotary=None, bnhd=False,
                   check_positions=True):
    """Fused input preparation of the cosine-attention module, one pass per tensor:
        q_out = keep * q / max(|q|, 1e-12),  k_out likewise,  v_out = keep * v / max(cnt ** sig[h], 1)
    converted to `out_dtype` (default: the input dtype) and returned as (B,H,N,D).  Replaces
    GPT_Trainer/GPTCosAttention.py:229-248 and BERT_Trainer/BertCosAttention.py:162-178.
    keep: (B,N) bool/0-1, True = real token; cnt: (B,N) number of kept keys each position attends to;
    sig: (H,) = sigmoid(norm_const).
    rotary=(table, position_ids): also applies the GPT-J rotary embedding to the first table.size(1) columns of
    q and k (GPTCosAttention.py:462-476); bnhd=True: q, k, v are given as (B,N,H,D), the layout the projections
    produce, and the head permute of :478-479 happens in the same pass."""
    _require_gpu(Q=q, K=k, V=v)
    b, h, n, dk, dv = _prep_shapes(q, k, v, bnhd)
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError("Q, K and V must have the same dtype")
    code = _dtype_code(q)
    out_dtype = out_dtype or q.dtype
    if out_dtype not in _DTYPES:
        raise ValueError("Only float32, float64, float16, and bfloat16 are supported")
    keep, cnt, sig = _prep_side_inputs(b, h, n, keep, cnt, sig, q.device)
    table, pos, rdim, rows = _rotary_args(rotary, b, n, dk, q.device, check_positions)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    qo, ko = (torch.empty((b, h, n, dk), dtype=out_dtype, device=q.device) for _ in range(2))
    vo = torch.empty((b, h, n, dv), dtype=out_dtype, device=q.device)
    L = _loader.lib()
    with _on(q.device):
        rc = L.cott_prep_ex_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), qo.data_ptr(), ko.data_ptr(), vo.data_ptr(),
                                _ptr(keep), _ptr(cnt), _ptr(sig), _ptr(table), _ptr(pos), rdim, rows, int(bool(bnhd)),
                                b, h, n, dk, dv, code, _DTYPES[out_dtype], _stream(q.device))
    _check(rc, "cott_prep_ex_fwd")
    return qo, ko, vo


def prepare_inputs_backward(q, k, v, gq, gk, gv, keep=None, cnt=None, sig=None, want_dsig=False, rotary=None,
                            bnhd=False, check_positions=True):
    """Gradients of `prepare_inputs` with respect to q, k, v (their dtype and layout) and, if asked, to sig (H,).
    gq, gk, gv: gradients with respect to the outputs, (B,H,N,D)."""
    _require_gpu(Q=q, K=k, V=v, gq=gq, gk=gk, gv=gv)
    b, h, n, dk, dv = _prep_shapes(q, k, v, bnhd)
    if gq.shape != (b, h, n, dk) or gk.shape != (b, h, n, dk) or gv.shape != (b, h, n, dv):
        raise RuntimeError("gradient shapes must be (B,H,N,D)")
    if not (q.dtype == k.dtype == v.dtype) or not (gq.dtype == gk.dtype == gv.dtype):
        raise RuntimeError("q, k, v share one dtype and their gradients share one dtype")
    code, gcode = _dtype_code(q), _dtype_code(gq)
    keep, cnt, sig = _prep_side_inputs(b, h, n, keep, cnt, sig, q.device)
    table, pos, rdim, rows = _rotary_args(rotary, b, n, dk, q.device, check_positions)
    q, k, v, gq, gk, gv = (t.contiguous() for t in (q, k, v, gq, gk, gv))
    dq, dk_, dv_ = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    drows = torch.empty((b, h, n), dtype=torch.float32, device=q.device) if (want_dsig and sig is not None) else None
    L = _loader.lib()
    with _on(q.device):
        rc = L.cott_prep_ex_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), gq.data_ptr(), gk.data_ptr(), gv.data_ptr(),
                                dq.data_ptr(), dk_.data_ptr(), dv_.data_ptr(), _ptr(drows), _ptr(keep), _ptr(cnt),
                                _ptr(sig), _ptr(table), _ptr(pos), rdim, rows, int(bool(bnhd)), b, h, n, dk, dv, code,
                                gcode, _stream(q.device))
    _check(rc, "cott_prep_ex_bwd")
    dsig = drows.sum(dim=(0, 2)) if drows is not None else None
    return dq, dk_, dv_, dsig
