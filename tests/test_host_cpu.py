"""CPU-side checks: the oracle reproduces the committed golden fixtures, the C-ABI library loads and
exports every symbol the header declares, and the host layer rejects what the reference rejects.
No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from util import load_golden, rel_l2

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- oracle vs golden fixtures -------------------------------------------------------------------

@pytest.mark.parametrize("name", ["causal_cfg1_1x2x128x64.npz", "causal_odd_1x2x63x32_dv48.npz"])
def test_oracle_reproduces_causal_golden(oracle, name):
    g = load_golden(name)
    assert rel_l2(oracle.causal(g["q"], g["k"], g["v"]), g["o"]) < 1e-14
    assert rel_l2(oracle.causal(g["q"], g["k"], g["v"], True), g["o_rev"]) < 1e-14
    for got, key in zip(oracle.causal_bwd(g["q"], g["k"], g["v"], g["g"]), ("dq", "dk", "dv")):
        assert rel_l2(got, g[key]) < 1e-14
    # the golden outputs are themselves consistent with the O(N^2) form
    assert rel_l2(oracle.causal_masked(g["q"], g["k"], g["v"]), g["o"]) < 1e-12


def test_oracle_reproduces_noncausal_and_decode_golden(oracle):
    g = load_golden("noncausal_2x2x50x32.npz")
    assert rel_l2(oracle.noncausal(g["q"], g["k"], g["v"]), g["o"]) < 1e-14
    for got, key in zip(oracle.noncausal_bwd(g["q"], g["k"], g["v"], g["g"]), ("dq", "dk", "dv")):
        assert rel_l2(got, g[key]) < 1e-14
    d = load_golden("decode_2x2x32x48_4steps.npz")
    state = d["s0"].astype(np.float64).copy()
    for t in range(d["q"].shape[0]):
        assert rel_l2(oracle.decode_step(state, d["q"][t], d["k"][t], d["v"][t]), d["o"][t]) < 1e-14
    assert rel_l2(state, d["s_final"]) < 1e-14


# ---- the C ABI -------------------------------------------------------------------------------------

def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "cottention.h")).read()
    return sorted(set(re.findall(r"COTT_API[^;(]*?\b(cott_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from cottention_transformer_amd import _loader
    names = _declared_symbols()
    assert {"cott_causal_fwd", "cott_causal_bwd", "cott_noncausal_fwd", "cott_noncausal_bwd", "cott_decode_step",
            "cott_last_error", "cott_version"} <= set(names)
    lib = _loader.lib()                     # builds with hipcc if no shared object is present
    raw = ctypes.CDLL(_loader.lib_path())
    for n in names:
        assert hasattr(raw, n), f"{n} declared in include/cottention.h but not exported"
    assert set(names) == set(_loader.SIGNATURES), "ctypes signatures out of step with the header"
    assert lib.cott_version() >= 100


def test_alias_query_follows_the_kernel_family():
    """cott_causal_fwd_may_alias_v: the MFMA kernels (16-bit and fp32, head dims 32..128 in steps of 16) may write o
    over v; fp64 and other head dims (plain-FMA kernels, operands declared __restrict__) may not."""
    from cottention_transformer_amd import _loader
    f = _loader.lib().cott_causal_fwd_may_alias_v
    assert f(8, 16, 2048, 64, 64, _loader.BF16) == 1 and f(1, 16, 65536, 128, 128, _loader.F16) == 1
    assert f(1, 2, 300, 64, 64, _loader.F32) == 1 and f(1, 2, 300, 48, 80, _loader.BF16) == 1
    assert f(1, 2, 300, 64, 64, _loader.F64) == 0
    assert f(1, 2, 300, 64, 20, _loader.F32) == 0 and f(1, 2, 300, 256, 256, _loader.BF16) == 0
    assert f(1, 2, 300, 40, 64, _loader.BF16) == 0  # (a shape cott_causal_fwd refuses)


def test_workspace_queries_are_pure_host_functions():
    from cottention_transformer_amd import _loader
    L = _loader.lib()
    # few heads, long sequence: the sequence is cut into groups, each with an fp32 state slot per problem
    ws = L.cott_causal_workspace_bytes(1, 2, 8192, 64, 64, _loader.BF16)
    assert ws > 0 and ws % (64 * 32 * 4) == 0
    # headline shape: B*H (x2 column halves) already fills the chip -> one group -> no workspace
    assert L.cott_causal_workspace_bytes(8, 16, 2048, 64, 64, _loader.BF16) == 0
    # fp32 has MFMA kernels too and is cut the same way; fp64 takes the plain-FMA path -> none
    assert L.cott_causal_workspace_bytes(1, 2, 8192, 64, 64, _loader.F32) > 0
    # (no column halves in fp32.  33..64 columns run from split bf16 operands, one workgroup per CU: 128 heads in two
    # groups, the one group that is summed cut into two pieces with a slot each; other widths stay on the fp32 matrix
    # pipe, two workgroups per CU: 128 heads of 32 columns in four groups)
    assert L.cott_causal_workspace_bytes(8, 16, 2048, 64, 64, _loader.F32) == 2 * 2 * 128 * 64 * 64 * 4
    assert L.cott_causal_workspace_bytes(8, 16, 2048, 32, 32, _loader.F32) == 4 * 128 * 32 * 32 * 4
    assert L.cott_causal_workspace_bytes(32, 16, 2048, 64, 64, _loader.F32) == 0
    assert L.cott_causal_workspace_bytes(1, 2, 8192, 64, 64, _loader.F64) == 0
    # Few heads, long sequence (groups needed with or without column halves): whole problems in 16 groups of 16
    # chunks, 16 heads x 16 groups x 128 x 128 floats ...
    assert L.cott_causal_workspace_bytes(1, 16, 16384, 128, 128, _loader.BF16) == 16 * 16 * 128 * 128 * 4
    # ... but with only 4 chunks per group that way, two column halves in 8 groups of 8 chunks
    assert L.cott_causal_workspace_bytes(1, 16, 4096, 128, 128, _loader.BF16) == 2 * 16 * 8 * 128 * 64 * 4
    # fp32 non-causal always stages K^T V through the workspace
    assert L.cott_noncausal_workspace_bytes(32, 12, 512, 64, 64, _loader.F32) > 0
    assert L.cott_causal_bwd_workspace_bytes(1, 2, 8192, 64, 64, _loader.BF16) > 0
    # non-causal: many heads -> one fused launch per head, no workspace; few heads -> group slots
    assert L.cott_noncausal_workspace_bytes(32, 12, 512, 64, 64, _loader.BF16) == 0
    assert L.cott_noncausal_workspace_bytes(1, 2, 8192, 64, 64, _loader.BF16) > 0


def test_c_abi_argument_errors_without_a_gpu():
    from cottention_transformer_amd import _loader
    L = _loader.lib()
    # D_attn % 16 and D_attn >= 32: combined_kernel_general.cu:372-374
    assert L.cott_causal_fwd(16, 16, 16, 16, 1, 1, 8, 24, 32, _loader.F32, 0, None, 0, None) == _loader.ERR_INVALID
    assert "divisible by 16" in _loader.last_error()
    assert L.cott_causal_fwd(16, 16, 16, 16, 1, 1, 8, 16, 32, _loader.F32, 0, None, 0, None) == _loader.ERR_INVALID
    assert "16*2" in _loader.last_error()
    assert L.cott_causal_fwd(16, 16, 16, 16, 1, 1, 8, 64, 64, 9, 0, None, 0, None) == _loader.ERR_INVALID
    assert L.cott_causal_fwd(None, 16, 16, 16, 1, 1, 8, 64, 64, _loader.F32, 0, None, 0, None) == _loader.ERR_INVALID
    assert L.cott_causal_fwd(8, 16, 16, 16, 1, 1, 8, 64, 64, _loader.F32, 0, None, 0, None) == _loader.ERR_INVALID
    assert "aligned" in _loader.last_error()
    # missing workspace on the grouped MFMA path
    assert L.cott_causal_fwd(16, 16, 16, 16, 1, 1, 4096, 64, 64, _loader.BF16, 0, None, 0, None) == _loader.ERR_WORKSPACE
    # empty problems are a no-op
    assert L.cott_causal_fwd(None, None, None, None, 0, 4, 128, 64, 64, _loader.BF16, 0, None, 0, None) == _loader.OK
    assert L.cott_decode_step(16, 16, 16, 16, 16, 1, 1, 32, 30, _loader.F32, None) == _loader.ERR_UNSUPPORTED
    # decode on raw projections: one wavefront per head needs Dv in {32,64,128,256} and Dk <= 256
    assert L.cott_decode_step_prep(16, 16, 16, 16, 16, None, 1.0, None, 0, 0, 0, 1, 1, 512, 64, _loader.BF16,
                                   None) == _loader.ERR_UNSUPPORTED
    assert L.cott_decode_step_prep(16, 16, 16, 16, 16, None, 1.0, 16, 0, 3, 8, 1, 1, 64, 64, _loader.BF16,
                                   None) == _loader.ERR_INVALID
    assert "rotary_dim" in _loader.last_error()
    assert L.cott_decode_step_prep(None, None, None, None, None, None, 1.0, None, 0, 0, 0, 0, 4, 64, 64, _loader.BF16,
                                   None) == _loader.OK
    # o / d_o in the projection layout (B,N,H,D): 16-bit MFMA shapes only, 32-bit offsets inside a batch element
    assert L.cott_causal_fwd_bnhd(16, 16, 16, 16, 1, 2, 64, 64, 64, _loader.F32, None, 0, None) == _loader.ERR_UNSUPPORTED
    assert "bf16 / fp16" in _loader.last_error()
    assert L.cott_causal_bwd_bnhd(16, 16, 16, 16, 16, 16, 16, 1, 2, 64, 256, 256, _loader.BF16, None, 0,
                                  None) == _loader.ERR_UNSUPPORTED
    assert "head dims" in _loader.last_error()
    assert L.cott_noncausal_fwd_bnhd(16, 16, 16, 16, 1, 4096, 8192, 64, 64, _loader.BF16, None, 0,
                                     None) == _loader.ERR_UNSUPPORTED
    assert "2^30" in _loader.last_error()
    assert L.cott_causal_fwd_bnhd(None, None, None, None, 0, 4, 128, 64, 64, _loader.BF16, None, 0, None) == _loader.OK
    # preparation inside the forward kernel: 16-bit MFMA shapes, rotary width a multiple of 8, one group per head
    prep = lambda *shape_dtype, rot=None, rdim=0, rows=0: L.cott_causal_fwd_prep(
        16, 16, 16, 16, None, None, None, None, None, None, rot, None, 0, rdim, rows, 0, 0, *shape_dtype, None, 0, None)
    assert prep(8, 16, 256, 64, 64, _loader.F32) == _loader.ERR_UNSUPPORTED
    assert "bf16 / fp16" in _loader.last_error()
    assert prep(8, 16, 256, 256, 64, _loader.BF16) == _loader.ERR_UNSUPPORTED
    assert prep(8, 16, 256, 64, 64, _loader.BF16, rot=16, rdim=12, rows=8) == _loader.ERR_INVALID
    assert "rotary_dim" in _loader.last_error()
    assert prep(1, 2, 4096, 64, 64, _loader.BF16) == _loader.ERR_WORKSPACE         # sequence groups: needs the workspace
    assert "workspace" in _loader.last_error()
    assert prep(0, 16, 256, 64, 64, _loader.BF16) == _loader.OK
    assert prep(8, 16, 256, 128, 32, _loader.BF16) == _loader.ERR_UNSUPPORTED      # 128-wide q / k rows need value tiles of 64+
    assert L.cott_causal_fwd_prep_supported(8, 16, 256, 64, 128, _loader.BF16, 64) == 1
    assert L.cott_causal_fwd_prep_supported(8, 16, 256, 128, 128, _loader.BF16, 64) == 1
    assert L.cott_causal_fwd_prep_supported(1, 16, 65536, 128, 128, _loader.BF16, 64) == 1   # cut into sequence groups
    assert L.cott_causal_fwd_prep_supported(1, 2, 4096, 64, 64, _loader.BF16, 0) == 1
    assert L.cott_causal_fwd_prep_supported(8, 16, 256, 128, 32, _loader.BF16, 0) == 0
    # the form the modules choose: only where the one launch has measured faster
    assert L.cott_causal_fwd_prep_preferred(8, 16, 2048, 64, 64, _loader.BF16, 64) == 1
    assert L.cott_causal_fwd_prep_preferred(8, 16, 256, 128, 128, _loader.BF16, 64) == 1
    assert L.cott_causal_fwd_prep_preferred(1, 16, 65536, 128, 128, _loader.BF16, 64) == 1
    assert L.cott_causal_fwd_prep_preferred(2, 12, 8192, 128, 128, _loader.BF16, 64) == 0      # column halves in groups
    assert L.cott_causal_fwd_prep_preferred(1, 16, 65536, 64, 64, _loader.BF16, 64) == 1       # whole problems in groups
    assert L.cott_causal_fwd_prep_preferred(8, 16, 2048, 64, 64, _loader.F32, 0) == 0
    # ... and inside the non-causal kernel: 16-bit, a head must fit one workgroup
    ncprep = lambda *shape_dtype, cnt=None, sig=None: L.cott_noncausal_fwd_prep(
        16, 16, 16, 16, None, None, None, None, cnt, sig, 1, 1, *shape_dtype, None)
    assert ncprep(32, 12, 512, 64, 64, _loader.F32) == _loader.ERR_UNSUPPORTED
    assert "bf16 / fp16" in _loader.last_error()
    assert ncprep(32, 12, 512, 64, 64, _loader.BF16, cnt=16) == _loader.ERR_INVALID
    assert "cnt and sig" in _loader.last_error()
    assert ncprep(1, 2, 4096, 64, 64, _loader.BF16) == _loader.ERR_UNSUPPORTED
    assert "one workgroup" in _loader.last_error()
    assert ncprep(0, 12, 512, 64, 64, _loader.BF16) == _loader.OK
    assert L.cott_noncausal_fwd_prep_supported(32, 12, 512, 64, 64, _loader.BF16) == 1
    assert L.cott_noncausal_fwd_prep_supported(16, 16, 512, 128, 128, _loader.BF16) == 1
    assert L.cott_noncausal_fwd_prep_supported(32, 12, 512, 64, 64, _loader.F32) == 0
    assert L.cott_noncausal_fwd_prep_supported(1, 2, 4096, 64, 64, _loader.BF16) == 0


def test_no_alloc_entry_point_checks_and_its_scratch_symbol(tmp_path):
    """Argument checks of cott_causal_fwd_noalloc need no GPU; and the built-in scratch array must be a GLOBAL
    symbol of the library's gfx950 code object, or the runtime cannot resolve it (hipGetSymbolAddress)."""
    import shutil
    import subprocess
    from cottention_transformer_amd import _loader
    L = _loader.lib()
    assert L.cott_noalloc_scratch_bytes() == 48 << 20
    assert L.cott_causal_fwd_noalloc(16, 16, 16, 16, 1, 1, 8, 24, 32, _loader.F32, 0, None) == _loader.ERR_INVALID
    assert "divisible by 16" in _loader.last_error()
    assert L.cott_causal_fwd_noalloc(None, 16, 16, 16, 1, 1, 8, 64, 64, _loader.F32, 0, None) == _loader.ERR_INVALID
    assert L.cott_causal_fwd_noalloc(None, None, None, None, 0, 4, 128, 64, 64, _loader.BF16, 0, None) == _loader.OK
    # every plan of the forward pass fits the built-in scratch: at most two group-state workgroups per CU with a
    # 64 KiB slot each, plus the slots of the last group, which no workgroup fills (G / (G - 1) <= 3 / 2 with pieces)
    # (test_launch_plans_over_device_geometries sweeps random shapes)
    for shape in ((1, 16, 65536, 128, 128), (1, 1, 1 << 20, 128, 128), (3, 5, 30000, 64, 128), (5, 16, 16384, 128, 128)):
        for dt in (_loader.BF16, _loader.F32):
            assert L.cott_causal_workspace_bytes(*shape, dt) <= L.cott_noalloc_scratch_bytes()
    objdump, readelf = "/opt/rocm/llvm/bin/llvm-objdump", "/opt/rocm/llvm/bin/llvm-readelf"
    if not (os.path.exists(objdump) and os.path.exists(readelf)):
        pytest.skip("llvm-objdump / llvm-readelf not installed")
    lib = shutil.copy(_loader.lib_path(), tmp_path / "lib.so")
    subprocess.run([objdump, "--offloading", str(lib)], check=True, stdout=subprocess.DEVNULL, cwd=tmp_path)
    rows = []
    for f in os.listdir(tmp_path):
        if "gfx950" in f:
            out = subprocess.run([readelf, "-s", "--wide", str(tmp_path / f)], check=True, capture_output=True, text=True).stdout
            rows += [l for l in out.splitlines() if l.split()[-1:] == ["_ZL7scratch"]]
    assert rows, "scratch array not found in the device code objects"
    assert all("GLOBAL" in l and str(48 << 20) in l for l in rows), rows


def test_saved_states_plan_and_argument_checks():
    """cott_causal_saved_plan answers without a GPU (256 CUs in 8 XCDs assumed); the two entry points that use the
    plan check their arguments before anything is launched."""
    import ctypes
    from cottention_transformer_amd import _loader
    L = _loader.lib()

    def plan(*shape_and_dtype):
        cpc, cuts, slot, ws = ctypes.c_int(-1), ctypes.c_int(-1), ctypes.c_int(-1), ctypes.c_size_t(1)
        rc = L.cott_causal_saved_plan(*shape_and_dtype, ctypes.byref(cpc), ctypes.byref(cuts), ctypes.byref(slot),
                                      ctypes.byref(ws))
        return rc, cpc.value, cuts.value, slot.value, ws.value
    # long-context benchmark configuration: the backward pass runs 5 groups of 205 chunks per head
    rc, cpc, cuts, slot, ws = plan(1, 16, 65536, 128, 128, _loader.BF16)
    assert (rc, cpc, cuts, slot) == (_loader.OK, 205, 5, 128 * 128) and ws > 0
    assert cuts * cpc >= 1024 > (cuts - 1) * cpc
    # headline shape: dQ beside the (dK, dV) pair workgroups starts from the sum over the whole sequence, one slot
    assert plan(8, 16, 2048, 64, 64, _loader.BF16) == (_loader.OK, 32, 1, 64 * 64, 0)
    # ... likewise pairs cut into groups
    assert plan(1, 16, 65536, 64, 64, _loader.BF16)[:4] == (_loader.OK, 128, 8, 64 * 64)
    # three separate problems of one group each (128-wide heads), column halves, fp32: no saved states
    for shape in ((8, 16, 2048, 128, 128, _loader.BF16), (4, 16, 2048, 128, 64, _loader.BF16),
                  (1, 16, 65536, 128, 128, _loader.F32)):
        assert plan(*shape)[:4] == (_loader.OK, 0, 0, 0)
    assert L.cott_causal_saved_plan(1, 16, 65536, 128, 128, _loader.BF16, None, None, None, None) == _loader.ERR_INVALID
    # the saving forward refuses cuts that do not fit the sequence, other dtypes and null pointers
    fwd, bwd = L.cott_causal_fwd_save, L.cott_causal_bwd_saved
    assert fwd(16, 16, 16, 16, 16, 205, 6, 1, 16, 65536, 128, 128, _loader.BF16, None, 0, None) == _loader.ERR_INVALID
    assert "do not fit" in _loader.last_error()
    assert fwd(16, 16, 16, 16, 16, 205, 5, 1, 16, 65536, 128, 128, _loader.F32, None, 0, None) == _loader.ERR_UNSUPPORTED
    assert fwd(16, 16, 16, 16, None, 205, 5, 1, 16, 65536, 128, 128, _loader.BF16, None, 0, None) == _loader.ERR_INVALID
    assert fwd(None, None, None, None, None, 1, 1, 0, 16, 64, 128, 128, _loader.BF16, None, 0, None) == _loader.OK
    # the backward pass refuses shapes without a plan and states cut for another plan
    assert bwd(*[16] * 8, 1, 1, 4, 16, 2048, 128, 64, _loader.BF16, None, 0, None) == _loader.ERR_UNSUPPORTED
    assert "takes no saved states" in _loader.last_error()
    assert bwd(*[16] * 8, 200, 5, 1, 16, 65536, 128, 128, _loader.BF16, None, 0, None) == _loader.ERR_INVALID
    assert "this shape needs 5 of 205" in _loader.last_error()
    assert bwd(*[16] * 7, None, 205, 5, 1, 16, 65536, 128, 128, _loader.BF16, None, 0, None) == _loader.ERR_INVALID


# ---- host layer mirrors the reference's checks ----------------------------------------------------

def test_host_rejects_cpu_tensors_like_the_reference():
    import cottention_transformer_amd as ct
    q = torch.randn(1, 2, 8, 32)
    with pytest.raises(RuntimeError, match="Q must be a CUDA tensor"):   # combined_kernel_general.cu:355
        ct.causal_dot_product(q, q, q)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ct.decode_step(torch.zeros(1, 2, 32, 32), q[:, :, 0], q[:, :, 0], q[:, :, 0])


def test_dropin_module_names_resolve():
    import sys
    sys.path.insert(0, os.path.join(ROOT, "cottention_transformer_amd", "Cuda_Kernel"))
    try:
        import Custom_Kernel
        import FastAttention
        import FastAttention2
        from FastAttention2 import kernel
    finally:
        sys.path.pop(0)
    for name in ("float32", "float64", "float16", "bfloat16"):
        assert callable(getattr(kernel, name))
        assert callable(getattr(FastAttention.forward, name)) and callable(getattr(FastAttention.backward, name))
    for name in ("forward_float32", "forward_float16", "forward_bfloat16", "backward_float32", "backward_float16",
                 "backward_bfloat16"):                                            # Cuda_Kernel/pybind.cpp:10-27
        assert callable(getattr(FastAttention, name))
    assert issubclass(Custom_Kernel.CustomAttention, torch.autograd.Function)
    assert FastAttention2.kernel is kernel
    q = torch.randn(1, 2, 8, 32)
    with pytest.raises(RuntimeError, match="Q must be a CUDA tensor"):
        kernel.float32(q, q, q, 1, False, False)
    with pytest.raises(ValueError):                                               # Custom_Kernel.py:31-32
        Custom_Kernel.CustomAttention.apply(q.to(torch.int32), q, q)


def test_plan_queries_stay_sane_over_random_shapes():
    """The host-side planner behind the workspace, saved-state and fused-preparation queries, over 400 seeded shapes
    (no GPU involved): sizes are multiples of 16 bytes and bounded by what a full chip of 64 KiB state slots per
    problem can need, a saved-state plan's cuts fit the sequence, and the `supported` answers agree with their
    documented preconditions."""
    import ctypes
    import random
    from cottention_transformer_amd import _loader
    L = _loader.lib()
    rnd = random.Random(7)
    for _ in range(400):
        b = rnd.choice([1, 2, 3, 8, 32, 100]); h = rnd.choice([1, 2, 8, 12, 16])
        n = rnd.choice([1, 63, 64, 65, 512, 2048, 4097, 16384, 65536])
        dk = rnd.choice([32, 48, 64, 96, 128]); dv = rnd.choice([32, 64, 80, 128])
        dt = rnd.choice([_loader.BF16, _loader.F16, _loader.F32])
        if n * max(dk, dv) > 1 << 30:
            continue
        nchunks = (n + 63) // 64
        for fn in (L.cott_causal_workspace_bytes, L.cott_causal_bwd_workspace_bytes, L.cott_noncausal_workspace_bytes):
            ws = fn(b, h, n, dk, dv, dt)
            # at most a few hundred workgroups hold a slot of 128 x 128 floats each, per problem (six with halves)
            assert ws % 16 == 0 and 0 <= ws <= 6 * 4096 * 128 * 128 * 4, (fn.__name__, b, h, n, dk, dv, dt, ws)
        cpc, cuts, slot, wsb = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0), ctypes.c_size_t(0)
        rc = L.cott_causal_saved_plan(b, h, n, dk, dv, dt, ctypes.byref(cpc), ctypes.byref(cuts), ctypes.byref(slot),
                                      ctypes.byref(wsb))
        assert rc == _loader.OK
        if cuts.value > 0:
            assert dt != _loader.F32 and nchunks >= 16
            assert cpc.value >= 1 and (cuts.value - 1) * cpc.value <= nchunks - 1
            assert slot.value >= dk * dv and wsb.value % 16 == 0
        sup = L.cott_causal_fwd_prep_supported(b, h, n, dk, dv, dt, 0)
        if sup:  # (any plan, also with sequence groups: the entry point takes the forward pass's workspace)
            assert dt != _loader.F32 and dk <= 128
        sup = L.cott_noncausal_fwd_prep_supported(b, h, n, dk, dv, dt)
        if sup:
            assert dt != _loader.F32 and dk <= 128 and dv <= 128
            assert L.cott_noncausal_workspace_bytes(b, h, n, dk, dv, dt) == 0


@pytest.mark.parametrize("cus,xcds", [(256, 8), (304, 8), (128, 4), (64, 2), (32, 1), (80, 8)])
def test_launch_plans_over_device_geometries(cus, xcds):
    """The launch planner's rules were measured on one part (256 CUs in 8 XCDs) but follow the CU and XCD counts of the
    device.  With those counts given (cott_plan_geometry), over seeded random shapes: every grid is a whole number of
    XCD rounds and stays within a few workgroups per CU unless the heads alone exceed that; groups cover the sequence;
    the cuts cott_causal_saved_plan names are the groups the gradient launch that takes the states is cut into; the
    workspace sizes follow from the plan (one padded state per head, group, piece and op with sums of its own at most);
    and on parts of up to 256 CUs every forward plan fits the built-in array of cott_causal_fwd_noalloc."""
    import ctypes
    import random
    from cottention_transformer_amd import _loader
    L = _loader.lib()
    assert L.cott_plan_geometry(7, 2) == _loader.ERR_INVALID
    assert L.cott_plan_geometry(cus, xcds) == _loader.OK
    try:
        rnd = random.Random(cus * 31 + xcds)
        sets, nsets = (ctypes.c_int * 64)(), ctypes.c_int(0)
        pad = lambda d: 32 if d <= 32 else (64 if d <= 64 else 128)
        seen_groups = seen_pair = seen_comp = 0
        for _ in range(300):
            b = rnd.choice([1, 2, 3, 5, 8, 32, 100]); h = rnd.choice([1, 2, 8, 12, 16])
            n = rnd.choice([1, 63, 64, 65, 512, 2048, 4097, 16384, 65536])
            dk = rnd.choice([32, 48, 64, 96, 128]); dv = rnd.choice([32, 64, 80, 128])
            dt = rnd.choice([_loader.BF16, _loader.F16, _loader.F32])
            bh, nchunks = b * h, (n + 63) // 64
            cpc, cuts, slot, wsb = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0), ctypes.c_size_t(0)
            assert L.cott_causal_saved_plan(b, h, n, dk, dv, dt, ctypes.byref(cpc), ctypes.byref(cuts),
                                            ctypes.byref(slot), ctypes.byref(wsb)) == _loader.OK
            for which, saved in ((0, 0), (1, 0), (1, 1), (2, 0), (3, 0)):
                assert L.cott_plan_describe(which, saved, b, h, n, dk, dv, dt, sets, ctypes.byref(nsets)) == _loader.OK
                assert 1 <= nsets.value <= 3, (which, b, h, n, dk, dv, dt)
                ops_total, slots = 0, 0
                for s in range(nsets.value):
                    cnt, halves, G, cpg, sub, pair, comp, grid = sets[8 * s: 8 * s + 8]
                    case = (cus, xcds, which, saved, b, h, n, dk, dv, dt, s, tuple(sets[8 * s: 8 * s + 8]))
                    ops_total += cnt
                    assert halves in (1, 2) and 1 <= G <= nchunks and 1 <= sub <= 4, case
                    assert (G - 1) * cpg < nchunks <= G * cpg, case           # the groups cover the sequence, none is empty
                    per_unit = 2 if pair else cnt * halves
                    assert grid % (xcds * per_unit) == 0 and grid >= bh * G * per_unit, case
                    assert grid < (bh * G + xcds) * per_unit, case             # less than one XCD round of padding
                    # cutting into groups never pushes a launch past two workgroups per CU (the fp32 matrix-pipe
                    # kernels aim at two per CU); what exceeds that is heads times ops alone
                    if G > 1:
                        assert bh * per_unit * G <= 2 * cus, case
                        seen_groups += 1
                    seen_pair += pair
                    seen_comp += comp
                    slots += cnt * halves * bh * G * sub
                    if which == 1 and saved and cuts.value > 0 and (pair or comp):
                        assert (G, cpg) == (cuts.value, cpc.value), case     # the forward pass cuts where this launch does
                assert ops_total == (3 if which in (1, 3) else 1)
                if which == 2:
                    nc_slots = slots
                    continue
                if which == 3:  # one query serves the non-causal forward and gradients: the larger of the two
                    ws, slots = L.cott_noncausal_workspace_bytes(b, h, n, dk, dv, dt), max(slots, nc_slots)
                elif which == 1:
                    ws = wsb.value if (saved and cuts.value > 0) else L.cott_causal_bwd_workspace_bytes(b, h, n, dk, dv, dt)
                else:
                    ws = L.cott_causal_workspace_bytes(b, h, n, dk, dv, dt)
                # (a column half's slot is half a padded state; ops that take their states from elsewhere have none)
                assert ws % 16 == 0 and ws <= slots * pad(dk) * pad(dv) * 4, (cus, which, saved, b, h, n, dk, dv, dt, ws)
                if which == 0 and cus <= 256:
                    assert ws <= L.cott_noalloc_scratch_bytes(), (cus, b, h, n, dk, dv, dt, ws)
        assert seen_groups > 50 and seen_pair > 5 and seen_comp > 5
    finally:
        assert L.cott_plan_geometry(0, 0) == _loader.OK
