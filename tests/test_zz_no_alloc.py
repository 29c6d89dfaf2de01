"""The entry point that allocates nothing (cott_causal_fwd_noalloc) against cott_causal_fwd, through the C ABI:
same kernels on the library's built-in scratch instead of a caller workspace, so the outputs are equal bit for bit.
Two calls in a row, the second on a smaller input, so that what the first left in the scratch is seen not to matter."""
import os

import pytest
import torch

from util import inputs, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, F32 = torch.bfloat16, torch.float32


@pytest.fixture(scope="module")
def L():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from cottention_transformer_amd import _loader
    assert os.path.exists(_loader.lib_path()), "libcottention_hip.so must be prebuilt in-tree"
    return _loader.lib()


def both(L, q, k, v, code, rev=0):
    from cottention_transformer_amd import _loader
    b, h, n, dk = q.shape
    dv = v.shape[3]
    st = torch.cuda.current_stream().cuda_stream
    need = L.cott_causal_workspace_bytes(b, h, n, dk, dv, code)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
    want, got = torch.empty_like(v), torch.full_like(v, float("nan"))
    rc = L.cott_causal_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), want.data_ptr(), b, h, n, dk, dv, code, rev,
                           ws.data_ptr() if need else None, need, st)
    assert rc == 0, _loader.last_error()
    rc = L.cott_causal_fwd_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), got.data_ptr(), b, h, n, dk, dv, code, rev, st)
    assert rc == 0, _loader.last_error()
    torch.cuda.synchronize()
    return want, got, need


@pytest.mark.parametrize("dt", [BF, F32], ids=["bf16", "fp32"])
def test_no_alloc_entry_point_equals_workspace_entry_point(L, oracle, dt):
    from cottention_transformer_amd import _loader
    code = _loader.BF16 if dt == BF else _loader.F32
    assert L.cott_noalloc_scratch_bytes() == 48 << 20
    # first long sequences in many groups of 128-wide heads, then a smaller, ragged one: all use the scratch
    # (the first shape, 80 heads in three groups of three pieces each, has the largest slot array of all plans: 45 MiB)
    for (b, h, n, d, rev) in ((5, 16, 16384, 128, 0), (1, 4, 8192, 128, 0), (1, 2, 1023, 64, 0), (1, 2, 1023, 64, 1)):
        print("no-alloc", (b, h, n, d, rev, dt), flush=True)
        q, k, v, _ = inputs(b, h, n, d, d, dt, seed=n + rev)
        want, got, need = both(L, q.to(DEV), k.to(DEV), v.to(DEV), code, rev)
        assert need > 0, "the shape must use group-state slots"
        assert torch.equal(got, want)
        if n < 2000:
            assert rel_l2(got, oracle.causal(q, k, v, bool(rev))) <= (2e-2 if dt == BF else 1e-4)
    # a shape that needs no slots at all takes the same path without touching the scratch
    q, k, v, _ = inputs(8, 32, 256, 64, 64, dt, seed=1)
    want, got, need = both(L, q.to(DEV), k.to(DEV), v.to(DEV), code)
    assert torch.equal(got, want)


def test_no_alloc_entry_point_in_a_hip_graph(L):
    """What the entry point is for: recorded into a HIP graph (no allocation may happen under capture).  The size
    query before the capture resolves the scratch address; every replay, with eager work and a synchronisation
    between replays, equals cott_causal_fwd bit for bit."""
    from cottention_transformer_amd import _loader
    b, h, n, d = 1, 4, 4096, 64
    assert L.cott_causal_workspace_bytes(b, h, n, d, d, _loader.BF16) > 0, "the shape must use group-state slots"
    q, k, v, _ = (x.to(DEV) for x in inputs(b, h, n, d, d, BF, seed=7))
    out = torch.full_like(v, float("nan"))
    assert L.cott_noalloc_scratch_bytes() == 48 << 20            # resolves the symbol, outside the capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        rc = L.cott_causal_fwd_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), b, h, n, d, d, _loader.BF16,
                                       0, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, _loader.last_error()
    for rep in range(3):
        new = [x.to(DEV) for x in inputs(b, h, n, d, d, BF, seed=70 + rep)[:3]]
        for dst, src in zip((q, k, v), new):
            dst.copy_(src)
        graph.replay()
        want, _, _ = both(L, *new, _loader.BF16)                 # eager calls (they use the scratch too) and a sync
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {rep}"


def test_no_alloc_entry_point_rejects_like_the_workspace_entry_point(L):
    from cottention_transformer_amd import _loader
    z = torch.zeros(1, 1, 64, 64, dtype=BF, device=DEV)
    p = z.data_ptr()
    assert L.cott_causal_fwd_noalloc(p, p, p, p, 1, 1, 64, 40, 64, _loader.BF16, 0, None) == _loader.ERR_INVALID
    assert b"divisible by 16" in L.cott_last_error()
    assert L.cott_causal_fwd_noalloc(None, p, p, p, 1, 1, 64, 64, 64, _loader.BF16, 0, None) == _loader.ERR_INVALID
    assert L.cott_causal_fwd_noalloc(None, None, None, None, 0, 1, 64, 64, 64, _loader.BF16, 0, None) == 0
