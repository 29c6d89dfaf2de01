"""`FastAttention2.kernel.{float32,float64,float16,bfloat16}(Q, K, V, block_size, inplace=False,
reversed=False) -> Tensor` -- the bindings of Cuda_Kernel/combined_kernel_general.cu:444-454, with the
host-side behaviour of forward_<T> (:352-429) reproduced in Python over the HIP library."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import _bootstrap  # noqa: E402,F401

import torch  # noqa: E402

from cottention_transformer_amd import ops  # noqa: E402
from cottention_transformer_amd.autograd import _autocast_target  # noqa: E402


def _entry(half_entry):
    def call(Q, K, V, block_size=1, inplace=False, reversed=False):
        # block_size is accepted and ignored, as in the reference (never read in forward_<T>).
        for name, t in (("Q", Q), ("K", K), ("V", V)):
            if not t.is_cuda:
                raise RuntimeError(f"{name} must be a CUDA tensor")                      # :355-357
        if Q.size(3) != K.size(3):
            raise RuntimeError("Q and K must have the same dimension")                   # :365
        d_attn = Q.size(3)
        if d_attn % 16 != 0:
            raise RuntimeError("D_attn must be divisible by 16")                         # :372
        if d_attn < 32:
            raise RuntimeError("D_attn must be greater than or equal to 16*2")           # :374
        if not Q.dtype.is_floating_point or Q.dtype not in (torch.float32, torch.float64, torch.float16,
                                                            torch.bfloat16):
            raise RuntimeError("Unsupported data type")                                  # :387
        dt = _autocast_target(Q, half_entry=half_entry)                                  # :377-389
        if inplace:
            # the reference makes V the output tensor (:403-404); here the kernels write into V's memory where
            # the library allows the alias (ops.causal_dot_product(into_v=True))
            if V.dtype != dt or not V.is_contiguous():
                raise RuntimeError("inplace=True needs a contiguous V of the compute dtype")
            return ops.causal_dot_product(Q.contiguous().to(dt), K.contiguous().to(dt), V, bool(reversed),
                                          into_v=True)
        out = ops.causal_dot_product(Q.contiguous().to(dt), K.contiguous().to(dt), V.contiguous().to(dt),
                                     bool(reversed))                                     # :397-421
        return out
    return call


float32 = _entry(False)
float64 = _entry(False)
float16 = _entry(True)
bfloat16 = _entry(False)
