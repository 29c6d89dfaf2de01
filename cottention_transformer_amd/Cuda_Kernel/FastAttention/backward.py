"""`FastAttention.backward.<dtype>(Q, K, V, prev_grad, block_size) -> [Q_grad, K_grad, V_grad]`: the
fused three-gradient entry point of Cuda_Kernel/backwardv2_comb.cu:172-224 (bindings :241-247)."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import _bootstrap  # noqa: E402,F401

from cottention_transformer_amd import ops  # noqa: E402


def _entry():
    def call(Q, K, V, prev_grad, block_size=1):
        if block_size > 1:
            raise ValueError("block_size > 1 is not supported")  # std::invalid_argument, backward.cu:400-402
        dt = Q.dtype
        return list(ops.causal_backward(Q, K.to(dt), V.to(dt), prev_grad.to(dt)))
    return call


float32 = float64 = float16 = bfloat16 = _entry()
