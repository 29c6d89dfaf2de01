"""`FastAttention.forward.<dtype>(Q, K, V, block_size, inplace=False) -> Tensor`: the causal forward
of Cuda_Kernel/forward.cu:402-455 (bindings :470-476); one head dim D for Q, K and V."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from FastAttention2 import kernel as _kernel  # noqa: E402


def _entry(fn):
    def call(Q, K, V, block_size=1, inplace=False):
        return fn(Q, K, V, block_size, inplace, False)
    return call


float32, float64 = _entry(_kernel.float32), _entry(_kernel.float64)
float16, bfloat16 = _entry(_kernel.float16), _entry(_kernel.bfloat16)
