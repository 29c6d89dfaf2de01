"""Drop-in for the reference's Cuda_Kernel/Custom_Kernel.py: `from Custom_Kernel import CustomAttention`
(GPT_Trainer/GPTCosAttention.py:18, Cuda_Kernel/speed_test.py:2) resolves here when this directory
is on sys.path.  CustomAttention.apply(Q, K, V) -> O with tensors (N, H, S, D)."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import _bootstrap  # noqa: E402,F401

import FastAttention2 as FastAttention  # noqa: E402,F401  (same aliasing as Custom_Kernel.py:2)
from FastAttention2 import kernel  # noqa: E402,F401
from cottention_transformer_amd.autograd import CustomAttention, NonCausalAttention  # noqa: E402,F401

__all__ = ["CustomAttention", "NonCausalAttention", "FastAttention", "kernel"]
