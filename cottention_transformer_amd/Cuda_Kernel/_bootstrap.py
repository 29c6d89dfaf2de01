"""Makes the `cottention_transformer_amd` package importable when only this directory is on
sys.path (the reference's callers do `sys.path.append("Cuda_Kernel")`, GPT_Trainer/GPTCosAttention.py:17)."""
import os
import sys

_ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if _ROOT not in sys.path:
    sys.path.insert(0, _ROOT)
