"""Drop-in for the reference's GPT_Trainer/GPTCosAttention.py: `from GPTCosAttention import GPTCosAttention`
(GPT_Trainer/Trainer.py:27, fast_infer.py:17, infer.py:14) or `from GPT_Trainer.GPTCosAttention import ...`
(Trainer.py:23) resolves here when this directory, or its parent, is on sys.path."""
import os
import sys

_ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if _ROOT not in sys.path:
    sys.path.insert(0, _ROOT)

from cottention_transformer_amd.autograd import CustomAttention  # noqa: E402,F401
from cottention_transformer_amd.modules import GPTCosAttention, apply_rotary, rotary_table  # noqa: E402,F401

__all__ = ["GPTCosAttention", "CustomAttention"]
