"""Drop-in for the reference's BERT_Trainer/BertCosAttention.py: `from BertCosAttention import BertCosAttention`
(BERT_Trainer/Trainer.py:26) or `from BERT_Trainer.BertCosAttention import BertCosAttention` (Trainer.py:23,
tests/MemoryTest.py:5) resolves here when this directory, or its parent, is on sys.path."""
import os
import sys

_ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if _ROOT not in sys.path:
    sys.path.insert(0, _ROOT)

from cottention_transformer_amd.modules import BertCosAttention  # noqa: E402,F401

__all__ = ["BertCosAttention"]
