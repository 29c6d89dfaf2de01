"""MI355X-native cosine linear attention (causal, non-causal and recurrent-decode forms).

The compute path is libcottention_hip.so (hand-written HIP for gfx950) behind the C ABI of
include/cottention.h; this package is the torch-facing host side.  `Cuda_Kernel/` holds modules
named like the reference's extension (`FastAttention2.kernel`, `FastAttention.forward/backward`,
`Custom_Kernel.CustomAttention`) so its callers import them unchanged.
"""
from .ops import (causal_backward, causal_dot_product, causal_dot_product_prepared, causal_dot_product_saving, causal_prefill, decode_step, decode_step_prepared,  # noqa: F401
                  fused_preparation_supported, fused_preparation_preferred, merged_heads_supported,
                  noncausal_backward, noncausal_dot_product, noncausal_dot_product_prepared,
                  noncausal_fused_preparation_supported, prepare_inputs, prepare_inputs_backward, saved_states_plan)

__all__ = ["causal_dot_product", "causal_dot_product_prepared", "causal_dot_product_saving", "saved_states_plan", "fused_preparation_supported", "fused_preparation_preferred", "PreparedCausalAttention",
           "causal_prefill", "causal_backward", "merged_heads_supported", "noncausal_dot_product",
           "noncausal_backward", "noncausal_dot_product_prepared", "noncausal_fused_preparation_supported",
           "PreparedNonCausalAttention", "decode_step", "decode_step_prepared",
           "prepare_inputs", "prepare_inputs_backward", "CustomAttention", "CustomAttentionMergedHeads", "NonCausalAttention", "NonCausalAttentionMergedHeads",
           "PrepareInputs"]


def __getattr__(name):
    if name in __all__ and name[0].isupper():
        from . import autograd
        return getattr(autograd, name)
    raise AttributeError(name)
