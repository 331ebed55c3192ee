"""MI355X-native ring attention: the reference package's public names (``__init__.py:3``)
on top of hand-written gfx950 kernels."""
from .bias import (BiasFn, BlockBias, alibi_bias, alibi_slopes, causal_bias, prefix_lm_bias,
                   segment_bias, sliding_window_bias)
from .ring import (RingAxis, bwd_block, clear_plan_cache, fwd_block, precompute_delta, ring_attention,
                   ring_attention_with_lse, ring_self_attention)

__all__ = [
    "ring_attention", "ring_self_attention", "ring_attention_with_lse", "RingAxis", "fwd_block",
    "bwd_block", "precompute_delta", "clear_plan_cache", "BiasFn", "BlockBias", "causal_bias", "segment_bias",
    "sliding_window_bias", "prefix_lm_bias", "alibi_bias", "alibi_slopes",
]
