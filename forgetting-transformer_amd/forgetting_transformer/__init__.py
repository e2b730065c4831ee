"""Forgetting Attention for AMD MI355X (gfx950).

Same import path and call signature as the reference package
(``src/forgetting_transformer/__init__.py:1-3``)::

    from forgetting_transformer import forgetting_attention
"""
from .ops.forgetting_attention import (forgetting_attention, forgetting_attention_from_logits,
                                         forgetting_attention_norm_gate, qk_norm_threshold)
from .ops.norm_gate import group_norm, group_norm_gated, rms_norm
from .ops.token_shift import token_shift
from .fgate_cache import FgateDynamicCache

__version__ = "0.1.0"
__all__ = ["forgetting_attention", "forgetting_attention_from_logits", "forgetting_attention_norm_gate", "qk_norm_threshold", "group_norm",
           "group_norm_gated", "rms_norm", "token_shift", "FgateDynamicCache"]
