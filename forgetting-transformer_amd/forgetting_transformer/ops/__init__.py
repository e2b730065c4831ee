from .forgetting_attention import (forgetting_attention, forgetting_attention_from_logits,
                                         forgetting_attention_norm_gate, qk_norm_threshold)
from .norm_gate import group_norm, group_norm_gated, rms_norm
from .token_shift import token_shift

__all__ = ["forgetting_attention", "forgetting_attention_from_logits", "forgetting_attention_norm_gate", "qk_norm_threshold", "group_norm",
           "group_norm_gated", "rms_norm", "token_shift"]
