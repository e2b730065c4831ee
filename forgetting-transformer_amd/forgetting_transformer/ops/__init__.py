from .forgetting_attention import forgetting_attention, forgetting_attention_from_logits
from .norm_gate import group_norm_gated
from .token_shift import token_shift

__all__ = ["forgetting_attention", "forgetting_attention_from_logits", "group_norm_gated", "token_shift"]
