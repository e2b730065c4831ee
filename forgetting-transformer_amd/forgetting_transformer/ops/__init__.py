from .forgetting_attention import forgetting_attention, forgetting_attention_from_logits
from .token_shift import token_shift

__all__ = ["forgetting_attention", "forgetting_attention_from_logits", "token_shift"]
