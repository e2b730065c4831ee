from .forgetting_attention import forgetting_attention
from .token_shift import token_shift

__all__ = ["forgetting_attention", "token_shift"]
