from .forgetting_attention import forgetting_attention

__all__ = ["forgetting_attention"]
