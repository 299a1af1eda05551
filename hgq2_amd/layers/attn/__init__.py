from .mha import QMultiHeadAttention

__all__ = ['QMultiHeadAttention']
