"""Module-path alias: the reference exposes the compressed-attention entry point as
nsa.triton_attention.flash_attn_func (nsa/triton_attention.py:549).  Nothing here is Triton."""
from .compressed_attn import flash_attn_func  # noqa: F401
