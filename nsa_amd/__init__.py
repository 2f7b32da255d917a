"""MI355X-native Native Sparse Attention, forward and backward (hand-written gfx950 kernels behind a C ABI).

Module layout mirrors the reference package so that `import nsa_amd as nsa` is a drop-in for that
path: nsa.selection_attention, nsa.nsa.NSAAttention, nsa.compression_kv.*,
nsa.triton_attention.flash_attn_func, nsa.selection_attn.parallel_nsa."""
from .selection_attn import parallel_nsa as selection_attention  # noqa: F401
from .selection_attn import parallel_nsa, sliding_window_attn  # noqa: F401
from .compressed_attn import flash_attn_func  # noqa: F401
from .compression_kv import (KVCompressor, KVCompressorVarlen, calc_compressed_len,  # noqa: F401
                             compress_kv)

__all__ = ["selection_attention", "parallel_nsa", "sliding_window_attn", "flash_attn_func", "KVCompressor",
           "KVCompressorVarlen", "calc_compressed_len", "compress_kv", "NSAAttention", "install_as_nsa"]


def __getattr__(name):
    if name == "NSAAttention":
        from .nsa import NSAAttention
        return NSAAttention
    raise AttributeError(name)


def install_as_nsa():
    """Registers this package under the reference's import name `nsa` (and its submodules)."""
    import importlib
    import sys
    me = sys.modules[__name__]
    sys.modules["nsa"] = me
    for sub in ("nsa", "compression_kv", "triton_attention", "selection_attn"):
        sys.modules["nsa." + sub] = importlib.import_module(__name__ + "." + sub)
    return me
