"""The reference's naive compressed-attention interface on top of the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Same names, argument order and return values as the reference's nsa/torch_attention.py
(construct_local_mask :12-48, get_indices :51-61, attention_ref :66-163), so that a test written
against the reference's oracle reads the same here.  Nothing is computed in this file that
oracle/nsa_oracle.py does not already define: these are thin adapters between the reference's batched
[B, T, H, D] layout (compressed keys already repeated to the query heads) and the oracle's
per-sequence functions.  The shipped package never imports this module.

Only what the NSA path uses is built: the block-causal mask (window_size[0] < 0), no padding masks,
no bias, no dropout, no softcap; anything else raises NotImplementedError instead of guessing.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import nsa_oracle as O


def construct_local_mask(seqlen_q, seqlen_k, block_stride, block_size, window_size=(-1, -1),
                         query_padding_mask=None, key_padding_mask=None, device=None, key_leftpad=None):
    """bool [seqlen_q, seqlen_k], True where compressed row c is HIDDEN from query row t:
    c * block_stride + block_size > t (nsa/torch_attention.py:41)."""
    if window_size[0] >= 0 or query_padding_mask is not None or key_padding_mask is not None or key_leftpad is not None:
        raise NotImplementedError("only the block-causal mask of the NSA path is restated")
    rows = torch.arange(seqlen_q, device=device, dtype=torch.long)[:, None]
    first_seeing_row = torch.arange(seqlen_k, device=device, dtype=torch.long) * block_stride + block_size
    return first_seeing_row[None, :] > rows


def get_indices(s, pool_num_kv_head=0, pool_kernel_size=0, pool_stride=0, pool_padding=0, select_block_count=0):
    """s [B, Hq, T, Nc] per-head importance -> int64 [B, T, Hkv, S] (nsa/torch_attention.py:51-61):
    sum over the query heads of each kv head, ceil-mode average pool, top-k."""
    B, Hq, T, Nc = s.shape
    G = Hq // pool_num_kv_head
    imp = s.reshape(B, pool_num_kv_head, G, T, Nc).sum(2).float()              # [B, Hkv, T, Nc]
    pooled = O.pool_scores_direct(imp, pool_kernel_size, pool_stride, pool_padding)
    out = torch.stack([O.select_blocks(pooled[b].transpose(0, 1), select_block_count) for b in range(B)])
    return out                                                                  # [B, T, Hkv, S]


def attention_ref(q, k, v, block_stride, block_size, query_padding_mask=None, key_padding_mask=None,
                  attn_bias=None, dropout_p=0.0, dropout_mask=None, causal=False, window_size=(-1, -1),
                  softcap=0.0, upcast=False, reorder_ops=False, key_leftpad=None, scale: Optional[float] = None,
                  pool_num_kv_head=0, pool_kernel_size=0, pool_stride=0, pool_padding=0, select_block_count=0):
    """q [B, T, Hq, D], k / v [B, Nc, Hq, D] (compressed rows repeated to the query heads, as
    KVCompressor returns them) -> (output [B, T, Hq, Dv] in q's dtype, indices [B, T, Hkv, S]).
    The oracle always accumulates in fp32 (the reference does so only with upcast=True)."""
    if (query_padding_mask is not None or key_padding_mask is not None or attn_bias is not None or dropout_p != 0.0
            or dropout_mask is not None or softcap != 0.0 or key_leftpad is not None or window_size[0] >= 0):
        raise NotImplementedError("only the NSA path of attention_ref is restated")
    B, T, Hq, D = q.shape
    outs, idxs = [], []
    for b in range(B):
        if causal:
            o = O.compressed_attention(q[b], k[b], v[b], block_size, block_stride, scale)
        else:                                    # every compressed row visible: a block that ends before row 0
            o = O.compressed_attention(q[b], k[b], v[b], -k.shape[1] * block_stride, block_stride, scale)
        outs.append(o.to(q.dtype))
        if select_block_count > 0:
            G = Hq // pool_num_kv_head
            pooled = O.importance_scores(q[b], k[b][:, ::G], pool_kernel_size, pool_stride, pool_padding)
            idxs.append(O.select_blocks(pooled, select_block_count))
    return torch.stack(outs), (torch.stack(idxs) if idxs else None)
