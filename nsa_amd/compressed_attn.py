"""Compressed attention + block selection with the interface of the reference's
nsa/triton_attention.py::flash_attn_func (:419-476, :549).  Semantics are those of the reference's
torch path (nsa/torch_attention.py:66-163): the importance softmax is over all compressed rows of
the raw, unscaled scores.  When q, k or v requires grad the call goes through an autograd function
whose backward (nsa/triton_attention.py:478-546 in the reference) is nsa_cmp_attn_bwd; the block
indices carry no gradient."""
from __future__ import annotations

import math

import torch

from . import ops
from .autograd import CmpAttnFn, needs_grad


def flash_attn_func(q, k, v, block_stride, block_size, causal, sm_scale, pool_num_kv_head=0,
                    pool_kernel_size=0, pool_stride=0, pool_padding=0, select_block_count=0):
    """q [B,T,Hq,D]; k, v = compressed keys/values [B,Nc,H,D] with H = Hq (each kv head repeated
    Hq/pool_num_kv_head times, as KVCompressor(group=...) returns them) or H = pool_num_kv_head.
    Returns (o [B,T,Hq,Dv], indices int64 [B,T,pool_num_kv_head,select_block_count])."""
    B, T, Hq, D = q.shape
    _, Nc, H, Dv = v.shape
    hkv = pool_num_kv_head if pool_num_kv_head else H
    if H != hkv and H != Hq:
        raise ValueError("compressed k/v must carry Hq or pool_num_kv_head heads")
    rep = H // hkv
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    select = select_block_count > 0 and pool_kernel_size > 0
    cu = ops.uniform_cu(B, T, q.device)
    cu_cmp = ops.uniform_cu(B, Nc, q.device)
    if needs_grad(q, k, v):
        # one row set per kv head; the gradient of a head-repeated k / v lands on the head that is read
        ckp = k[:, :, ::rep].reshape(B * Nc, hkv, D)
        cvp = v[:, :, ::rep].reshape(B * Nc, hkv, Dv)
        sel = (pool_kernel_size, pool_stride, pool_padding, select_block_count, Nc, True) if select else None
        o, idx = CmpAttnFn.apply(q.reshape(B * T, Hq, D), ckp, cvp, cu, cu_cmp, B, block_size, block_stride,
                                 float(sm_scale), bool(causal), sel)
        return o.view(B, T, Hq, Dv), (None if idx is None else idx.view(B, T, hkv, select_block_count))
    with torch.no_grad():
        return _flash_attn_nograd(q, k, v, cu, cu_cmp, hkv, rep, block_stride, block_size, causal, sm_scale,
                                  pool_kernel_size, pool_stride, pool_padding, select_block_count, select)


def _flash_attn_nograd(q, k, v, cu, cu_cmp, hkv, rep, block_stride, block_size, causal, sm_scale, pool_kernel_size,
                       pool_stride, pool_padding, select_block_count, select):
    B, T, Hq, D = q.shape
    _, Nc, H, Dv = v.shape
    if (k.stride(-1) != 1 or k.stride(0) != Nc * k.stride(1) or k.data_ptr() % 16 or k.stride(1) % 8
            or k.stride(2) % 8):
        k = k.contiguous()
    vc = v if v.is_contiguous() else v.contiguous()
    cvt = ops.transpose(vc.view(B * Nc, H, Dv), cu_cmp, B, heads=hkv, head_stride=rep * Dv)
    o, idx, _ = ops.cmp_attn_select(
        q.reshape(B * T, Hq, D), k, cvt, cu, cu_cmp, B, hkv, Dv, k.stride(1), rep * k.stride(2), block_size,
        block_stride, pool_kernel_size, pool_stride, pool_padding, select_block_count, Nc, sm_scale,
        causal=bool(causal), select=select)
    o = o.view(B, T, Hq, Dv)
    if idx is not None:
        idx = idx.view(B, T, hkv, select_block_count)
    return o, idx
