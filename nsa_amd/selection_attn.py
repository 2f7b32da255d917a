"""Selected-block + sliding-window attention with the interface of the reference's
nsa/selection_attn.py::parallel_nsa (:740-814).  When q, k, v or a gate requires grad the two
branches run un-fused through an autograd function (backward: nsa_slc_swa_bwd, the counterpart of
nsa/selection_attn.py:715-737) and the gates are applied with torch ops as in :808-811."""
from __future__ import annotations

from typing import Optional, Union

import torch

from . import ops
from .autograd import GateCombineFn, SlcSwaFn, needs_grad


def _packed(x, B, T):
    return x.reshape(B * T, *x.shape[2:])


def sliding_window_attn(q, k, v, window_size: int, scale: Optional[float] = None,
                        cu_seqlens: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Token t attends the last `window_size` tokens up to and including itself.
    q [B,T,HQ,K], k [B,T,H,K], v [B,T,H,V] (B == 1 with cu_seqlens) -> [B,T,HQ,V]."""
    B, T, HQ, K = q.shape
    if scale is None:
        scale = K ** -0.5
    if cu_seqlens is not None:
        assert B == 1, "batch size must be 1 when cu_seqlens are provided"
        cu = cu_seqlens.to(torch.int32)
    else:
        cu = ops.uniform_cu(B, T, q.device)
    nb = cu.numel() - 1
    if needs_grad(q, k, v):
        _, o = SlcSwaFn.apply(_packed(q, B, T), _packed(k, B, T), _packed(v, B, T), None, None, cu, nb, 64,
                              window_size, float(scale))
        return o.view(B, T, HQ, v.shape[-1])
    with torch.no_grad():
        vt = ops.transpose(_packed(v, B, T), cu, nb)
        o = ops.swa(_packed(q, B, T), _packed(k, B, T), vt, cu, nb, window_size, scale)
    return o.view(B, T, HQ, v.shape[-1])


def parallel_nsa(q: torch.Tensor,
                 k: torch.Tensor,
                 v: torch.Tensor,
                 g_slc: torch.Tensor,
                 g_swa: torch.Tensor,
                 block_indices: torch.LongTensor,
                 block_counts: Optional[Union[torch.LongTensor, int]] = None,
                 block_size: int = 64,
                 window_size: int = 0,
                 scale: Optional[float] = None,
                 cu_seqlens: Optional[torch.LongTensor] = None,
                 head_first: bool = False) -> torch.Tensor:
    """o = g_slc * selected_attention + g_swa * sliding_attention.

    q [B,T,HQ,K], k [B,T,H,K], v [B,T,H,V], g_* [B,T,HQ], block_indices [B,T,H,S] (block numbers
    local to the sequence), block_counts None | int | [B,T,H]; head_first swaps dims 1 and 2.
    With cu_seqlens (B must be 1) the tensors are packed sequences.  GQA groups of 1..16 heads and of 32, 48,
    64, ... heads run (the reference takes multiples of 16 only); the backward of a group beyond 16 heads runs as
    one call per sub-group of 16 heads.
    A count tensor limits the picks of a (token, head) in the forward as well, which the reference's forward
    kernel does too (nsa/selection_attn.py:431-434)."""
    if scale is None:
        scale = k.shape[-1] ** -0.5
    if cu_seqlens is not None:
        assert q.shape[0] == 1, "batch size must be 1 when cu_seqlens are provided"
    if head_first:
        q, k, v, block_indices = (x.transpose(1, 2) for x in (q, k, v, block_indices))
        g_slc, g_swa = (x.transpose(1, 2) for x in (g_slc, g_swa))
        if isinstance(block_counts, torch.Tensor):
            block_counts = block_counts.transpose(1, 2)
    B, T, HQ, K = q.shape
    H, V = k.shape[2], v.shape[-1]
    if HQ % H != 0 or (HQ // H > 16 and (HQ // H) % 16 != 0):
        raise NotImplementedError("GQA group size must divide HQ and be at most 16 or a multiple of 16")
    if isinstance(block_counts, int):
        block_indices = block_indices[:, :, :, :block_counts]
        block_counts = None
    cu = cu_seqlens.to(torch.int32) if cu_seqlens is not None else ops.uniform_cu(B, T, q.device)
    nb = cu.numel() - 1
    qp, kp, vp = _packed(q, B, T), _packed(k, B, T), _packed(v, B, T)
    counts = None if block_counts is None else block_counts.reshape(B * T, H)
    idx = block_indices.reshape(B * T, H, -1)
    if needs_grad(q, k, v, g_slc, g_swa):
        o_slc, o_swa = SlcSwaFn.apply(qp, kp, vp, idx, counts, cu, nb, block_size, window_size, float(scale))
        gs = g_slc.reshape(B * T, HQ).to(q.dtype)
        gw = g_swa.reshape(B * T, HQ).to(q.dtype) if o_swa is not None else torch.zeros_like(gs)
        o = GateCombineFn.apply(torch.stack((gs, gw, torch.zeros_like(gs)), -1), o_slc, o_swa, None, 0)
    else:
        with torch.no_grad():
            o = _parallel_nsa_nograd(qp, kp, vp, idx, counts, g_slc, g_swa, cu, nb, block_size, window_size, scale)
    o = o.view(B, T, HQ, V)
    if head_first:
        o = o.transpose(1, 2)
    return o


def _parallel_nsa_nograd(qp, kp, vp, idx, counts, g_slc, g_swa, cu, nb, block_size, window_size, scale):
    total, HQ = qp.shape[0], qp.shape[1]
    H, V = kp.shape[1], vp.shape[-1]
    vt = ops.transpose(vp, cu, nb)
    ws = ops.slc_workspace(qp, H, V, idx.shape[-1], block_size, nb) if window_size > 0 else None
    if ws is not None:
        # fused schedule: per-block partial results, merged in the window kernel's epilogue
        ops.slc_partials(qp, kp, vt, idx, counts, cu, nb, block_size, scale, ws)
        o = ops.swa_merge(qp, kp, vt, ws, idx.shape[-1], g_slc.reshape(total, HQ), g_swa.reshape(total, HQ), None,
                          None, cu, nb, block_size, window_size, scale)
    else:
        o = None
        if window_size > 0:       # the same schedule in token slabs when the one-slab workspace is too large
            o = ops.slc_swa_fused(qp, kp, vt, idx, counts, g_slc.reshape(total, HQ), g_swa.reshape(total, HQ), None,
                                  None, cu, nb, block_size, window_size, scale)
    if ws is None and o is None:
        o_swa = ops.swa(qp, kp, vt, cu, nb, window_size, scale) if window_size > 0 else None
        o = ops.slc_combine(qp, kp, vt, idx, counts, g_slc.reshape(total, HQ),
                            g_swa.reshape(total, HQ) if o_swa is not None else None, None, o_swa, None, cu, nb,
                            block_size, scale)
    return o
