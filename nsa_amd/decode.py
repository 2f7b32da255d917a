"""Single-token NSA decode on a KV cache laid out for the gfx950 kernels.

The reference has no cache and no decode path.  One step is defined as the last row of the prefill
forward over the cached tokens (mean-pool compressor): block importance over every cached compressed
row, top-n blocks, selected + sliding-window + compressed attention, gated sum."""
from __future__ import annotations

import math
from typing import Optional

import torch

from . import _lib
from .ops import _dtype_code, _ptr, _stream


def _round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


class NSADecodeCache:
    """Per-sequence caches: keys row-major, values key-contiguous, plus their block-compressed
    versions (mean over `block` tokens every `stride`)."""

    def __init__(self, batch, ctx_capacity, hkv, dk, dv, block=32, stride=16, dtype=torch.bfloat16, device="cuda"):
        self.batch, self.hkv, self.dk, self.dv = batch, hkv, dk, dv
        self.block, self.stride = block, stride
        self.ctx_cap = _round_up(ctx_capacity, 64)
        nc = (self.ctx_cap - block) // stride + 1 if self.ctx_cap >= block else 1
        self.nc_cap = _round_up(nc, 64)
        z = dict(dtype=dtype, device=device)
        self.k = torch.zeros(batch, self.ctx_cap, hkv, dk, **z)
        self.vt = torch.zeros(batch, hkv, dv, self.ctx_cap, **z)
        self.ck = torch.zeros(batch, self.nc_cap, hkv, dk, **z)
        self.cvt = torch.zeros(batch, hkv, dv, self.nc_cap, **z)
        self.ctx_lens = torch.zeros(batch, dtype=torch.int32, device=device)

    @torch.no_grad()
    def fill(self, k: torch.Tensor, v: torch.Tensor):
        """Loads a prefilled context: k [B,T,Hkv,Dk], v [B,T,Hkv,Dv] (same T for every sequence)."""
        from . import ops
        B, T = k.shape[:2]
        self.k[:, :T] = k
        self.vt[:, :, :, :T] = v.permute(0, 2, 3, 1)
        nc = (T - self.block) // self.stride + 1 if T >= self.block else 0
        if nc > 0:
            cu = ops.uniform_cu(B, T, k.device)
            cu_out = ops.uniform_cu(B, nc, k.device)
            ck = ops.compress(k.reshape(B * T, self.hkv, self.dk), cu, cu_out, B * nc, self.block, self.stride)
            cv = ops.compress(v.reshape(B * T, self.hkv, self.dv), cu, cu_out, B * nc, self.block, self.stride)
            self.ck[:, :nc] = ck.view(B, nc, self.hkv, self.dk)
            self.cvt[:, :, :, :nc] = cv.view(B, nc, self.hkv, self.dv).permute(0, 2, 3, 1)
        self.ctx_lens.fill_(T)

    @torch.no_grad()
    def append(self, k_new: torch.Tensor, v_new: torch.Tensor):
        """k_new [B,Hkv,Dk], v_new [B,Hkv,Dv]: the next token of every sequence."""
        pos = self.ctx_lens.clone()
        k_new, v_new = k_new.contiguous(), v_new.contiguous()      # keep the copies alive across the launch
        rc = _lib.load().nsa_decode_append(_ptr(k_new), _ptr(v_new), _ptr(self.k),
                                           _ptr(self.vt), _ptr(self.ck), _ptr(self.cvt), _ptr(pos), self.batch,
                                           self.hkv, self.dk, self.dv, self.ctx_cap, self.nc_cap, self.block,
                                           self.stride, _dtype_code(self.k), _stream())
        _lib.check(rc, "nsa_decode_append")
        self.ctx_lens += 1


@torch.no_grad()
def nsa_decode_step(q: torch.Tensor, cache: NSADecodeCache, gates: Optional[torch.Tensor] = None,
                    selection_block: int = 64, selected_block_count: int = 16, sliding_window: int = 512,
                    scale: Optional[float] = None, gate_activation: Optional[str] = None,
                    return_indices: bool = False):
    """q [B,Hq,Dk]: queries of the newest cached token.  gates [B,Hq,3] (selected, sliding,
    compressed; pre-activation if gate_activation == "sigmoid").  Returns out [B,Hq,Dv]
    (and int32 block indices [B,Hkv,S])."""
    if not q.is_cuda:
        raise RuntimeError("NSA kernels run on the GPU only")
    B, hq, dk = q.shape
    q = q.contiguous()
    if scale is None:
        scale = 1.0 / math.sqrt(dk)
    out = torch.empty(B, hq, cache.dv, dtype=q.dtype, device=q.device)
    idx = torch.empty(B, cache.hkv, selected_block_count, dtype=torch.int32, device=q.device) \
        if return_indices else None
    if gates is not None:
        gates = gates.to(q.dtype).contiguous()
    pool_k = selection_block // cache.stride + 1
    pool_s = selection_block // cache.stride
    pool_p = cache.block // cache.stride - 2
    act = _lib.GATE_SIGMOID if gate_activation == "sigmoid" else _lib.GATE_IDENTITY
    rc = _lib.load().nsa_decode_step(
        _ptr(q), _ptr(cache.k), _ptr(cache.vt), _ptr(cache.ck), _ptr(cache.cvt), _ptr(cache.ctx_lens), _ptr(gates),
        _ptr(out), _ptr(idx), B, hq, cache.hkv, dk, cache.dv, cache.ctx_cap, cache.nc_cap, cache.block, cache.stride,
        selection_block, pool_k, pool_s, pool_p, selected_block_count, sliding_window, float(scale), act,
        _dtype_code(q), _stream())
    _lib.check(rc, "nsa_decode_step")
    return (out, idx) if return_indices else out
