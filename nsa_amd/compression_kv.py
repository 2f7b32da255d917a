"""KV block compression with the interface of the reference's nsa/compression_kv.py.

calc_compressed_len (compression_kv.py:9-10), compress_kv (:178-217, :269), KVCompressorVarlen
(:272-289) and KVCompressor (:292-312) keep their names, argument order, parameter names/shapes and
return arity.  The arithmetic runs in the HIP kernels of libnsa_hip.so, forward and backward (the
backward of :220-266 through nsa_compress_bwd when an input or a parameter requires grad).
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
from torch.nn import init

from . import ops
from .autograd import CompressFn, needs_grad


def calc_compressed_len(x, stride, size):
    """Rows the functional compressor emits for a sequence of x tokens (one fewer than a Conv1d)."""
    return (x - size) // stride


def conv_compressed_len(x, stride, size):
    """Rows nn.Conv1d(kernel=size, stride=stride) emits for x tokens."""
    return 0 if x < size else (x - size) // stride + 1


def compress_kv(k, v, w_k, w_v, cu_seq_len, block_stride, block_size):
    """k, v [total, H, D]; w_* [block_size*D, D] (row j*D+i); cu_seq_len int32 [B+1].
    Returns (ck, cv, cu_out_len): bf16 [sum Nc', H, D] with Nc' = (T - block_size)//block_stride."""
    cu = cu_seq_len.to(torch.int32)
    cu_out = ops.compressed_offsets(cu, block_size, block_stride, extra=0)
    out_rows = int(cu_out[-1].item())      # the reference syncs here as well (cu_seq_len.tolist())
    if needs_grad(k, v, w_k, w_v):
        kk = k if k.dtype in (torch.bfloat16, torch.float32, torch.float16) else k.to(torch.bfloat16)
        vv = v if v.dtype in (torch.bfloat16, torch.float32, torch.float16) else v.to(torch.bfloat16)
        ck = CompressFn.apply(kk, w_k.to(kk.dtype), None, cu, cu_out, out_rows, block_size, block_stride)
        cv = CompressFn.apply(vv, w_v.to(vv.dtype), None, cu, cu_out, out_rows, block_size, block_stride)
        return ck.to(torch.bfloat16), cv.to(torch.bfloat16), cu_out
    with torch.no_grad():
        return _compress_kv_nograd(k, v, w_k, w_v, cu, cu_out, out_rows, block_stride, block_size)


def _compress_kv_nograd(k, v, w_k, w_v, cu, cu_out, out_rows, block_stride, block_size):
    wk_t = w_k.detach().t().contiguous()
    wv_t = w_v.detach().t().contiguous()
    kk = k if k.dtype in (torch.bfloat16, torch.float32, torch.float16) else k.to(torch.bfloat16)
    vv = v if v.dtype in (torch.bfloat16, torch.float32, torch.float16) else v.to(torch.bfloat16)
    if kk.dtype != vv.dtype:
        vv = vv.to(kk.dtype)
    ck, cv = ops.compress_kv(kk, vv, cu, cu_out, out_rows, block_size, block_stride, wk_t, wv_t)
    return ck.to(torch.bfloat16), cv.to(torch.bfloat16), cu_out


class KVCompressorVarlen(nn.Module):
    def __init__(self, block_stride, block_size, head_dim, device, dtype):
        factory_kwargs = {"device": device, "dtype": dtype}
        super().__init__()
        self.block_stride = block_stride
        self.block_size = block_size
        self.k_weight = nn.Parameter(torch.empty(block_size * head_dim, head_dim, **factory_kwargs))
        self.v_weight = nn.Parameter(torch.empty(block_size * head_dim, head_dim, **factory_kwargs))
        self.reset_parameters()

    def forward(self, k, v, cu_seq_len, group=None):
        return compress_kv(k, v, self.k_weight, self.v_weight, cu_seq_len, self.block_stride, self.block_size)

    def reset_parameters(self) -> None:
        init.kaiming_uniform_(self.k_weight, a=math.sqrt(5))
        init.kaiming_uniform_(self.v_weight, a=math.sqrt(5))


class KVCompressor(nn.Module):
    """Conv1d-parameterised compressor (weight [D, D, block], bias [D], shared over heads).

    mode="conv" is the reference; mode="mean" ignores the parameters and averages each window
    (the conv with eye/block weights and zero bias)."""

    def __init__(self, block_stride, block_size, head_dim, device=None, dtype=None, mode: str = "conv",
                 v_head_dim: Optional[int] = None):
        super().__init__()
        factory_kwargs = {"device": device, "dtype": dtype}
        self.block_stride = block_stride
        self.block_size = block_size
        self.mode = mode
        v_head_dim = head_dim if v_head_dim is None else v_head_dim     # the reference has one head_dim for both
        self.compressor_k = nn.Conv1d(head_dim, head_dim, block_size, block_stride, **factory_kwargs)
        self.compressor_v = nn.Conv1d(v_head_dim, v_head_dim, block_size, block_stride, **factory_kwargs)

    def _wt(self, conv: nn.Conv1d) -> torch.Tensor:
        """[o, i, j] -> [o, j*D + i], the layout the kernels read.  The no-grad path asks for it on every forward, so
        the copy is kept until the parameter changes (another tensor, another storage, or an in-place update)."""
        w = conv.weight.detach()
        key = (id(conv.weight), w.data_ptr(), conv.weight._version, w.dtype, w.device)
        cache = self.__dict__.setdefault("_wt_cache", {})
        hit = cache.get(id(conv))
        if hit is None or hit[0] != key:
            hit = (key, w.permute(0, 2, 1).reshape(w.shape[0], -1).contiguous())
            cache[id(conv)] = hit
        return hit[1]

    @staticmethod
    def _w_lin(conv: nn.Conv1d) -> torch.Tensor:
        # [o, i, j] -> [j*D + i, o], differentiable
        w = conv.weight
        return w.permute(2, 1, 0).reshape(-1, w.shape[0])

    def compress_packed(self, k, v, cu_seq_len, seq_len: Optional[int] = None):
        """Un-repeated result: (ck, cv [sum Nc, H, D], cu_cmp int32 [B+1], max Nc or None)."""
        params = () if self.mode == "mean" else tuple(self.parameters())
        if needs_grad(k, v, *params):
            return self._compress_packed(k, v, cu_seq_len, seq_len, True)
        with torch.no_grad():
            return self._compress_packed(k, v, cu_seq_len, seq_len, False)

    def _compress_packed(self, k, v, cu_seq_len, seq_len, train):
        cu = cu_seq_len.to(torch.int32)
        batch = cu.numel() - 1
        nc = conv_compressed_len(seq_len, self.block_stride, self.block_size) if seq_len is not None else None
        if nc:
            cu_out = ops.uniform_cu(batch, nc, k.device)
            rows = nc * batch
        else:                       # ragged lengths, or sequences shorter than one block (no rows at all)
            cu_out = ops.compressed_offsets(cu, self.block_size, self.block_stride, extra=1)
            rows = k.shape[0] // self.block_stride + batch
            nc = None
        if train:
            if self.mode == "mean":
                wk = wv = bk = bv = None
            else:
                wk, wv = self._w_lin(self.compressor_k).to(k.dtype), self._w_lin(self.compressor_v).to(v.dtype)
                bk, bv = self.compressor_k.bias, self.compressor_v.bias
            ck = CompressFn.apply(k, wk, bk, cu, cu_out, rows, self.block_size, self.block_stride)
            cv = CompressFn.apply(v, wv, bv, cu, cu_out, rows, self.block_size, self.block_stride)
        elif self.mode == "mean":
            ck, cv = ops.compress_kv(k, v, cu, cu_out, rows, self.block_size, self.block_stride)
        else:
            ck, cv = ops.compress_kv(k, v, cu, cu_out, rows, self.block_size, self.block_stride,
                                     self._wt(self.compressor_k), self._wt(self.compressor_v),
                                     self.compressor_k.bias, self.compressor_v.bias)
        return ck, cv, cu_out, nc

    def forward(self, k, v, cu_seq_len, group=None):
        """k, v [B*T, H, D] with B = len(cu_seq_len)-1 equal-length sequences.
        Returns (ck, cv [B, Nc, H*group, D], cu_seq_len) like the reference."""
        BT, H, D = k.shape
        B = cu_seq_len.shape[0] - 1
        T = BT // B
        cu = ops.uniform_cu(B, T, k.device)
        ck, cv, _, nc = self.compress_packed(k, v, cu, seq_len=T)
        ck = ck.view(B, nc, H, D)
        cv = cv.view(B, nc, H, v.shape[-1])
        if group is not None:
            ck = ck.repeat_interleave(group, dim=2)
            cv = cv.repeat_interleave(group, dim=2)
        return ck, cv, cu_seq_len
