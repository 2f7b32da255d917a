"""An attention layer around NSAAttention: fused q/k/v projection with the gating Linear folded in,
rotary embedding on a slice of the q/k heads, NSA core, output projection, prefill and decode.

The reference ends at the attention module (nsa/nsa.py:15-135): its caller projects, rotates and
hands in q, k, v, and the module computes the gate logits with a Linear on q (nsa/nsa.py:61,117).
Here the logits of head h, gating(q_h) = Wg (Wq_h x + bq_h) + bg, are 3 more output columns of the
projection GEMM with weight Wg Wq_h, so they cost no pass over q; one HIP pass then splits the
GEMM's packed rows into contiguous q, k, v, gate logits and rotates the rotary channels of q and k
on the way.  With a rotation the folded gate reads q before it is rotated (a Linear on the rotated
q is position dependent and does not fold); without rotation it is exactly the reference's gate.

Parameter names follow the common decoder-layer convention (`q_proj`, `k_proj`, `v_proj`,
`o_proj`), the NSA parameters live under `attn.` with the reference's names."""
from __future__ import annotations

import math
from typing import Optional

import torch
from torch import nn
import torch.nn.functional as F

from . import ops
from .autograd import QkvRopeFn, needs_grad
from .decode import NSADecodeCache, NSAPagedDecodeCache, nsa_decode_step
from .nsa import NSAAttention


def _round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


class NSAAttentionLayer(nn.Module):
    """hidden_states -> attention output of the same shape.

    qk_head_dim / v_head_dim: head sizes of q,k and of v (e.g. 192 / 128); rope_dim: how many
    trailing channels of every q and k head are rotary (192 = 128 content + 64 rotary); 0 = none.
    rope_interleaved pairs channels (2i, 2i+1) instead of (i, i + rope_dim/2)."""

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, qk_head_dim: int = 128,
                 v_head_dim: Optional[int] = None, rope_dim: int = 0, rope_theta: float = 10000.0,
                 rope_interleaved: bool = False, bias: bool = False, compression_stride: int = 16,
                 compression_block: int = 32, selection_block: int = 64, selected_block_count: int = 16,
                 sliding_window: int = 512, compressor_mode: str = "conv", gate_activation: Optional[str] = None,
                 softmax_scale: Optional[float] = None, device=None, dtype=None):
        super().__init__()
        v_head_dim = qk_head_dim if v_head_dim is None else v_head_dim
        if num_heads % num_kv_heads != 0:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if rope_dim < 0 or rope_dim > qk_head_dim or rope_dim % (8 if rope_interleaved else 16) != 0 or \
                (qk_head_dim - rope_dim) % 8 != 0:
            raise ValueError("rope_dim must be a multiple of 16 (8 when interleaved) that leaves an 8-aligned "
                             "content part")
        kw = dict(device=device, dtype=dtype)
        self.hidden_size, self.hq, self.hkv = hidden_size, num_heads, num_kv_heads
        self.dk, self.dv, self.rope_dim, self.rope_interleaved = qk_head_dim, v_head_dim, rope_dim, rope_interleaved
        self.q_proj = nn.Linear(hidden_size, num_heads * qk_head_dim, bias=bias, **kw)
        self.k_proj = nn.Linear(hidden_size, num_kv_heads * qk_head_dim, bias=bias, **kw)
        self.v_proj = nn.Linear(hidden_size, num_kv_heads * v_head_dim, bias=bias, **kw)
        self.o_proj = nn.Linear(num_heads * v_head_dim, hidden_size, bias=bias, **kw)
        self.attn = NSAAttention(qk_head_dim, True, softmax_scale, compression_stride=compression_stride,
                                 compression_block=compression_block, selection_block=selection_block,
                                 selected_block_count=selected_block_count, sliding_window=sliding_window,
                                 compressor_mode=compressor_mode, gate_activation=gate_activation,
                                 v_head_dim=v_head_dim, **kw)
        if rope_dim:
            inv = 1.0 / (rope_theta ** (torch.arange(0, rope_dim, 2, dtype=torch.float32, device=device) / rope_dim))
        else:
            inv = None
        self.register_buffer("inv_freq", inv, persistent=False)
        # packed row of the fused projection: [q | k | v | gate logits | padding to a multiple of 8]
        nq, nk, nv = num_heads * qk_head_dim, num_kv_heads * qk_head_dim, num_kv_heads * v_head_dim
        self.offsets = (0, nq, nq + nk, nq + nk + nv)
        self.ld = _round_up(nq + nk + nv + 3 * num_heads, 8)
        self._fused = None          # (key, weight, bias) of the last inference call

    # ------------------------------------------------------------------ fused projection weights
    def fused_projection(self):
        """Weight [ld, hidden] and bias [ld] of the one GEMM that yields q, k, v and the gate logits."""
        wq, gw, gb = self.q_proj.weight, self.attn.gating.weight, self.attn.gating.bias
        f = torch.float32
        w_fold = torch.einsum("od,hdx->hox", gw.to(f), wq.to(f).view(self.hq, self.dk, -1)).reshape(3 * self.hq, -1)
        b_fold = gb.to(f).repeat(self.hq)
        if self.q_proj.bias is not None:
            b_fold = b_fold + (self.q_proj.bias.to(f).view(self.hq, self.dk) @ gw.to(f).t()).reshape(-1)
        pad = self.ld - self.offsets[3] - 3 * self.hq
        dt = wq.dtype

        def bias_of(lin):
            return lin.bias if lin.bias is not None else torch.zeros(lin.out_features, dtype=dt, device=wq.device)

        weight = torch.cat([wq, self.k_proj.weight, self.v_proj.weight, w_fold.to(dt),
                            torch.zeros(pad, wq.shape[1], dtype=dt, device=wq.device)])
        bias = torch.cat([bias_of(self.q_proj), bias_of(self.k_proj), bias_of(self.v_proj), b_fold.to(dt),
                          torch.zeros(pad, dtype=dt, device=wq.device)])
        return weight, bias

    def _projection_params(self):
        ps = [self.q_proj.weight, self.k_proj.weight, self.v_proj.weight, self.attn.gating.weight,
              self.attn.gating.bias]
        return ps + [l.bias for l in (self.q_proj, self.k_proj, self.v_proj) if l.bias is not None]

    def _fused_cached(self):
        ps = self._projection_params()
        key = tuple((p.data_ptr(), p._version) for p in ps)
        if self._fused is None or self._fused[0] != key:
            with torch.no_grad():
                self._fused = (key,) + self.fused_projection()
        return self._fused[1], self._fused[2]

    # ------------------------------------------------------------------ forward
    def forward(self, hidden_states: torch.Tensor, attention_mask=None, position_ids: Optional[torch.Tensor] = None,
                past_key_value=None, output_attentions: bool = False, use_cache: bool = False,
                cu_seqlens: Optional[torch.Tensor] = None, max_seqlen: Optional[int] = None,
                return_indices: bool = False, **_):
        """hidden_states [B, T, hidden] (equal-length sequences) or [total, hidden] with cu_seqlens
        (packed ragged sequences, max_seqlen = the longest).  Causal attention only: padding is
        expressed through cu_seqlens, so attention_mask must be None.  past_key_value: an
        NSADecodeCache / NSAPagedDecodeCache; with T == 1 the call is one decode step on it (the
        new token is appended first), with T > 1 the prompt is attended and its keys/values are
        loaded into the cache.  Returns (attention output shaped like hidden_states, None); with
        return_indices the second item is the int32 block ids [total, Hkv, S] the queries picked."""
        if attention_mask is not None:
            raise NotImplementedError("pass ragged batches packed with cu_seqlens; the kernels are causal")
        if output_attentions:
            raise NotImplementedError("sparse attention keeps no attention matrix")
        shape = hidden_states.shape
        if hidden_states.dim() == 3:
            B, T = shape[:2]
            if cu_seqlens is None:
                cu_seqlens = ops.uniform_cu(B, T, hidden_states.device)
            x = hidden_states.reshape(B * T, shape[2])
            uniform_len = T
        else:
            if cu_seqlens is None:
                raise ValueError("packed hidden_states [total, hidden] need cu_seqlens")
            x, uniform_len = hidden_states, None
            B, T = cu_seqlens.numel() - 1, None
            if max_seqlen is None:
                max_seqlen = int((cu_seqlens[1:] - cu_seqlens[:-1]).max())
        cache = past_key_value
        if cache is not None and T == 1:
            return self._decode(x, cache).view(shape), None
        train = needs_grad(x, *self.parameters())
        weight, bias = self.fused_projection() if train else self._fused_cached()
        positions = None if position_ids is None else position_ids.reshape(-1).to(torch.int32)
        rope = (self.inv_freq, positions, cu_seqlens, self.dk - self.rope_dim, self.rope_dim, self.rope_interleaved)
        if train:
            packed = F.linear(x, weight, bias)
            q, k, v, gates = QkvRopeFn.apply(packed, self.hq, self.hkv, self.dk, self.dv, self.offsets, *rope, True)
        else:
            with torch.no_grad():
                packed = F.linear(x, weight, bias)
                q, k, v, gates = ops.qkv_rope_split(packed, self.hq, self.hkv, self.dk, self.dv, self.offsets, *rope)
        o = self.attn(q, k, v, cu_seqlens, 0 if uniform_len is not None else max_seqlen, gates=gates,
                      return_indices=return_indices)
        idx = None
        if return_indices:
            o, idx = o
        if cache is not None:
            if uniform_len is None:
                raise NotImplementedError("loading a cache from a packed ragged prompt: fill it per sequence")
            cache.fill(k.view(B, T, self.hkv, self.dk), v.view(B, T, self.hkv, self.dv))
        out = self.o_proj(o.reshape(x.shape[0], self.hq * self.dv))
        return out.view(shape), idx

    @torch.no_grad()
    def _decode(self, x, cache):
        if not isinstance(cache, (NSADecodeCache, NSAPagedDecodeCache)):
            raise TypeError("past_key_value must be an NSADecodeCache or NSAPagedDecodeCache")
        if self.attn.compressor.mode != "mean":
            raise NotImplementedError("the decode cache compresses by mean pooling (compressor_mode='mean')")
        weight, bias = self._fused_cached()
        packed = F.linear(x, weight, bias)
        q, k_new, v_new, gates = ops.qkv_rope_split(
            packed, self.hq, self.hkv, self.dk, self.dv, self.offsets, self.inv_freq, cache.ctx_lens, None,
            self.dk - self.rope_dim, self.rope_dim, self.rope_interleaved)
        cache.append(k_new, v_new)
        a = self.attn
        scale = a.softmax_scale if a.softmax_scale not in (None, True) else 1.0 / math.sqrt(self.dk)
        o = nsa_decode_step(q, cache, gates, a.selection_block_size, a.selected_block_count, a.sliding_window, scale,
                            a.gate_activation)
        return self.o_proj(o.reshape(x.shape[0], self.hq * self.dv))
