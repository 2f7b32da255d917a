"""CPU oracle for an attention layer built around the NSA forward: projections, rotary embedding,
gating, NSA core, output projection.  TEST INFRASTRUCTURE ONLY (same rules as nsa_oracle.py: only
tests, the smoke check and the benchmark's cpu_baseline leg import it).

The reference stops at the attention module: nsa/nsa.py:83-135 receives q, k, v already projected
and rotated, and derives the gate logits from that q with its own Linear (nsa/nsa.py:61,117).  The
layer restated here is the caller it implies, written un-fused so that a fused implementation
(gating folded into the projection GEMM, split + rotation in one pass) has something to be checked
against:

  rope_rotate          rotary embedding of channels [rope_off, rope_off+rope_dim) of each head
  layer_forward        x -> q,k,v = Linear(x); gate logits = gating(q) (nsa/nsa.py:117, on the
                       projected q before the rotation); q,k rotated; NSA forward (nsa_oracle);
                       out = Linear(o)

How it is pinned (tests/test_oracle_pins.py, none of which retypes the rotation formula):
  rope_rotate   multiplication by torch.polar(1, angle) on complex pairs; the two pairings agree
                up to the channel permutation that maps one onto the other; position 0 is the
                identity; norms are preserved; <rope(q,m), rope(k,n)> depends on m-n only
  layer_forward composition of F.linear, rope_rotate and the pinned NSA oracle
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch
import torch.nn.functional as F

from . import nsa_oracle as O


def positions_from_cu(cu_seqlens: Sequence[int]) -> torch.Tensor:
    return torch.cat([torch.arange(int(e) - int(s)) for s, e in zip(cu_seqlens[:-1], cu_seqlens[1:])])


def rope_rotate(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, rope_off: int, rope_dim: int,
                interleaved: bool = False, inverse: bool = False, math_dtype=torch.float32) -> torch.Tensor:
    """x [total, H, D]; angle of pair i at position p is p * inv_freq[i] (computed in fp32 as the
    usual implementations do, then used in math_dtype).  Pair i = channels (i, i + rope_dim/2) of
    the rotary range, or (2i, 2i+1) when interleaved.  Returns math_dtype."""
    out = x.to(math_dtype).clone()
    ang = (positions.to(torch.float32)[:, None] * inv_freq.to(torch.float32)[None, :]).to(math_dtype)
    if inverse:
        ang = -ang
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    r = out[..., rope_off:rope_off + rope_dim]
    if interleaved:
        a, b = r[..., 0::2], r[..., 1::2]
        rot = torch.stack([a * cos - b * sin, b * cos + a * sin], dim=-1).flatten(-2)
    else:
        a, b = r[..., :rope_dim // 2], r[..., rope_dim // 2:]
        rot = torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)
    out[..., rope_off:rope_off + rope_dim] = rot
    return out


def layer_forward(x, w_q, w_k, w_v, w_o, gating_w, gating_b, cu_seqlens, p: O.NSAParams, hq, hkv, dk, dv,
                  inv_freq=None, rope_off=0, rope_dim=0, interleaved=False, gate_activation=None, compressor=None,
                  b_q=None, b_k=None, b_v=None, b_o=None, positions=None, return_parts=False,
                  math_dtype=torch.float32, force_idx=None):
    """x [total, hidden] (packed sequences), w_q [hq*dk, hidden], w_k [hkv*dk, hidden], w_v
    [hkv*dv, hidden], w_o [hidden, hq*dv], gating_w [3, dk], gating_b [3].  Every tensor the un-fused
    layer would materialise (q, k, v, gate logits, attention output) is rounded to x.dtype; with
    x in float64 nothing is rounded, which is the form autograd runs through for gradient checks.
    force_idx [total, hkv, S] replaces the block picks (so that score ties cannot differ)."""
    dt = x.dtype
    f = math_dtype
    total = x.shape[0]

    def lin(inp, w, b):
        return F.linear(inp.to(f), w.to(f), None if b is None else b.to(f))

    q = lin(x, w_q, b_q).to(dt).view(total, hq, dk)
    k = lin(x, w_k, b_k).to(dt).view(total, hkv, dk)
    v = lin(x, w_v, b_v).to(dt).view(total, hkv, dv)
    logits = lin(q, gating_w, gating_b).to(dt)                      # [total, hq, 3]
    if inv_freq is not None:
        pos = positions_from_cu(cu_seqlens) if positions is None else positions
        q = rope_rotate(q, pos, inv_freq, rope_off, rope_dim, interleaved, math_dtype=f).to(dt)
        k = rope_rotate(k, pos, inv_freq, rope_off, rope_dim, interleaved, math_dtype=f).to(dt)
    gates = torch.sigmoid(logits.to(f)).to(dt) if gate_activation == "sigmoid" else logits
    outs = []
    for s, e in zip(cu_seqlens[:-1], cu_seqlens[1:]):
        s, e = int(s), int(e)
        outs.append(O.nsa_forward_single(q[s:e], k[s:e], v[s:e], gates[s:e], p, compressor, math_dtype,
                                         force_idx=None if force_idx is None else force_idx[s:e]))
    o = torch.cat(outs, 0)
    out = lin(o.reshape(total, hq * dv), w_o, b_o).to(dt)
    if return_parts:
        return out, dict(q=q, k=k, v=v, logits=logits, o=o)
    return out
