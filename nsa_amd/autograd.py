"""torch.autograd glue over the backward entry points of the C ABI.  Every Function works on packed
tensors ([total, heads, dim]); the forward calls the same kernels as the inference path (asking them
for the log-sum-exp per row), the backward calls nsa_compress_bwd / nsa_cmp_attn_bwd /
nsa_slc_swa_bwd.  No arithmetic happens here.

Counterparts in the reference: _compress_kv (nsa/compression_kv.py:178-266), _attention
(nsa/triton_attention.py:419-546), ParallelNSAFunction (nsa/selection_attn.py:679-737)."""
from __future__ import annotations

import torch

from . import ops


def needs_grad(*tensors) -> bool:
    """True when a call has to build an autograd graph."""
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


class CompressFn(torch.autograd.Function):
    """x [total,H,D] -> [rows,H,D].  w_lin None = mean pooling, else [block*D, D] (row j*D+i, column o)
    with an optional bias [D]."""

    @staticmethod
    def forward(ctx, x, w_lin, bias, cu, cu_out, rows, block, stride):
        wt = None if w_lin is None else w_lin.detach().t().contiguous()
        out = ops.compress(x, cu, cu_out, rows, block, stride, wt, None if bias is None else bias.detach())
        ctx.save_for_backward(x, w_lin, bias, cu, cu_out)
        ctx.geom = (block, stride)
        return out

    @staticmethod
    def backward(ctx, d_out):
        x, w_lin, bias, cu, cu_out = ctx.saved_tensors
        block, stride = ctx.geom
        if w_lin is None:
            dx = ops.compress_bwd(d_out, cu, cu_out, x.shape[0], block, stride)
            return dx, None, None, None, None, None, None, None
        dx, dw, db = ops.compress_bwd(d_out, cu, cu_out, x.shape[0], block, stride, x=x, w_lin=w_lin.detach(),
                                      want_dw=ctx.needs_input_grad[1],
                                      want_dbias=bias is not None and ctx.needs_input_grad[2])
        dw = None if dw is None else dw.to(w_lin.dtype)
        db = None if db is None else db.to(bias.dtype)
        return dx, dw, db, None, None, None, None, None


class CmpAttnFn(torch.autograd.Function):
    """Compressed attention (+ block selection, which has no gradient).  q [total,Hq,Dk], ck
    [rows,Hkv,Dk], cv [rows,Hkv,Dv] packed over cu_cmp.  select = None or (pool_kernel, pool_stride,
    pool_pad, top_n, max_nc, idx64).  Returns (o, indices or None)."""

    @staticmethod
    def forward(ctx, q, ck, cv, cu, cu_cmp, batch, block, stride, scale, causal, select):
        q, ck, cv = q.contiguous(), ck.contiguous(), cv.contiguous()
        hkv, dk, dv = ck.shape[1], ck.shape[2], cv.shape[2]
        cvt = ops.transpose(cv, cu_cmp, batch)
        o, lse_raw, lse = ops.cmp_attn(q, ck, cvt, cu, cu_cmp, batch, hkv, dv, hkv * dk, dk, block, stride, scale,
                                       causal=causal, want_lse_attn=True)
        idx = None
        if select is not None:
            pk, ps, pp, top_n, max_nc, idx64 = select
            idx, _ = ops.block_select(q, ck, lse_raw, cu, cu_cmp, batch, hkv, hkv * dk, dk, pk, ps, pp, top_n, max_nc,
                                      idx64=idx64)
            ctx.mark_non_differentiable(idx)
        ctx.save_for_backward(q, ck, cv, o, lse, cu, cu_cmp)
        ctx.geom = (batch, block, stride, scale, causal)
        return o, idx

    @staticmethod
    def backward(ctx, d_o, _d_idx=None):
        q, ck, cv, o, lse, cu, cu_cmp = ctx.saved_tensors
        batch, block, stride, scale, causal = ctx.geom
        dq, dck, dcv = ops.cmp_attn_bwd(q, ck, cv, o, d_o, lse, cu, cu_cmp, batch, block, stride, scale, causal=causal)
        return dq, dck, dcv, None, None, None, None, None, None, None, None


class SlcSwaFn(torch.autograd.Function):
    """Selected-block attention (idx not None) and sliding-window attention (window > 0), ungated.
    q [total,Hq,Dk], k [total,Hkv,Dk], v [total,Hkv,Dv].  Returns (o_slc or None, o_swa or None)."""

    @staticmethod
    def forward(ctx, q, k, v, idx, counts, cu, batch, block_size, window, scale):
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        vt = ops.transpose(v, cu, batch)
        o_slc = lse_slc = o_swa = lse_swa = None
        ws = None
        if idx is not None and window > 0:
            ws = ops.slc_workspace(q, k.shape[1], v.shape[2], idx.shape[-1], block_size, batch)
        if ws is not None:
            # both branches: the fused schedule (partials per block, merged in the window kernel's epilogue),
            # which leaves the two ungated outputs and their log-sum-exps; its gated sum is not used here
            ops.slc_partials(q, k, vt, idx, counts, cu, batch, block_size, scale, ws)
            _, o_slc, o_swa, lse_slc, lse_swa = ops.swa_merge(q, k, vt, ws, idx.shape[-1], None, None, None, None, cu,
                                                               batch, block_size, window, scale, want_branches=True)
        fused = None
        if ws is None and idx is not None and window > 0:
            # the same schedule in token slabs when its one-slab workspace is beyond ops.SLC_WORKSPACE_LIMIT
            fused = ops.slc_swa_fused(q, k, vt, idx, counts, None, None, None, None, cu, batch, block_size, window, scale,
                                      want_branches=True)
        if fused is not None:
            _, o_slc, o_swa, lse_slc, lse_swa = fused
        elif ws is None:
            if idx is not None:
                o_slc, lse_slc = ops.slc_combine(q, k, vt, idx, counts, None, None, None, None, None, cu, batch,
                                                 block_size, scale, block_major=True, want_lse=True)
            if window > 0:
                o_swa, lse_swa = ops.swa(q, k, vt, cu, batch, window, scale, want_lse=True)
        ctx.save_for_backward(q, k, v, o_slc, lse_slc, o_swa, lse_swa, idx, counts, cu)
        ctx.geom = (batch, block_size, window, scale)
        return o_slc, o_swa

    @staticmethod
    def backward(ctx, d_slc, d_swa):
        q, k, v, o_slc, lse_slc, o_swa, lse_swa, idx, counts, cu = ctx.saved_tensors
        batch, block_size, window, scale = ctx.geom
        if o_slc is None:
            d_slc = None
        if o_swa is None:
            d_swa = None
        dq, dk, dv = ops.slc_swa_bwd(q, k, v, o_slc, d_slc, lse_slc, o_swa, d_swa, lse_swa, idx, counts, cu, batch,
                                     block_size, window, scale)
        return dq, dk, dv, None, None, None, None, None, None, None


class GateLinearFn(torch.autograd.Function):
    """Gate logits [total,Hq,3] = q . weight^T + bias (the gating nn.Linear of nsa/nsa.py:61)."""

    @staticmethod
    def forward(ctx, q, weight, bias):
        q = q.contiguous()
        ctx.save_for_backward(q, weight, bias)
        return ops.gate_logits(q, weight.detach(), None if bias is None else bias.detach())

    @staticmethod
    def backward(ctx, d_gates):
        q, weight, bias = ctx.saved_tensors
        dq, dw, db = ops.gate_bwd(q, weight.detach(), d_gates, want_dbias=bias is not None)
        return dq, dw.to(weight.dtype), None if db is None else db.to(bias.dtype)


class GateCombineFn(torch.autograd.Function):
    """out = sum_b act(gate_logits[..., b]) * o_b, b = (selected, sliding, compressed)."""

    @staticmethod
    def forward(ctx, gate_logits, o_slc, o_swa, o_cmp, gate_act):
        ctx.save_for_backward(gate_logits, o_slc, o_swa, o_cmp)
        ctx.gate_act = gate_act
        return ops.gate_combine(gate_logits, o_slc, o_swa, o_cmp, gate_act)

    @staticmethod
    def backward(ctx, d_out):
        gate_logits, o_slc, o_swa, o_cmp = ctx.saved_tensors
        d_slc, d_swa, d_cmp, d_gl = ops.gate_combine_bwd(gate_logits, d_out, o_slc, o_swa, o_cmp, ctx.gate_act)
        return d_gl.to(gate_logits.dtype), d_slc, d_swa, d_cmp, None


class NSACoreFn(torch.autograd.Function):
    """The three branches and their gated sum as one node (what NSAAttention's training path runs):
    q [total,Hq,Dk], ck / cv [rows,Hkv,D] packed over cu_cmp, k / v [total,Hkv,D], gate_logits
    [total,Hq,3] -> (out [total,Hq,Dv], indices int32 [total,Hkv,S]).  One node lets the backward hand
    the gates to the attention kernels as per-row scales together with the unscaled row sums
    <d_out, o_b>, so neither scaled copies of d_out nor separate row-sum passes are needed."""

    @staticmethod
    def forward(ctx, q, ck, cv, k, v, gate_logits, cu, cu_cmp, batch, block, stride, sel_block, window, scale,
                causal, select, gate_act):
        q, ck, cv, k, v = (t.contiguous() for t in (q, ck, cv, k, v))
        hkv, dk, dv = ck.shape[1], ck.shape[2], cv.shape[2]
        cvt, vt = ops.transpose(cv, cu_cmp, batch), ops.transpose(v, cu, batch)
        o_cmp, lse_raw, lse_cmp = ops.cmp_attn(q, ck, cvt, cu, cu_cmp, batch, hkv, dv, hkv * dk, dk, block, stride,
                                               scale, causal=causal, want_lse_attn=True)
        pk, ps, pp, top_n, max_nc = select
        idx, _ = ops.block_select(q, ck, lse_raw, cu, cu_cmp, batch, hkv, hkv * dk, dk, pk, ps, pp, top_n, max_nc,
                                  idx64=False)
        ws = ops.slc_workspace(q, hkv, dv, idx.shape[-1], sel_block, batch) if window > 0 else None
        gl = gate_logits.reshape(-1, 3)
        if ws is not None and gl.dtype == q.dtype:
            # the inference schedule (partials per block, merged in the window kernel's epilogue), which also
            # leaves the ungated branch outputs and their log-sum-exps for the backward
            ops.slc_partials(q, k, vt, idx, None, cu, batch, sel_block, scale, ws)
            g_slc, g_swa, g_cmp = (gl[:, i].view(q.shape[0], q.shape[1]) for i in range(3))
            out, o_slc, o_swa, lse_slc, lse_swa = ops.swa_merge(
                q, k, vt, ws, idx.shape[-1], g_slc, g_swa, g_cmp, o_cmp, cu, batch, sel_block, window, scale,
                gate_act=gate_act, want_branches=True)
        fused = None
        if ws is None and window > 0 and gl.dtype == q.dtype:
            g_slc, g_swa, g_cmp = (gl[:, i].view(q.shape[0], q.shape[1]) for i in range(3))
            fused = ops.slc_swa_fused(q, k, vt, idx, None, g_slc, g_swa, g_cmp, o_cmp, cu, batch, sel_block, window,
                                      scale, gate_act=gate_act, want_branches=True)
        if fused is not None:
            out, o_slc, o_swa, lse_slc, lse_swa = fused
        elif ws is None or gl.dtype != q.dtype:
            o_slc, lse_slc = ops.slc_combine(q, k, vt, idx, None, None, None, None, None, None, cu, batch, sel_block,
                                             scale, block_major=True, want_lse=True)
            o_swa = lse_swa = None
            if window > 0:
                o_swa, lse_swa = ops.swa(q, k, vt, cu, batch, window, scale, want_lse=True)
            out = ops.gate_combine(gate_logits, o_slc, o_swa, o_cmp, gate_act)
        ctx.save_for_backward(q, ck, cv, k, v, gate_logits, o_cmp, lse_cmp, o_slc, lse_slc, o_swa, lse_swa, idx, cu,
                              cu_cmp)
        ctx.geom = (batch, block, stride, sel_block, window, scale, causal, gate_act)
        ctx.mark_non_differentiable(idx)
        return out, idx

    @staticmethod
    def backward(ctx, d_out, _d_idx=None):
        q, ck, cv, k, v, gate_logits, o_cmp, lse_cmp, o_slc, lse_slc, o_swa, lse_swa, idx, cu, cu_cmp = \
            ctx.saved_tensors
        batch, block, stride, sel_block, window, scale, causal, gate_act = ctx.geom
        d_out = d_out.contiguous()
        _, _, _, d_gl, st = ops.gate_combine_bwd(gate_logits, d_out, o_slc, o_swa, o_cmp, gate_act, want_scaled=False,
                                                 want_stats=True)
        dq_c, dck, dcv = ops.cmp_attn_bwd(q, ck, cv, None, d_out, lse_cmp, cu, cu_cmp, batch, block, stride, scale,
                                          causal=causal, delta=st[2], rowscale=st[5])
        dq, dk, dv = ops.slc_swa_bwd(q, k, v, None, d_out, lse_slc, None, d_out if o_swa is not None else None,
                                     lse_swa, idx, None, cu, batch, sel_block, window, scale, delta_slc=st[0],
                                     delta_swa=st[1], rowscale_slc=st[3], rowscale_swa=st[4], dq_add=dq_c)
        return (dq, dck, dcv, dk, dv, d_gl.to(gate_logits.dtype)) + (None,) * 11


class QkvRopeFn(torch.autograd.Function):
    """Packed projection rows -> (q, k, v, gate logits or None) with the rotary embedding on q and k;
    the backward gathers the four gradients into packed rows with the inverse rotation."""

    @staticmethod
    def forward(ctx, packed, hq, hkv, dk, dv, offsets, inv_freq, positions, cu, rope_off, rope_dim, interleaved,
                with_gates):
        ctx.rows, ctx.like = packed.shape[0], (packed.dtype, packed.device)
        ctx.meta = (packed.shape[1], offsets, inv_freq, positions, cu, rope_off, rope_dim, interleaved, with_gates,
                    (hq, hkv, dk, dv))
        q, k, v, g = ops.qkv_rope_split(packed, hq, hkv, dk, dv, offsets, inv_freq, positions, cu, rope_off, rope_dim,
                                        interleaved, with_gates)
        if g is None:
            return q, k, v
        return q, k, v, g

    @staticmethod
    def backward(ctx, dq, dk_, dv_, dg=None):
        ld, offsets, inv_freq, positions, cu, rope_off, rope_dim, interleaved, with_gates, (hq, hkv, dk, dv) = ctx.meta

        def dense(g, heads, dim):
            if g is not None:
                return g
            return torch.zeros(ctx.rows, heads, dim, dtype=ctx.like[0], device=ctx.like[1])

        dq, dk_, dv_ = dense(dq, hq, dk), dense(dk_, hkv, dk), dense(dv_, hkv, dv)
        if with_gates:
            dg = dense(dg, hq, 3)
        d_packed = ops.qkv_rope_pack(dq, dk_, dv_, dg if with_gates else None, ld, offsets, inv_freq, positions, cu,
                                     rope_off, rope_dim, interleaved)
        return (d_packed,) + (None,) * 12
