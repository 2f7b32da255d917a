"""Thin tensor-level wrappers over the C ABI: they check layouts, allocate outputs with torch and
enqueue the kernels on the current stream.  No arithmetic happens in Python."""
from __future__ import annotations

import ctypes as C
import math
import os
from typing import Optional, Tuple

import torch

from . import _lib


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return _lib.NSA_BF16
    if t.dtype == torch.float32:
        return _lib.NSA_F32
    if t.dtype == torch.float16:
        return _lib.NSA_F16
    raise TypeError("NSA kernels take bfloat16, float16 or float32 tensors, got %s" % t.dtype)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("NSA kernels run on the GPU only; got a %s tensor" % t.device)


def _dense(t: torch.Tensor) -> torch.Tensor:
    """Contiguous and 16-byte aligned."""
    if not t.is_contiguous() or t.data_ptr() % 16:
        t = t.contiguous()
        if t.data_ptr() % 16:
            t = t.clone()
    return t


def pool_bins(nc: int, kernel: int, stride: int, pad: int) -> int:
    """Bins of a ceil-mode average pool (kernel, stride, pad) over nc columns."""
    if nc <= 0 or nc + 2 * pad < kernel:
        return 0
    ns = -(-(nc + 2 * pad - kernel) // stride) + 1
    if (ns - 1) * stride >= nc + pad:
        ns -= 1
    return ns


def head_subgroups(hq: int, hkv: int) -> int:
    """Sub-groups of 16 query heads per kv head: 1 for GQA groups up to 16; groups of 32, 48, 64, ... heads (the
    reference's HQ % (16 * H) == 0, nsa/selection_attn.py:800) run as G / 16 sub-groups that share the keys,
    values and block picks of their kv head."""
    g = hq // hkv
    return g // 16 if g > 16 and g % 16 == 0 else 1


def transposed_cols(total_rows: int, batch: int) -> int:
    return _lib.load().nsa_transposed_cols(total_rows, batch)


def uniform_cu(batch: int, length: int, device) -> torch.Tensor:
    if length == 0:
        return torch.zeros(batch + 1, dtype=torch.int32, device=device)
    return torch.arange(0, (batch + 1) * length, length, dtype=torch.int32, device=device)


def compressed_offsets(cu_seqlens: torch.Tensor, block: int, stride: int, extra: int = 1) -> torch.Tensor:
    """Row offsets of every sequence in the packed compressed tensor, computed on the device.
    extra = 1: Conv1d count (len-block)//stride + 1;  extra = 0: the functional count."""
    lens = (cu_seqlens[1:] - cu_seqlens[:-1]).to(torch.int64)
    nc = torch.where(lens >= block, (lens - block) // stride + extra, torch.zeros_like(lens)).clamp_(min=0)
    out = torch.zeros(cu_seqlens.numel(), dtype=torch.int32, device=cu_seqlens.device)
    out[1:] = torch.cumsum(nc, 0).to(torch.int32)
    return out


def transpose(x: torch.Tensor, cu: torch.Tensor, batch: int, heads: Optional[int] = None,
              head_stride: Optional[int] = None) -> torch.Tensor:
    """x [rows, H, dim] (last dim contiguous) -> key-contiguous [heads, dim, cols].
    heads/head_stride let a caller read every (H/heads)-th head of a head-repeated tensor."""
    _need_cuda(x, cu)
    rows, H, dim = x.shape
    if x.stride(2) != 1 or x.data_ptr() % 16:
        x = _dense(x)
    heads = H if heads is None else heads
    head_stride = x.stride(1) if head_stride is None else head_stride
    cols = transposed_cols(rows, batch)
    out = torch.empty(heads, dim, cols, dtype=x.dtype, device=x.device)
    lib = _lib.load()
    rc = lib.nsa_transpose_fwd(_ptr(x), _ptr(out), _ptr(cu), batch, heads, dim, x.stride(0), head_stride,
                               cols, _dtype_code(x), _stream())
    _lib.check(rc, "nsa_transpose_fwd")
    return out


def compress(x: torch.Tensor, cu_seqlens: torch.Tensor, cu_out: torch.Tensor, out_rows: int, block: int,
             stride: int, wt: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [total, H, D] -> [out_rows, H, D]; wt None = mean over each window, else [D, block*D]."""
    _need_cuda(x, cu_seqlens, cu_out)
    x = _dense(x)
    total, H, D = x.shape
    out = torch.empty(out_rows, H, D, dtype=x.dtype, device=x.device)
    if wt is not None:
        wt = _dense(wt.to(x.dtype))
        if tuple(wt.shape) != (D, block * D):
            raise ValueError("weight must be [dim, block*dim], got %s" % (tuple(wt.shape),))
    if bias is not None:
        bias = _dense(bias.to(x.dtype))
    if out_rows == 0:
        return out
    lib = _lib.load()
    rc = lib.nsa_compress_fwd(_ptr(x), _ptr(wt), _ptr(bias), _ptr(out), _ptr(cu_seqlens), _ptr(cu_out),
                              cu_seqlens.numel() - 1, out_rows, H, D, block, stride, _dtype_code(x), _stream())
    _lib.check(rc, "nsa_compress_fwd")
    return out


def compress_kv(k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor, cu_out: torch.Tensor, out_rows: int,
                block: int, stride: int, wk_t=None, wv_t=None, bk=None, bv=None):
    """k [total, H, Dk], v [total, H, Dv] -> (ck [out_rows, H, Dk], cv [out_rows, H, Dv]).  Without weights
    (mean over each window) both tensors go through one launch; w*_t are [D, block*D] as in compress()."""
    _need_cuda(k, v, cu_seqlens, cu_out)
    k, v = _dense(k), _dense(v)
    total, H, Dk = k.shape
    if v.shape[0] != total or v.shape[1] != H or v.dtype != k.dtype:
        raise ValueError("k and v must share tokens, heads and dtype: %s vs %s" % (tuple(k.shape), tuple(v.shape)))
    Dv = v.shape[2]
    ck = torch.empty(out_rows, H, Dk, dtype=k.dtype, device=k.device)
    cv = torch.empty(out_rows, H, Dv, dtype=v.dtype, device=v.device)
    if (wk_t is None) != (wv_t is None):
        raise ValueError("give both weights or neither")
    if wk_t is not None:
        wk_t, wv_t = _dense(wk_t.to(k.dtype)), _dense(wv_t.to(v.dtype))
        if tuple(wk_t.shape) != (Dk, block * Dk) or tuple(wv_t.shape) != (Dv, block * Dv):
            raise ValueError("weights must be [dim, block*dim], got %s and %s" % (tuple(wk_t.shape), tuple(wv_t.shape)))
    bk = None if bk is None else _dense(bk.to(k.dtype))
    bv = None if bv is None else _dense(bv.to(v.dtype))
    if out_rows == 0:
        return ck, cv
    lib = _lib.load()
    rc = lib.nsa_compress_kv_fwd(_ptr(k), _ptr(v), _ptr(wk_t), _ptr(wv_t), _ptr(bk), _ptr(bv), _ptr(ck), _ptr(cv),
                                 _ptr(cu_seqlens), _ptr(cu_out), cu_seqlens.numel() - 1, out_rows, H, Dk, Dv, block,
                                 stride, _dtype_code(k), _stream())
    _lib.check(rc, "nsa_compress_kv_fwd")
    return ck, cv


def cmp_attn_select(q, ck, cvt, cu_seqlens, cu_cmp, batch, hkv, dv, ck_row_stride, ck_head_stride, block,
                    stride, pool_kernel, pool_stride, pool_pad, top_n, max_nc, scale, causal=True,
                    select=True, idx64=True, want_pooled=False):
    """q [total,Hq,Dk] packed; ck any tensor whose rows are reachable with the two strides;
    cvt [hkv, dv, cols].  Returns (o [total,Hq,dv], indices [total,hkv,top_n] or None, pooled or None)."""
    _need_cuda(q, ck, cvt, cu_seqlens, cu_cmp)
    q = _dense(q)
    total, hq, dk = q.shape
    o = torch.empty(total, hq, dv, dtype=q.dtype, device=q.device)
    max_ns = pool_bins(max_nc, pool_kernel, pool_stride, pool_pad) if select else 0
    idx = pooled = None
    lse = torch.empty(total, hq, dtype=torch.float32, device=q.device)
    if select:
        idx = torch.empty(total, hkv, top_n, dtype=torch.int64 if idx64 else torch.int32, device=q.device)
        # always given: with it the library runs its two-kernel schedule (window sums, then top-n); one row per
        # sub-group of 16 heads, the block scores end up in the first row of every kv head
        pooled = torch.empty(total, hkv, head_subgroups(hq, hkv), max(max_ns, 1), dtype=torch.float32, device=q.device)
    lib = _lib.load()
    rc = lib.nsa_cmp_attn_select_fwd(
        _ptr(q), _ptr(ck), _ptr(cvt), _ptr(o), _ptr(idx), _ptr(pooled), _ptr(lse), _ptr(cu_seqlens), _ptr(cu_cmp),
        batch,
        total, hq, hkv, dk, dv, ck_row_stride, ck_head_stride, cvt.shape[-1], block, stride, pool_kernel,
        pool_stride, pool_pad, max(top_n, 1), max_ns, max(max_ns, 1), int(bool(want_pooled)), float(scale),
        int(bool(causal)), int(idx64), _dtype_code(q), _stream())
    _lib.check(rc, "nsa_cmp_attn_select_fwd")
    return o, idx, (pooled[:, :, 0] if want_pooled else None)


def cmp_select_single_pass(q, hkv, dv, pool_kernel, pool_stride, pool_pad, top_n, max_nc) -> bool:
    """Whether cmp_select runs this shape as one kernel (one pass over the compressed keys)."""
    return bool(_lib.load().nsa_cmp_select_single_pass(q.shape[1], hkv, q.shape[2], dv, pool_kernel, pool_stride,
                                                       pool_pad, top_n, max_nc, _dtype_code(q)))


def cmp_pack(ck, cv, cu_cmp, batch):
    """ck [rows,H,Dk], cv [rows,H,Dv] (row-major, last dim contiguous) -> their fragment-major copy, which the
    one-pass kernel of cmp_select streams: a flat tensor of H * chunks * 64 * (Dk + Dv) elements and `chunks`."""
    _need_cuda(ck, cv, cu_cmp)
    rows, h, dk = ck.shape
    dv = cv.shape[2]
    if ck.stride(2) != 1 or ck.data_ptr() % 16:
        ck = _dense(ck)
    if cv.stride(2) != 1 or cv.data_ptr() % 16:
        cv = _dense(cv)
    lib = _lib.load()
    chunks = lib.nsa_cmp_pack_chunks(rows, batch)
    frag = torch.empty(h * chunks * 64 * (dk + dv), dtype=ck.dtype, device=ck.device)
    rc = lib.nsa_cmp_pack_fwd(_ptr(ck), _ptr(cv), _ptr(frag), _ptr(cu_cmp), batch, rows, h, dk, dv, ck.stride(0),
                              ck.stride(1), cv.stride(0), cv.stride(1), chunks, _dtype_code(ck), _stream())
    _lib.check(rc, "nsa_cmp_pack_fwd")
    return frag, chunks


def cmp_select(q, ck, cvt, cu_seqlens, cu_cmp, batch, hkv, dv, ck_row_stride, ck_head_stride, block, stride,
               pool_kernel, pool_stride, pool_pad, top_n, max_nc, scale, causal=True, idx64=False,
               want_pooled=False, want_lse_attn=False, gate_weight=None, gate_bias=None, single_pass=None,
               frag=None):
    """Compressed attention and block selection in one library call, as the reference's `_attention.forward`
    (nsa/triton_attention.py:419-476).  Returns a dict: o [total,Hq,dv], indices [total,hkv,top_n], and on request
    pooled [total,hkv,Ns], lse_attn [total,Hq] (what the backward reads), gates [total,Hq,3] (the gating Linear on q
    when gate_weight [3,Dk] is given).
    single_pass: None = one kernel when the shape qualifies (cmp_select_single_pass) and `frag` is given, otherwise
    compressed attention, window sums and top-n as three launches; False = always the latter; True = the one kernel
    or an error.  frag: (tensor, chunks) from cmp_pack; cvt may be None when only the one kernel is to run."""
    _need_cuda(q, ck, cu_seqlens, cu_cmp)
    q = _dense(q)
    total, hq, dk = q.shape
    lib = _lib.load()
    max_ns = pool_bins(max_nc, pool_kernel, pool_stride, pool_pad)
    fused = single_pass is not False and frag is not None and cmp_select_single_pass(
        q, hkv, dv, pool_kernel, pool_stride, pool_pad, max(top_n, 1), max_nc)
    frag_t, frag_chunks = frag if frag is not None else (None, 0)
    o = torch.empty(total, hq, dv, dtype=q.dtype, device=q.device)
    idx = torch.empty(total, hkv, top_n, dtype=torch.int64 if idx64 else torch.int32, device=q.device)
    lse_attn = torch.empty(total, hq, dtype=torch.float32, device=q.device) if want_lse_attn else None
    # the one kernel needs neither the importance log-sum-exp nor a hand-over buffer for the window sums
    lse = None if fused else torch.empty(total, hq, dtype=torch.float32, device=q.device)
    pooled = None
    if want_pooled or not fused:
        pooled = torch.empty(total, hkv, head_subgroups(hq, hkv), max(max_ns, 1), dtype=torch.float32, device=q.device)
    w = b = gates = None
    if gate_weight is not None:
        _need_cuda(gate_weight)
        w = _dense(gate_weight.to(q.dtype))
        b = None if gate_bias is None else gate_bias.to(q.dtype).contiguous()
        gates = torch.empty(total, hq, 3, dtype=q.dtype, device=q.device)
    mode = -1 if single_pass is None else int(bool(single_pass))
    rc = lib.nsa_cmp_select_fwd(
        _ptr(q), _ptr(ck), _ptr(cvt), _ptr(frag_t), frag_chunks, _ptr(o), _ptr(idx), _ptr(pooled), _ptr(lse),
        _ptr(lse_attn), _ptr(w), _ptr(b),
        _ptr(gates), _ptr(cu_seqlens), _ptr(cu_cmp), batch, total, hq, hkv, dk, dv, ck_row_stride, ck_head_stride,
        cvt.shape[-1] if cvt is not None else 0, block, stride, pool_kernel, pool_stride, pool_pad, max(top_n, 1), max_nc, max_ns, max(max_ns, 1),
        int(bool(want_pooled)), float(scale), int(bool(causal)), int(idx64), _dtype_code(q), mode, _stream())
    _lib.check(rc, "nsa_cmp_select_fwd")
    return dict(o=o, indices=idx, pooled=pooled[:, :, 0] if want_pooled else None, lse_attn=lse_attn, gates=gates,
                single_pass=fused)


def cmp_attn(q, ck, cvt, cu_seqlens, cu_cmp, batch, hkv, dv, ck_row_stride, ck_head_stride, block, stride, scale,
             causal=True, want_lse_attn=False, gate_weight=None, gate_bias=None):
    """Compressed attention only.  Returns (o [total,Hq,dv], lse float32 [total,Hq]) where lse is the
    log-sum-exp of the raw scores over all compressed rows (what block_select reads); with
    want_lse_attn a third tensor: the log-sum-exp of the scaled visible scores (what the backward reads).
    gate_weight [3,Dk] (+ gate_bias [3]): the same kernel also evaluates the gating Linear on q and the gate
    logits [total,Hq,3] are returned as one more tensor."""
    _need_cuda(q, ck, cvt, cu_seqlens, cu_cmp)
    q = _dense(q)
    total, hq, dk = q.shape
    o = torch.empty(total, hq, dv, dtype=q.dtype, device=q.device)
    lse = torch.empty(total, hq, dtype=torch.float32, device=q.device)
    lse_attn = torch.empty(total, hq, dtype=torch.float32, device=q.device) if want_lse_attn else None
    if gate_weight is not None:
        _need_cuda(gate_weight)
        w = _dense(gate_weight.to(q.dtype))
        b = None if gate_bias is None else gate_bias.to(q.dtype).contiguous()
        gates = torch.empty(total, hq, 3, dtype=q.dtype, device=q.device)
        rc = _lib.load().nsa_cmp_attn_gate_fwd(
            _ptr(q), _ptr(ck), _ptr(cvt), _ptr(o), _ptr(lse), _ptr(lse_attn), _ptr(w), _ptr(b), _ptr(gates),
            _ptr(cu_seqlens), _ptr(cu_cmp), batch, total, hq, hkv, dk, dv, ck_row_stride, ck_head_stride,
            cvt.shape[-1], block, stride, float(scale), int(bool(causal)), _dtype_code(q), _stream())
        _lib.check(rc, "nsa_cmp_attn_gate_fwd")
        return (o, lse, lse_attn, gates) if want_lse_attn else (o, lse, gates)
    rc = _lib.load().nsa_cmp_attn_fwd(_ptr(q), _ptr(ck), _ptr(cvt), _ptr(o), _ptr(lse), _ptr(lse_attn),
                                      _ptr(cu_seqlens), _ptr(cu_cmp), batch, total, hq, hkv, dk, dv, ck_row_stride,
                                      ck_head_stride, cvt.shape[-1], block, stride, float(scale), int(bool(causal)),
                                      _dtype_code(q), _stream())
    _lib.check(rc, "nsa_cmp_attn_fwd")
    return (o, lse, lse_attn) if want_lse_attn else (o, lse)


def block_select(q, ck, lse, cu_seqlens, cu_cmp, batch, hkv, ck_row_stride, ck_head_stride, pool_kernel,
                 pool_stride, pool_pad, top_n, max_nc, idx64=True, want_pooled=False):
    """Block importance + top-n from the lse that cmp_attn wrote.  Returns (indices, pooled or None)."""
    _need_cuda(q, ck, lse, cu_seqlens, cu_cmp)
    q = _dense(q)
    total, hq, dk = q.shape
    max_ns = pool_bins(max_nc, pool_kernel, pool_stride, pool_pad)
    idx = torch.empty(total, hkv, top_n, dtype=torch.int64 if idx64 else torch.int32, device=q.device)
    # always given: with it the library runs its two-kernel schedule (window sums, then top-n); one row per
    # sub-group of 16 heads, the block scores end up in the first row of every kv head
    pooled = torch.empty(total, hkv, head_subgroups(hq, hkv), max(max_ns, 1), dtype=torch.float32, device=q.device)
    rc = _lib.load().nsa_block_select_fwd(_ptr(q), _ptr(ck), _ptr(lse), _ptr(idx), _ptr(pooled), _ptr(cu_seqlens),
                                          _ptr(cu_cmp), batch, total, hq, hkv, dk, ck_row_stride, ck_head_stride,
                                          pool_kernel, pool_stride, pool_pad, top_n, max_ns, max(max_ns, 1),
                                          int(bool(want_pooled)), int(idx64), _dtype_code(q), _stream())
    _lib.check(rc, "nsa_block_select_fwd")
    return idx, (pooled[:, :, 0] if want_pooled else None)


def swa(q, k, vt, cu_seqlens, batch, window, scale, want_lse=False):
    """Sliding-window attention; with want_lse returns (o, lse float32 [total,Hq])."""
    _need_cuda(q, k, vt, cu_seqlens)
    q, k = _dense(q), _dense(k)
    total, hq, dk = q.shape
    hkv, dv = vt.shape[0], vt.shape[1]
    o = torch.empty(total, hq, dv, dtype=q.dtype, device=q.device)
    lse = torch.empty(total, hq, dtype=torch.float32, device=q.device) if want_lse else None
    lib = _lib.load()
    rc = lib.nsa_swa_fwd(_ptr(q), _ptr(k), _ptr(vt), _ptr(o), _ptr(lse), _ptr(cu_seqlens), batch, total, hq, hkv,
                         dk, dv, vt.shape[-1], window, float(scale), _dtype_code(q), _stream())
    _lib.check(rc, "nsa_swa_fwd")
    return (o, lse) if want_lse else o


def _gate_views(gates, q):
    """gates: list of [total, Hq] tensors or None.  Returns (tensors, common element stride)."""
    live = [g for g in gates if g is not None]
    if not live:
        return gates, 1
    hq = q.shape[1]
    s = live[0].stride(-1) if live[0].dim() == 2 else 0
    ok = all(g.dim() == 2 and g.dtype == q.dtype and g.stride(1) == s and g.stride(0) == hq * s and s > 0
             and g.data_ptr() % g.element_size() == 0 for g in live)
    if ok:
        return gates, s
    return [None if g is None else g.to(q.dtype).contiguous() for g in gates], 1


# Bytes the block-major selected attention may take for its pair list and partial results in one piece (8.3 GiB at
# 32768 tokens x 4 kv heads x 16 picks); beyond, the fused schedule walks the tokens in slabs of this size.
SLC_WORKSPACE_LIMIT = int(os.environ.get("NSA_SLC_WORKSPACE_LIMIT", 16 << 30))


def slc_combine(q, k, vt, indices, counts, g_slc, g_swa, g_cmp, o_swa, o_cmp, cu_seqlens, batch, block_size,
                scale, gate_act=0, block_major=None, want_lse=False):
    """block_major: None = use the block-major schedule when the shape has one and its workspace
    fits SLC_WORKSPACE_LIMIT; False = token-major kernel; True = require block-major.
    want_lse (block-major only): returns (out, lse float32 [total,Hq] of the selected branch)."""
    _need_cuda(q, k, vt, indices, cu_seqlens)
    q, k = _dense(q), _dense(k)
    total, hq, dk = q.shape
    hkv, dv = vt.shape[0], vt.shape[1]
    if indices.dtype not in (torch.int32, torch.int64):
        raise TypeError("block indices must be int32 or int64")
    indices = indices.contiguous()
    top_n = indices.shape[-1]
    if counts is not None:
        counts = counts.to(torch.int32).contiguous()
    (g_slc, g_swa, g_cmp), gs = _gate_views([g_slc, g_swa, g_cmp], q)
    o_swa = None if o_swa is None else _dense(o_swa)
    o_cmp = None if o_cmp is None else _dense(o_cmp)
    out = torch.empty(total, hq, dv, dtype=q.dtype, device=q.device)
    lse = torch.empty(total, hq, dtype=torch.float32, device=q.device) if want_lse else None
    lib = _lib.load()
    ws, ws_bytes = None, 0
    if block_major is not False:
        need = lib.nsa_slc_workspace_bytes(total, batch, hkv * head_subgroups(hq, hkv), dk, dv, top_n, block_size,
                                           _dtype_code(q))
        if need > 0 and (block_major or need <= SLC_WORKSPACE_LIMIT):
            ws = torch.empty(need, dtype=torch.uint8, device=q.device)
            ws_bytes = need
        elif block_major:
            raise NotImplementedError("no block-major selected attention for this shape / dtype")
    rc = lib.nsa_slc_combine_fwd(
        _ptr(q), _ptr(k), _ptr(vt), _ptr(indices), _ptr(counts), _ptr(g_slc), _ptr(g_swa), _ptr(g_cmp), gs,
        _ptr(o_swa), _ptr(o_cmp), _ptr(out), _ptr(lse), _ptr(cu_seqlens), batch, total, hq, hkv, dk, dv,
        vt.shape[-1], top_n, block_size, float(scale), int(indices.dtype == torch.int64), gate_act, _dtype_code(q),
        _ptr(ws), ws_bytes, _stream())
    _lib.check(rc, "nsa_slc_combine_fwd")
    return (out, lse) if want_lse else out


def slc_workspace(q, hkv, dv, top_n, block_size, batch):
    """Workspace tensor of the block-major selected attention, or None when the shape has none."""
    total, hq, dk = q.shape
    need = _lib.load().nsa_slc_swa_fused_workspace_bytes(total, batch, hq, hkv, dk, dv, top_n, block_size,
                                                         _dtype_code(q), 0)
    if need <= 0 or need > SLC_WORKSPACE_LIMIT:
        return None
    return torch.empty(need, dtype=torch.uint8, device=q.device)


def slc_partials(q, k, vt, indices, counts, cu_seqlens, batch, block_size, scale, workspace):
    """First half of the fused schedule: one partial softmax state per (token, pick) into `workspace`."""
    _need_cuda(q, k, vt, indices, cu_seqlens, workspace)
    q, k = _dense(q), _dense(k)
    total, hq, dk = q.shape
    hkv, dv = vt.shape[0], vt.shape[1]
    if indices.dtype not in (torch.int32, torch.int64):
        raise TypeError("block indices must be int32 or int64")
    indices = indices.contiguous()
    if counts is not None:
        counts = counts.to(torch.int32).contiguous()
    rc = _lib.load().nsa_slc_partials_fwd(
        _ptr(q), _ptr(k), _ptr(vt), _ptr(indices), _ptr(counts), _ptr(cu_seqlens), batch, total, hq, hkv, dk, dv,
        vt.shape[-1], indices.shape[-1], block_size, float(scale), int(indices.dtype == torch.int64),
        _dtype_code(q), _ptr(workspace), workspace.numel(), _stream())
    _lib.check(rc, "nsa_slc_partials_fwd")
    return workspace


def swa_merge(q, k, vt, workspace, top_n, g_slc, g_swa, g_cmp, o_cmp, cu_seqlens, batch, block_size, window,
              scale, gate_act=0, want_branches=False):
    """Second half: sliding-window attention whose epilogue merges the partials slc_partials left in
    `workspace` (same sizes, top_n picks per token and kv head), applies the gates and adds the
    compressed branch.  Returns the final output [total,Hq,dv]; with want_branches also what a backward
    pass keeps: (out, o_slc, o_swa, lse_slc, lse_swa), the ungated branch outputs and their float32
    [total,Hq] log-sum-exps."""
    _need_cuda(q, k, vt, cu_seqlens, workspace)
    q, k = _dense(q), _dense(k)
    total, hq, dk = q.shape
    hkv, dv = vt.shape[0], vt.shape[1]
    (g_slc, g_swa, g_cmp), gs = _gate_views([g_slc, g_swa, g_cmp], q)
    o_cmp = None if o_cmp is None else _dense(o_cmp)
    out = torch.empty(total, hq, dv, dtype=q.dtype, device=q.device)
    o_slc = o_swa = lse_slc = lse_swa = None
    if want_branches:
        o_slc, o_swa = torch.empty_like(out), torch.empty_like(out)
        lse_slc = torch.empty(total, hq, dtype=torch.float32, device=q.device)
        lse_swa = torch.empty_like(lse_slc)
    rc = _lib.load().nsa_swa_merge_fwd(
        _ptr(q), _ptr(k), _ptr(vt), _ptr(g_slc), _ptr(g_swa), _ptr(g_cmp), gs, _ptr(o_cmp), _ptr(out),
        _ptr(cu_seqlens), batch, total, hq, hkv, dk, dv, vt.shape[-1], window, top_n, block_size, float(scale),
        gate_act, _dtype_code(q), _ptr(o_slc), _ptr(o_swa), _ptr(lse_slc), _ptr(lse_swa), _ptr(workspace),
        workspace.numel(), _stream())
    _lib.check(rc, "nsa_swa_merge_fwd")
    return (out, o_slc, o_swa, lse_slc, lse_swa) if want_branches else out


def slc_swa_fused(q, k, vt, indices, counts, g_slc, g_swa, g_cmp, o_cmp, cu_seqlens, batch, block_size, window, scale,
                  gate_act=0, want_branches=False, workspace_limit=None):
    """slc_partials + swa_merge as one call that walks the tokens in slabs sized to a workspace of at most
    workspace_limit bytes (default SLC_WORKSPACE_LIMIT): what a context too long for the one-slab workspace
    runs.  Returns as swa_merge; None when the shape has no block-major schedule."""
    _need_cuda(q, k, vt, indices, cu_seqlens)
    q, k = _dense(q), _dense(k)
    total, hq, dk = q.shape
    hkv, dv = vt.shape[0], vt.shape[1]
    if indices.dtype not in (torch.int32, torch.int64):
        raise TypeError("block indices must be int32 or int64")
    indices = indices.contiguous()
    top_n = indices.shape[-1]
    if counts is not None:
        counts = counts.to(torch.int32).contiguous()
    lib = _lib.load()
    limit = SLC_WORKSPACE_LIMIT if workspace_limit is None else int(workspace_limit)
    geom = (total, batch, hq, hkv, dk, dv, top_n, block_size, _dtype_code(q))
    need = lib.nsa_slc_swa_fused_workspace_bytes(*geom, 0)
    if need <= 0:
        return None
    if need > limit:        # the entry point takes the largest slab these bytes hold; one tile is the least
        need = max(limit, lib.nsa_slc_swa_fused_workspace_bytes(*geom, 1))
    ws = torch.empty(need, dtype=torch.uint8, device=q.device)
    (g_slc, g_swa, g_cmp), gs = _gate_views([g_slc, g_swa, g_cmp], q)
    o_cmp = None if o_cmp is None else _dense(o_cmp)
    out = torch.empty(total, hq, dv, dtype=q.dtype, device=q.device)
    o_slc = o_swa = lse_slc = lse_swa = None
    if want_branches:
        o_slc, o_swa = torch.empty_like(out), torch.empty_like(out)
        lse_slc = torch.empty(total, hq, dtype=torch.float32, device=q.device)
        lse_swa = torch.empty_like(lse_slc)
    rc = lib.nsa_slc_swa_fused_fwd(
        _ptr(q), _ptr(k), _ptr(vt), _ptr(indices), _ptr(counts), _ptr(g_slc), _ptr(g_swa), _ptr(g_cmp), gs,
        _ptr(o_cmp), _ptr(out), _ptr(cu_seqlens), batch, total, hq, hkv, dk, dv, vt.shape[-1], window, top_n,
        block_size, float(scale), int(indices.dtype == torch.int64), gate_act, _dtype_code(q), _ptr(o_slc),
        _ptr(o_swa), _ptr(lse_slc), _ptr(lse_swa), _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "nsa_slc_swa_fused_fwd")
    return (out, o_slc, o_swa, lse_slc, lse_swa) if want_branches else out


def gate_logits(q, weight, bias=None):
    """q [total,Hq,D], weight [3,D], bias [3] -> gate logits [total,Hq,3] (selected, sliding, compressed)."""
    _need_cuda(q, weight)
    q = _dense(q)
    total, hq, dim = q.shape
    weight = weight.to(q.dtype).contiguous()
    bias = None if bias is None else bias.to(q.dtype).contiguous()
    out = torch.empty(total, hq, 3, dtype=q.dtype, device=q.device)
    rc = _lib.load().nsa_gate_fwd(_ptr(q), _ptr(weight), _ptr(bias), _ptr(out), total * hq, dim, _dtype_code(q),
                                  _stream())
    _lib.check(rc, "nsa_gate_fwd")
    return out


def _subgroup(t, hkv, rep, r):
    """Heads of sub-group r (16 of the rep * 16 query heads of every kv head) of a [total, Hq, ...] tensor, as a
    contiguous [total, hkv * 16, ...] tensor."""
    if t is None:
        return None
    return t.reshape(t.shape[0], hkv, rep, 16, *t.shape[2:])[:, :, r].reshape(t.shape[0], hkv * 16, *t.shape[2:]).contiguous()


def cmp_attn_bwd(q, ck, cv, o, d_o, lse_attn, cu_seqlens, cu_cmp, batch, block, stride, scale, causal=True,
                 delta=None, rowscale=None):
    """Backward of the compressed attention.  q [total,Hq,Dk], ck [rows,Hkv,Dk], cv [rows,Hkv,Dv]
    (packed over cu_cmp), o / d_o [total,Hq,Dv], lse_attn from cmp_attn(want_lse_attn=True).
    delta (float32 [total,Hq]) = rowsum(o*d_o) if already known (o may then be None); rowscale (float32
    [total,Hq]) = a per-row gate applied to d_o inside the kernels.  Returns (dq, dck, dcv)."""
    _need_cuda(q, ck, cv, d_o, lse_attn, cu_seqlens, cu_cmp)
    rep = head_subgroups(q.shape[1], cv.shape[1])
    if rep > 1:
        # groups of 32, 48, 64 ... heads: one call per sub-group of 16 heads (they share ck / cv, so the key
        # gradients of the calls add up; summed in float32, rounded once)
        hkv = cv.shape[1]
        dq = torch.empty_like(q).view(q.shape[0], hkv, rep, 16, q.shape[2])
        dck = torch.zeros(ck.shape, dtype=torch.float32, device=q.device)
        dcv = torch.zeros(cv.shape, dtype=torch.float32, device=q.device)
        for r in range(rep):
            part = cmp_attn_bwd(_subgroup(q, hkv, rep, r), ck, cv, _subgroup(o, hkv, rep, r), _subgroup(d_o, hkv, rep, r),
                                _subgroup(lse_attn, hkv, rep, r), cu_seqlens, cu_cmp, batch, block, stride, scale,
                                causal=causal, delta=_subgroup(delta, hkv, rep, r),
                                rowscale=_subgroup(rowscale, hkv, rep, r))
            dq[:, :, r] = part[0].view(q.shape[0], hkv, 16, q.shape[2])
            dck += part[1]
            dcv += part[2]
        return dq.view(q.shape), dck.to(ck.dtype), dcv.to(cv.dtype)
    q, ck, cv, d_o = (_dense(t) for t in (q, ck, cv, d_o))
    o = None if o is None else _dense(o)
    total, hq, dk = q.shape
    rows, hkv, dv = cv.shape
    dq, dck, dcv = torch.empty_like(q), torch.empty_like(ck), torch.empty_like(cv)
    lib = _lib.load()
    need = lib.nsa_cmp_attn_bwd_workspace_bytes(total, rows, hq, hkv, dk, dv)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    rc = lib.nsa_cmp_attn_bwd(_ptr(q), _ptr(ck), _ptr(cv), _ptr(o), _ptr(d_o), _ptr(lse_attn), _ptr(delta),
                              _ptr(rowscale), _ptr(cu_seqlens), _ptr(cu_cmp), batch, total, rows, hq, hkv, dk, dv, block, stride, float(scale),
                              int(bool(causal)), _dtype_code(q), _ptr(dq), _ptr(dck), _ptr(dcv), _ptr(ws),
                              ws.numel(), _stream())
    _lib.check(rc, "nsa_cmp_attn_bwd")
    return dq, dck, dcv


def slc_swa_bwd(q, k, v, o_slc, d_o_slc, lse_slc, o_swa, d_o_swa, lse_swa, indices, counts, cu_seqlens, batch,
                block_size, window, scale, delta_slc=None, delta_swa=None, rowscale_slc=None, rowscale_swa=None,
                dq_add=None):
    """Backward of the selected (o_slc / d_o_slc / lse_slc, or None) and sliding (o_swa / d_o_swa /
    lse_swa, or None) branches.  v is the row-major [total,Hkv,Dv] tensor.  delta_* / rowscale_* as in
    cmp_attn_bwd (with delta_* the matching o_* may be None).  dq_add (optional, shape of q): added to dq
    by the kernel that writes it (the compressed branch's dq).  Returns (dq, dk, dv), each the sum over
    the branches given."""
    _need_cuda(q, k, v, cu_seqlens)
    rep = head_subgroups(q.shape[1], v.shape[1])
    if rep > 1:
        hkv = v.shape[1]
        sub = lambda t, r: _subgroup(t, hkv, rep, r)     # noqa: E731
        dq = torch.empty_like(q).view(q.shape[0], hkv, rep, 16, q.shape[2])
        dk_sum = torch.zeros(k.shape, dtype=torch.float32, device=q.device)
        dv_sum = torch.zeros(v.shape, dtype=torch.float32, device=q.device)
        for r in range(rep):
            part = slc_swa_bwd(sub(q, r), k, v, sub(o_slc, r), sub(d_o_slc, r), sub(lse_slc, r), sub(o_swa, r),
                               sub(d_o_swa, r), sub(lse_swa, r), indices, counts, cu_seqlens, batch, block_size, window,
                               scale, delta_slc=sub(delta_slc, r), delta_swa=sub(delta_swa, r),
                               rowscale_slc=sub(rowscale_slc, r), rowscale_swa=sub(rowscale_swa, r),
                               dq_add=sub(dq_add, r))
            dq[:, :, r] = part[0].view(q.shape[0], hkv, 16, q.shape[2])
            dk_sum += part[1]
            dv_sum += part[2]
        return dq.view(q.shape), dk_sum.to(k.dtype), dv_sum.to(v.dtype)
    q, k, v = _dense(q), _dense(k), _dense(v)
    total, hq, dk = q.shape
    hkv, dv = v.shape[1], v.shape[2]
    slc, swa_ = d_o_slc is not None, d_o_swa is not None
    top_n = 0
    if slc:
        if indices.dtype not in (torch.int32, torch.int64):
            raise TypeError("block indices must be int32 or int64")
        indices = indices.contiguous()
        top_n = indices.shape[-1]
        counts = None if counts is None else counts.to(torch.int32).contiguous()
        o_slc, d_o_slc = (None if o_slc is None else _dense(o_slc)), _dense(d_o_slc)
    if swa_:
        o_swa, d_o_swa = (None if o_swa is None else _dense(o_swa)), _dense(d_o_swa)
    dq, dk_out, dv_out = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    if dq_add is not None:
        if dq_add.shape != q.shape or dq_add.dtype != q.dtype:
            raise ValueError("dq_add must have the shape and dtype of q")
        dq_add = _dense(dq_add)
    lib = _lib.load()
    geom = (total, batch, hq, hkv, dk, dv, top_n, block_size, _dtype_code(q))
    need = lib.nsa_slc_swa_bwd_workspace_bytes(*geom)
    if need > SLC_WORKSPACE_LIMIT:      # token slabs: the call takes the largest slab these bytes hold
        need = max(SLC_WORKSPACE_LIMIT, lib.nsa_slc_swa_bwd_slab_workspace_bytes(*geom, 1))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    rc = lib.nsa_slc_swa_bwd(
        _ptr(q), _ptr(k), _ptr(v), _ptr(o_slc if slc else None), _ptr(o_swa if swa_ else None),
        _ptr(d_o_slc if slc else None), _ptr(d_o_swa if swa_ else None), _ptr(lse_slc if slc else None),
        _ptr(lse_swa if swa_ else None), _ptr(delta_slc if slc else None), _ptr(delta_swa if swa_ else None),
        _ptr(rowscale_slc if slc else None), _ptr(rowscale_swa if swa_ else None),
        _ptr(indices if slc else None), _ptr(counts if slc else None),
        _ptr(cu_seqlens), batch, total, hq, hkv, dk, dv, top_n, block_size, window if swa_ else 0, float(scale),
        int(slc and indices.dtype == torch.int64), _dtype_code(q), _ptr(dq_add), _ptr(dq), _ptr(dk_out), _ptr(dv_out),
        _ptr(ws),
        ws.numel(), _stream())
    _lib.check(rc, "nsa_slc_swa_bwd")
    return dq, dk_out, dv_out


def compress_bwd(d_out, cu_seqlens, cu_out, total, block, stride, x=None, w_lin=None, want_dw=True,
                 want_dbias=False):
    """Backward of compress().  d_out [rows, H, D].  Mean pooling: w_lin None -> returns dx.  Weighted:
    w_lin [block*D, D] (row j*D+i, column o), x the forward input -> (dx, dw float32 or None,
    dbias float32 or None)."""
    _need_cuda(d_out, cu_seqlens, cu_out)
    d_out = _dense(d_out)
    rows, H, D = d_out.shape
    dx = torch.empty(total, H, D, dtype=d_out.dtype, device=d_out.device)
    dw = dbias = None
    if w_lin is not None:
        w_lin = _dense(w_lin.to(d_out.dtype))
        if tuple(w_lin.shape) != (block * D, D):
            raise ValueError("weight must be [block*dim, dim], got %s" % (tuple(w_lin.shape),))
        if want_dw:
            x = _dense(x)
            dw = torch.empty(block * D, D, dtype=torch.float32, device=d_out.device)
        if want_dbias:
            dbias = torch.empty(D, dtype=torch.float32, device=d_out.device)
    if rows == 0:
        dx.zero_()
        for t in (dw, dbias):
            if t is not None:
                t.zero_()
    else:
        rc = _lib.load().nsa_compress_bwd(_ptr(x if dw is not None else None), _ptr(w_lin), _ptr(d_out), _ptr(dx),
                                          _ptr(dw), _ptr(dbias), _ptr(cu_seqlens), _ptr(cu_out),
                                          cu_seqlens.numel() - 1, total, rows, H, D, block, stride,
                                          _dtype_code(d_out), _stream())
        _lib.check(rc, "nsa_compress_bwd")
    return dx if w_lin is None else (dx, dw, dbias)


def gate_bwd(q, weight, d_gates, want_dbias=True):
    """Backward of gate_logits: returns (dq [total,Hq,D], dweight float32 [3,D], dbias float32 [3] or None)."""
    _need_cuda(q, weight, d_gates)
    q = _dense(q)
    total, hq, dim = q.shape
    weight = weight.to(q.dtype).contiguous()
    d_gates = d_gates.to(q.dtype).contiguous()
    dq = torch.empty_like(q)
    dw = torch.empty(3, dim, dtype=torch.float32, device=q.device)
    db = torch.empty(3, dtype=torch.float32, device=q.device) if want_dbias else None
    rc = _lib.load().nsa_gate_bwd(_ptr(q), _ptr(weight), _ptr(d_gates), _ptr(dq), _ptr(dw), _ptr(db), total * hq, dim,
                                  _dtype_code(q), _stream())
    _lib.check(rc, "nsa_gate_bwd")
    return dq, dw, db


def gate_combine(gate_logits, o_slc, o_swa, o_cmp, gate_act=0):
    """out = sum_b act(gate_logits[..., b]) * o_b over (selected, sliding, compressed); o_swa / o_cmp may be None."""
    _need_cuda(gate_logits, o_slc)
    gl = _dense(gate_logits.to(o_slc.dtype))
    o_slc = _dense(o_slc)
    o_swa = None if o_swa is None else _dense(o_swa)
    o_cmp = None if o_cmp is None else _dense(o_cmp)
    total, hq, dv = o_slc.shape
    out = torch.empty_like(o_slc)
    rc = _lib.load().nsa_gate_combine_fwd(_ptr(gl), _ptr(o_slc), _ptr(o_swa), _ptr(o_cmp), _ptr(out), total * hq, dv,
                                          gate_act, _dtype_code(o_slc), _stream())
    _lib.check(rc, "nsa_gate_combine_fwd")
    return out


def gate_combine_bwd(gate_logits, d_out, o_slc, o_swa, o_cmp, gate_act=0, want_scaled=True, want_stats=False):
    """Returns (d_o_slc, d_o_swa or None, d_o_cmp or None, d_gate_logits [total,Hq,3]) and, with want_stats,
    a fifth tensor float32 [6, total, Hq]: <d_out, o_b> for b = selected, sliding, compressed, then the
    activated gates (the delta / rowscale inputs of the attention backward).  want_scaled=False skips the
    scaled copies (they come back as None)."""
    _need_cuda(gate_logits, d_out, o_slc)
    gl = _dense(gate_logits.to(o_slc.dtype))
    d_out, o_slc = _dense(d_out), _dense(o_slc)
    o_swa = None if o_swa is None else _dense(o_swa)
    o_cmp = None if o_cmp is None else _dense(o_cmp)
    total, hq, dv = o_slc.shape
    if not (want_scaled or want_stats):
        raise ValueError("gate_combine_bwd: nothing requested")
    d_slc = torch.empty_like(o_slc) if want_scaled else None
    d_swa = None if o_swa is None or not want_scaled else torch.empty_like(o_slc)
    d_cmp = None if o_cmp is None or not want_scaled else torch.empty_like(o_slc)
    d_gl = torch.empty(total, hq, 3, dtype=o_slc.dtype, device=o_slc.device)
    stats = torch.empty(6, total, hq, dtype=torch.float32, device=o_slc.device) if want_stats else None
    rc = _lib.load().nsa_gate_combine_bwd(_ptr(gl), _ptr(d_out), _ptr(o_slc), _ptr(o_swa), _ptr(o_cmp), _ptr(d_slc),
                                          _ptr(d_swa), _ptr(d_cmp), _ptr(d_gl), _ptr(stats), total * hq, dv, gate_act,
                                          _dtype_code(o_slc), _stream())
    _lib.check(rc, "nsa_gate_combine_bwd")
    return (d_slc, d_swa, d_cmp, d_gl, stats) if want_stats else (d_slc, d_swa, d_cmp, d_gl)


def _qkv_rope(packed, q, k, v, gates, offsets, inv_freq, positions, cu_seqlens, rope_off, rope_dim, interleaved,
              pack):
    total, hq, dk = q.shape
    hkv, dv = v.shape[1], v.shape[2]
    q_off, k_off, v_off, g_off = offsets
    batch = 0 if cu_seqlens is None else cu_seqlens.numel() - 1
    rc = _lib.load().nsa_qkv_rope(_ptr(packed), _ptr(q), _ptr(k), _ptr(v), _ptr(gates), _ptr(inv_freq),
                                  _ptr(positions), _ptr(cu_seqlens), batch, total, packed.shape[1], q_off, k_off,
                                  v_off, g_off, hq, hkv, dk, dv, rope_off, rope_dim, int(bool(interleaved)),
                                  int(pack), _dtype_code(packed), _stream())
    _lib.check(rc, "nsa_qkv_rope")


def _rope_operands(inv_freq, positions, cu_seqlens, ref):
    if inv_freq is not None:
        inv_freq = inv_freq.to(device=ref.device, dtype=torch.float32).contiguous()
        if positions is not None:
            positions = positions.to(device=ref.device, dtype=torch.int32).contiguous()
        elif cu_seqlens is None:
            raise ValueError("a rotation needs positions or cu_seqlens")
    if cu_seqlens is not None:
        cu_seqlens = cu_seqlens.to(device=ref.device, dtype=torch.int32).contiguous()
    return inv_freq, positions, cu_seqlens


def qkv_rope_split(packed, hq, hkv, dk, dv, offsets, inv_freq=None, positions=None, cu_seqlens=None, rope_off=0,
                   rope_dim=0, interleaved=False, with_gates=True):
    """packed [total, ld] (a projection GEMM's output: q, k, v and 3*hq gate-logit columns at the
    element offsets (q_off, k_off, v_off, g_off)) -> q [total,hq,dk], k [total,hkv,dk], v
    [total,hkv,dv], gates [total,hq,3] or None; channels [rope_off, rope_off+rope_dim) of every q and
    k head are rotated by position * inv_freq[i] (positions int32 [total], or the offset inside the
    sequence from cu_seqlens)."""
    _need_cuda(packed)
    packed = _dense(packed)
    total = packed.shape[0]
    inv_freq, positions, cu_seqlens = _rope_operands(inv_freq, positions, cu_seqlens, packed)
    z = dict(dtype=packed.dtype, device=packed.device)
    q, k, v = torch.empty(total, hq, dk, **z), torch.empty(total, hkv, dk, **z), torch.empty(total, hkv, dv, **z)
    gates = torch.empty(total, hq, 3, **z) if with_gates else None
    _qkv_rope(packed, q, k, v, gates, offsets, inv_freq, positions, cu_seqlens, rope_off, rope_dim, interleaved, 0)
    return q, k, v, gates


def qkv_rope_pack(dq, dk_, dv_, dgates, ld, offsets, inv_freq=None, positions=None, cu_seqlens=None, rope_off=0,
                  rope_dim=0, interleaved=False):
    """Transpose of qkv_rope_split: gradients of q, k, v (and gate logits, or None) -> gradient of the
    packed rows [total, ld] (columns outside the four ranges are zero), inverse rotation applied."""
    _need_cuda(dq, dk_, dv_)
    dq, dk_, dv_ = _dense(dq), _dense(dk_), _dense(dv_)
    dgates = None if dgates is None else _dense(dgates)
    inv_freq, positions, cu_seqlens = _rope_operands(inv_freq, positions, cu_seqlens, dq)
    total, hq, dk = dq.shape
    hkv, dv = dv_.shape[1], dv_.shape[2]
    covered = hq * dk + hkv * dk + hkv * dv + (0 if dgates is None else 3 * hq)
    alloc = torch.empty if covered == ld else torch.zeros
    packed = alloc(total, ld, dtype=dq.dtype, device=dq.device)
    _qkv_rope(packed, dq, dk_, dv_, dgates, offsets, inv_freq, positions, cu_seqlens, rope_off, rope_dim,
              interleaved, 1)
    return packed
