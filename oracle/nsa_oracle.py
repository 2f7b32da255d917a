"""CPU oracle for the Native Sparse Attention forward path.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain torch on the CPU, the algorithm of the reference's
naive path.  It is the checker for the HIP kernels: only tests, the smoke check
and the benchmark's cpu_baseline leg may import it.  The shipped package never
does, and fails loudly when its HIP library is missing.

Reference lines each function follows (paths inside the reference tree):

  compressed_len_conv / compressed_len_functional
        nsa/compression_kv.py:292-312 (Conv1d output count), :9-10 (functional count)
  compress_weighted / compress_meanpool
        nsa/compression_kv.py:26-57 (windowed matmul, weight [l*D, D]),
        :298-307 (Conv1d with bias); tests/test_compression_kv.py:28-42
  pool_geometry / pool_scores
        nsa/torch_attention.py:51-58 (sum over the GQA group, avg_pool1d, ceil_mode=True);
        pool parameters nsa/nsa.py:57-59
  importance_scores / select_blocks
        nsa/torch_attention.py:121-125 (softmax of the *unscaled, unmasked* q.ck),
        :59-60 (topk, [B,T,Hkv,S])
  compressed_attention
        nsa/torch_attention.py:41 (block c is hidden from row t iff c*d + l > t),
        :126-160 (scale, mask, softmax, rows with nothing visible -> 0, PV)
  selected_attention / sliding_attention
        tests/test_parallel_nsa.py:115-156 (token ids of a block, mask i<0 | i>t | c>=count,
        window [max(0,t-W+1), t]); empty selection -> 0 as nsa/selection_attn.py:451-481
  gated_combine
        nsa/selection_attn.py:808-811 and nsa/nsa.py:133
  nsa_forward
        nsa/nsa.py:90-135

How it is pinned (tests/test_oracle_*.py, none of which retypes these formulas):
  compress_*          F.conv1d with permuted weights; unfold().mean(); triple loop
  pool_*              torch.nn.functional.avg_pool1d(ceil_mode=True); sum(imp) == G
  compressed_attention F.scaled_dot_product_attention with a boolean mask; rows t<l are 0
  selected/sliding    all blocks selected == causal SDPA; W>=T == causal SDPA; S=0 == banded
                      SDPA; per-token python loop on tiny inputs
  varlen              packed == concatenation of per-sequence runs
  decode              == last row of the prefill result
No function here is "parity unpinned".

Precision model: inputs (bf16 or fp32) are upcast once; every sum, softmax and
comparison runs in `math_dtype` (fp32 by default, fp64 for pinning); ck/cv are
rounded to the input dtype where the reference materialises them; the final
output is rounded once.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch


# ----------------------------------------------------------------------------- counts

def compressed_len_conv(T: int, block: int, stride: int) -> int:
    """Rows produced by a Conv1d(kernel=block, stride=stride) over T tokens."""
    return 0 if T < block else (T - block) // stride + 1


def compressed_len_functional(T: int, block: int, stride: int) -> int:
    """Row count of the varlen functional compressor: one fewer than the Conv1d count."""
    return max((T - block) // stride, 0)


# ----------------------------------------------------------------------------- compression

def compress_weighted(x: torch.Tensor, w_lin: torch.Tensor, bias: Optional[torch.Tensor],
                      block: int, stride: int, n_out: int,
                      math_dtype=torch.float32, out_dtype=None) -> torch.Tensor:
    """x [T,H,D], w_lin [block*D, Do] with row index j*D+i -> out [n_out,H,Do].

    out[n,h,o] = bias[o] + sum_j sum_i x[n*stride+j, h, i] * w_lin[j*D+i, o]
    """
    T, H, D = x.shape
    Do = w_lin.shape[1]
    out_dtype = out_dtype or x.dtype
    xm = x.to(math_dtype)
    wm = w_lin.to(math_dtype).reshape(block, D, Do)
    out = torch.zeros(n_out, H, Do, dtype=math_dtype)
    for j in range(block):
        rows = xm[j: j + (n_out - 1) * stride + 1: stride] if n_out > 0 else xm[:0]
        out += torch.einsum("nhi,io->nho", rows, wm[j])
    if bias is not None:
        out += bias.to(math_dtype)
    return out.to(out_dtype)


def compress_meanpool(x: torch.Tensor, block: int, stride: int, n_out: int,
                      math_dtype=torch.float32, out_dtype=None) -> torch.Tensor:
    """Mean over each window of `block` rows: the weighted compressor with eye/block weights."""
    T, H, D = x.shape
    out_dtype = out_dtype or x.dtype
    xm = x.to(math_dtype)
    out = torch.zeros(n_out, H, D, dtype=math_dtype)
    for j in range(block):
        if n_out > 0:
            out += xm[j: j + (n_out - 1) * stride + 1: stride]
    return (out / block).to(out_dtype)


# ----------------------------------------------------------------------------- pooling

def pool_geometry(Nc: int, kernel: int, stride: int, pad: int) -> Tuple[int, torch.Tensor]:
    """Number of pooled bins and the divisor of each (ceil_mode, padding counted in the divisor)."""
    if Nc + 2 * pad < kernel:
        return 0, torch.zeros(0)
    Ns = -(-(Nc + 2 * pad - kernel) // stride) + 1
    if (Ns - 1) * stride >= Nc + pad:
        Ns -= 1
    div = torch.empty(Ns)
    for j in range(Ns):
        start = j * stride - pad
        end = min(start + kernel, Nc + pad)
        div[j] = end - start
    return Ns, div


def pool_scores(imp: torch.Tensor, kernel: int, stride: int, pad: int) -> torch.Tensor:
    """imp [..., Nc] -> pooled [..., Ns]: window j covers columns [j*stride-pad, j*stride-pad+kernel)."""
    Nc = imp.shape[-1]
    Ns, div = pool_geometry(Nc, kernel, stride, pad)
    csum = torch.zeros(*imp.shape[:-1], Nc + 1, dtype=imp.dtype)
    csum[..., 1:] = imp.cumsum(-1)
    lo = torch.tensor([min(max(j * stride - pad, 0), Nc) for j in range(Ns)])
    hi = torch.tensor([min(max(j * stride - pad + kernel, 0), Nc) for j in range(Ns)])
    return (csum[..., hi] - csum[..., lo]) / div.to(imp.dtype)


def pool_scores_direct(imp: torch.Tensor, kernel: int, stride: int, pad: int) -> torch.Tensor:
    """Same as pool_scores without the prefix-sum (no cancellation); slower."""
    Nc = imp.shape[-1]
    Ns, div = pool_geometry(Nc, kernel, stride, pad)
    out = torch.zeros(*imp.shape[:-1], Ns, dtype=imp.dtype)
    for j in range(Ns):
        lo = max(j * stride - pad, 0)
        hi = min(j * stride - pad + kernel, Nc)
        if hi > lo:
            out[..., j] = imp[..., lo:hi].sum(-1)
    return out / div.to(imp.dtype)


# ----------------------------------------------------------------------------- compressed branch

def _group(hq: int, hkv: int) -> int:
    assert hq % hkv == 0
    return hq // hkv


def _row_chunks(T: int, rows: Optional[torch.Tensor], chunk: int):
    """Yields (positions in the output, token indices) for all rows or for the subset `rows`."""
    ids = torch.arange(T) if rows is None else rows.to(torch.int64)
    for i in range(0, ids.numel(), chunk):
        yield slice(i, min(i + chunk, ids.numel())), ids[i:i + chunk]


def importance_scores(q: torch.Tensor, ck: torch.Tensor, kernel: int, stride: int, pad: int,
                      math_dtype=torch.float32, row_chunk: int = 1024, rows=None) -> torch.Tensor:
    """q [T,Hq,D], ck [Nc,Hkv,D] -> pooled block scores [T,Hkv,Ns] (or [len(rows),Hkv,Ns]).

    p = softmax over ALL Nc columns of the raw q.ck (no scale, no causal mask), summed
    over the G query heads of each kv head, then average-pooled.
    """
    T, Hq, D = q.shape
    Nc, Hkv, _ = ck.shape
    G = _group(Hq, Hkv)
    Ns, _ = pool_geometry(Nc, kernel, stride, pad)
    ckm = ck.to(math_dtype)
    n_out = T if rows is None else len(rows)
    out = torch.zeros(n_out, Hkv, Ns, dtype=math_dtype)
    for pos, ids in _row_chunks(T, rows, row_chunk):
        qm = q[ids].to(math_dtype).reshape(-1, Hkv, G, D)
        s = torch.einsum("thgd,chd->thgc", qm, ckm)
        p = torch.softmax(s, dim=-1).sum(2)                       # [t,Hkv,Nc]
        out[pos] = pool_scores_direct(p, kernel, stride, pad)
    return out


def select_blocks(pooled: torch.Tensor, top_n: int) -> torch.Tensor:
    """pooled [T,Hkv,Ns] -> int64 [T,Hkv,top_n], descending score; -1 pads when Ns < top_n."""
    T, Hkv, Ns = pooled.shape
    n = min(top_n, Ns)
    idx = torch.full((T, Hkv, top_n), -1, dtype=torch.int64)
    if n > 0:
        idx[..., :n] = torch.topk(pooled, n, dim=-1).indices
    return idx


def compressed_attention(q: torch.Tensor, ck: torch.Tensor, cv: torch.Tensor, block: int,
                         stride: int, scale: Optional[float] = None,
                         math_dtype=torch.float32, row_chunk: int = 1024, rows=None) -> torch.Tensor:
    """q [T,Hq,Dk], ck [Nc,Hkv,Dk], cv [Nc,Hkv,Dv] -> [T,Hq,Dv] in math_dtype.

    Column c is visible to row t iff c*stride + block <= t.  Rows that see nothing give 0.
    """
    T, Hq, Dk = q.shape
    Nc, Hkv, Dv = cv.shape
    G = _group(Hq, Hkv)
    scale = 1.0 / math.sqrt(Dk) if scale is None else scale
    ckm, cvm = ck.to(math_dtype), cv.to(math_dtype)
    out = torch.zeros(T if rows is None else len(rows), Hq, Dv, dtype=math_dtype)
    col_end = torch.arange(Nc) * stride + block                   # first row that may see c
    for pos, ids in _row_chunks(T, rows, row_chunk):
        qm = q[ids].to(math_dtype).reshape(-1, Hkv, G, Dk)
        vis = col_end[None, :] <= ids[:, None]                    # [t,Nc]
        s = torch.einsum("thgd,chd->thgc", qm, ckm) * scale
        s = s.masked_fill(~vis[:, None, None, :], float("-inf"))
        m = s.amax(-1, keepdim=True)
        m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
        e = torch.exp(s - m)
        z = e.sum(-1, keepdim=True)
        p = torch.where(z > 0, e / z.clamp_min(1e-300), torch.zeros_like(e))
        o = torch.einsum("thgc,chv->thgv", p, cvm)
        out[pos] = o.reshape(-1, Hq, Dv)
    return out


# ----------------------------------------------------------------------------- selected / sliding

def _masked_attention(qm, km, vm, allowed, scale):
    """qm [t,Hkv,G,Dk], km [Tk,Hkv,Dk], vm [Tk,Hkv,Dv], allowed [t,Hkv,Tk] -> [t,Hkv,G,Dv].  `allowed` is a boolean
    mask, or an integer count of how many times the key enters the softmax (0 = masked)."""
    s = torch.einsum("thgd,khd->thgk", qm, km) * scale
    s = s.masked_fill((allowed == 0)[:, :, None, :], float("-inf"))
    m = s.amax(-1, keepdim=True)
    m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    e = torch.exp(s - m)
    if allowed.dtype != torch.bool:
        e = e * allowed[:, :, None, :].to(e.dtype)
    z = e.sum(-1, keepdim=True)
    p = torch.where(z > 0, e / z.clamp_min(1e-300), torch.zeros_like(e))
    return torch.einsum("thgk,khv->thgv", p, vm)


def selected_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                       block_indices: torch.Tensor, block_counts, block_size: int,
                       scale: Optional[float] = None, math_dtype=torch.float32,
                       row_chunk: int = 512, rows=None) -> torch.Tensor:
    """One sequence.  q [T,Hq,Dk], k [T,Hkv,Dk], v [T,Hkv,Dv], block_indices [T,Hkv,S] (block
    numbers local to the sequence).  Entry i of row t is used iff i < count, idx >= 0 and
    idx*block_size <= t; it contributes keys [idx*bs, min(idx*bs+bs-1, t)].  No usable entry -> 0.
    A block id that occurs twice among a row's used entries enters the softmax twice, as in the reference's gather
    (tests/test_parallel_nsa.py:133-146: k and v are gathered per entry, so a repeated block's keys are repeated).
    """
    T, Hq, Dk = q.shape
    _, Hkv, Dv = v.shape
    G = _group(Hq, Hkv)
    S = block_indices.shape[-1]
    scale = 1.0 / math.sqrt(Dk) if scale is None else scale
    km, vm = k.to(math_dtype), v.to(math_dtype)
    out = torch.zeros(T if rows is None else len(rows), Hq, Dv, dtype=math_dtype)
    if isinstance(block_counts, int):
        counts = torch.full((T, Hkv), block_counts, dtype=torch.int64)
    elif block_counts is None:
        counts = torch.full((T, Hkv), S, dtype=torch.int64)
    else:
        counts = block_counts.to(torch.int64)
    nblk = (T + block_size - 1) // block_size
    for pos, ids in _row_chunks(T, rows, row_chunk):
        n = ids.numel()
        idx = block_indices[ids].to(torch.int64)                           # [n,Hkv,S]
        use = (torch.arange(S)[None, None, :] < counts[ids][:, :, None]) & (idx >= 0) \
            & (idx * block_size <= ids[:, None, None])
        blk = torch.zeros(n, Hkv, nblk + 1, dtype=torch.int64)             # times each block is used
        tgt = torch.where(use, idx, torch.full_like(idx, nblk)).clamp(max=nblk)
        blk.scatter_add_(2, tgt, torch.ones_like(tgt))
        blk = blk[..., :nblk]
        allowed = blk.repeat_interleave(block_size, dim=2)[..., :T]        # [n,Hkv,T]
        allowed = allowed * (torch.arange(T)[None, None, :] <= ids[:, None, None])
        qm = q[ids].to(math_dtype).reshape(n, Hkv, G, Dk)
        out[pos] = _masked_attention(qm, km, vm, allowed, scale).reshape(n, Hq, Dv)
    return out


def sliding_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int,
                      scale: Optional[float] = None, math_dtype=torch.float32,
                      row_chunk: int = 512, rows=None) -> torch.Tensor:
    """One sequence.  Row t attends keys [max(0, t-window+1), t]."""
    T, Hq, Dk = q.shape
    _, Hkv, Dv = v.shape
    G = _group(Hq, Hkv)
    scale = 1.0 / math.sqrt(Dk) if scale is None else scale
    km, vm = k.to(math_dtype), v.to(math_dtype)
    out = torch.zeros(T if rows is None else len(rows), Hq, Dv, dtype=math_dtype)
    cols = torch.arange(T)
    for pos, ids in _row_chunks(T, rows, row_chunk):
        lo = max(0, int(ids.min()) - window + 1)
        hi = int(ids.max()) + 1
        allowed = (cols[None, lo:hi] <= ids[:, None]) & (cols[None, lo:hi] > ids[:, None] - window)
        allowed = allowed[:, None, :].expand(-1, Hkv, -1)
        qm = q[ids].to(math_dtype).reshape(ids.numel(), Hkv, G, Dk)
        out[pos] = _masked_attention(qm, km[lo:hi], vm[lo:hi], allowed, scale).reshape(-1, Hq, Dv)
    return out


def gated_combine(g_slc, o_slc, g_swa, o_swa, g_cmp=None, o_cmp=None):
    """out = g_slc*o_slc + g_swa*o_swa (+ g_cmp*o_cmp); gates [T,Hq], branches [T,Hq,Dv]."""
    out = g_slc.unsqueeze(-1) * o_slc
    if o_swa is not None:
        out = out + g_swa.unsqueeze(-1) * o_swa
    if o_cmp is not None:
        out = out + g_cmp.unsqueeze(-1) * o_cmp
    return out


# ----------------------------------------------------------------------------- slow loops (tiny inputs)

def selected_sliding_loop(q, k, v, block_indices, block_counts, block_size, window, scale=None):
    """Per-token python loop over one sequence in fp64; returns (o_slc, o_swa)."""
    T, Hq, Dk = q.shape
    _, Hkv, Dv = v.shape
    G = Hq // Hkv
    S = block_indices.shape[-1]
    scale = 1.0 / math.sqrt(Dk) if scale is None else scale
    qd, kd, vd = q.double(), k.double(), v.double()
    o_slc = torch.zeros(T, Hq, Dv, dtype=torch.float64)
    o_swa = torch.zeros(T, Hq, Dv, dtype=torch.float64)
    for t in range(T):
        for h in range(Hkv):
            cnt = S if block_counts is None else (
                block_counts if isinstance(block_counts, int) else int(block_counts[t, h]))
            toks = []
            for i in range(min(cnt, S)):
                b = int(block_indices[t, h, i])
                if b < 0 or b * block_size > t:
                    continue
                toks.extend(range(b * block_size, min(b * block_size + block_size - 1, t) + 1))
            for g in range(G):
                hq = h * G + g
                if toks:
                    sc = (kd[toks, h] @ qd[t, hq]) * scale
                    o_slc[t, hq] = torch.softmax(sc, 0) @ vd[toks, h]
                if window > 0:
                    lo = max(0, t - window + 1)
                    sc = (kd[lo:t + 1, h] @ qd[t, hq]) * scale
                    o_swa[t, hq] = torch.softmax(sc, 0) @ vd[lo:t + 1, h]
    return o_slc, o_swa


def compress_loop(x, w_lin, bias, block, stride, n_out):
    """Triple loop in fp64: flatten each window of one head and multiply by the weight."""
    T, H, D = x.shape
    out = torch.zeros(n_out, H, w_lin.shape[1], dtype=torch.float64)
    for n in range(n_out):
        win = x[n * stride:n * stride + block].double()
        for h in range(H):
            out[n, h] = win[:, h, :].reshape(1, -1) @ w_lin.double()
            if bias is not None:
                out[n, h] += bias.double()
    return out


# ----------------------------------------------------------------------------- full forward

class NSAParams:
    def __init__(self, block=32, stride=16, sel_block=64, top_n=16, window=512, scale=None):
        self.block, self.stride, self.sel_block = block, stride, sel_block
        self.top_n, self.window, self.scale = top_n, window, scale
        self.pool_kernel = sel_block // stride + 1
        self.pool_pad = block // stride - 2
        self.pool_stride = sel_block // stride


def nsa_forward_single(q, k, v, gates, p: NSAParams, compressor=None,
                       math_dtype=torch.float32, return_parts=False, force_idx=None, rows=None,
                       compressed=None):
    """One sequence.  q [T,Hq,Dk], k [T,Hkv,Dk], v [T,Hkv,Dv], gates [T,Hq,3] already activated,
    ordered (selected, sliding, compressed).  compressor: None -> mean-pool, else a dict with
    'wk','wv' ([block*D, D] row j*D+i) and optional 'bk','bv'.  Returns [T,Hq,Dv] in q.dtype.
    force_idx [T,Hkv,S] replaces the selected block ids (the returned 'idx_own' keeps the oracle's own).
    rows (sorted token ids) restricts the computation to those query rows: every result then has
    len(rows) rows.  A sequence too short for one pooled bin selects nothing (the reference's
    avg_pool1d would raise there); its compressed and sliding branches are still computed.
    """
    T = q.shape[0]
    Hkv = k.shape[1]
    Nc = compressed_len_conv(T, p.block, p.stride)
    if compressed is not None:         # (ck, cv) computed earlier by one of the compress_* functions
        ck, cv = compressed
    elif compressor is None:
        ck = compress_meanpool(k, p.block, p.stride, Nc, math_dtype)
        cv = compress_meanpool(v, p.block, p.stride, Nc, math_dtype)
    else:
        ck = compress_weighted(k, compressor["wk"], compressor.get("bk"), p.block, p.stride, Nc, math_dtype)
        cv = compress_weighted(v, compressor["wv"], compressor.get("bv"), p.block, p.stride, Nc, math_dtype)
    n_rows = T if rows is None else len(rows)
    Ns = pool_geometry(Nc, p.pool_kernel, p.pool_stride, p.pool_pad)[0] if Nc > 0 else 0
    if Ns > 0:
        pooled = importance_scores(q, ck, p.pool_kernel, p.pool_stride, p.pool_pad, math_dtype, rows=rows)
        idx_own = select_blocks(pooled, p.top_n)
    else:
        pooled = torch.zeros(n_rows, Hkv, 0, dtype=math_dtype)
        idx_own = torch.full((n_rows, Hkv, p.top_n), -1, dtype=torch.int64)
    if Nc > 0:
        o_cmp = compressed_attention(q, ck, cv, p.block, p.stride, p.scale, math_dtype, rows=rows)
    else:
        o_cmp = torch.zeros(n_rows, q.shape[1], v.shape[2], dtype=math_dtype)
    if force_idx is not None:          # branch parity independent of how score ties were broken
        idx_full = force_idx.to(torch.int64)
        idx = idx_full if rows is None else idx_full[rows]
    else:
        idx = idx_own
        if rows is None:
            idx_full = idx
        else:
            idx_full = torch.full((T, Hkv, p.top_n), -1, dtype=torch.int64)
            idx_full[rows] = idx
    o_slc = selected_attention(q, k, v, idx_full, None, p.sel_block, p.scale, math_dtype, rows=rows)
    o_swa = sliding_attention(q, k, v, p.window, p.scale, math_dtype, rows=rows) if p.window > 0 else None
    gm = gates.to(math_dtype) if rows is None else gates[rows].to(math_dtype)
    out = gated_combine(gm[..., 0], o_slc, gm[..., 1], o_swa, gm[..., 2], o_cmp).to(q.dtype)
    if return_parts:
        return out, dict(ck=ck, cv=cv, pooled=pooled, idx=idx, idx_own=idx_own, o_cmp=o_cmp, o_slc=o_slc,
                         o_swa=o_swa)
    return out


def nsa_forward_varlen(q, k, v, gates, cu_seqlens: Sequence[int], p: NSAParams, compressor=None,
                       math_dtype=torch.float32):
    """Packed sequences: each one is run on its own and the results are concatenated."""
    outs = []
    for b in range(len(cu_seqlens) - 1):
        s, e = int(cu_seqlens[b]), int(cu_seqlens[b + 1])
        outs.append(nsa_forward_single(q[s:e], k[s:e], v[s:e], gates[s:e], p, compressor, math_dtype))
    return torch.cat(outs, 0)


def nsa_decode_step(q_last, k_cache, v_cache, gates_last, p: NSAParams, math_dtype=torch.float32,
                    return_parts=False, force_idx=None):
    """One new token per sequence.  q_last [Hq,Dk] is the query at position ctx-1, k_cache
    [ctx,Hkv,Dk] / v_cache [ctx,Hkv,Dv] already hold that token.  Defined as the last row of the
    prefill forward on the same cache (mean-pool compressor), computed here without the other rows.
    force_idx [Hkv,S]: blocks to attend in the selected branch instead of the oracle's own picks
    (which are still returned in parts["idx"]), so that outputs stay comparable when a tie flips a pick.
    """
    ctx = k_cache.shape[0]
    t = ctx - 1
    Hq, Dk = q_last.shape
    Hkv, Dv = v_cache.shape[1:]
    Nc = compressed_len_conv(ctx, p.block, p.stride)
    q1 = q_last[None]
    ck = compress_meanpool(k_cache, p.block, p.stride, Nc, math_dtype)
    cv = compress_meanpool(v_cache, p.block, p.stride, Nc, math_dtype)
    parts = {}
    scale = 1.0 / math.sqrt(Dk) if p.scale is None else p.scale
    if Nc > 0 and pool_geometry(Nc, p.pool_kernel, p.pool_stride, p.pool_pad)[0] > 0:
        pooled = importance_scores(q1, ck, p.pool_kernel, p.pool_stride, p.pool_pad, math_dtype)
        idx = select_blocks(pooled, p.top_n)[0]                        # [Hkv,S]
        parts["pooled"] = pooled[0]
    else:
        idx = torch.full((Hkv, p.top_n), -1, dtype=torch.int64)
    use_idx = idx if force_idx is None else force_idx
    n_vis = min(max((t - p.block) // p.stride + 1, 0), Nc) if t >= p.block else 0
    if n_vis > 0:
        s = torch.einsum("hgd,chd->hgc", q_last.to(math_dtype).reshape(Hkv, -1, Dk),
                         ck[:n_vis].to(math_dtype)) * scale
        o_cmp = torch.einsum("hgc,chv->hgv", torch.softmax(s, -1), cv[:n_vis].to(math_dtype))
        o_cmp = o_cmp.reshape(Hq, Dv)
    else:
        o_cmp = torch.zeros(Hq, Dv, dtype=math_dtype)
    scale = 1.0 / math.sqrt(Dk) if p.scale is None else p.scale
    G = Hq // Hkv
    qm = q_last.to(math_dtype).reshape(Hkv, G, Dk)
    o_slc = torch.zeros(Hkv, G, Dv, dtype=math_dtype)
    o_swa = torch.zeros(Hkv, G, Dv, dtype=math_dtype)
    for h in range(Hkv):
        toks = []
        for b in (int(x) for x in use_idx[h] if x >= 0 and int(x) * p.sel_block <= t):    # a repeated id counts twice
            toks.extend(range(b * p.sel_block, min(b * p.sel_block + p.sel_block - 1, t) + 1))
        if toks:
            tk = torch.tensor(toks)
            s = (qm[h] @ k_cache[tk, h].to(math_dtype).T) * scale
            o_slc[h] = torch.softmax(s, -1) @ v_cache[tk, h].to(math_dtype)
        if p.window > 0:
            lo = max(0, t - p.window + 1)
            s = (qm[h] @ k_cache[lo:, h].to(math_dtype).T) * scale
            o_swa[h] = torch.softmax(s, -1) @ v_cache[lo:, h].to(math_dtype)
    gm = gates_last.to(math_dtype)
    out = gated_combine(gm[:, 0], o_slc.reshape(Hq, Dv), gm[:, 1],
                        o_swa.reshape(Hq, Dv) if p.window > 0 else None, gm[:, 2], o_cmp)
    out = out.to(q_last.dtype)
    if return_parts:
        parts.update(idx=idx, o_cmp=o_cmp, o_slc=o_slc.reshape(Hq, Dv), o_swa=o_swa.reshape(Hq, Dv))
        return out, parts
    return out


# ----------------------------------------------------------------------------- index parity rule

def compare_selection(idx_test: torch.Tensor, idx_ref: torch.Tensor, pooled_ref: torch.Tensor,
                      tol: float = 1e-3):
    """Set comparison per (t, h).  A differing entry is excused iff its oracle score is within
    `tol` of the oracle's S-th largest score.  Returns (n_rows, n_exact, n_excused, n_fail)."""
    T, H, S = idx_ref.shape
    Ns = pooled_ref.shape[-1]
    n_exact = n_exc = n_fail = 0
    a = idx_test.to(torch.int64).sort(-1).values
    b = idx_ref.to(torch.int64).sort(-1).values
    same = (a == b).all(-1)
    n_exact = int(same.sum())
    bad = (~same).nonzero()
    for t, h in bad.tolist():
        sa = set(int(x) for x in idx_test[t, h] if x >= 0)
        sb = set(int(x) for x in idx_ref[t, h] if x >= 0)
        if len(sa) != len(sb) or any(x >= Ns for x in sa):
            n_fail += 1
            continue
        tau = min(float(pooled_ref[t, h, j]) for j in sb)
        ok = all(abs(float(pooled_ref[t, h, j]) - tau) <= tol for j in (sa ^ sb))
        if ok:
            n_exc += 1
        else:
            n_fail += 1
    return T * H, n_exact, n_exc, n_fail
