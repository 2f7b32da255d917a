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
        self._max_len = 0        # longest sequence, tracked on the host so that append() never waits for the GPU

    @torch.no_grad()
    def fill(self, k: torch.Tensor, v: torch.Tensor):
        """Loads a prefilled context: k [B,T,Hkv,Dk], v [B,T,Hkv,Dv] (same T for every sequence)."""
        from . import ops
        B, T = k.shape[:2]
        if T > self.ctx_cap:
            raise RuntimeError(f"{T} tokens do not fit the cache capacity of {self.ctx_cap}")
        self._max_len = T
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
        """k_new [B,Hkv,Dk], v_new [B,Hkv,Dv]: the next token of every sequence.  Raises once the longest
        sequence (as filled and appended through this object) has reached the capacity: the kernel would
        drop the token and later steps would attend a stale last row."""
        if self._max_len >= self.ctx_cap:
            raise RuntimeError(f"a sequence would exceed the cache capacity of {self.ctx_cap} tokens")
        self._max_len += 1
        pos = self.ctx_lens.clone()
        k_new, v_new = k_new.contiguous(), v_new.contiguous()      # keep the copies alive across the launch
        rc = _lib.load().nsa_decode_append(_ptr(k_new), _ptr(v_new), _ptr(self.k),
                                           _ptr(self.vt), _ptr(self.ck), _ptr(self.cvt), _ptr(pos), self.batch,
                                           self.hkv, self.dk, self.dv, self.ctx_cap, self.nc_cap, self.block,
                                           self.stride, _dtype_code(self.k), _stream())
        _lib.check(rc, "nsa_decode_append")
        self.ctx_lens += 1


class NSAPagedDecodeCache:
    """The same caches with K and V in a pool of 64-token pages shared by all sequences (one page =
    one selection block of the default configuration), so that sequences of very different lengths
    do not reserve their maximum.  Layout per page: keys [64, Hkv, Dk] row-major, values
    [Hkv, Dv, 64] key-contiguous.  block_table[b, i] is the page that holds tokens [64 i, 64 i + 64)
    of sequence b; unused entries point at page 0, which is never handed out and stays zero.  The
    compressed caches are small (1/stride of the tokens) and stay contiguous per sequence.

    Page bookkeeping (free list, lengths) lives on the host, so no call here waits for the GPU."""

    PAGE = 64

    def __init__(self, batch, num_pages, max_ctx, hkv, dk, dv, block=32, stride=16, dtype=torch.bfloat16,
                 device="cuda"):
        if block > self.PAGE:
            raise ValueError("the compression block may span at most one page boundary (block <= 64)")
        self.batch, self.hkv, self.dk, self.dv = batch, hkv, dk, dv
        self.block, self.stride = block, stride
        self.max_pages = _round_up(max_ctx, self.PAGE) // self.PAGE
        self.ctx_cap = self.max_pages * self.PAGE
        nc = (self.ctx_cap - block) // stride + 1 if self.ctx_cap >= block else 1
        self.nc_cap = _round_up(nc, 64)
        z = dict(dtype=dtype, device=device)
        self.num_pages = num_pages + 1                           # page 0 is the shared all-zero page
        self.k_pool = torch.zeros(self.num_pages, self.PAGE, hkv, dk, **z)
        self.v_pool_t = torch.zeros(self.num_pages, hkv, dv, self.PAGE, **z)
        self.ck = torch.zeros(batch, self.nc_cap, hkv, dk, **z)
        self.cvt = torch.zeros(batch, hkv, dv, self.nc_cap, **z)
        self.block_table = torch.zeros(batch, self.max_pages, dtype=torch.int32, device=device)
        self.ctx_lens = torch.zeros(batch, dtype=torch.int32, device=device)
        self._free = list(range(self.num_pages - 1, 0, -1))
        self._pages = [[] for _ in range(batch)]
        self._lens = [0] * batch

    @property
    def free_pages(self) -> int:
        return len(self._free)

    def _grow(self, b: int, new_len: int):
        """Makes sure sequence b owns pages for new_len tokens; returns the (slot, page) pairs added.
        All or nothing: on an error the sequence keeps exactly the pages it had."""
        need = (new_len + self.PAGE - 1) // self.PAGE
        if need > self.max_pages:
            raise RuntimeError(f"sequence {b} would exceed the cache capacity of {self.ctx_cap} tokens")
        if need - len(self._pages[b]) > len(self._free):
            raise RuntimeError("the K/V page pool is exhausted")
        added = []
        while len(self._pages[b]) < need:
            pg = self._free.pop()
            added.append((len(self._pages[b]), pg))
            self._pages[b].append(pg)
        return added

    def _publish(self, entries):
        """entries: (sequence, slot, page) triples to write into the device block table."""
        if not entries:
            return
        e = torch.tensor(entries, dtype=torch.int64)
        self.block_table[e[:, 0].to(self.block_table.device), e[:, 1].to(self.block_table.device)] = \
            e[:, 2].to(device=self.block_table.device, dtype=torch.int32)

    def release(self, b: int):
        """Returns the pages of sequence b to the pool and empties it."""
        self._free.extend(reversed(self._pages[b]))
        self._pages[b] = []
        self._lens[b] = 0
        self.block_table[b].zero_()
        self.ctx_lens[b] = 0

    @torch.no_grad()
    def fill(self, k: torch.Tensor, v: torch.Tensor, seq: Optional[int] = None):
        """Loads a prefilled context.  k [B,T,Hkv,Dk], v [B,T,Hkv,Dv] for every sequence (seq None,
        B == batch), or k [T,Hkv,Dk], v [T,Hkv,Dv] for sequence `seq` alone."""
        from . import ops
        if seq is not None:
            k, v, seqs = k.unsqueeze(0), v.unsqueeze(0), [seq]
        else:
            seqs = list(range(self.batch))
        B, T = k.shape[:2]
        if B != len(seqs):
            raise ValueError(f"fill() got {B} sequences for {len(seqs)} cache slots")
        held = sum(len(self._pages[b]) for b in seqs)
        if len(seqs) * ((T + self.PAGE - 1) // self.PAGE) > len(self._free) + held:
            raise RuntimeError("the K/V page pool is exhausted")       # before any sequence is touched
        entries = []
        for b in seqs:
            if self._lens[b]:
                self.release(b)
            entries += [(b, slot, pg) for slot, pg in self._grow(b, T)]
            self._lens[b] = T
        self._publish(entries)
        P, Tp = self.PAGE, _round_up(T, self.PAGE)
        if T > 0:
            pages = torch.tensor([self._pages[b][:Tp // P] for b in seqs], dtype=torch.int64, device=k.device)
            kp = torch.zeros(B, Tp, self.hkv, self.dk, dtype=k.dtype, device=k.device)
            vp = torch.zeros(B, Tp, self.hkv, self.dv, dtype=v.dtype, device=v.device)
            kp[:, :T], vp[:, :T] = k, v
            self.k_pool[pages.reshape(-1)] = kp.view(B * (Tp // P), P, self.hkv, self.dk)
            self.v_pool_t[pages.reshape(-1)] = vp.view(B * (Tp // P), P, self.hkv, self.dv).permute(0, 2, 3, 1)
        nc = (T - self.block) // self.stride + 1 if T >= self.block else 0
        sq = torch.tensor(seqs, dtype=torch.int64, device=k.device)
        if nc > 0:
            cu = ops.uniform_cu(B, T, k.device)
            cu_out = ops.uniform_cu(B, nc, k.device)
            ck = ops.compress(k.reshape(B * T, self.hkv, self.dk).contiguous(), cu, cu_out, B * nc, self.block,
                              self.stride)
            cv = ops.compress(v.reshape(B * T, self.hkv, self.dv).contiguous(), cu, cu_out, B * nc, self.block,
                              self.stride)
            self.ck[sq, :nc] = ck.view(B, nc, self.hkv, self.dk)
            self.cvt[sq, :, :, :nc] = cv.view(B, nc, self.hkv, self.dv).permute(0, 2, 3, 1)
        self.ctx_lens[sq] = T

    def reserve_next(self):
        """Host half of append(): makes sure every sequence owns the page of its next token and
        publishes new table entries.  Separate so that the device half can live in a captured graph."""
        fresh = sum(self._lens[b] % self.PAGE == 0 for b in range(self.batch))
        if fresh > len(self._free):
            raise RuntimeError("the K/V page pool is exhausted")       # before any sequence has grown
        if max(self._lens) >= self.ctx_cap:
            raise RuntimeError(f"a sequence would exceed the cache capacity of {self.ctx_cap} tokens")
        entries = []
        for b in range(self.batch):
            entries += [(b, slot, pg) for slot, pg in self._grow(b, self._lens[b] + 1)]
            self._lens[b] += 1
        self._publish(entries)

    @torch.no_grad()
    def append_reserved(self, k_new: torch.Tensor, v_new: torch.Tensor):
        """Device half of append(): writes the token (and a compressed row when one completes)."""
        pos = self.ctx_lens.clone()
        k_new, v_new = k_new.contiguous(), v_new.contiguous()
        rc = _lib.load().nsa_decode_append_paged(_ptr(k_new), _ptr(v_new), _ptr(self.k_pool), _ptr(self.v_pool_t),
                                                 _ptr(self.block_table), self.max_pages, _ptr(self.ck),
                                                 _ptr(self.cvt), _ptr(pos), self.batch, self.hkv, self.dk, self.dv,
                                                 self.nc_cap, self.block, self.stride, _dtype_code(self.k_pool),
                                                 _stream())
        _lib.check(rc, "nsa_decode_append_paged")
        self.ctx_lens += 1

    def append(self, k_new: torch.Tensor, v_new: torch.Tensor):
        """k_new [B,Hkv,Dk], v_new [B,Hkv,Dv]: the next token of every sequence."""
        self.reserve_next()
        self.append_reserved(k_new, v_new)


@torch.no_grad()
def nsa_decode_step(q: torch.Tensor, cache, gates: Optional[torch.Tensor] = None,
                    selection_block: int = 64, selected_block_count: int = 16, sliding_window: int = 512,
                    scale: Optional[float] = None, gate_activation: Optional[str] = None,
                    return_indices: bool = False, splits: Optional[int] = None, out: Optional[torch.Tensor] = None,
                    indices: Optional[torch.Tensor] = None, static_scratch: bool = False):
    """q [B,Hq,Dk]: queries of the newest cached token; cache: NSADecodeCache or NSAPagedDecodeCache.  gates [B,Hq,3] (selected, sliding,
    compressed; pre-activation if gate_activation == "sigmoid").  Returns out [B,Hq,Dv]
    (and int32 block indices [B,Hkv,S]).

    splits: how many workgroups share one (sequence, kv head) pair.  0 = one (the kernel the batch-64
    benchmark runs); None = chosen from the batch: up to 64 pairs a single workgroup per pair leaves
    most of the chip idle and its ~60 us critical path sets the step time, so the work is split 8 ways
    (three launches, partial results in a workspace kept on the cache object).  Caches with more
    compressed rows than one workgroup keeps in registers (contexts beyond ~36k tokens) always take the
    split schedule, whose first launch cuts the compressed rows into slices of at most 384.  So do GQA groups of
    32, 48 or 64 heads: every 16 heads run as a pair of their own, the picks come from the whole group.

    out [B,Hq,Dv] / indices int32 [B,Hkv,S]: result buffers of the caller (allocated here when None).
    static_scratch: run the split schedule with its partial results in the library's own fixed device array
    (nsa_decode_step_split_static): with `out` (and `indices`) given, the call then allocates nothing, for
    callers that must not (graph capture, serving loops).  Calls that overlap on one GPU race on that array."""
    if not q.is_cuda:
        raise RuntimeError("NSA kernels run on the GPU only")
    B, hq, dk = q.shape
    q = q.contiguous()
    if scale is None:
        scale = 1.0 / math.sqrt(dk)
    if out is None:
        out = torch.empty(B, hq, cache.dv, dtype=q.dtype, device=q.device)
    elif out.shape != (B, hq, cache.dv) or out.dtype != q.dtype or not out.is_contiguous():
        raise ValueError("out must be a contiguous [B,Hq,Dv] tensor of q's dtype")
    idx = indices
    if idx is None and return_indices:
        idx = torch.empty(B, cache.hkv, selected_block_count, dtype=torch.int32, device=q.device)
    elif idx is not None and (idx.shape != (B, cache.hkv, selected_block_count) or idx.dtype != torch.int32
                              or not idx.is_contiguous()):
        raise ValueError("indices must be a contiguous int32 [B,Hkv,S] tensor")
    if gates is not None:
        gates = gates.to(q.dtype).contiguous()
    pool_k = selection_block // cache.stride + 1
    pool_s = selection_block // cache.stride
    pool_p = cache.block // cache.stride - 2
    act = _lib.GATE_SIGMOID if gate_activation == "sigmoid" else _lib.GATE_IDENTITY
    paged = isinstance(cache, NSAPagedDecodeCache)
    lib = _lib.load()
    long_cache = cache.nc_cap > lib.nsa_decode_max_compressed()
    group = hq // cache.hkv if hq % cache.hkv == 0 else 0
    sub_groups = group // 16 if group > 16 and group % 16 == 0 else 1    # 16-head sub-groups per kv head
    # the one-workgroup kernel holds nc_cap / 2 + 4 pooled bins (pooling strides of 2 and more): selection blocks of
    # one compression stride make more and run on the split schedule, which holds 3136
    span = cache.nc_cap + 2 * pool_p - pool_k
    ns_cap = 0 if span < 0 else (span + pool_s - 1) // pool_s + 1
    one_wg_bins = min((cache.nc_cap + 1) // 2 + 4, 1156)
    many_bins = ns_cap > one_wg_bins
    if sub_groups > 1 or many_bins:
        # groups of 32, 48, 64 heads: the split schedule runs every 16 heads as a pair of their own
        long_cache = True
    if static_scratch and splits == 0:
        raise ValueError("static_scratch runs the split schedule: pass splits=None or a positive split count "
                         "(splits=0 asks for the one-workgroup step, which has no scratch buffer)")
    if splits is None:
        pairs = B * cache.hkv * sub_groups
        # measured at 32k context: 8 splits halve the step up to 32 pairs and still win at 64 (46 vs 64 us);
        # at 128 pairs one workgroup per pair is as fast and needs no workspace
        splits = 8 if pairs <= 64 and selected_block_count <= 64 else 0
        if long_cache and splits == 0:
            splits = 1 if pairs > 64 else 8       # the compressed rows are sliced whatever `splits` says
    elif splits == 0 and sub_groups > 1:
        raise NotImplementedError("the one-workgroup decode step is built for GQA groups of at most 16 heads "
                                  "(pass splits=None or a positive split count)")
    elif splits == 0 and many_bins:
        raise NotImplementedError("the one-workgroup decode step holds %d pooled bins per sequence, this geometry "
                                  "makes up to %d (pass splits=None or a positive split count)"
                                  % (one_wg_bins, ns_cap))
    elif splits == 0 and long_cache:
        raise NotImplementedError(
            "the one-workgroup decode step keeps at most %d compressed rows per sequence; this cache holds up "
            "to %d (pass splits=None or a positive split count)" % (lib.nsa_decode_max_compressed(), cache.nc_cap))
    if static_scratch:
        splits = splits or 8          # None that resolved to the one-workgroup step: the split schedule all the same
        k_c, v_c = (cache.k_pool, cache.v_pool_t) if paged else (cache.k, cache.vt)
        rc = lib.nsa_decode_step_split_static(
            _ptr(q), _ptr(k_c), _ptr(v_c), _ptr(cache.block_table) if paged else None,
            cache.max_pages if paged else 0, _ptr(cache.ck), _ptr(cache.cvt), _ptr(cache.ctx_lens), _ptr(gates),
            _ptr(out), _ptr(idx), B, hq, cache.hkv, dk, cache.dv, cache.ctx_cap, cache.nc_cap, cache.block,
            cache.stride, selection_block, pool_k, pool_s, pool_p, selected_block_count, sliding_window,
            float(scale), act, _dtype_code(q), splits, _stream())
        _lib.check(rc, "nsa_decode_step_split_static")
        return (out, idx) if return_indices else out
    if splits:
        need = lib.nsa_decode_split_pooled_workspace_bytes(B, cache.hkv * sub_groups, cache.dv, cache.nc_cap, splits,
                                                           pool_k, pool_s, pool_p)
        ws = getattr(cache, "_split_ws", None)
        if ws is None or ws.numel() < need:
            ws = cache._split_ws = torch.empty(need, dtype=torch.uint8, device=q.device)
        k_c, v_c = (cache.k_pool, cache.v_pool_t) if paged else (cache.k, cache.vt)
        rc = lib.nsa_decode_step_split(
            _ptr(q), _ptr(k_c), _ptr(v_c), _ptr(cache.block_table) if paged else None,
            cache.max_pages if paged else 0, _ptr(cache.ck), _ptr(cache.cvt), _ptr(cache.ctx_lens), _ptr(gates),
            _ptr(out), _ptr(idx), B, hq, cache.hkv, dk, cache.dv, cache.ctx_cap, cache.nc_cap, cache.block,
            cache.stride, selection_block, pool_k, pool_s, pool_p, selected_block_count, sliding_window,
            float(scale), act, _dtype_code(q), splits, _ptr(ws), ws.numel(), _stream())
        _lib.check(rc, "nsa_decode_step_split")
        return (out, idx) if return_indices else out
    if paged:
        rc = _lib.load().nsa_decode_step_paged(
            _ptr(q), _ptr(cache.k_pool), _ptr(cache.v_pool_t), _ptr(cache.block_table), cache.max_pages,
            _ptr(cache.ck), _ptr(cache.cvt), _ptr(cache.ctx_lens), _ptr(gates), _ptr(out), _ptr(idx), B, hq,
            cache.hkv, dk, cache.dv, cache.nc_cap, cache.block, cache.stride, selection_block, pool_k, pool_s,
            pool_p, selected_block_count, sliding_window, float(scale), act, _dtype_code(q), _stream())
        _lib.check(rc, "nsa_decode_step_paged")
        return (out, idx) if return_indices else out
    rc = _lib.load().nsa_decode_step(
        _ptr(q), _ptr(cache.k), _ptr(cache.vt), _ptr(cache.ck), _ptr(cache.cvt), _ptr(cache.ctx_lens), _ptr(gates),
        _ptr(out), _ptr(idx), B, hq, cache.hkv, dk, cache.dv, cache.ctx_cap, cache.nc_cap, cache.block, cache.stride,
        selection_block, pool_k, pool_s, pool_p, selected_block_count, sliding_window, float(scale), act,
        _dtype_code(q), _stream())
    _lib.check(rc, "nsa_decode_step")
    return (out, idx) if return_indices else out


class NSADecodeGraph:
    """One decode iteration (cache append of the new token, then the attention step for its query)
    captured as a HIP graph and replayed per token, so that a serving loop pays one graph launch
    instead of the launches and allocations of the eager path.  Inputs are copied into fixed
    buffers; the result is returned as a view of a fixed buffer that the next call overwrites.

    Works on both cache kinds; with a paged cache the page bookkeeping (host only, plus a small
    table update when a sequence crosses a page boundary) runs before the replay, outside the
    graph.  The graph holds no memset nodes: the kernels clear what they need themselves."""

    def __init__(self, cache, hq: int, selection_block: int = 64, selected_block_count: int = 16,
                 sliding_window: int = 512, scale: Optional[float] = None, gate_activation: Optional[str] = None,
                 use_gates: bool = True, return_indices: bool = False):
        self.cache = cache
        self.paged = isinstance(cache, NSAPagedDecodeCache)
        dt = (cache.k_pool if self.paged else cache.k).dtype
        dev = cache.ctx_lens.device
        B = cache.batch
        self.q = torch.zeros(B, hq, cache.dk, dtype=dt, device=dev)
        self.k_new = torch.zeros(B, cache.hkv, cache.dk, dtype=dt, device=dev)
        self.v_new = torch.zeros(B, cache.hkv, cache.dv, dtype=dt, device=dev)
        self.gates = torch.zeros(B, hq, 3, dtype=dt, device=dev) if use_gates else None
        self._kw = dict(selection_block=selection_block, selected_block_count=selected_block_count,
                        sliding_window=sliding_window, scale=scale, gate_activation=gate_activation,
                        return_indices=return_indices)
        self.graph = None
        self.out = self.indices = None
        self._steps = 0             # tokens appended through this object
        self._base_len = None       # longest sequence at the first call (read from the device once)

    def _iteration(self):
        if self.paged:
            self.cache.append_reserved(self.k_new, self.v_new)
        else:
            self.cache.append(self.k_new, self.v_new)
        r = nsa_decode_step(self.q, self.cache, self.gates, **self._kw)
        self.out, self.indices = r if self._kw["return_indices"] else (r, None)

    @torch.no_grad()
    def step(self, q=None, k_new=None, v_new=None, gates=None):
        """q [B,Hq,Dk], k_new [B,Hkv,Dk], v_new [B,Hkv,Dv] of the next token, gates [B,Hq,3]; None
        for an operand that the caller has already written into self.q / k_new / v_new / gates."""
        if self.paged:
            self.cache.reserve_next()
        elif int(self.cache.ctx_cap) <= self._host_len():
            raise RuntimeError(f"a sequence would exceed the cache capacity of {self.cache.ctx_cap} tokens")
        elif self.graph is not None:
            self.cache._max_len += 1     # a replay appends without passing through cache.append()
        for buf, src in ((self.q, q), (self.k_new, k_new), (self.v_new, v_new), (self.gates, gates)):
            if buf is not None and src is not None and src is not buf:
                buf.copy_(src)       # producers that write into the buffers themselves pass None (or the buffer)
        if self.graph is None:
            # the capture itself does not execute, so it stands for no token: replayed below
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                self._iteration()
            self.graph = g
        self.graph.replay()
        self._steps += 1
        return (self.out, self.indices) if self._kw["return_indices"] else self.out

    def _host_len(self) -> int:
        """Longest sequence, tracked on the host (one read of the device lengths at the first call;
        appends made behind this object's back are not seen)."""
        if self._base_len is None:
            self._base_len = int(self.cache.ctx_lens.max())
        return self._base_len + self._steps
