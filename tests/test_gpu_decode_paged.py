"""GPU tests of the paged K/V cache: the decode step over a pool of 64-token pages with a shuffled
page table must equal the step over contiguous caches bit for bit (the kernels do the same
arithmetic in the same order, only addresses differ), and appending through the page table must
leave the same tokens in the pool as a bulk fill."""
import random

import pytest
import torch

from tests.util import max_abs, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _paged(batch, pages, max_ctx, Hkv, Dk, Dv, dtype, seed):
    from nsa_amd.decode import NSAPagedDecodeCache
    c = NSAPagedDecodeCache(batch, pages, max_ctx, Hkv, Dk, Dv, dtype=dtype, device=DEV)
    random.Random(seed).shuffle(c._free)           # pages of a sequence end up scattered over the pool
    return c


def _gather(cache, b):
    """tokens of sequence b read back through the page table: k [T,Hkv,Dk], v [T,Hkv,Dv]"""
    T = cache._lens[b]
    pages = torch.tensor(cache._pages[b], dtype=torch.int64, device=DEV)
    k = cache.k_pool[pages].reshape(-1, cache.hkv, cache.dk)[:T]
    v = cache.v_pool_t[pages].permute(0, 3, 1, 2).reshape(-1, cache.hkv, cache.dv)[:T]
    return k, v


@pytest.mark.parametrize("dtype,Hq,Hkv,Dk,Dv,S,W", [
    (torch.bfloat16, 64, 4, 128, 128, 16, 512),
    (torch.bfloat16, 32, 2, 192, 128, 4, 128),
    (torch.bfloat16, 4, 1, 64, 64, 3, 17),
    (torch.float32, 8, 2, 64, 64, 4, 64),
])
def test_paged_step_equals_contiguous_step(dtype, Hq, Hkv, Dk, Dv, S, W):
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    ctxs = [2048, 1000, 513, 64, 65, 33, 1]
    B, T = len(ctxs), max(ctxs)
    k = randn(B, T, Hkv, Dk, seed=700, scale=0.5, dtype=dtype).to(DEV)
    v = randn(B, T, Hkv, Dv, seed=701, scale=0.5, dtype=dtype).to(DEV)
    q = randn(B, Hq, Dk, seed=702, scale=0.5, dtype=dtype).to(DEV)
    gl = randn(B, Hq, 3, seed=703, dtype=dtype).to(DEV)
    paged = _paged(B, sum((c + 63) // 64 for c in ctxs) + 3, T, Hkv, Dk, Dv, dtype, seed=1)
    outs, idxs = [], []
    for b, c in enumerate(ctxs):
        paged.fill(k[b, :c], v[b, :c], seq=b)
        flat = NSADecodeCache(1, T, Hkv, Dk, Dv, dtype=dtype, device=DEV)
        flat.fill(k[b:b + 1, :c], v[b:b + 1, :c])
        o, i = nsa_decode_step(q[b:b + 1], flat, gl[b:b + 1], 64, S, W, gate_activation="sigmoid",
                               return_indices=True)
        outs.append(o)
        idxs.append(i)
    assert paged.free_pages == 3
    out, idx = nsa_decode_step(q, paged, gl, 64, S, W, gate_activation="sigmoid", return_indices=True)
    assert torch.equal(idx, torch.cat(idxs))
    assert torch.equal(out, torch.cat(outs))
    assert torch.isfinite(out.float()).all()


def test_paged_step_cfg5_shape():
    """benchmark decode shape per sequence (ctx 32768, Hq 64 / Hkv 4, D 128, top-16, window 512)."""
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    B, T, Hq, Hkv, D = 4, 32768, 64, 4, 128
    dtype = torch.bfloat16
    k = randn(B, T, Hkv, D, seed=710, scale=0.5, dtype=dtype).to(DEV)
    v = randn(B, T, Hkv, D, seed=711, scale=0.5, dtype=dtype).to(DEV)
    q = randn(B, Hq, D, seed=712, scale=0.5, dtype=dtype).to(DEV)
    flat = NSADecodeCache(B, T, Hkv, D, D, dtype=dtype, device=DEV)
    flat.fill(k, v)
    paged = _paged(B, B * T // 64, T, Hkv, D, D, dtype, seed=2)
    paged.fill(k, v)
    a, ia = nsa_decode_step(q, flat, None, 64, 16, 512, return_indices=True)
    b, ib = nsa_decode_step(q, paged, None, 64, 16, 512, return_indices=True)
    assert torch.equal(ia, ib) and torch.equal(a, b)


def test_paged_append_matches_bulk_fill_and_recycles_pages():
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    B, T0, steps, Hkv, Dk, Dv = 3, 100, 90, 2, 64, 64
    dtype = torch.bfloat16
    k = randn(B, T0 + steps, Hkv, Dk, seed=720, dtype=dtype).to(DEV)
    v = randn(B, T0 + steps, Hkv, Dv, seed=721, dtype=dtype).to(DEV)
    inc = _paged(B, 12, 256, Hkv, Dk, Dv, dtype, seed=3)
    # a sequence that is filled and released first leaves stale data in the recycled pages
    inc.fill(k[0, :150] * 3, v[0, :150] * 3, seq=1)
    inc.release(1)
    assert inc.free_pages == 12
    inc.fill(k[:, :T0], v[:, :T0])
    for s in range(steps):
        inc.append(k[:, T0 + s], v[:, T0 + s])
    assert inc.free_pages == 12 - B * 3
    ref = NSADecodeCache(B, T0 + steps, Hkv, Dk, Dv, dtype=dtype, device=DEV)
    ref.fill(k, v)
    assert torch.equal(inc.ctx_lens, ref.ctx_lens)
    for b in range(B):
        kb, vb = _gather(inc, b)
        assert torch.equal(kb, k[b]) and torch.equal(vb, v[b])
    nc = (T0 + steps - 32) // 16 + 1
    assert max_abs(inc.ck[:, :nc], ref.ck[:, :nc]) <= 4e-3
    assert max_abs(inc.cvt[..., :nc], ref.cvt[..., :nc]) <= 4e-3
    q = randn(B, 8, Dk, seed=722, dtype=dtype).to(DEV)
    a = nsa_decode_step(q, inc, None, 64, 2, 32)
    b = nsa_decode_step(q, ref, None, 64, 2, 32)
    assert max_abs(a, b) <= 2e-2
    with pytest.raises(RuntimeError, match="exhausted"):
        for _ in range(200):
            inc.append(k[:, 0], v[:, 0])


@pytest.mark.parametrize("paged", [False, True])
def test_decode_graph_replays_match_eager_steps(paged):
    """append + step captured once and replayed per token: every replay must equal the eager
    iteration on a twin cache, with eager work and synchronisations between the replays."""
    from nsa_amd.decode import NSADecodeCache, NSADecodeGraph, nsa_decode_step
    B, T0, steps, Hq, Hkv, D = 3, 500, 80, 16, 2, 128
    dtype = torch.bfloat16
    k = randn(B, T0 + steps, Hkv, D, seed=730, scale=0.5, dtype=dtype).to(DEV)
    v = randn(B, T0 + steps, Hkv, D, seed=731, scale=0.5, dtype=dtype).to(DEV)
    q = randn(steps, B, Hq, D, seed=732, scale=0.5, dtype=dtype).to(DEV)
    gl = randn(steps, B, Hq, 3, seed=733, dtype=dtype).to(DEV)

    def make():
        if paged:
            return _paged(B, B * 10 + 2, T0 + steps, Hkv, D, D, dtype, seed=4)
        return NSADecodeCache(B, T0 + steps, Hkv, D, D, dtype=dtype, device=DEV)

    ca, cb = make(), make()
    ca.fill(k[:, :T0], v[:, :T0])
    cb.fill(k[:, :T0], v[:, :T0])
    graph = NSADecodeGraph(ca, Hq, 64, 4, 128, gate_activation="sigmoid", return_indices=True)
    for s in range(steps):
        out, idx = graph.step(q[s], k[:, T0 + s], v[:, T0 + s], gl[s])
        cb.append(k[:, T0 + s], v[:, T0 + s])
        ref, ref_idx = nsa_decode_step(q[s], cb, gl[s], 64, 4, 128, gate_activation="sigmoid", return_indices=True)
        torch.cuda.synchronize()
        assert torch.equal(idx, ref_idx), s
        assert torch.equal(out, ref), s
    assert torch.equal(ca.ctx_lens, cb.ctx_lens) and int(ca.ctx_lens[0]) == T0 + steps
    assert torch.equal(ca.ck, cb.ck) and torch.equal(ca.cvt, cb.cvt)
    if not paged:
        assert torch.equal(ca.k, cb.k) and torch.equal(ca.vt, cb.vt)
        with pytest.raises(RuntimeError, match="capacity"):
            for _ in range(64):
                graph.step(q[0], k[:, 0], v[:, 0], gl[0])
