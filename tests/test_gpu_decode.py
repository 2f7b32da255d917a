"""GPU parity of the decode step and the cache append, through the C ABI, against the CPU oracle
(decode == last row of the prefill forward on the cached tokens)."""
import math

import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import TOL, max_abs, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _make(B, T, Hq, Hkv, Dk, Dv, seed, dtype, scale=0.5):
    q = randn(B, Hq, Dk, seed=seed, scale=scale, dtype=dtype)
    k = randn(B, T, Hkv, Dk, seed=seed + 1, scale=scale, dtype=dtype)
    v = randn(B, T, Hkv, Dv, seed=seed + 2, scale=scale, dtype=dtype)
    gl = randn(B, Hq, 3, seed=seed + 3, dtype=dtype)
    return q, k, v, gl


def _check(dtype, ctxs, Hq, Hkv, Dk, Dv, S, W, seed, which=None, splits=None, paged=False, sel_block=64, block=32,
           stride=16):
    """One decode step through the C ABI against the CPU oracle on the same cache contents.
    splits: None = the schedule nsa_decode_step picks from the batch, 0 = the one-workgroup kernel
    (what the batch-64 benchmark times), > 0 = that many workgroups per pair.  paged: K/V in a shuffled
    page pool.  The picks are checked under the tie rule and must be the oracle's own in >= 99 % of the
    rows; outputs are compared with the kernel's picks forced into the oracle, so a tie never hides them."""
    import random
    from nsa_amd.decode import NSADecodeCache, NSAPagedDecodeCache, nsa_decode_step
    B, T = len(ctxs), max(ctxs)
    q, k, v, gl = _make(B, T, Hq, Hkv, Dk, Dv, seed, dtype)
    if paged:
        cache = NSAPagedDecodeCache(B, sum((c + 63) // 64 for c in ctxs) + 2, T, Hkv, Dk, Dv, block=block, stride=stride,
                                    dtype=dtype, device=DEV)
        random.Random(seed).shuffle(cache._free)
        for b, c in enumerate(ctxs):
            cache.fill(k[b, :c].to(DEV), v[b, :c].to(DEV), seq=b)
    else:
        cache = NSADecodeCache(B, T, Hkv, Dk, Dv, block=block, stride=stride, dtype=dtype, device=DEV)
        cache.fill(k.to(DEV), v.to(DEV))
        cache.ctx_lens.copy_(torch.tensor(ctxs, dtype=torch.int32))
    out, idx = nsa_decode_step(q.to(DEV), cache, gl.to(DEV), sel_block, S, W, gate_activation="sigmoid",
                               return_indices=True, splits=splits)
    out, idx = out.cpu(), idx.cpu().long()
    p = O.NSAParams(block, stride, sel_block, S, W)
    gates = torch.sigmoid(gl.float()).to(dtype)
    worst, stats = 0.0, [0, 0, 0, 0]
    for b in (range(B) if which is None else which):
        c = ctxs[b]
        ref, parts = O.nsa_decode_step(q[b], k[b, :c], v[b, :c], gates[b], p, return_parts=True, force_idx=idx[b])
        if "pooled" in parts:
            r = O.compare_selection(idx[b][None], parts["idx"][None], parts["pooled"][None], 1e-3)
            stats = [x + y for x, y in zip(stats, r)]
            assert r[3] == 0
        else:
            assert (idx[b] == -1).all()
        worst = max(worst, max_abs(out[b], ref))
    print("decode", dtype, ctxs[:6], (Hq, Hkv, Dk, Dv, S, W), "splits", splits, "paged", paged, "max_abs", worst,
          "rows/exact/excused/fail", stats)
    assert torch.isfinite(out).all()
    assert worst <= TOL[dtype]
    assert stats[1] >= 0.99 * stats[0]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_decode_one_workgroup_step_does_not_depend_on_the_batch_slot(dtype):
    """The one-workgroup kernel runs its window phase at three different points of the step, by workgroup number;
    the output is (compressed + window) + selected whatever that order, so the same sequence gives the same bits
    in every batch slot."""
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    B, T, Hq, Hkv, D, S, W = 7, 1500, 32, 2, 128, 8, 200
    q, k, v, gl = _make(1, T, Hq, Hkv, D, D, 130, dtype)
    q, k, v, gl = (x.expand(B, *x.shape[1:]).contiguous() for x in (q, k, v, gl))
    cache = NSADecodeCache(B, T, Hkv, D, D, dtype=dtype, device=DEV)
    cache.fill(k.to(DEV), v.to(DEV))
    out, idx = nsa_decode_step(q.to(DEV), cache, gl.to(DEV), 64, S, W, gate_activation="sigmoid", return_indices=True,
                               splits=0)
    for b in range(1, B):         # 14 workgroups: every slot parity of (sequence, kv head) modulo 3 occurs
        assert torch.equal(idx[b], idx[0]), (b, idx[b], idx[0])
        assert torch.equal(out[b], out[0]), (b, float((out[b].float() - out[0].float()).abs().max()))


SCHEDULES = [None, 0]      # chosen from the batch (split for small batches) / one workgroup per pair


@pytest.mark.parametrize("splits", SCHEDULES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_decode_small_ragged_contexts(dtype, splits):
    _check(dtype, [1024, 1000, 513, 64, 40, 33, 20, 1], 64, 4, 128, 128, 4, 128, seed=100, splits=splits)


@pytest.mark.parametrize("splits", SCHEDULES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_decode_gqa4_d64(dtype, splits):
    _check(dtype, [1024, 777], 4, 1, 64, 64, 4, 128, seed=110, splits=splits)


@pytest.mark.parametrize("splits", SCHEDULES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_decode_dqk192(splits, dtype):
    _check(dtype, [2048, 1536], 32, 2, 192, 128, 16, 512, seed=120, splits=splits)


@pytest.mark.parametrize("splits", SCHEDULES)
def test_decode_cfg5_context_subset(splits):
    """benchmark config 5 shape per sequence (ctx 32768, Hq64/Hkv4, D128, top-16, window 512), batch 4."""
    _check(torch.bfloat16, [32768, 32768, 32767, 32000], 64, 4, 128, 128, 16, 512, seed=130, splits=splits)


def test_decode_cfg5_full_batch_default_dispatch():
    """benchmark config 5 as the benchmark runs it: batch 64 x ctx 32768 = 256 (sequence, kv head) pairs, which
    the default dispatch sends to the one-workgroup kernel; six sampled sequences against the oracle."""
    _check(torch.bfloat16, [32768] * 64, 64, 4, 128, 128, 16, 512, seed=131, which=[0, 1, 17, 31, 42, 63])


@pytest.mark.parametrize("splits", SCHEDULES)
@pytest.mark.parametrize("dtype,Hq,Hkv,Dk,Dv,S,W", [
    (torch.bfloat16, 64, 4, 128, 128, 16, 512),
    (torch.bfloat16, 32, 2, 192, 128, 4, 128),
    (torch.float16, 32, 2, 128, 128, 8, 100),
    (torch.float32, 8, 2, 64, 64, 4, 64),
])
def test_paged_decode_against_oracle(dtype, Hq, Hkv, Dk, Dv, S, W, splits):
    """The paged kernels (one workgroup per pair and split) against the oracle, not only against the
    contiguous kernels: shuffled page pool, ragged contexts across page boundaries."""
    _check(dtype, [2048, 1000, 513, 65, 64, 33, 1], Hq, Hkv, Dk, Dv, S, W, seed=135, splits=splits, paged=True)


def test_paged_decode_cfg5_batch_one_workgroup():
    """ctx 32768 per sequence on the paged one-workgroup kernel (batch 68 -> 272 pairs by default dispatch)."""
    _check(torch.bfloat16, [32768] * 66 + [32767, 20000], 64, 4, 128, 128, 16, 512, seed=136, which=[0, 33, 66, 67],
           paged=True)


@pytest.mark.parametrize("splits", [None, 1, 3])
@pytest.mark.parametrize("dtype,Hq,Hkv,Dk,Dv,S,W,paged", [
    (torch.bfloat16, 32, 1, 128, 128, 8, 128, False),
    (torch.float16, 64, 2, 64, 64, 4, 100, False),
    (torch.bfloat16, 96, 2, 192, 128, 16, 512, True),
    (torch.bfloat16, 64, 1, 128, 128, 6, 64, True),
    (torch.float32, 32, 1, 64, 64, 4, 0, False),
])
def test_decode_groups_of_32_48_64_heads(dtype, Hq, Hkv, Dk, Dv, S, W, paged, splits):
    """GQA groups beyond 16 heads (the reference admits every multiple of 16, nsa/selection_attn.py:800): each 16
    heads run as a pair of their own on the kv head's caches, the picks come from the importance of the whole
    group (compare_selection checks them against the oracle's sum over all heads)."""
    _check(dtype, [2048, 1000, 513, 65, 33, 1], Hq, Hkv, Dk, Dv, S, W, seed=140, splits=splits, paged=paged)


def test_decode_big_group_long_context_and_refusal():
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    _check(torch.bfloat16, [40000, 12345], 32, 1, 128, 128, 16, 512, seed=141)
    cache = NSADecodeCache(1, 256, 1, 64, 64, device=DEV)
    cache.fill(torch.zeros(1, 256, 1, 64, dtype=torch.bfloat16, device=DEV),
               torch.zeros(1, 256, 1, 64, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(NotImplementedError):
        nsa_decode_step(torch.zeros(1, 32, 64, dtype=torch.bfloat16, device=DEV), cache, splits=0)
    with pytest.raises(RuntimeError):        # a group of 24 heads is neither <= 16 nor a multiple of 16
        nsa_decode_step(torch.zeros(1, 24, 64, dtype=torch.bfloat16, device=DEV), cache)


@pytest.mark.parametrize("ctx", [65536, 131072])
def test_decode_long_context(ctx):
    """Caches beyond what one workgroup keeps in registers (2304 compressed rows) run on the sliced schedule."""
    _check(torch.bfloat16, [ctx, ctx - 37], 64, 4, 128, 128, 16, 512, seed=137)


def test_decode_long_context_large_batch_and_paged():
    """66 pairs of 49152 tokens: beyond the register kernel, above the small-batch threshold; then paged."""
    _check(torch.bfloat16, [49152] * 33, 32, 2, 64, 64, 16, 512, seed=138, which=[0, 16, 32])
    _check(torch.bfloat16, [49152, 40000], 32, 2, 64, 64, 16, 512, seed=139, paged=True)


def test_decode_equals_last_prefill_row_on_gpu():
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    from nsa_amd.nsa import NSAAttention
    T, Hq, Hkv, D, S, W = 2048, 64, 4, 128, 16, 512
    dtype = torch.bfloat16
    q = randn(T, Hq, D, seed=140, scale=0.5, dtype=dtype)
    k = randn(T, Hkv, D, seed=141, scale=0.5, dtype=dtype)
    v = randn(T, Hkv, D, seed=142, scale=0.5, dtype=dtype)
    gl = randn(T, Hq, 3, seed=143, dtype=dtype)
    m = NSAAttention(D, True, selected_block_count=S, sliding_window=W, dtype=dtype, compressor_mode="mean",
                     gate_activation="sigmoid").to(DEV)
    cu = torch.tensor([0, T], dtype=torch.int32, device=DEV)
    full, idx_full = m(q.to(DEV), k.to(DEV), v.to(DEV), cu, 0, gates=gl.to(DEV), return_indices=True)
    cache = NSADecodeCache(1, T, Hkv, D, D, dtype=dtype, device=DEV)
    cache.fill(k[None].to(DEV), v[None].to(DEV))
    out, idx = nsa_decode_step(q[-1:].to(DEV), cache, gl[-1:].to(DEV), 64, S, W, gate_activation="sigmoid",
                               return_indices=True)
    assert torch.equal(idx[0].sort(-1).values.cpu(), idx_full[-1].sort(-1).values.cpu().int())
    err = max_abs(out[0], full[-1])
    print("decode vs prefill last row max_abs", err)
    assert err <= 2e-2


def test_cache_append_matches_bulk_fill():
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    B, T0, steps, Hkv, Dk, Dv = 3, 100, 45, 2, 64, 64
    dtype = torch.bfloat16
    k = randn(B, T0 + steps, Hkv, Dk, seed=150, dtype=dtype).to(DEV)
    v = randn(B, T0 + steps, Hkv, Dv, seed=151, dtype=dtype).to(DEV)
    inc = NSADecodeCache(B, T0 + steps, Hkv, Dk, Dv, dtype=dtype, device=DEV)
    inc.fill(k[:, :T0], v[:, :T0])
    for s in range(steps):
        inc.append(k[:, T0 + s], v[:, T0 + s])
    ref = NSADecodeCache(B, T0 + steps, Hkv, Dk, Dv, dtype=dtype, device=DEV)
    ref.fill(k, v)
    assert torch.equal(inc.ctx_lens, ref.ctx_lens)
    assert torch.equal(inc.k, ref.k) and torch.equal(inc.vt, ref.vt)
    assert max_abs(inc.ck, ref.ck) <= 4e-3 and max_abs(inc.cvt, ref.cvt) <= 4e-3
    # and the caches are usable: a decode step on both gives the same result
    q = randn(B, 8, Dk, seed=152, dtype=dtype).to(DEV)
    a = nsa_decode_step(q, inc, None, 64, 2, 32)
    b = nsa_decode_step(q, ref, None, 64, 2, 32)
    assert max_abs(a, b) <= 2e-2


def test_decode_one_workgroup_kernel_rejects_what_it_cannot_hold():
    """The register kernel refuses caches beyond its 2304 compressed rows and pooling geometries that make more
    bins than it holds (half the compressed rows: a 16-token selection block at stride 16 = windows of 2 every 1)."""
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    cache = NSADecodeCache(1, 65536, 1, 64, 64, dtype=torch.bfloat16, device=DEV)
    q = torch.zeros(1, 4, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(NotImplementedError):
        nsa_decode_step(q, cache, splits=0)
    small = NSADecodeCache(1, 4096, 1, 64, 64, dtype=torch.bfloat16, device=DEV)
    nsa_decode_step(q, small, selection_block=32, splits=0)  # its wide build (oracle cases below)
    nsa_decode_step(q, small, selection_block=32)            # the split schedule (oracle cases below)


@pytest.mark.parametrize("splits", [None, 0, 1, 5])
@pytest.mark.parametrize("dtype,Hq,Hkv,Dk,Dv,S,W,sel_block,paged", [
    (torch.bfloat16, 16, 1, 128, 128, 8, 128, 32, False),
    (torch.float16, 32, 2, 64, 64, 16, 100, 32, True),
    (torch.bfloat16, 8, 2, 192, 128, 4, 64, 128, False),
    (torch.bfloat16, 64, 2, 128, 128, 6, 0, 32, False),
    (torch.float32, 4, 1, 64, 64, 3, 32, 96, True),
])
def test_decode_other_selection_block_sizes(dtype, Hq, Hkv, Dk, Dv, S, W, sel_block, paged, splits):
    """Selection blocks of 32 keys (the reference's own selection test, tests/test_parallel_nsa.py:169; pooling
    windows of 3 every 2, twice the bins of the default: the wide build of the one-workgroup kernel), 96 and 128
    keys, on both schedules (windows of s + 1 rows every s, s = 1, 2, 4, 8, go to the bins as runs of rows of equal
    bin, others row by row)."""
    if splits == 0 and Hq // Hkv > 16:
        pytest.skip("the one-workgroup kernel takes groups of at most 16 heads")
    _check(dtype, [2048, 1000, 513, 100, 65, 33, 1], Hq, Hkv, Dk, Dv, S, W, seed=150, splits=splits, paged=paged,
           sel_block=sel_block)


@pytest.mark.parametrize("splits", [None, 0, 3])
@pytest.mark.parametrize("dtype,Hq,Hkv,Dk,Dv,S,W,block,stride,sel_block,paged", [
    (torch.bfloat16, 16, 1, 128, 128, 8, 128, 64, 16, 64, False),       # pooling windows of 5 every 4, padding 2
    (torch.float16, 32, 2, 64, 64, 4, 100, 64, 16, 64, True),
    (torch.bfloat16, 8, 2, 192, 128, 4, 64, 64, 16, 128, False),        # 9 every 8, padding 2
    (torch.float32, 4, 1, 64, 64, 3, 32, 64, 32, 64, False),            # 3 every 2, stride 32
])
def test_decode_other_compression_geometries(dtype, Hq, Hkv, Dk, Dv, S, W, block, stride, sel_block, paged, splits):
    """Compression blocks of 64 tokens (what the reference's own compression benchmark uses,
    tests/benchmark_compression_kv_bwd.py:9) pad the pooled row by block / stride - 2 columns: both decode
    schedules against the oracle."""
    _check(dtype, [2048, 1000, 513, 100, 65, 33, 1], Hq, Hkv, Dk, Dv, S, W, seed=155, splits=splits, paged=paged,
           sel_block=sel_block, block=block, stride=stride)


def test_decode_selection_block_32_long_context():
    _check(torch.bfloat16, [50000, 20001], 16, 1, 128, 128, 16, 512, seed=151, sel_block=32)
    _check(torch.bfloat16, [3000] * 70, 16, 1, 64, 64, 4, 64, seed=152, sel_block=32, which=[0, 69])   # 70 pairs: one workgroup each
    _check(torch.bfloat16, [3000] * 70, 16, 1, 64, 64, 4, 64, seed=153, sel_block=32, which=[1, 68], splits=1)


def test_cache_append_beyond_capacity_raises():
    from nsa_amd.decode import NSADecodeCache
    cache = NSADecodeCache(2, 64, 1, 64, 64, dtype=torch.bfloat16, device=DEV)
    k = randn(2, 63, 1, 64, seed=160, dtype=torch.bfloat16).to(DEV)
    cache.fill(k, k)
    cache.append(k[:, 0], k[:, 0])
    with pytest.raises(RuntimeError):
        cache.append(k[:, 0], k[:, 0])
    assert int(cache.ctx_lens.max()) == 64


def test_decode_randomized_sweep():
    """Seeded sweep over ragged context lengths, group sizes, top-n and window, both dtypes."""
    g = torch.Generator().manual_seed(77)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=g))]

    for case in range(20):
        B = pick([1, 2, 3, 5])
        ctxs = [int(torch.randint(1, 900, (1,), generator=g)) for _ in range(B)]
        if case % 5 == 0:
            ctxs[0] = pick([1, 31, 32, 33, 63, 64, 65, 95, 96, 127, 128])
        G, Hkv = pick([1, 2, 4, 8, 16]), pick([1, 2])
        D = pick([64, 128])
        S, W = pick([1, 3, 4, 16]), pick([1, 17, 64, 128, 512])
        dtype = pick([torch.bfloat16, torch.float32])
        if dtype == torch.float32 and D == 128 and G == 16:
            G = 4                                  # keep the sweep to shapes every dtype is built for
        print("case", case, ctxs, G, Hkv, D, S, W, dtype)
        _check(dtype, ctxs, G * Hkv, Hkv, D, D, S, W, seed=400 + case, splits=[None, 0][case % 2],
               paged=case % 3 == 2)


def test_decode_randomized_sweep_split_schedule_only_shapes():
    """The same sweep over what only the split schedule serves: GQA groups of 32 and 48 heads, selection blocks
    of 32, 96 and 128 keys (128 also runs on the one-workgroup kernel; here with explicit split counts)."""
    g = torch.Generator().manual_seed(78)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=g))]

    for case in range(16):
        B = pick([1, 2, 3, 5])
        ctxs = [int(torch.randint(1, 1500, (1,), generator=g)) for _ in range(B)]
        if case % 4 == 0:
            ctxs[0] = pick([1, 31, 32, 33, 47, 48, 63, 64, 65, 95, 96, 127, 128, 129])
        G, Hkv = pick([2, 8, 16, 32, 48]), pick([1, 2])
        sel_block = pick([32, 32, 96, 128]) if G <= 16 else pick([32, 64])
        D = pick([64, 128])
        S, W = pick([1, 3, 4, 16]), pick([0, 17, 64, 512])
        dtype = pick([torch.bfloat16, torch.float16])
        print("case", case, ctxs, G, Hkv, D, S, W, sel_block, dtype)
        _check(dtype, ctxs, G * Hkv, Hkv, D, D, S, W, seed=500 + case, splits=[None, 1, 2, 7][case % 4],
               paged=case % 3 == 1, sel_block=sel_block)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("splits", [1, 2, 3, 8, 16])
def test_split_step_equals_one_workgroup_step(dtype, splits):
    """The small-batch schedule (work of a pair spread over `splits` workgroups, three launches) against
    the one-workgroup kernel: same block picks, outputs equal up to the order of fp32 sums."""
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    ctxs = [2048, 1500, 1025, 513, 96, 64, 33, 31, 5, 1]
    B, T = len(ctxs), max(ctxs)
    Hq, Hkv, D, S, W = 32, 2, 128, 4, 128
    q, k, v, gl = _make(B, T, Hq, Hkv, D, D, 900, dtype)
    cache = NSADecodeCache(B, T, Hkv, D, D, dtype=dtype, device=DEV)
    cache.fill(k.to(DEV), v.to(DEV))
    cache.ctx_lens.copy_(torch.tensor(ctxs, dtype=torch.int32))
    kw = dict(selection_block=64, selected_block_count=S, sliding_window=W, gate_activation="sigmoid",
              return_indices=True)
    ref, ref_idx = nsa_decode_step(q.to(DEV), cache, gl.to(DEV), splits=0, **kw)
    out, idx = nsa_decode_step(q.to(DEV), cache, gl.to(DEV), splits=splits, **kw)
    assert torch.equal(idx, ref_idx)
    err = max_abs(out, ref)
    print("split", splits, dtype, "max_abs vs one workgroup", err)
    assert err <= (1e-5 if dtype == torch.float32 else 8e-3)


def test_split_step_long_context_and_paged():
    """ctx 32768 (2047 compressed rows, every slice and bin boundary in use), contiguous and paged, group 16."""
    import random
    from nsa_amd.decode import NSADecodeCache, NSAPagedDecodeCache, nsa_decode_step
    B, T, Hq, Hkv, D = 2, 32768, 64, 4, 128
    dtype = torch.bfloat16
    q, k, v, gl = _make(B, T, Hq, Hkv, D, D, 910, dtype)
    flat = NSADecodeCache(B, T, Hkv, D, D, dtype=dtype, device=DEV)
    flat.fill(k.to(DEV), v.to(DEV))
    paged = NSAPagedDecodeCache(B, B * T // 64, T, Hkv, D, D, dtype=dtype, device=DEV)
    random.Random(5).shuffle(paged._free)
    paged.fill(k.to(DEV), v.to(DEV))
    kw = dict(selection_block=64, selected_block_count=16, sliding_window=512, gate_activation="sigmoid",
              return_indices=True)
    ref, ref_idx = nsa_decode_step(q.to(DEV), flat, gl.to(DEV), splits=0, **kw)
    for cache in (flat, paged):
        for splits in (6, 8):
            out, idx = nsa_decode_step(q.to(DEV), cache, gl.to(DEV), splits=splits, **kw)
            assert torch.equal(idx, ref_idx)
            assert max_abs(out, ref) <= 8e-3
    auto, _ = nsa_decode_step(q.to(DEV), flat, gl.to(DEV), **kw)           # 8 pairs: the split path by default
    assert max_abs(auto, ref) <= 8e-3


@pytest.mark.parametrize("S,W", [(1, 0), (64, 0), (64, 2048), (16, 1)])
def test_split_step_extreme_selection_and_window(S, W):
    """No window at all, one pick, more picks than blocks, a window longer than the context."""
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    ctxs = [1999, 640, 70]
    B, T, Hq, Hkv, D = len(ctxs), max(ctxs), 16, 2, 64
    dtype = torch.float32
    q, k, v, gl = _make(B, T, Hq, Hkv, D, D, 920, dtype)
    cache = NSADecodeCache(B, T, Hkv, D, D, dtype=dtype, device=DEV)
    cache.fill(k.to(DEV), v.to(DEV))
    cache.ctx_lens.copy_(torch.tensor(ctxs, dtype=torch.int32))
    kw = dict(selection_block=64, selected_block_count=S, sliding_window=W, return_indices=True)
    ref, ref_idx = nsa_decode_step(q.to(DEV), cache, gl.to(DEV), splits=0, **kw)
    out, idx = nsa_decode_step(q.to(DEV), cache, gl.to(DEV), splits=8, **kw)
    assert torch.equal(idx, ref_idx)
    assert torch.isfinite(out).all() and max_abs(out, ref) <= 1e-5
