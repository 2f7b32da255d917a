"""GPU parity: every kernel is called through the C ABI (via the thin ctypes wrappers) and compared
with the CPU oracle on the same seeded inputs.  Bars: bf16 max-abs <= 2e-2, fp32 <= 1e-4, selected
block sets identical except where the oracle's scores tie within 1e-3."""
import math
import random

import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import ROW_TOL, TOL, make_qkv, max_abs, ragged_cu, randn, sample_rows, within

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _ops():
    from nsa_amd import ops
    return ops


def _cu(lens):
    return torch.tensor(ragged_cu(lens), dtype=torch.int32, device=DEV)


# ------------------------------------------------------------------------------ compression
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("lens,H,D,l,d", [([1024], 1, 64, 32, 16), ([300, 31, 64, 1000], 4, 128, 32, 16),
                                          ([200, 77], 2, 192, 64, 16)])
def test_compress_mean(dtype, lens, H, D, l, d):
    ops = _ops()
    x = randn(sum(lens), H, D, seed=1, dtype=dtype)
    cu = _cu(lens)
    cu_out = ops.compressed_offsets(cu, l, d, extra=1)
    ncs = [O.compressed_len_conv(t, l, d) for t in lens]
    assert cu_out.cpu().tolist() == ragged_cu(ncs)
    out = ops.compress(x.to(DEV), cu, cu_out, sum(ncs), l, d)
    ref = torch.cat([O.compress_meanpool(x[s:e], l, d, n) for s, e, n in
                     zip(ragged_cu(lens)[:-1], ragged_cu(lens)[1:], ncs)])
    err = max_abs(out, ref)
    print("compress_mean", dtype, lens, "max_abs", err)
    assert err <= ROW_TOL[dtype]
    # closed form on the first sequence
    if ncs[0] > 0:
        cf = x[:lens[0]].float().unfold(0, l, d).mean(-1).to(dtype)
        assert max_abs(out[:ncs[0]], cf) <= ROW_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("lens,H,Dk,Dv,l,d", [([1024], 1, 64, 64, 32, 16), ([300, 31, 64, 1000], 4, 192, 128, 32, 16),
                                              ([200, 77], 2, 64, 128, 40, 8), ([31], 2, 32, 32, 32, 16),
                                              ([300, 17, 16, 1000, 33], 4, 128, 64, 16, 8),
                                              ([100, 45], 1, 32, 32, 32, 16)])
def test_compress_kv_pair(dtype, lens, H, Dk, Dv, l, d):
    """K and V through the paired entry point (one launch for mean pooling, head dims may differ, windows that
    are not a multiple of the kernel's load round, a sequence with no compressed row) against the oracle, and
    bit-identical to the one-tensor entry point."""
    ops = _ops()
    k = randn(sum(lens), H, Dk, seed=1, dtype=dtype)
    v = randn(sum(lens), H, Dv, seed=2, dtype=dtype)
    cu = _cu(lens)
    cu_out = ops.compressed_offsets(cu, l, d, extra=1)
    ncs = [O.compressed_len_conv(t, l, d) for t in lens]
    ck, cv = ops.compress_kv(k.to(DEV), v.to(DEV), cu, cu_out, sum(ncs), l, d)
    assert ck.shape == (sum(ncs), H, Dk) and cv.shape == (sum(ncs), H, Dv)
    if sum(ncs) == 0:
        return
    for x, got in ((k, ck), (v, cv)):
        ref = torch.cat([O.compress_meanpool(x[s:e], l, d, n) for s, e, n in
                         zip(ragged_cu(lens)[:-1], ragged_cu(lens)[1:], ncs)])
        assert max_abs(got, ref) <= ROW_TOL[dtype]
        assert torch.equal(got, ops.compress(x.to(DEV), cu, cu_out, sum(ncs), l, d))
    # learned compressor through the same entry point: the two GEMM launches
    if Dk == Dv and l == 32:
        wk = randn(l * Dk, Dk, seed=3, dtype=dtype, scale=0.05)
        wv = randn(l * Dv, Dv, seed=4, dtype=dtype, scale=0.05)
        ck2, cv2 = ops.compress_kv(k.to(DEV), v.to(DEV), cu, cu_out, sum(ncs), l, d, wk.t().contiguous().to(DEV),
                                   wv.t().contiguous().to(DEV))
        # (the GEMM adds its split-K partial sums in LDS in whatever order they arrive: equal up to rounding)
        tol = 1e-5 if dtype == torch.float32 else TOL[dtype]      # one unit in the last place of an O(1) value
        assert max_abs(ck2, ops.compress(k.to(DEV), cu, cu_out, sum(ncs), l, d, wk.t().contiguous().to(DEV))) <= tol
        assert max_abs(cv2, ops.compress(v.to(DEV), cu, cu_out, sum(ncs), l, d, wv.t().contiguous().to(DEV))) <= tol


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("lens,H,D,l,d,extra", [([256, 100], 2, 64, 32, 16, 1), ([1024] * 2, 2, 128, 64, 16, 0),
                                                ([90], 1, 32, 8, 4, 1)])
def test_compress_weighted(dtype, lens, H, D, l, d, extra):
    ops = _ops()
    x = randn(sum(lens), H, D, seed=2, dtype=dtype)
    w_lin = randn(l * D, D, seed=3, scale=1.0 / math.sqrt(l * D), dtype=dtype)
    bias = randn(D, seed=4, dtype=dtype) if extra else None
    cu = _cu(lens)
    cu_out = ops.compressed_offsets(cu, l, d, extra=extra)
    ncs = [O.compressed_len_conv(t, l, d) if extra else O.compressed_len_functional(t, l, d) for t in lens]
    assert cu_out.cpu().tolist() == ragged_cu(ncs)
    out = ops.compress(x.to(DEV), cu, cu_out, sum(ncs), l, d, w_lin.t().contiguous().to(DEV),
                       None if bias is None else bias.to(DEV))
    ref = torch.cat([O.compress_weighted(x[s:e], w_lin, bias, l, d, n) for s, e, n in
                     zip(ragged_cu(lens)[:-1], ragged_cu(lens)[1:], ncs)])
    err = max_abs(out, ref)
    print("compress_weighted", dtype, lens, "max_abs", err)
    assert err <= TOL[dtype]


def test_transpose_layout():
    ops = _ops()
    lens = [70, 5, 129]
    x = randn(sum(lens), 3, 64, seed=5, dtype=torch.bfloat16)
    cu = _cu(lens)
    out = ops.transpose(x.to(DEV), cu, len(lens)).cpu()
    from nsa_amd import _lib
    lib = _lib.load()
    cuh = ragged_cu(lens)
    seen = torch.zeros(out.shape[-1], dtype=torch.bool)
    for b, (s, e) in enumerate(zip(cuh[:-1], cuh[1:])):
        off = lib.nsa_transposed_offset(s, b)
        assert off % 8 == 0
        assert torch.equal(out[:, :, off:off + e - s], x[s:e].permute(1, 2, 0))
        seen[off:off + e - s] = True
    assert torch.count_nonzero(out[:, :, ~seen]) == 0


# ------------------------------------------------------------------------------ compressed attention + selection
def _cmp_case(dtype, lens, Hq, Hkv, Dk, Dv, l, d, lsel, S, seed, scale_in=1.0, late_key_scale=None, min_exact=0.99,
              key_scale_range=None, softmax_scale=None):
    ops = _ops()
    p = O.NSAParams(l, d, lsel, S, 0)
    T = sum(lens)
    q, k, v, _ = make_qkv(T, Hq, Hkv, Dk, Dv, seed, dtype, scale_in)
    if late_key_scale is not None:          # keys of the later half of the packed tokens blown up
        k = k.clone()
        k[T // 2:] *= late_key_scale
    if key_scale_range is not None:         # (first token, end token, factor)
        k = k.clone()
        k[key_scale_range[0]:key_scale_range[1]] *= key_scale_range[2]
    cu = _cu(lens)
    cu_cmp = ops.compressed_offsets(cu, l, d, extra=1)
    ncs = [O.compressed_len_conv(t, l, d) for t in lens]
    ck = ops.compress(k.to(DEV), cu, cu_cmp, sum(ncs), l, d)
    cv = ops.compress(v.to(DEV), cu, cu_cmp, sum(ncs), l, d)
    cvt = ops.transpose(cv, cu_cmp, len(lens))
    scale = 1.0 / math.sqrt(Dk) if softmax_scale is None else softmax_scale
    o, idx, pooled = ops.cmp_attn_select(q.to(DEV), ck, cvt, cu, cu_cmp, len(lens), Hkv, Dv, ck.stride(0),
                                         ck.stride(1), l, d, p.pool_kernel, p.pool_stride, p.pool_pad, S,
                                         max(ncs), scale, want_pooled=True)
    torch.cuda.synchronize()
    worst = _cmp_check(dtype, lens, ncs, q, ck, cv, o.cpu(), idx.cpu(), pooled.cpu(), p, l, d, S, scale, scale_in,
                       min_exact, "cmp (three launches)", (Hq, Hkv, Dk, Dv))
    # the same through the one-call entry point; shapes that qualify run there as ONE kernel (one pass over the
    # compressed keys, window sums kept per head in registers), everything else as the three launches above
    r = ops.cmp_select(q.to(DEV), ck, cvt, cu, cu_cmp, len(lens), Hkv, Dv, ck.stride(0), ck.stride(1), l, d,
                       p.pool_kernel, p.pool_stride, p.pool_pad, S, max(ncs), scale, idx64=True, want_pooled=True,
                       want_lse_attn=True, frag=ops.cmp_pack(ck, cv, cu_cmp, len(lens)) if dtype != torch.float32 and
                       (Dk, Dv) in ((64, 64), (128, 128), (192, 128)) else None)
    torch.cuda.synchronize()
    if r["single_pass"]:
        w2 = _cmp_check(dtype, lens, ncs, q, ck, cv, r["o"].cpu(), r["indices"].cpu(), r["pooled"].cpu(), p, l, d, S,
                        scale, scale_in, min_exact, "cmp (single pass)", (Hq, Hkv, Dk, Dv))
        worst = {k: max(worst[k], w2[k]) if k in ("o", "pooled", "fail") else worst[k] for k in worst}
        # log-sum-exp of the scaled visible scores, as the three-launch schedule writes it for the backward
        ref_lse = ops.cmp_attn(q.to(DEV), ck, cvt, cu, cu_cmp, len(lens), Hkv, Dv, ck.stride(0), ck.stride(1), l, d, scale,
                               want_lse_attn=True)[2]
        fin = torch.isfinite(ref_lse)
        assert torch.equal(fin, torch.isfinite(r["lse_attn"]))
        assert float((ref_lse[fin] - r["lse_attn"][fin]).abs().max()) <= 2e-3 if fin.any() else True
    else:
        assert torch.equal(r["o"].cpu(), o.cpu()) and torch.equal(r["indices"].cpu(), idx.cpu())
    return worst


def _cmp_check(dtype, lens, ncs, q, ck, cv, o, idx, pooled, p, l, d, S, scale, scale_in, min_exact, what, shape):
    cuh, cuc = ragged_cu(lens), ragged_cu(ncs)
    worst = dict(o=0.0, pooled=0.0, rows=0, exact=0, excused=0, fail=0)
    for b in range(len(lens)):
        s, e = cuh[b], cuh[b + 1]
        ckb, cvb = ck[cuc[b]:cuc[b + 1]].cpu(), cv[cuc[b]:cuc[b + 1]].cpu()
        if ncs[b] == 0:
            assert torch.count_nonzero(o[s:e]) == 0
            assert (idx[s:e] == -1).all()
            continue
        ref_o = O.compressed_attention(q[s:e], ckb, cvb, l, d, scale)
        worst["o"] = max(worst["o"], max_abs(o[s:e], ref_o))
        assert torch.count_nonzero(o[s:s + min(l, e - s)]) == 0          # rows that see nothing
        ref_p = O.importance_scores(q[s:e], ckb, p.pool_kernel, p.pool_stride, p.pool_pad)
        Ns = ref_p.shape[-1]
        if Ns == 0:
            assert (idx[s:e] == -1).all()
            continue
        worst["pooled"] = max(worst["pooled"], max_abs(pooled[s:e, :, :Ns], ref_p))
        ref_idx = O.select_blocks(ref_p, S)
        n, ex, exc, fail = O.compare_selection(idx[s:e], ref_idx, ref_p, 1e-3)
        worst["rows"] += n; worst["exact"] += ex; worst["excused"] += exc; worst["fail"] += fail
        # descending order of the kernel's own scores
        got = torch.gather(pooled[s:e, :, :Ns], 2, idx[s:e].clamp(min=0))
        got = torch.where(idx[s:e] >= 0, got, torch.full_like(got, -1.0))
        assert (got[..., :-1] >= got[..., 1:]).all()
    print(what, dtype, lens, shape, worst)
    assert worst["o"] <= TOL[dtype] * max(1.0, scale_in)      # |v| grows with scale_in, and with it one bf16 ulp of o
    assert worst["pooled"] <= 1e-3
    assert worst["fail"] == 0
    assert worst["exact"] >= min_exact * worst["rows"]   # the tie rule is for the remainder, not a hiding place
    return worst


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_cmp_select_cfg1_shape(dtype):
    _cmp_case(dtype, [1024], 4, 1, 64, 64, 32, 16, 64, 4, seed=0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_cmp_select_g16(dtype):
    _cmp_case(dtype, [2048], 32, 2, 128, 128, 32, 16, 64, 16, seed=10, scale_in=0.5)


def test_cmp_select_dqk192_ragged():
    _cmp_case(torch.bfloat16, [700, 31, 1055, 64, 1000], 32, 2, 192, 128, 32, 16, 64, 4, seed=20, scale_in=0.5)


def test_cmp_select_block64_padded_pool():
    # l=64,d=16 -> pool kernel 5 stride 4 pad 2 (padding counted in the divisor)
    _cmp_case(torch.bfloat16, [1024, 333], 16, 1, 64, 64, 64, 16, 64, 4, seed=30)


@pytest.mark.parametrize("dtype,lens,Hq,Hkv,Dk,Dv,l,d,lsel,S", [
    (torch.bfloat16, [2100, 333, 70, 1], 64, 4, 128, 128, 64, 16, 64, 16),     # windows of 5 every 4, padding 2
    (torch.float16, [1500, 65], 32, 2, 192, 128, 32, 8, 64, 8),                # 9 every 8, padding 2
    (torch.bfloat16, [1024, 40], 16, 1, 64, 64, 32, 8, 32, 4),                 # 5 every 4, padding 2, stride 8
    (torch.bfloat16, [1300, 257, 31], 16, 2, 128, 128, 32, 16, 16, 16),        # 2 every 1 (16-key selection blocks)
    (torch.bfloat16, [900, 100], 8, 2, 64, 64, 32, 16, 16, 5),                 # 2 every 1, two tokens per tile
    (torch.bfloat16, [700], 4, 1, 128, 128, 64, 16, 128, 3),                   # 9 every 8, padding 2, four tokens per tile
    (torch.bfloat16, [1200, 90], 64, 2, 128, 128, 64, 16, 32, 6),              # a group of 32 heads, 3 every 2, padding 2
    (torch.float32, [800, 130], 16, 1, 64, 64, 64, 16, 64, 4),
])
def test_cmp_select_other_pooling_geometries(dtype, lens, Hq, Hkv, Dk, Dv, l, d, lsel, S):
    """Compression blocks beyond two strides pad the pooled row (pool_pad = block / stride - 2 columns on either
    side, counted in the divisor); selection blocks of one stride pool windows of 2 columns every column.  Both run
    on the two-kernel selection with the stream shifted by the padding."""
    _cmp_case(dtype, lens, Hq, Hkv, Dk, Dv, l, d, lsel, S, seed=60, scale_in=0.5)


def test_cmp_select_groups_of_32_48_64_heads():
    """GQA groups the reference's selected attention takes (HQ a multiple of 16 * H, nsa/selection_attn.py:800):
    sub-groups of 16 heads share the compressed keys; the block scores are the sum over all heads of the group."""
    _cmp_case(torch.bfloat16, [1500, 200], 64, 2, 128, 128, 32, 16, 64, 16, seed=43, scale_in=0.5)    # G=32
    _cmp_case(torch.bfloat16, [1024], 48, 1, 64, 64, 32, 16, 64, 4, seed=44, scale_in=0.5)            # G=48
    _cmp_case(torch.float32, [700], 64, 1, 64, 64, 32, 16, 64, 8, seed=45, scale_in=0.5)              # G=64, fp32
    _cmp_case(torch.bfloat16, [2048], 64, 2, 192, 128, 32, 16, 64, 16, seed=46, scale_in=0.5)         # G=32, Dqk 192


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_cmp_select_scores_beyond_the_fixed_reference(dtype):
    """Inputs on which the kernel's common pass (one fixed softmax reference per row) must give way to its exact
    pass: raw scores spread over hundreds of units, so exponentials against an early reference overflow; and keys
    whose later half is 200 times larger, so that rows in the first half see only scores ~1000 below the largest
    hidden one (a softmax referenced to the hidden maximum would return 0 for them)."""
    # near one-hot softmaxes leave most bins at (almost) exactly 0: many genuine ties, so only the tie rule applies
    _cmp_case(dtype, [1024, 300], 32, 2, 64, 64, 32, 16, 64, 4, seed=47, scale_in=8.0, min_exact=0.0)
    _cmp_case(dtype, [1024], 16, 1, 128, 128, 32, 16, 64, 16, seed=48, scale_in=1.0, late_key_scale=200.0, min_exact=0.0)
    _cmp_case(dtype, [2048], 64, 4, 192 if dtype == torch.bfloat16 else 128, 128, 32, 16, 64, 16, seed=49, scale_in=3.0,
              min_exact=0.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_cmp_select_scores_between_the_float16_and_float32_ranges(dtype):
    """Probabilities against the fixed reference that an fp32 sum holds easily and a float16 operand does not.  With
    a softmax scale of 1 the attention logits are the raw scores, so the importance sum (fp32, overflows only 69 nats
    above the reference) raises no alarm.  (a) Later keys 6.5 times larger: visible logits 15-40 nats above the largest
    score of the first 32 compressed rows, probabilities of 1e7..1e17 -- infinite as float16.  (b) Keys of tokens
    288..543 (compressed rows 17..32) 6 times larger: tokens below 288 see none of them, yet their reference is the
    maximum over rows 0..31, so their visible probabilities are ~1e-9 -- zero as float16.  Both must come out as
    under a running maximum (nsa/torch_attention.py:126-148)."""
    a = _cmp_case(dtype, [1024, 200], 16, 1, 64, 64, 32, 16, 64, 4, seed=51, scale_in=1.0, softmax_scale=1.0,
                  key_scale_range=(512, 1024, 6.5), min_exact=0.0)
    b = _cmp_case(dtype, [1024], 32, 2, 64, 64, 32, 16, 64, 4, seed=52, scale_in=1.0, softmax_scale=1.0,
                  key_scale_range=(288, 544, 6.0), min_exact=0.0)
    # head dim 32: sqrt(32) = 5.7 raw units per nat, so a visible logit 11.1-12.2 nats above the reference overflows
    # float16 (> 65504) while the raw-score exponential stays below the fp32 alarm
    c = _cmp_case(dtype, [1024], 16, 1, 32, 32, 32, 16, 64, 4, seed=53, scale_in=1.0, key_scale_range=(512, 1024, 14.5),
                  min_exact=0.0)
    assert all(math.isfinite(w["o"]) for w in (a, b, c))


def test_cmp_select_odd_groups():
    _cmp_case(torch.float32, [500], 6, 2, 64, 64, 32, 16, 64, 2, seed=40)      # G=3 -> padded to 4
    _cmp_case(torch.float32, [500], 8, 1, 32, 32, 32, 16, 64, 2, seed=41)      # G=8
    _cmp_case(torch.float32, [300], 2, 2, 32, 32, 32, 16, 64, 2, seed=42)      # G=1


# ------------------------------------------------------------------------------ sliding window
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("lens,Hq,Hkv,Dk,Dv,W", [([1024], 4, 1, 64, 64, 128), ([777, 40, 513], 32, 2, 128, 128, 512),
                                                 ([600], 16, 1, 192, 128, 100), ([130], 8, 2, 32, 32, 1),
                                                 ([300], 6, 2, 64, 64, 1000), ([500, 77], 64, 2, 128, 128, 128),
                                                 ([300], 48, 1, 64, 64, 64)])
def test_swa(dtype, lens, Hq, Hkv, Dk, Dv, W):
    ops = _ops()
    T = sum(lens)
    q, k, v, _ = make_qkv(T, Hq, Hkv, Dk, Dv, 50, dtype, 0.7)
    cu = _cu(lens)
    vt = ops.transpose(v.to(DEV), cu, len(lens))
    scale = 1.0 / math.sqrt(Dk)
    o = ops.swa(q.to(DEV), k.to(DEV), vt, cu, len(lens), W, scale).cpu()
    cuh = ragged_cu(lens)
    err = 0.0
    for s, e in zip(cuh[:-1], cuh[1:]):
        err = max(err, max_abs(o[s:e], O.sliding_attention(q[s:e], k[s:e], v[s:e], W, scale)))
    print("swa", dtype, lens, (Hq, Hkv, Dk, Dv, W), "max_abs", err)
    assert err <= TOL[dtype]


# ------------------------------------------------------------------------------ selected blocks + combine
def _random_indices(T, Hkv, S, bs, seed, poison=True):
    g = torch.Generator().manual_seed(seed)
    nblk = (T + bs - 1) // bs
    idx = torch.full((T, Hkv, S), nblk + 3, dtype=torch.int64)       # out-of-range padding
    for t in range(T):
        for h in range(Hkv):
            perm = torch.randperm(nblk, generator=g)[:S]             # past and future blocks, no duplicates
            idx[t, h, :len(perm)] = perm
    if poison:
        idx[0] = nblk + 1
        idx[T // 2, :, 0] = -5
    return idx


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("lens,Hq,Hkv,Dk,Dv,S,bs", [([256], 16, 1, 32, 32, 2, 32), ([512, 100], 32, 2, 128, 128, 8, 64),
                                                   ([384], 4, 1, 64, 64, 4, 64), ([200], 16, 1, 192, 128, 3, 64),
                                                   ([160], 6, 2, 64, 64, 3, 16), ([512, 100], 64, 2, 128, 128, 8, 64),
                                                   ([300], 48, 1, 64, 64, 3, 32),
                                                   # other selection block sizes on the 64-key schedule: parts of
                                                   # a block (8, 16, 32 keys) and several blocks per pick (128, 192)
                                                   ([300, 90], 16, 1, 64, 64, 5, 32), ([300], 8, 2, 128, 128, 4, 8),
                                                   ([700], 16, 1, 64, 64, 3, 128), ([900, 100], 32, 2, 192, 128, 2, 192),
                                                   # groups of 8, 6 and 2 heads: 2 resp. 4 pairs share a score tile
                                                   ([330, 77], 16, 2, 128, 128, 5, 64), ([300], 12, 2, 64, 64, 3, 32),
                                                   ([500], 2, 1, 192, 128, 16, 64)])
def test_slc_only(dtype, lens, Hq, Hkv, Dk, Dv, S, bs):
    ops = _ops()
    T = sum(lens)
    q, k, v, gl = make_qkv(T, Hq, Hkv, Dk, Dv, 60, dtype, 0.7)
    cu = _cu(lens)
    cuh = ragged_cu(lens)
    idx = torch.cat([_random_indices(e - s, Hkv, S, bs, 61 + s) for s, e in zip(cuh[:-1], cuh[1:])])
    g = torch.Generator().manual_seed(62)
    counts = torch.randint(0, S + 1, (T, Hkv), generator=g)
    vt = ops.transpose(v.to(DEV), cu, len(lens))
    scale = 1.0 / math.sqrt(Dk)
    has_block_major = dtype != torch.float32 and (bs in (8, 16, 32) or bs % 64 == 0) and Dk >= 64
    modes = ((False, torch.int64, False), (True, torch.int32, False)) + \
        (((False, torch.int32, True), (True, torch.int64, True)) if has_block_major else ())
    for use_counts, dt_idx, block_major in modes:
        o = ops.slc_combine(q.to(DEV), k.to(DEV), vt, idx.to(dt_idx).to(DEV),
                            counts.to(DEV) if use_counts else None, None, None, None, None, None, cu,
                            len(lens), bs, scale, block_major=block_major).cpu()
        err = 0.0
        for s, e in zip(cuh[:-1], cuh[1:]):
            ref = O.selected_attention(q[s:e], k[s:e], v[s:e], idx[s:e], counts[s:e] if use_counts else None,
                                       bs, scale)
            err = max(err, max_abs(o[s:e], ref))
            assert torch.count_nonzero(o[s]) == 0                     # poisoned row: empty selection -> 0
        print("slc", dtype, lens, (Hq, Hkv, Dk, Dv, S, bs), "counts", use_counts, "block_major", block_major,
              "max_abs", err)
        assert err <= TOL[dtype]


@pytest.mark.parametrize("lens,Hq,Hkv,Dk,Dv,S,W", [([512, 100], 32, 2, 128, 128, 8, 128), ([200], 16, 1, 192, 128, 3, 64),
                                                  ([384], 4, 1, 64, 64, 4, 512), ([700, 330], 24, 2, 64, 64, 16, 256),
                                                  ([700, 330], 64, 2, 128, 128, 16, 256), ([400], 48, 1, 192, 128, 4, 64),
                                                  ([700, 130], 16, 2, 128, 128, 16, 100), ([520], 3, 1, 64, 64, 7, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_partials_and_window_merge(lens, Hq, Hkv, Dk, Dv, S, W, dtype):
    """nsa_slc_partials_fwd + nsa_swa_merge_fwd against nsa_swa_fwd + nsa_slc_combine_fwd (token-major
    kernel) and against the oracle, with counts, invalid picks, gates and a compressed-branch input."""
    ops = _ops()
    bs = 64
    T = sum(lens)
    q, k, v, gl = make_qkv(T, Hq, Hkv, Dk, Dv, 160, dtype, 0.7)
    cu = _cu(lens)
    cuh = ragged_cu(lens)
    idx = torch.cat([_random_indices(e - s, Hkv, S, bs, 161 + s) for s, e in zip(cuh[:-1], cuh[1:])])
    counts = torch.randint(0, S + 1, (T, Hkv), generator=torch.Generator().manual_seed(162))
    o_cmp = randn(T, Hq, Dv, seed=163, dtype=dtype)
    vt = ops.transpose(v.to(DEV), cu, len(lens))
    scale = 1.0 / math.sqrt(Dk)
    gd = gl.to(DEV)
    g_slc, g_swa, g_cmp = (gd[..., i] for i in range(3))
    qd, kd = q.to(DEV), k.to(DEV)
    for use_counts, dt_idx in ((False, torch.int32), (True, torch.int64)):
        cd = counts.to(DEV) if use_counts else None
        idd = idx.to(dt_idx).to(DEV)
        ws = ops.slc_workspace(qd, Hkv, Dv, S, bs, len(lens))
        assert ws is not None
        ops.slc_partials(qd, kd, vt, idd, cd, cu, len(lens), bs, scale, ws)
        fused = ops.swa_merge(qd, kd, vt, ws, S, g_slc, g_swa, g_cmp, o_cmp.to(DEV), cu, len(lens), bs, W,
                              scale, gate_act=1).cpu()
        o_swa = ops.swa(qd, kd, vt, cu, len(lens), W, scale)
        split = ops.slc_combine(qd, kd, vt, idd, cd, g_slc, g_swa, g_cmp, o_swa, o_cmp.to(DEV), cu, len(lens), bs,
                                scale, gate_act=1, block_major=False).cpu()
        sg = torch.sigmoid(gl.float())
        err = 0.0
        for s, e in zip(cuh[:-1], cuh[1:]):
            slc = O.selected_attention(q[s:e], k[s:e], v[s:e], idx[s:e], counts[s:e] if use_counts else None, bs, scale)
            swa = O.sliding_attention(q[s:e], k[s:e], v[s:e], W, scale)
            ref = sg[s:e, :, 0:1] * slc.float() + sg[s:e, :, 1:2] * swa.float() + sg[s:e, :, 2:3] * o_cmp[s:e].float()
            err = max(err, max_abs(fused[s:e], ref))
        d = max_abs(fused, split)
        print("fused", lens, (Hq, Hkv, Dk, Dv, S, W), "counts", use_counts, "vs oracle", err, "vs split kernels", d)
        # two kernels that each round once to bf16: where |out| > 4 they may differ by one unit in the last place
        assert err <= TOL[dtype] and within(fused, split, dtype, large_values=True), (err, d)
        # the same launch can also leave what a backward pass keeps: the ungated branch outputs and their
        # log-sum-exps, equal to those of the stand-alone kernels
        out2, b_slc, b_swa, l_slc, l_swa = ops.swa_merge(qd, kd, vt, ws, S, g_slc, g_swa, g_cmp, o_cmp.to(DEV), cu,
                                                         len(lens), bs, W, scale, gate_act=1, want_branches=True)
        r_slc, rl_slc = ops.slc_combine(qd, kd, vt, idd, cd, None, None, None, None, None, cu, len(lens), bs, scale,
                                        block_major=True, want_lse=True)
        r_swa, rl_swa = ops.swa(qd, kd, vt, cu, len(lens), W, scale, want_lse=True)
        assert torch.equal(out2.cpu(), fused)
        assert torch.equal(b_slc, r_slc) and torch.equal(b_swa, r_swa) and torch.equal(l_swa, rl_swa)
        fin = torch.isfinite(rl_slc)
        assert torch.equal(fin, torch.isfinite(l_slc)) and torch.equal(l_slc[~fin], rl_slc[~fin])
        assert float((l_slc[fin] - rl_slc[fin]).abs().max()) <= 1e-5 if fin.any() else True


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_parallel_nsa_api_like_reference_test(dtype):
    """Shape of the reference's own test (B=2,T=64,H=1,HQ=16,D=32,S=2,bs=32,W=128, ones gates,
    random counts, two rows forced to an empty selection), fp16 replaced by bf16/fp32."""
    import nsa_amd
    B, T, H, HQ, D, S, bs, W = 2, 64, 1, 16, 32, 2, 32, 128
    q = randn(B, T, HQ, D, seed=70, dtype=dtype)
    k = randn(B, T, H, D, seed=71, dtype=dtype)
    v = randn(B, T, H, D, seed=72, dtype=dtype)
    g_slc = torch.ones(B, T, HQ, dtype=dtype)
    g_swa = torch.ones(B, T, HQ, dtype=dtype)
    gen = torch.Generator().manual_seed(73)
    idx = torch.full((B, T, H, S), T, dtype=torch.long)
    for b in range(B):
        for t in range(T):
            perm = torch.randperm(max(1, t // bs), generator=gen)[:S]
            idx[b, t, 0, :len(perm)] = perm
    idx = idx.sort(-1)[0]
    idx[0, 0, 0, 0] = 4
    idx[1, 63, 0, 0] = 7
    idx[1, 63, 0, 1] = 9
    counts = torch.randint(1, S + 1, (B, T, H), generator=gen)
    out = nsa_amd.selection_attention(q.to(DEV), k.to(DEV), v.to(DEV), g_slc.to(DEV), g_swa.to(DEV), idx.to(DEV),
                                      counts.to(DEV), bs, W).cpu()
    for b in range(B):
        slc, swa = O.selected_sliding_loop(q[b], k[b], v[b], idx[b], counts[b], bs, W)
        ref = slc + swa
        err = max_abs(out[b], ref)
        print("parallel_nsa", dtype, "batch", b, "max_abs", err)
        assert err <= TOL[dtype]
    # head_first and int block_counts
    out_hf = nsa_amd.parallel_nsa(q.transpose(1, 2).to(DEV), k.transpose(1, 2).to(DEV), v.transpose(1, 2).to(DEV),
                                  g_slc.transpose(1, 2).to(DEV), g_swa.transpose(1, 2).to(DEV),
                                  idx.transpose(1, 2).to(DEV), 1, bs, W, head_first=True).cpu()
    slc, swa = O.selected_sliding_loop(q[0], k[0], v[0], idx[0], 1, bs, W)
    assert max_abs(out_hf[0].transpose(0, 1), slc + swa) <= TOL[dtype]


@pytest.mark.parametrize("lens,Hq,Hkv,Dk,Dv,S,W,bs", [([3000], 16, 1, 64, 64, 8, 100, 64),
                                                     ([700, 1, 330, 64, 1500], 32, 2, 128, 128, 16, 256, 64),
                                                     ([90] * 11 + [400, 33], 64, 2, 64, 64, 4, 64, 32),
                                                     ([1200, 500], 16, 1, 192, 128, 3, 512, 128)])
def test_token_slabs_equal_one_slab(lens, Hq, Hkv, Dk, Dv, S, W, bs):
    """nsa_slc_swa_fused_fwd with a workspace for a fraction of the tokens (several slabs, slab edges inside
    sequences, more than 8 sequences, a GQA group of 32 heads, 32- and 128-key selection blocks) against the
    two-call schedule with the one-slab workspace: bit-identical outputs, branch outputs and log-sum-exps."""
    ops = _ops()
    from nsa_amd import _lib
    dtype = torch.bfloat16
    T = sum(lens)
    q, k, v, gl = make_qkv(T, Hq, Hkv, Dk, Dv, 500, dtype, 0.7)
    cu, cuh = _cu(lens), ragged_cu(lens)
    idx = torch.cat([_random_indices(e - s, Hkv, S, bs, 501 + s, poison=e - s > 2) for s, e in zip(cuh[:-1], cuh[1:])])
    g = torch.Generator().manual_seed(502)
    counts = torch.randint(0, S + 1, (T, Hkv), generator=g).to(DEV)
    qd, kd, idxd = q.to(DEV), k.to(DEV), idx.to(torch.int32).to(DEV)
    vt = ops.transpose(v.to(DEV), cu, len(lens))
    gates = [gl[..., i].contiguous().to(DEV) for i in range(3)]
    o_cmp = randn(T, Hq, Dv, seed=503, dtype=dtype).to(DEV)
    scale = 1.0 / math.sqrt(Dk)
    ws = ops.slc_workspace(qd, Hkv, Dv, S, bs, len(lens))
    ops.slc_partials(qd, kd, vt, idxd, counts, cu, len(lens), bs, scale, ws)
    ref = ops.swa_merge(qd, kd, vt, ws, S, *gates, o_cmp, cu, len(lens), bs, W, scale, gate_act=1, want_branches=True)
    lib = _lib.load()
    geom = (T, len(lens), Hq, Hkv, Dk, Dv, S, bs, 0)
    full = lib.nsa_slc_swa_fused_workspace_bytes(*geom, 0)
    assert full == ws.numel()
    for frac in (1, 3, 7):
        limit = lib.nsa_slc_swa_fused_workspace_bytes(*geom, (T + frac - 1) // frac) if frac > 1 else full
        assert frac == 1 or limit < full
        got = ops.slc_swa_fused(qd, kd, vt, idxd, counts, *gates, o_cmp, cu, len(lens), bs, W, scale, gate_act=1,
                                want_branches=True, workspace_limit=limit)
        for name, a, b in zip(("out", "o_slc", "o_swa", "lse_slc", "lse_swa"), got, ref):
            assert torch.equal(a, b), (name, frac)
    print("slabs", lens, (Hq, Hkv, Dk, Dv, S, W, bs), "workspace", full, "->", limit)


@pytest.mark.parametrize("H", [2, 1])          # GQA groups of 16 and of 32 heads
@pytest.mark.parametrize("dtype,bs,W", [(torch.bfloat16, 64, 128), (torch.bfloat16, 32, 48), (torch.float32, 32, 16)])
def test_parallel_nsa_packed_cu_seqlens_and_tensor_counts(dtype, bs, W, H):
    """The public call in its varlen form (nsa/selection_attn.py:792-793: B == 1, packed [1,total,...]
    tensors, block ids local to each sequence) with a per-(token, head) count tensor (:431-434), random
    gates; every sequence against the per-token loop oracle."""
    import nsa_amd
    lens = [200, 64, 1, 333, 97]
    T, HQ, D, S = sum(lens), 32, 64, 3
    q = randn(1, T, HQ, D, seed=90, scale=0.7, dtype=dtype)
    k = randn(1, T, H, D, seed=91, scale=0.7, dtype=dtype)
    v = randn(1, T, H, D, seed=92, dtype=dtype)
    g_slc = randn(1, T, HQ, seed=93, dtype=dtype)
    g_swa = randn(1, T, HQ, seed=94, dtype=dtype)
    gen = torch.Generator().manual_seed(95)
    cuh = ragged_cu(lens)
    idx = torch.full((1, T, H, S), -1, dtype=torch.long)
    for s0, e0 in zip(cuh[:-1], cuh[1:]):
        L = e0 - s0
        idx[0, s0:e0] = _random_indices(L, H, S, bs, int(torch.randint(0, 1 << 30, (1,), generator=gen)))
    counts = torch.randint(0, S + 1, (1, T, H), generator=gen)
    cu = torch.tensor(cuh, dtype=torch.long, device=DEV)
    out = nsa_amd.parallel_nsa(q.to(DEV), k.to(DEV), v.to(DEV), g_slc.to(DEV), g_swa.to(DEV), idx.to(DEV),
                               counts.to(DEV), bs, W, cu_seqlens=cu).cpu()
    assert out.shape == (1, T, HQ, D)
    for s0, e0 in zip(cuh[:-1], cuh[1:]):
        slc, swa = O.selected_sliding_loop(q[0, s0:e0], k[0, s0:e0], v[0, s0:e0], idx[0, s0:e0], counts[0, s0:e0], bs, W)
        ref = g_slc[0, s0:e0, :, None].float() * slc + g_swa[0, s0:e0, :, None].float() * swa
        assert within(out[0, s0:e0], ref, dtype, large_values=True), max_abs(out[0, s0:e0], ref)


@pytest.mark.parametrize("dtype,W", [(torch.bfloat16, 64), (torch.float16, 0), (torch.float32, 64), (torch.float32, 0)])
def test_parallel_nsa_repeated_block_ids(dtype, W):
    """block_indices that list a block twice (every row) or three times: the reference's naive loop gathers keys
    and values per entry, so the block's keys enter the softmax once per occurrence
    (tests/test_parallel_nsa.py:133-146).  16-bit inputs take the block-major schedule (one partial result per
    (token, entry) pair), fp32 the token-major kernel."""
    import nsa_amd
    B, T, HQ, H, D, S, bs = 2, 320, 16, 2, 64, 6, 32
    q = randn(B, T, HQ, D, seed=120, scale=0.7, dtype=dtype)
    k = randn(B, T, H, D, seed=121, scale=0.7, dtype=dtype)
    v = randn(B, T, H, D, seed=122, dtype=dtype)
    g_slc = randn(B, T, HQ, seed=123, dtype=dtype)
    g_swa = randn(B, T, HQ, seed=124, dtype=dtype)
    idx = torch.stack([_random_indices(T, H, S, bs, 125 + b, poison=False) for b in range(B)])
    idx[..., 1] = idx[..., 0]
    idx[:, T // 2:, 0, 4] = idx[:, T // 2:, 0, 0]
    out = nsa_amd.parallel_nsa(q.to(DEV), k.to(DEV), v.to(DEV), g_slc.to(DEV), g_swa.to(DEV), idx.to(DEV), None, bs,
                               W).cpu()
    once = idx.clone()
    once[..., 1] = -1
    differs = 0.0
    for b in range(B):
        slc, swa = O.selected_sliding_loop(q[b], k[b], v[b], idx[b], None, bs, W)
        ref = g_slc[b, :, :, None].float() * slc + g_swa[b, :, :, None].float() * swa
        assert within(out[b], ref, dtype, large_values=True), max_abs(out[b], ref)
        differs = max(differs, max_abs(slc, O.selected_attention(q[b], k[b], v[b], once[b], None, bs)))
    assert differs > 0.05          # counting the repeated block once would have been visible


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_sliding_window_attn_public_call(dtype):
    """nsa_amd.sliding_window_attn in both forms (batched equal lengths; packed with cu_seqlens)."""
    import nsa_amd
    B, T, HQ, H, D, W = 2, 300, 16, 2, 64, 100
    q = randn(B, T, HQ, D, seed=96, scale=0.7, dtype=dtype)
    k = randn(B, T, H, D, seed=97, scale=0.7, dtype=dtype)
    v = randn(B, T, H, D, seed=98, dtype=dtype)
    out = nsa_amd.sliding_window_attn(q.to(DEV), k.to(DEV), v.to(DEV), W).cpu()
    for b in range(B):
        assert max_abs(out[b], O.sliding_attention(q[b], k[b], v[b], W)) <= TOL[dtype]
    lens = [77, 300, 1, 222]
    cuh = ragged_cu(lens)
    qp, kp, vp = (x.reshape(1, B * T, *x.shape[2:]) for x in (q, k, v))
    cu = torch.tensor(cuh, dtype=torch.long, device=DEV)
    outp = nsa_amd.sliding_window_attn(qp.to(DEV), kp.to(DEV), vp.to(DEV), W, cu_seqlens=cu).cpu()
    for s0, e0 in zip(cuh[:-1], cuh[1:]):
        assert max_abs(outp[0, s0:e0], O.sliding_attention(qp[0, s0:e0], kp[0, s0:e0], vp[0, s0:e0], W)) <= TOL[dtype]


# ------------------------------------------------------------------------------ whole forward
def _module_case(dtype, lens, Hq, Hkv, Dk, Dv, S, W, seed, scale_in, mode="mean", act="sigmoid", l=32, d=16, lsel=64,
                 rows_per_seq=None):
    """Whole forward through NSAAttention vs the oracle.  The oracle is run with the kernel's own
    block picks forced (so a flipped tie cannot hide a branch error) and the picks are compared
    separately under the 1e-3 tie rule.  rows_per_seq: check only that many sampled rows (+ edge
    rows) of every sequence, which keeps the dense oracle affordable at full sizes."""
    from nsa_amd.nsa import NSAAttention
    T = sum(lens)
    q, k, v, gl = make_qkv(T, Hq, Hkv, Dk, Dv, seed, dtype, scale_in)
    torch.manual_seed(seed)
    m = NSAAttention(Dk, causal=True, compression_stride=d, compression_block=l, selection_block=lsel,
                     selected_block_count=S, sliding_window=W, dtype=dtype, compressor_mode=mode,
                     gate_activation=act)
    comp = None
    if mode == "conv":
        assert Dk == Dv
        comp = dict(wk=m.compressor.compressor_k.weight.detach().permute(2, 1, 0).reshape(l * Dk, Dk).clone(),
                    wv=m.compressor.compressor_v.weight.detach().permute(2, 1, 0).reshape(l * Dk, Dk).clone(),
                    bk=m.compressor.compressor_k.bias.detach().clone(),
                    bv=m.compressor.compressor_v.bias.detach().clone())
    m = m.to(DEV)
    uniform = len(set(lens)) == 1
    cu = _cu(lens)
    with torch.no_grad():       # parameters require grad: without this the un-fused training path would run
        out, idx = m(q.to(DEV), k.to(DEV), v.to(DEV), cu, 0 if uniform else max(lens), gates=gl.to(DEV),
                 return_indices=True)
    out, idx = out.cpu(), idx.cpu().long()
    gates = torch.sigmoid(gl.float()).to(dtype) if act == "sigmoid" else gl
    p = O.NSAParams(l, d, lsel, S, W)
    cuh = ragged_cu(lens)
    err, ok = 0.0, True
    stats = [0, 0, 0, 0]
    for b, (s, e) in enumerate(zip(cuh[:-1], cuh[1:])):
        rows = None if rows_per_seq is None else sample_rows(e - s, rows_per_seq, seed + b)
        ref, parts = O.nsa_forward_single(q[s:e], k[s:e], v[s:e], gates[s:e], p, comp, return_parts=True,
                                          force_idx=idx[s:e], rows=rows)
        got = out[s:e] if rows is None else out[s:e][rows]
        err = max(err, max_abs(got, ref))
        if not within(got, ref, dtype, large_values=(act is None)):
            print("sequence", b, "of", e - s, "tokens: max-abs", max_abs(got, ref), "rows", rows)
        ok = ok and within(got, ref, dtype, large_values=(act is None))
        if parts["pooled"].shape[-1] > 0:
            r = O.compare_selection(idx[s:e] if rows is None else idx[s:e][rows], parts["idx_own"],
                                    parts["pooled"], 1e-3)
            stats = [a + c for a, c in zip(stats, r)]
    print("module", dtype, lens, (Hq, Hkv, Dk, Dv, S, W), mode, act, "max_abs", err, "rows/exact/excused/fail", stats)
    assert torch.isfinite(out).all()
    assert ok, "max-abs %.4g over the bar" % err
    assert stats[3] == 0
    assert stats[1] >= 0.99 * stats[0]                 # picks are the oracle's own, ties aside
    return out


def test_module_cfg1_fp32():
    """benchmark config 1: B1, T1024, Hq4, Hkv1, D64, fp32, mean-pool 32/16, blocks of 64, top-4, window 128."""
    _module_case(torch.float32, [1024], 4, 1, 64, 64, 4, 128, seed=0, scale_in=1.0)


def test_module_cfg2_shape_reduced_bf16():
    """benchmark config 2 at T=2048 (the full T=8192 case is test_module_cfg2_full)."""
    _module_case(torch.bfloat16, [2048], 64, 4, 128, 128, 16, 512, seed=1, scale_in=0.5)


def test_module_cfg4_shape_reduced_dqk192():
    _module_case(torch.bfloat16, [2048], 64, 4, 192, 128, 16, 512, seed=3, scale_in=0.5)


def test_module_fp16():
    """The dtype of the reference's own selection test: the whole forward in float16, ragged, Dqk 192."""
    _module_case(torch.float16, [1100, 64, 1000, 33, 1536], 32, 2, 128, 128, 16, 512, seed=21, scale_in=0.5)
    _module_case(torch.float16, [2048], 64, 4, 192, 128, 16, 512, seed=22, scale_in=0.5)
    _module_case(torch.float16, [1500], 64, 2, 128, 128, 16, 512, seed=23, scale_in=0.5)       # groups of 32 heads


@pytest.mark.parametrize("l,d,lsel,S,mode", [(64, 16, 64, 16, "mean"), (64, 16, 64, 8, "conv"), (32, 8, 64, 8, "mean"),
                                              (64, 32, 64, 6, "mean"), (32, 16, 16, 16, "mean")])
def test_module_other_compression_geometries(l, d, lsel, S, mode):
    """The whole forward with compression blocks of 64 tokens (the reference's compression benchmark,
    tests/benchmark_compression_kv_bwd.py:9), a compression stride of 8 or 32, and selection blocks of one stride."""
    _module_case(torch.bfloat16, [1300, 70, 1000, 33], 32, 2, 128, 128, S, 200, seed=24, scale_in=0.5, mode=mode, l=l,
                 d=d, lsel=lsel)


def test_module_varlen_ragged():
    _module_case(torch.bfloat16, [1100, 64, 1000, 33, 1536], 32, 2, 128, 128, 16, 512, seed=2, scale_in=0.5)


def test_module_many_short_sequences():
    """A serving-style batch: 150 ragged sequences (more than one 64-sequence run of the cooperative tile lookup),
    some shorter than a compression block, one of a single token."""
    rng = random.Random(11)
    lens = [rng.randint(1, 200) for _ in range(150)]
    lens[3], lens[70], lens[149] = 1, 31, 257
    _module_case(torch.bfloat16, lens, 16, 1, 64, 64, 4, 64, seed=12, scale_in=0.5, rows_per_seq=6)
    lens = [rng.randint(20, 400) for _ in range(20)]           # one partial run
    _module_case(torch.bfloat16, lens, 32, 2, 128, 128, 8, 128, seed=13, scale_in=0.5, rows_per_seq=6)


def test_module_groups_of_32_and_64_heads():
    """Hq 64 / Hkv 2 (what the reference's HQ % (16 * H) == 0 allows and a group limit of 16 refuses), ragged;
    Hq 64 / Hkv 1 with the reference's learned compressor and raw gates."""
    _module_case(torch.bfloat16, [1100, 64, 1000, 33, 1536], 64, 2, 128, 128, 16, 512, seed=7, scale_in=0.5)
    _module_case(torch.bfloat16, [2048], 64, 1, 128, 128, 16, 512, seed=8, scale_in=0.7, mode="conv", act=None)
    _module_case(torch.bfloat16, [1024], 96, 2, 192, 128, 8, 128, seed=9, scale_in=0.5)                # G=48, Dqk 192


def test_module_reference_defaults_conv_raw_gates():
    """Reference configuration: learned Conv1d compressor with bias, raw (un-activated) gates."""
    _module_case(torch.bfloat16, [1024, 1024], 16, 1, 128, 128, 16, 512, seed=5, scale_in=1.0, mode="conv", act=None)
    _module_case(torch.float32, [512], 16, 1, 64, 64, 4, 128, seed=6, scale_in=1.0, mode="conv", act=None)


def test_module_cfg2_full_size():
    """benchmark config 2 at its real size (T=8192, Hq64/Hkv4, D128, bf16); sampled rows."""
    _module_case(torch.bfloat16, [8192], 64, 4, 128, 128, 16, 512, seed=1, scale_in=0.5, rows_per_seq=160)


def test_module_cfg3_full_size_varlen():
    """benchmark config 3: 8 sequences with seeded lengths in [1024, 16384], packed; sampled rows, and
    the packed result must equal, bit for bit, each sequence run on its own."""
    from nsa_amd.nsa import NSAAttention
    g = torch.Generator().manual_seed(2)
    lens = [int(x) for x in torch.randint(1024, 16384 + 1, (8,), generator=g)]
    out = _module_case(torch.bfloat16, lens, 64, 4, 128, 128, 16, 512, seed=2, scale_in=0.5, rows_per_seq=40)
    q, k, v, gl = make_qkv(sum(lens), 64, 4, 128, 128, 2, torch.bfloat16, 0.5)
    m = NSAAttention(128, True, dtype=torch.bfloat16, compressor_mode="mean", gate_activation="sigmoid").to(DEV)
    cuh = ragged_cu(lens)
    for b in (0, 3, 7):
        s, e = cuh[b], cuh[b + 1]
        alone = m(q[s:e].to(DEV), k[s:e].to(DEV), v[s:e].to(DEV), _cu([e - s]), 0, gates=gl[s:e].to(DEV)).cpu()
        assert torch.equal(alone, out[s:e]), "sequence %d differs between packed and single runs" % b


def test_module_cfg4_full_size_dqk192():
    """benchmark config 4 (T=32768, Dqk192/Dv128, bf16); sampled rows."""
    _module_case(torch.bfloat16, [32768], 64, 4, 192, 128, 16, 512, seed=3, scale_in=0.5, rows_per_seq=96)


def test_module_long_context_more_than_512_bins():
    """T=40960: 2559 compressed rows, 640 pooled bins -> the 16-candidates-per-lane top-n kernel; one kv
    head of 16 q heads keeps the sampled-row oracle cheap."""
    _module_case(torch.bfloat16, [40960], 16, 1, 64, 64, 16, 512, seed=9, scale_in=0.5, rows_per_seq=96)


@pytest.mark.parametrize("T", [131072, 262144])
def test_module_long_context_beyond_1024_bins(T):
    """T=131072 / 262144: 2048 / 4096 pooled bins -> 32 / 64 top-n candidates per lane; sampled rows."""
    _module_case(torch.bfloat16, [T], 16, 1, 64, 64, 16, 512, seed=11, scale_in=0.5, rows_per_seq=48)


def test_module_group_of_12_heads_ragged():
    """GQA group of 12 (padded to 16 rows per token) with ragged sequences, one shorter than a bin."""
    _module_case(torch.bfloat16, [1500, 70, 36, 900], 24, 2, 128, 128, 8, 256, seed=10, scale_in=0.5)


@pytest.mark.parametrize("dtype,T,Hq,D", [(torch.bfloat16, 300, 16, 192), (torch.float32, 77, 4, 64),
                                          (torch.bfloat16, 1000, 64, 128)])
def test_gate_logits_match_linear(dtype, T, Hq, D):
    """nsa_gate_fwd against the Linear it stands for, evaluated in fp64 on the bf16/fp32 values: one
    rounding of the result is all that may differ."""
    ops = _ops()
    q = randn(T, Hq, D, seed=170, dtype=dtype)
    w = randn(3, D, seed=171, scale=0.2, dtype=dtype)
    b = randn(3, seed=172, dtype=dtype)
    got = ops.gate_logits(q.to(DEV), w.to(DEV), b.to(DEV)).cpu()
    ref = (q.double() @ w.double().t() + b.double())
    err = (got.double() - ref).abs()
    bar = ref.abs() * (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -20) + 1e-6
    print("gate", dtype, (T, Hq, D), "max_abs", err.max().item())
    assert (err <= bar).all()
    assert torch.equal(ops.gate_logits(q.to(DEV), w.to(DEV), None).cpu(),
                       ops.gate_logits(q.to(DEV), w.to(DEV), torch.zeros(3, dtype=dtype).to(DEV)).cpu())


def test_module_own_gating_equals_explicit_gates():
    """forward(gates=None) evaluates the module's gating Linear inside the compressed-attention kernel
    (nsa_cmp_attn_gate_fwd): those logits against the Linear in float64 (one rounding of the result may differ),
    against the stand-alone gate kernel, and fed back in through gates= (same output bit for bit)."""
    from nsa_amd.nsa import NSAAttention
    from nsa_amd.compression_kv import conv_compressed_len
    ops = _ops()
    for dtype, lens, Hq, Hkv, Dk, Dv in ((torch.bfloat16, [640], 32, 2, 128, 128), (torch.float16, [300, 77], 12, 2, 192, 128),
                                         (torch.float32, [200], 4, 1, 64, 64), (torch.bfloat16, [260], 64, 2, 64, 64)):
        T = sum(lens)
        q, k, v, _ = make_qkv(T, Hq, Hkv, Dk, Dv, 173, dtype, 0.5)
        torch.manual_seed(174)
        m = NSAAttention(Dk, causal=True, selected_block_count=8, sliding_window=128, dtype=dtype, compressor_mode="mean",
                         gate_activation="sigmoid").to(DEV)
        cu = _cu(lens)
        qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
        with torch.no_grad():
            a = m(qd, kd, vd, cu, max(lens))
            ck, cv, cu_cmp, _ = m.compressor.compress_packed(kd, vd, cu, seq_len=None)
            cvt = ops.transpose(cv, cu_cmp, len(lens))
            o1, lse1 = ops.cmp_attn(qd, ck, cvt, cu, cu_cmp, len(lens), Hkv, Dv, ck.stride(0), ck.stride(1), 32, 16,
                                    Dk ** -0.5)
            o2, lse2, gl = ops.cmp_attn(qd, ck, cvt, cu, cu_cmp, len(lens), Hkv, Dv, ck.stride(0), ck.stride(1), 32, 16,
                                        Dk ** -0.5, gate_weight=m.gating.weight, gate_bias=m.gating.bias)
            assert torch.equal(o1, o2) and torch.equal(lse1, lse2)            # the attention itself is untouched
            ref_gl = torch.nn.functional.linear(q.double(), m.gating.weight.detach().double().cpu(),
                                                m.gating.bias.detach().double().cpu())
            ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -20}[dtype]
            err = (gl.double().cpu() - ref_gl).abs()
            assert bool((err <= ref_gl.abs() * ulp + 1e-6).all()), float(err.max())
            sep = ops.gate_logits(qd, m.gating.weight, m.gating.bias)
            assert max_abs(gl, sep) <= (float(ref_gl.abs().max()) * 2 * ulp + 1e-6)
            b = m(qd, kd, vd, cu, max(lens), gates=gl)
        assert torch.equal(a, b)


def test_module_randomized_small_shapes():
    """Seeded sweep over ragged lengths (down to a single token), group sizes 1..16, top-n, window and
    both dtypes: every config is checked in full against the oracle."""
    g = torch.Generator().manual_seed(2025)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=g))]

    for case in range(28):
        nseq = pick([1, 1, 2, 3, 4])
        lens = [int(torch.randint(1, 400, (1,), generator=g)) for _ in range(nseq)]
        if case % 7 == 0:
            lens[0] = pick([1, 31, 32, 33, 47, 48, 63, 64, 65, 111, 112])
        G = pick([1, 2, 3, 4, 8, 12, 16])
        Hkv = pick([1, 2])
        D = pick([64, 128])
        S = pick([1, 2, 4, 7, 16])
        W = pick([1, 5, 64, 100, 512])
        dtype = pick([torch.bfloat16, torch.float32])
        mode = pick(["mean", "mean", "conv"])           # conv: the reference's learned Conv1d compressor
        act = pick(["sigmoid", "sigmoid", None])        # None: raw gate logits as in the reference
        print("case", case, lens, G, Hkv, D, S, W, dtype, mode, act)
        _module_case(dtype, lens, G * Hkv, Hkv, D, D, S, W, seed=300 + case, scale_in=0.6, mode=mode, act=act)


def test_module_randomized_groups_beyond_16_and_float16():
    """The same kind of sweep over what came later: GQA groups of 32 / 48 / 64 heads (sub-groups of 16), float16,
    Dqk 192, batches of many short sequences."""
    g = torch.Generator().manual_seed(4051)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=g))]

    for case in range(16):
        nseq = pick([1, 2, 3, 12, 40])
        lens = [int(torch.randint(1, 500 if nseq < 10 else 120, (1,), generator=g)) for _ in range(nseq)]
        if case % 5 == 0:
            lens[0] = pick([1, 32, 33, 63, 64, 65, 129])
        G = pick([16, 32, 48, 64]) if case % 2 == 0 else pick([4, 8, 16])
        Hkv = pick([1, 2])
        Dk, Dv = pick([(64, 64), (128, 128), (192, 128)])
        S = pick([2, 5, 16])
        W = pick([1, 64, 200, 512])
        dtype = torch.float16 if case % 2 == 1 else pick([torch.bfloat16, torch.float16])
        mode = "conv" if Dk == Dv and pick([0, 1, 1]) == 0 else "mean"
        act = pick(["sigmoid", "sigmoid", None])
        print("case", case, lens, G, Hkv, Dk, Dv, S, W, dtype, mode, act)
        _module_case(dtype, lens, G * Hkv, Hkv, Dk, Dv, S, W, seed=700 + case, scale_in=0.6, mode=mode, act=act,
                     rows_per_seq=None if sum(lens) <= 1500 else 24)


def test_module_randomized_selection_block_sizes_and_token_slabs(monkeypatch):
    """The sweep once more over what came last: selection blocks of 32 and 128 keys on the 64-key schedule, head
    dim 32, and (every second case) a workspace cap of 3 MB so that the selected branch runs in token slabs."""
    from nsa_amd import ops
    g = torch.Generator().manual_seed(5077)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=g))]

    for case in range(14):
        nseq = pick([1, 2, 3, 10])
        lens = [int(torch.randint(1, 700 if nseq < 10 else 150, (1,), generator=g)) for _ in range(nseq)]
        if case % 4 == 0:
            lens[0] = pick([1, 31, 32, 33, 64, 127, 128, 129])
        G = pick([4, 16, 16, 32])
        Hkv = pick([1, 2])
        Dk, Dv = pick([(32, 32), (64, 64), (128, 128), (192, 128)])
        lsel = pick([32, 32, 128, 64])
        S = pick([2, 5, 16]) if lsel <= 64 else pick([2, 4])
        W = pick([16, 64, 200, 512])
        dtype = pick([torch.bfloat16, torch.float16])
        act = pick(["sigmoid", "sigmoid", None])
        monkeypatch.setattr(ops, "SLC_WORKSPACE_LIMIT", 3 << 20 if case % 2 else 16 << 30)
        print("case", case, lens, G, Hkv, Dk, Dv, lsel, S, W, dtype, act, "slabs" if case % 2 else "one slab")
        _module_case(dtype, lens, G * Hkv, Hkv, Dk, Dv, S, W, seed=900 + case, scale_in=0.6, act=act, lsel=lsel,
                     rows_per_seq=None if sum(lens) <= 1500 else 24)


def test_flash_attn_func_api():
    import nsa_amd
    from nsa_amd.compression_kv import KVCompressor
    B, T, Hq, Hkv, D, l, d, S = 2, 1024, 16, 1, 128, 32, 16, 16
    dtype = torch.bfloat16
    q = randn(B * T, Hq, D, seed=80, dtype=dtype)
    k = randn(B * T, Hkv, D, seed=81, dtype=dtype)
    v = randn(B * T, Hkv, D, seed=82, dtype=dtype)
    torch.manual_seed(83)
    comp = KVCompressor(d, l, D, None, dtype)
    wk = comp.compressor_k.weight.detach().permute(2, 1, 0).reshape(l * D, D).clone()
    wv = comp.compressor_v.weight.detach().permute(2, 1, 0).reshape(l * D, D).clone()
    bk, bv = comp.compressor_k.bias.detach().clone(), comp.compressor_v.bias.detach().clone()
    comp = comp.to(DEV)
    cu = torch.arange(0, (B + 1) * T, T, dtype=torch.int32, device=DEV)
    ck, cv, _ = comp(k.to(DEV), v.to(DEV), cu, Hq // Hkv)
    Nc = O.compressed_len_conv(T, l, d)
    assert ck.shape == (B, Nc, Hq, D)
    o, idx = nsa_amd.flash_attn_func(q.view(B, T, Hq, D).to(DEV), ck, cv, d, l, True, None, Hkv, 5, 4, 0, S)
    assert o.shape == (B, T, Hq, D) and idx.shape == (B, T, Hkv, S) and idx.dtype == torch.int64
    o, idx = o.cpu(), idx.cpu()
    for b in range(B):
        sl = slice(b * T, (b + 1) * T)
        ckr = O.compress_weighted(k[sl], wk, bk, l, d, Nc)
        cvr = O.compress_weighted(v[sl], wv, bv, l, d, Nc)
        assert max_abs(ck[b, :, ::Hq // Hkv], ckr) <= 2e-2
        ref = O.compressed_attention(q[sl], ck[b, :, ::Hq // Hkv].cpu(), cv[b, :, ::Hq // Hkv].cpu(), l, d)
        assert max_abs(o[b], ref) <= 2e-2
        pooled = O.importance_scores(q[sl], ck[b, :, ::Hq // Hkv].cpu(), 5, 4, 0)
        r = O.compare_selection(idx[b], O.select_blocks(pooled, S), pooled, 1e-3)
        print("flash_attn_func batch", b, r)
        assert r[3] == 0 and r[1] >= 0.99 * r[0]


def test_error_paths():
    import nsa_amd
    from nsa_amd import ops
    q = torch.zeros(64, 40, 64, dtype=torch.bfloat16, device=DEV)      # G = 40 > 16
    k = torch.zeros(64, 1, 64, dtype=torch.bfloat16, device=DEV)
    cu = _cu([64])
    vt = ops.transpose(k, cu, 1)
    with pytest.raises(NotImplementedError):
        ops.swa(q, k, vt, cu, 1, 16, 0.1)
    with pytest.raises(TypeError):
        ops.swa(q.double(), k.double(), vt, cu, 1, 16, 0.1)
    with pytest.raises(ValueError):
        ops.swa(q[:, :4].contiguous(), k, vt, cu, 1, 16, -1.0)
    with pytest.raises(RuntimeError):
        ops.swa(q.cpu(), k, vt, cu, 1, 16, 0.1)
