"""GPU parity of the backward kernels: every gradient comes from the C ABI (nsa_cmp_attn_bwd,
nsa_slc_swa_bwd, nsa_compress_bwd through the ctypes wrappers and the autograd functions built on them)
and is compared with autograd through the CPU oracle's forward in float64 on the same seeded inputs.
Bars: max-abs error <= tol * max(1, max|reference gradient|) with tol 2e-2 for bf16 and 1e-4 for fp32."""
import math

import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import make_qkv, ragged_cu, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"
GTOL = {torch.bfloat16: 2e-2, torch.float32: 1e-4}


def _ops():
    from nsa_amd import ops
    return ops


def _cu(lens):
    return torch.tensor(ragged_cu(lens), dtype=torch.int32, device=DEV)


def _oracle_grads(fn, inputs, d_o):
    """d(sum(fn(*inputs) * d_o)) / d inputs in float64."""
    ins = [x.double().clone().requires_grad_(True) for x in inputs]
    out = fn(*ins)
    out.backward(d_o.double())
    return [x.grad if x.grad is not None else torch.zeros_like(x) for x in ins]


def _check(name, got, ref, dtype):
    a, b = got.double().cpu(), ref.double()
    assert torch.isfinite(a).all(), name + ": non-finite gradient"
    err = float((a - b).abs().max()) if a.numel() else 0.0
    mag = max(1.0, float(b.abs().max()) if b.numel() else 0.0)
    print("   %-4s max_abs %.3e  (max|ref| %.3f)" % (name, err, mag))
    assert err <= GTOL[dtype] * mag, "%s: %.3e > %.1e * %.3f" % (name, err, GTOL[dtype], mag)


# ------------------------------------------------------------------------------ sliding window
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("lens,Hq,Hkv,Dk,Dv,W", [([300], 16, 1, 64, 64, 128), ([257, 40, 130], 32, 2, 128, 128, 100),
                                                 ([200], 16, 1, 192, 128, 64), ([130], 8, 2, 64, 64, 1),
                                                 ([150], 6, 2, 64, 64, 1000)])
def test_swa_bwd(dtype, lens, Hq, Hkv, Dk, Dv, W):
    if dtype == torch.float32 and Dk == 192:
        pytest.skip("fp32 backward is built for head dims 64 and 128")
    ops = _ops()
    T = sum(lens)
    q, k, v, _ = make_qkv(T, Hq, Hkv, Dk, Dv, 150, dtype, 0.7)
    d_o = randn(T, Hq, Dv, seed=151, dtype=dtype)
    cu, cuh = _cu(lens), ragged_cu(lens)
    scale = 1.0 / math.sqrt(Dk)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    vt = ops.transpose(vd, cu, len(lens))
    o, lse = ops.swa(qd, kd, vt, cu, len(lens), W, scale, want_lse=True)
    dq, dk, dv = ops.slc_swa_bwd(qd, kd, vd, None, None, None, o, d_o.to(DEV), lse, None, None, cu, len(lens), 64,
                                 W, scale)
    print("swa_bwd", dtype, lens, (Hq, Hkv, Dk, Dv, W))
    for s, e in zip(cuh[:-1], cuh[1:]):
        rq, rk, rv = _oracle_grads(lambda a, b, c: O.sliding_attention(a, b, c, W, scale, math_dtype=torch.float64),
                                   [q[s:e], k[s:e], v[s:e]], d_o[s:e])
        # the saved log-sum-exp against the oracle's
        sc = torch.einsum("thgd,khd->thgk", q[s:e].double().view(e - s, Hkv, Hq // Hkv, Dk), k[s:e].double()) * scale
        pos = torch.arange(e - s)
        allowed = (pos[None, :] <= pos[:, None]) & (pos[None, :] > pos[:, None] - W)
        ref_lse = torch.logsumexp(sc.masked_fill(~allowed[:, None, None, :], float("-inf")), -1).reshape(e - s, Hq)
        assert float((lse[s:e].double().cpu() - ref_lse).abs().max()) <= (2e-2 if dtype == torch.bfloat16 else 1e-4)
        _check("dq", dq[s:e], rq, dtype)
        _check("dk", dk[s:e], rk, dtype)
        _check("dv", dv[s:e], rv, dtype)


# ------------------------------------------------------------------------------ compressed attention
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("lens,Hq,Hkv,Dk,Dv,l,d,causal", [([600], 16, 1, 64, 64, 32, 16, True),
                                                          ([1300, 20, 333], 32, 2, 128, 128, 32, 16, True),
                                                          ([2500], 16, 1, 192, 128, 32, 16, True),
                                                          ([260], 8, 2, 64, 64, 64, 16, True),
                                                          ([200], 4, 1, 64, 64, 32, 16, False)])
def test_cmp_attn_bwd(dtype, lens, Hq, Hkv, Dk, Dv, l, d, causal):
    if dtype == torch.float32 and Dk == 192:
        pytest.skip("fp32 backward is built for head dims 64 and 128")
    ops = _ops()
    T = sum(lens)
    ncs = [O.compressed_len_conv(t, l, d) for t in lens]
    NC = sum(ncs)
    q = randn(T, Hq, Dk, seed=160, scale=0.7, dtype=dtype)
    ck = randn(NC, Hkv, Dk, seed=161, scale=0.7, dtype=dtype)
    cv = randn(NC, Hkv, Dv, seed=162, scale=0.7, dtype=dtype)
    d_o = randn(T, Hq, Dv, seed=163, dtype=dtype)
    cu, cu_cmp = _cu(lens), _cu(ncs)
    cuh, cuc = ragged_cu(lens), ragged_cu(ncs)
    scale = 1.0 / math.sqrt(Dk)
    qd, ckd, cvd = q.to(DEV), ck.to(DEV), cv.to(DEV)
    cvt = ops.transpose(cvd, cu_cmp, len(lens))
    o, _, lse = ops.cmp_attn(qd, ckd, cvt, cu, cu_cmp, len(lens), Hkv, Dv, Hkv * Dk, Dk, l, d, scale, causal=causal,
                             want_lse_attn=True)
    dq, dck, dcv = ops.cmp_attn_bwd(qd, ckd, cvd, o, d_o.to(DEV), lse, cu, cu_cmp, len(lens), l, d, scale,
                                    causal=causal)
    print("cmp_bwd", dtype, lens, (Hq, Hkv, Dk, Dv, l, d, causal))
    for s, e, cs, ce in zip(cuh[:-1], cuh[1:], cuc[:-1], cuc[1:]):
        if ce == cs:                                    # shorter than one compression block: nothing to attend
            assert torch.count_nonzero(dq[s:e]) == 0
            continue
        if causal:
            fn = lambda a, b, c: O.compressed_attention(a, b, c, l, d, scale, math_dtype=torch.float64)
        else:       # every row visible: block 0, stride 0 makes column c visible from row 0 on
            fn = lambda a, b, c: O.compressed_attention(a, b, c, 0, 0, scale, math_dtype=torch.float64)
        rq, rk, rv = _oracle_grads(fn, [q[s:e], ck[cs:ce], cv[cs:ce]], d_o[s:e])
        _check("dq", dq[s:e], rq, dtype)
        _check("dck", dck[cs:ce], rk, dtype)
        _check("dcv", dcv[cs:ce], rv, dtype)
        if causal:
            assert torch.count_nonzero(dq[s:s + min(l, e - s)]) == 0      # rows that see nothing


# ------------------------------------------------------------------------------ selected blocks
def _random_indices(T, Hkv, S, bs, seed):
    g = torch.Generator().manual_seed(seed)
    nblk = (T + bs - 1) // bs
    idx = torch.full((T, Hkv, S), nblk + 3, dtype=torch.int64)
    for t in range(T):
        for h in range(Hkv):
            perm = torch.randperm(nblk, generator=g)[:S]
            idx[t, h, :len(perm)] = perm
    idx[0] = nblk + 1
    idx[T // 2, :, 0] = -5
    return idx


@pytest.mark.parametrize("lens,Hq,Hkv,Dk,Dv,S,W", [([384], 16, 1, 64, 64, 4, 0), ([512, 100], 32, 2, 128, 128, 8, 100),
                                                  ([330], 16, 1, 192, 128, 3, 64), ([700, 130], 24, 2, 64, 64, 16, 0),
                                                  ([200], 4, 1, 64, 64, 2, 32)])
def test_slc_swa_bwd(lens, Hq, Hkv, Dk, Dv, S, W):
    dtype, bs = torch.bfloat16, 64
    ops = _ops()
    T = sum(lens)
    q, k, v, _ = make_qkv(T, Hq, Hkv, Dk, Dv, 170, dtype, 0.7)
    d_slc = randn(T, Hq, Dv, seed=171, dtype=dtype)
    d_swa = randn(T, Hq, Dv, seed=172, dtype=dtype)
    cu, cuh = _cu(lens), ragged_cu(lens)
    idx = torch.cat([_random_indices(e - s, Hkv, S, bs, 173 + s) for s, e in zip(cuh[:-1], cuh[1:])])
    g = torch.Generator().manual_seed(174)
    counts = torch.randint(0, S + 1, (T, Hkv), generator=g)
    scale = 1.0 / math.sqrt(Dk)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    vt = ops.transpose(vd, cu, len(lens))
    for use_counts in (False, True):
        cd = counts.to(DEV) if use_counts else None
        o_slc, lse_slc = ops.slc_combine(qd, kd, vt, idx.to(DEV), cd, None, None, None, None, None, cu, len(lens), bs,
                                         scale, block_major=True, want_lse=True)
        o_swa = lse_swa = None
        if W > 0:
            o_swa, lse_swa = ops.swa(qd, kd, vt, cu, len(lens), W, scale, want_lse=True)
        dq, dk, dv = ops.slc_swa_bwd(qd, kd, vd, o_slc, d_slc.to(DEV), lse_slc, o_swa,
                                     d_swa.to(DEV) if W > 0 else None, lse_swa, idx.to(DEV), cd, cu, len(lens), bs,
                                     W, scale)
        print("slc_swa_bwd", lens, (Hq, Hkv, Dk, Dv, S, W), "counts", use_counts)
        for s, e in zip(cuh[:-1], cuh[1:]):
            cn = counts[s:e] if use_counts else None
            rq, rk, rv = _oracle_grads(
                lambda a, b, c: O.selected_attention(a, b, c, idx[s:e], cn, bs, scale, math_dtype=torch.float64),
                [q[s:e], k[s:e], v[s:e]], d_slc[s:e])
            if W > 0:
                wq, wk, wv = _oracle_grads(
                    lambda a, b, c: O.sliding_attention(a, b, c, W, scale, math_dtype=torch.float64),
                    [q[s:e], k[s:e], v[s:e]], d_swa[s:e])
                rq, rk, rv = rq + wq, rk + wk, rv + wv
            _check("dq", dq[s:e], rq, dtype)
            _check("dk", dk[s:e], rk, dtype)
            _check("dv", dv[s:e], rv, dtype)
