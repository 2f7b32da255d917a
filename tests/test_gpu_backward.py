"""GPU parity of the backward kernels: every gradient comes from the C ABI (nsa_cmp_attn_bwd,
nsa_slc_swa_bwd, nsa_compress_bwd through the ctypes wrappers and the autograd functions built on them)
and is compared with autograd through the CPU oracle's forward in float64 on the same seeded inputs.
Bars: max-abs error <= tol * max(1, max|reference gradient|) with tol 2e-2 for bf16, 4e-3 for fp16 and 1e-4
for fp32."""
import math

import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import make_qkv, ragged_cu, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"
GTOL = {torch.bfloat16: 2e-2, torch.float16: 4e-3, torch.float32: 1e-4}


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


def _check(name, got, ref, dtype, floor=1.0):
    a, b = got.double().cpu(), ref.double()
    assert torch.isfinite(a).all(), name + ": non-finite gradient"
    err = float((a - b).abs().max()) if a.numel() else 0.0
    mag = max(floor, float(b.abs().max()) if b.numel() else 0.0)
    print("   %-4s max_abs %.3e  (max|ref| %.3f)" % (name, err, mag))
    assert err <= GTOL[dtype] * mag, "%s: %.3e > %.1e * %.3f" % (name, err, GTOL[dtype], mag)


# ------------------------------------------------------------------------------ sliding window
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("lens,Hq,Hkv,Dk,Dv,W", [([300], 16, 1, 64, 64, 128), ([257, 40, 130], 32, 2, 128, 128, 100),
                                                 ([200], 16, 1, 192, 128, 64), ([130], 8, 2, 64, 64, 1),
                                                 ([150], 6, 2, 64, 64, 1000), ([190, 70], 16, 1, 32, 32, 50),
                                                 # 36 key tiles: several per XCD, windows that wrap around
                                                 ([1500, 700], 16, 2, 64, 64, 200)])
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
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("lens,Hq,Hkv,Dk,Dv,l,d,causal", [([600], 16, 1, 64, 64, 32, 16, True),
                                                          ([1300, 20, 333], 32, 2, 128, 128, 32, 16, True),
                                                          ([2500], 16, 1, 192, 128, 32, 16, True),
                                                          ([260], 8, 2, 64, 64, 64, 16, True),
                                                          ([200], 4, 1, 64, 64, 32, 16, False),
                                                          ([400, 90], 16, 2, 32, 32, 32, 16, True),
                                                          # 10 token items: more than one per XCD
                                                          ([5000], 16, 1, 64, 64, 32, 16, True)])
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
                                                  ([200], 4, 1, 64, 64, 2, 32), ([512, 100], 16, 2, 128, 128, 8, 100),
                                                  ([700, 130], 12, 2, 64, 64, 16, 0), ([330], 3, 1, 192, 128, 3, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_slc_swa_bwd(lens, Hq, Hkv, Dk, Dv, S, W, dtype):
    _slc_swa_bwd_case(lens, Hq, Hkv, Dk, Dv, S, W, dtype, 64)


@pytest.mark.parametrize("lens,Hq,Hkv,Dk,Dv,S,W,bs", [([300, 90], 16, 1, 64, 64, 5, 0, 32),
                                                     ([260], 8, 2, 128, 128, 4, 40, 8),
                                                     ([330], 16, 1, 192, 128, 6, 64, 16),
                                                     ([700], 16, 1, 64, 64, 3, 100, 128),
                                                     ([900, 100], 32, 2, 128, 128, 2, 0, 192),
                                                     ([300], 16, 1, 32, 32, 3, 64, 32), ([300], 4, 2, 32, 32, 3, 0, 64),
                                                     ([400, 90], 8, 1, 64, 64, 5, 0, 32),
                                                     ([333], 12, 4, 128, 128, 6, 50, 16)])
def test_slc_swa_bwd_other_selection_block_sizes(lens, Hq, Hkv, Dk, Dv, S, W, bs):
    """Selection blocks of 8, 16, 32 keys (the reference's own test uses 32, tests/test_parallel_nsa.py:169) run as
    masked parts of a 64-key block, blocks of 128, 192 keys as several 64-key blocks per pick."""
    _slc_swa_bwd_case(lens, Hq, Hkv, Dk, Dv, S, W, torch.bfloat16, bs)


@pytest.mark.parametrize("lens,Hq,Hkv,Dk,Dv,S,W,bs", [([1500, 700], 16, 2, 64, 64, 16, 200, 64),
                                                     ([90] * 11 + [400, 33], 16, 1, 128, 128, 4, 0, 32),
                                                     ([1000], 8, 1, 192, 128, 3, 64, 128)])
def test_slc_swa_bwd_in_token_slabs(monkeypatch, lens, Hq, Hkv, Dk, Dv, S, W, bs):
    """A workspace that holds a fraction of the (token, pick) pairs: the selected branch walks the tokens in slabs.
    Gradients against the oracle as in the one-slab cases, and dq bit-identical to the one-slab run (dk / dv are
    sums of fp32 atomics, equal to rounding)."""
    from nsa_amd import _lib
    ops = _ops()
    T = sum(lens)
    geom = (T, len(lens), Hq, Hkv, Dk, Dv, S, bs, 0)
    lib = _lib.load()
    full = lib.nsa_slc_swa_bwd_workspace_bytes(*geom)
    small = lib.nsa_slc_swa_bwd_slab_workspace_bytes(*geom, (T + 4) // 5)
    assert lib.nsa_slc_swa_bwd_slab_workspace_bytes(*geom, 1) < small < full
    one = _slc_swa_bwd_case(lens, Hq, Hkv, Dk, Dv, S, W, torch.bfloat16, bs)
    monkeypatch.setattr(ops, "SLC_WORKSPACE_LIMIT", small)
    slabs = _slc_swa_bwd_case(lens, Hq, Hkv, Dk, Dv, S, W, torch.bfloat16, bs)
    assert torch.equal(one[0], slabs[0])
    for a, b in zip(one[1:], slabs[1:]):
        assert float((a.double() - b.double()).abs().max()) <= 2.0 ** -7 * max(1.0, float(a.abs().max()))


def _slc_swa_bwd_case(lens, Hq, Hkv, Dk, Dv, S, W, dtype, bs):
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
    return dq, dk, dv


# ------------------------------------------------------------------------------ compression
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("S,W", [(16, 100), (4, 0), (0, 64)])
def test_slc_swa_bwd_dq_add(dtype, S, W):
    """dq_add is summed into dq by the kernel that writes it: dk / dv unchanged, dq = plain result + dq_add (to
    one rounding of the output type).  top_n 16 takes the unrolled merge, 4 the loop, 0 the window-only path."""
    if dtype == torch.float32 and S > 0:
        pytest.skip("the selected branch saves its log-sum-exp on the bf16 path only")
    lens, Hq, Hkv, D, bs = [300, 77], 16, 1, 64, 64
    ops = _ops()
    T = sum(lens)
    q, k, v, _ = make_qkv(T, Hq, Hkv, D, D, 180, dtype, 0.7)
    d_o = randn(T, Hq, D, seed=181, dtype=dtype).to(DEV)
    extra = randn(T, Hq, D, seed=182, dtype=dtype).to(DEV)
    cu, cuh = _cu(lens), ragged_cu(lens)
    scale = 1.0 / math.sqrt(D)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    vt = ops.transpose(vd, cu, len(lens))
    idx = o_slc = lse_slc = o_swa = lse_swa = None
    if S > 0:
        idx = torch.cat([_random_indices(e - s, Hkv, S, bs, 183 + s) for s, e in zip(cuh[:-1], cuh[1:])]).to(DEV)
        o_slc, lse_slc = ops.slc_combine(qd, kd, vt, idx, None, None, None, None, None, None, cu, len(lens), bs, scale,
                                         block_major=True, want_lse=True)
    if W > 0:
        o_swa, lse_swa = ops.swa(qd, kd, vt, cu, len(lens), W, scale, want_lse=True)
    args = (qd, kd, vd, o_slc, d_o if S > 0 else None, lse_slc, o_swa, d_o if W > 0 else None, lse_swa, idx, None, cu,
            len(lens), bs, W, scale)
    dq0, dk0, dv0 = ops.slc_swa_bwd(*args)
    dq1, dk1, dv1 = ops.slc_swa_bwd(*args, dq_add=extra)
    tol = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 1e-5}[dtype]
    for a, b in ((dk0, dk1), (dv0, dv1)):      # fp32 atomics: the order of the sums differs from run to run
        assert float((a.double() - b.double()).abs().max()) <= tol * max(1.0, float(a.abs().max()))
    ref = dq0.double() + extra.double()
    err = float((dq1.double() - ref).abs().max())
    mag = max(1.0, float(ref.abs().max()))
    assert err <= tol * mag, err
    with pytest.raises(ValueError):
        ops.slc_swa_bwd(*args, dq_add=extra[:, :, :32])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("lens,H,D,l,d", [([300], 1, 64, 32, 16), ([300, 31, 64, 1000], 4, 128, 32, 16),
                                          ([200, 77], 2, 192, 64, 16), ([90], 2, 32, 8, 4)])
def test_compress_mean_bwd(dtype, lens, H, D, l, d):
    ops = _ops()
    T = sum(lens)
    ncs = [O.compressed_len_conv(t, l, d) for t in lens]
    d_out = randn(sum(ncs), H, D, seed=180, dtype=dtype)
    cu, cu_out = _cu(lens), _cu(ncs)
    dx = ops.compress_bwd(d_out.to(DEV), cu, cu_out, T, l, d)
    cuh, cuc = ragged_cu(lens), ragged_cu(ncs)
    print("compress_mean_bwd", dtype, lens, (H, D, l, d))
    for s, e, cs, ce, n in zip(cuh[:-1], cuh[1:], cuc[:-1], cuc[1:], ncs):
        if n == 0:                                     # shorter than one block: no window, no gradient
            assert torch.count_nonzero(dx[s:e]) == 0
            continue
        x = torch.zeros(e - s, H, D)
        (rx,) = _oracle_grads(lambda a: O.compress_meanpool(a, l, d, n, math_dtype=torch.float64), [x], d_out[cs:ce])
        _check("dx", dx[s:e], rx, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("lens,H,D,l,d,extra", [([256, 100], 2, 64, 32, 16, 1), ([1024] * 2, 2, 128, 64, 16, 0),
                                                ([90, 7], 1, 32, 8, 4, 1), ([700], 4, 192, 32, 16, 1)])
def test_compress_weighted_bwd(dtype, lens, H, D, l, d, extra):
    ops = _ops()
    T = sum(lens)
    ncs = [O.compressed_len_conv(t, l, d) if extra else O.compressed_len_functional(t, l, d) for t in lens]
    x = randn(T, H, D, seed=181, dtype=dtype)
    w_lin = randn(l * D, D, seed=182, scale=1.0 / math.sqrt(l * D), dtype=dtype)
    bias = randn(D, seed=183, dtype=dtype) if extra else None
    d_out = randn(sum(ncs), H, D, seed=184, dtype=dtype)
    cu, cu_out = _cu(lens), _cu(ncs)
    dx, dw, db = ops.compress_bwd(d_out.to(DEV), cu, cu_out, T, l, d, x=x.to(DEV), w_lin=w_lin.to(DEV),
                                  want_dbias=bool(extra))
    cuh, cuc = ragged_cu(lens), ragged_cu(ncs)
    print("compress_weighted_bwd", dtype, lens, (H, D, l, d, extra))
    rw = torch.zeros(l * D, D, dtype=torch.float64)
    rb = torch.zeros(D, dtype=torch.float64)
    for s, e, cs, ce, n in zip(cuh[:-1], cuh[1:], cuc[:-1], cuc[1:], ncs):
        ins = [x[s:e], w_lin] + ([bias] if extra else [])
        fn = (lambda a, w, b: O.compress_weighted(a, w, b, l, d, n, math_dtype=torch.float64)) if extra else \
            (lambda a, w: O.compress_weighted(a, w, None, l, d, n, math_dtype=torch.float64))
        g = _oracle_grads(fn, ins, d_out[cs:ce])
        _check("dx", dx[s:e], g[0], dtype)
        rw += g[1]
        if extra:
            rb += g[2]
    _check("dw", dw, rw, dtype)
    if extra:
        _check("db", db, rb, dtype)


# ------------------------------------------------------------------------------ host API (autograd functions)
def _leaf(t):
    return t.to(DEV).requires_grad_(True)


def _module_backward_case(mode, lens, Hq, Hkv, Dk, Dv, act, S=4, W=64, seed=190, dtype=torch.bfloat16, sel_block=64):
    """NSAAttention end to end: gradients of every input and parameter against autograd through the
    oracle forward (float64, the module's own block picks forced so that score ties cannot differ)."""
    from nsa_amd.nsa import NSAAttention
    T = sum(lens)
    p = O.NSAParams(block=32, stride=16, sel_block=sel_block, top_n=S, window=W, scale=1.0 / math.sqrt(Dk))
    torch.manual_seed(5)
    mod = NSAAttention(Dk, causal=True, compression_stride=16, compression_block=32, selection_block=sel_block,
                       selected_block_count=S, sliding_window=W, device=DEV, dtype=dtype, compressor_mode=mode,
                       gate_activation=act)       # None: raw gates of either sign, as in the reference
    q, k, v, _ = make_qkv(T, Hq, Hkv, Dk, Dv, seed, dtype, 0.7)
    d_o = randn(T, Hq, Dv, seed=seed + 1, dtype=dtype)
    qd, kd, vd = _leaf(q), _leaf(k), _leaf(v)
    cu = _cu(lens)
    out, idx = mod(qd, kd, vd, cu, max_seqlen=max(lens), return_indices=True)
    out.backward(d_o.to(DEV))
    assert out.requires_grad and idx.dtype == torch.int32

    # oracle: same parameters, float64
    gw = mod.gating.weight.detach().cpu().double().requires_grad_(True)
    gb = mod.gating.bias.detach().cpu().double().requires_grad_(True)
    comp = None
    if mode == "conv":
        def lin(conv):
            w = conv.weight.detach().cpu().double()
            return w.permute(2, 1, 0).reshape(-1, w.shape[0]).requires_grad_(True)
        comp = {"wk": lin(mod.compressor.compressor_k), "wv": lin(mod.compressor.compressor_v),
                "bk": mod.compressor.compressor_k.bias.detach().cpu().double().requires_grad_(True),
                "bv": mod.compressor.compressor_v.bias.detach().cpu().double().requires_grad_(True)}
    qr, kr, vr = (t.double().clone().requires_grad_(True) for t in (q, k, v))
    cuh = ragged_cu(lens)
    outs = []
    for s, e in zip(cuh[:-1], cuh[1:]):
        gates = qr[s:e] @ gw.t() + gb
        gates = torch.sigmoid(gates) if act == "sigmoid" else gates
        outs.append(O.nsa_forward_single(qr[s:e], kr[s:e], vr[s:e], gates, p, comp, math_dtype=torch.float64,
                                         force_idx=idx[s:e].cpu()))
    ref = torch.cat(outs)
    ref.backward(d_o.double())
    print("module_bwd", mode, lens, (Hq, Hkv, Dk, Dv), act, S, W)
    big = act is None                       # raw gates: |out| and the gradients are several units large
    _check("out", out.detach(), ref.detach(), dtype, floor=4.0 if big else 1.0)
    _check("dq", qd.grad, qr.grad, dtype)
    _check("dk", kd.grad, kr.grad, dtype)
    _check("dv", vd.grad, vr.grad, dtype)
    _check("dgw", mod.gating.weight.grad, gw.grad, dtype)
    # the bias gradient is the sum of T * Hq gate-logit gradients, each rounded to the 16-bit dtype on its way
    # through autograd: an error of about eps * sqrt(T * Hq) times their size, whatever the sum itself comes to
    _check("dgb", mod.gating.bias.grad, gb.grad, dtype, floor=max(1.0, 0.1 * math.sqrt(T * Hq)))
    if mode == "conv":
        for name, conv in (("k", mod.compressor.compressor_k), ("v", mod.compressor.compressor_v)):
            w = comp["w" + name].grad                                  # [j*D+i, o] -> [o, i, j]
            D = conv.weight.shape[0]
            _check("dw" + name, conv.weight.grad, w.reshape(-1, D, D).permute(2, 1, 0), dtype)
            # the bias gradient is a sum of bf16-rounded rows that nearly cancel (shifting every key by a
            # constant does not change the attention): its error scales with the terms, as dw's does
            _check("db" + name, conv.bias.grad, comp["b" + name].grad, dtype, floor=max(1.0, float(w.abs().max())))


@pytest.mark.parametrize("mode,lens,Hq,Hkv,Dk,Dv,act", [("mean", [600], 16, 1, 64, 64, "sigmoid"),
                                                        ("mean", [300, 200, 40], 32, 2, 128, 128, "sigmoid"),
                                                        ("conv", [500], 16, 1, 64, 64, "sigmoid"),
                                                        ("mean", [400], 16, 1, 192, 128, "sigmoid"),
                                                        ("mean", [450], 32, 2, 64, 64, None)])
def test_module_backward(mode, lens, Hq, Hkv, Dk, Dv, act):
    _module_backward_case(mode, lens, Hq, Hkv, Dk, Dv, act)


@pytest.mark.parametrize("mode,lens,Hq,Hkv,Dk,Dv,act", [("mean", [300, 200, 40], 32, 2, 128, 128, "sigmoid"),
                                                        ("conv", [500], 16, 1, 64, 64, None),
                                                        ("mean", [400], 16, 1, 192, 128, "sigmoid")])
def test_module_backward_float16(mode, lens, Hq, Hkv, Dk, Dv, act):
    """float16, the dtype of the reference's own selection test (tests/test_parallel_nsa.py:169), through
    every backward kernel."""
    _module_backward_case(mode, lens, Hq, Hkv, Dk, Dv, act, dtype=torch.float16)


@pytest.mark.parametrize("mode,lens,Hq,Hkv,Dk,Dv,act", [("mean", [300, 120], 32, 1, 64, 64, "sigmoid"),
                                                        ("conv", [260], 96, 2, 128, 128, None),
                                                        ("mean", [200], 64, 1, 192, 128, "sigmoid")])
def test_module_backward_groups_of_32_48_64_heads(mode, lens, Hq, Hkv, Dk, Dv, act):
    """What the reference's HQ % (16 * H) == 0 admits beyond 16 heads (nsa/selection_attn.py:800): the backward runs
    one call per sub-group of 16 heads, the key / value gradients of the sub-groups add up."""
    _module_backward_case(mode, lens, Hq, Hkv, Dk, Dv, act)


@pytest.mark.parametrize("lens,Hq,Hkv,D,sel_block,S", [([400, 130], 16, 1, 64, 32, 6), ([500], 32, 2, 128, 128, 3),
                                                      ([300], 16, 1, 32, 32, 4)])
def test_module_backward_other_selection_block_sizes(lens, Hq, Hkv, D, sel_block, S):
    """Training through the module with selection blocks of 32 keys (what the reference's own selection test uses)
    and of 128 keys, and with head dim 32."""
    _module_backward_case("mean", lens, Hq, Hkv, D, D, "sigmoid", S=S, sel_block=sel_block)


def test_training_forward_in_token_slabs(monkeypatch):
    """With the one-slab workspace of the selected branch over ops.SLC_WORKSPACE_LIMIT the training forward runs the
    slab schedule (module and functional form); outputs and gradients as before."""
    from nsa_amd import ops
    monkeypatch.setattr(ops, "SLC_WORKSPACE_LIMIT", 2 << 20)
    _module_backward_case("mean", [700, 300, 90], 32, 2, 128, 128, "sigmoid", S=8, W=100)
    test_parallel_nsa_and_flash_attn_backward(torch.bfloat16, 2)


def test_module_backward_randomized_small_shapes():
    """Seeded sweep over ragged lengths (down to a single token and sequences without any compressed row),
    group sizes 1..16, top-n, window, both compressors and both gate conventions."""
    g = torch.Generator().manual_seed(4242)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=g))]

    for case in range(20):
        nseq = pick([1, 1, 2, 3, 4])
        lens = [int(torch.randint(1, 400, (1,), generator=g)) for _ in range(nseq)]
        if case % 5 == 0:
            lens[0] = pick([1, 31, 32, 33, 47, 48, 63, 64, 65, 111, 112])
        G = pick([1, 2, 3, 4, 8, 12, 16])
        Hkv = pick([1, 2])
        D = pick([64, 128])
        S = pick([1, 2, 4, 7, 16])
        W = pick([1, 5, 64, 100, 512])
        mode = pick(["mean", "mean", "conv"])
        act = pick(["sigmoid", "sigmoid", None])
        print("case", case, lens, G, Hkv, D, S, W, mode, act, flush=True)
        _module_backward_case(mode, lens, G * Hkv, Hkv, D, D, act, S=S, W=W, seed=400 + 3 * case)


def test_module_backward_randomized_block_sizes_and_groups():
    """The same sweep over selection blocks of 16, 32, 128 keys and GQA groups from 2 to 48 heads (the packed
    layouts of the small groups, the per-sub-group calls of the large ones), bf16 and fp16."""
    g = torch.Generator().manual_seed(4343)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=g))]

    for case in range(14):
        nseq = pick([1, 1, 2, 3])
        lens = [int(torch.randint(1, 400, (1,), generator=g)) for _ in range(nseq)]
        if case % 5 == 0:
            lens[0] = pick([1, 31, 32, 33, 47, 48, 63, 64, 65, 111, 112])
        G = pick([2, 4, 6, 8, 16, 32, 48])
        Hkv = pick([1, 2])
        D = pick([32, 64, 128]) if G <= 16 else pick([64, 128])
        sel_block = pick([16, 16, 32, 32, 128])       # (8 keys would be below the compression stride of 16)
        S = pick([1, 2, 4, 7]) if sel_block >= 32 else pick([3, 8, 16])
        W = pick([1, 64, 100, 512])
        dtype = pick([torch.bfloat16, torch.float16])
        print("case", case, lens, G, Hkv, D, S, W, sel_block, dtype, flush=True)
        _module_backward_case("mean", lens, G * Hkv, Hkv, D, D, "sigmoid", S=S, W=W, seed=700 + 3 * case, dtype=dtype,
                              sel_block=sel_block)


def test_module_no_grad_path_unchanged():
    """Without grad the fused inference schedule runs and agrees with the training-path output."""
    from nsa_amd.nsa import NSAAttention
    dtype, T, Hq, Hkv, D = torch.bfloat16, 700, 32, 2, 128
    mod = NSAAttention(D, causal=True, selected_block_count=4, sliding_window=128, device=DEV, dtype=dtype,
                       compressor_mode="mean", gate_activation="sigmoid")
    q, k, v, _ = make_qkv(T, Hq, Hkv, D, D, 195, dtype, 0.7)
    cu = _cu([T])
    with torch.no_grad():
        a = mod(q.to(DEV), k.to(DEV), v.to(DEV), cu)
    b = mod(_leaf(q), k.to(DEV), v.to(DEV), cu)
    assert not a.requires_grad and b.requires_grad
    assert float((a.float() - b.detach().float()).abs().max()) <= 2e-2


@pytest.mark.parametrize("dtype,Hkv", [(torch.bfloat16, 2), (torch.float16, 2), (torch.bfloat16, 1)])
def test_parallel_nsa_and_flash_attn_backward(dtype, Hkv):
    """The two functional entry points with the reference's tensor layouts ([B,T,H,D], head-repeated
    compressed keys): gradients of q, k, v and the gates.  Hkv 1 = a GQA group of 32 heads."""
    import nsa_amd
    B, T, Hq, D, S, W, bs = 2, 256, 32, 64, 3, 32, 64
    scale = 1.0 / math.sqrt(D)
    q = randn(B, T, Hq, D, seed=200, scale=0.7, dtype=dtype)
    k = randn(B, T, Hkv, D, seed=201, scale=0.7, dtype=dtype)
    v = randn(B, T, Hkv, D, seed=202, scale=0.7, dtype=dtype)
    g1 = torch.sigmoid(randn(B, T, Hq, seed=203)).to(dtype)
    g2 = torch.sigmoid(randn(B, T, Hq, seed=204)).to(dtype)
    d_o = randn(B, T, Hq, D, seed=205, dtype=dtype)
    idx = torch.stack([_random_indices(T, Hkv, S, bs, 206 + b) for b in range(B)])
    leaves = [_leaf(t) for t in (q, k, v, g1, g2)]
    o = nsa_amd.parallel_nsa(*leaves, idx.to(DEV), block_size=bs, window_size=W, scale=scale)
    o.backward(d_o.to(DEV))
    refs = [t.double().clone().requires_grad_(True) for t in (q, k, v, g1, g2)]
    outs = []
    for b in range(B):
        o_slc = O.selected_attention(refs[0][b], refs[1][b], refs[2][b], idx[b], None, bs, scale, math_dtype=torch.float64)
        o_swa = O.sliding_attention(refs[0][b], refs[1][b], refs[2][b], W, scale, math_dtype=torch.float64)
        outs.append(O.gated_combine(refs[3][b], o_slc, refs[4][b], o_swa))
    ref = torch.stack(outs)
    ref.backward(d_o.double())
    print("parallel_nsa_bwd")
    _check("out", o.detach(), ref.detach(), dtype)
    for name, a, r in zip(("dq", "dk", "dv", "dg1", "dg2"), leaves, refs):
        _check(name, a.grad, r.grad, dtype)

    # compressed attention on head-repeated compressed keys, as KVCompressor(group=...) hands them over
    Nc, l, d = O.compressed_len_conv(T, 32, 16), 32, 16
    ck = randn(B, Nc, Hkv, D, seed=207, scale=0.7, dtype=dtype)
    cv = randn(B, Nc, Hkv, D, seed=208, scale=0.7, dtype=dtype)
    qd, ckd, cvd = _leaf(q), _leaf(ck), _leaf(cv)
    G = Hq // Hkv
    o2, idx2 = nsa_amd.flash_attn_func(qd, ckd.repeat_interleave(G, dim=2), cvd.repeat_interleave(G, dim=2), d, l, True,
                                       scale, Hkv, 5, 4, 0, 2)
    o2.backward(d_o.to(DEV))
    assert idx2.shape == (B, T, Hkv, 2) and not idx2.requires_grad
    rq, rck, rcv = (t.double().clone().requires_grad_(True) for t in (q, ck, cv))
    ref2 = torch.stack([O.compressed_attention(rq[b], rck[b], rcv[b], l, d, scale, math_dtype=torch.float64)
                        for b in range(B)])
    ref2.backward(d_o.double())
    print("flash_attn_func_bwd")
    _check("out", o2.detach(), ref2.detach(), dtype)
    _check("dq", qd.grad, rq.grad, dtype)
    _check("dck", ckd.grad, rck.grad, dtype)
    _check("dcv", cvd.grad, rcv.grad, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_parallel_nsa_backward_in_the_shape_of_the_reference_test(dtype):
    """The reference's own selection test (tests/test_parallel_nsa.py:168-236): B 2, T 64, H 1, HQ 16, D 32, S 2,
    32-key selection blocks, window 128, float16, gates of ones that require grad, random counts, two rows with an
    unusable first pick; forward and every gradient it compares (dq, dk, dv, dg_slc) plus dg_swa."""
    import nsa_amd
    B, T, H, HQ, D, S, bs, W = 2, 64, 1, 16, 32, 2, 32, 128
    q = randn(B, T, HQ, D, seed=300, dtype=dtype)
    k = randn(B, T, H, D, seed=301, dtype=dtype)
    v = randn(B, T, H, D, seed=302, dtype=dtype)
    g_slc, g_swa = torch.ones(B, T, HQ, dtype=dtype), torch.ones(B, T, HQ, dtype=dtype)
    d_o = randn(B, T, HQ, D, seed=303, dtype=dtype)
    gen = torch.Generator().manual_seed(304)
    idx = torch.full((B, T, H, S), T, dtype=torch.long)
    for b in range(B):
        for t in range(T):
            perm = torch.randperm(max(1, t // bs), generator=gen)[:S]
            idx[b, t, 0, :len(perm)] = perm
    idx = idx.sort(-1)[0]
    idx[0, 0, 0, 0] = 4
    idx[1, 63, 0, 0] = 7
    counts = torch.randint(1, S + 1, (B, T, H), generator=gen)
    leaves = [_leaf(t) for t in (q, k, v, g_slc, g_swa)]
    o = nsa_amd.selection_attention(*leaves, idx.to(DEV), counts.to(DEV), bs, W)
    o.backward(d_o.to(DEV))
    scale = D ** -0.5
    refs = [t.double().clone().requires_grad_(True) for t in (q, k, v, g_slc, g_swa)]
    outs = []
    for b in range(B):
        o_slc = O.selected_attention(refs[0][b], refs[1][b], refs[2][b], idx[b], counts[b], bs, scale,
                                     math_dtype=torch.float64)
        o_swa = O.sliding_attention(refs[0][b], refs[1][b], refs[2][b], W, scale, math_dtype=torch.float64)
        outs.append(O.gated_combine(refs[3][b], o_slc, refs[4][b], o_swa))
    ref = torch.stack(outs)
    ref.backward(d_o.double())
    print("reference test shape", dtype)
    _check("out", o.detach(), ref.detach(), dtype)
    for name, a, r in zip(("dq", "dk", "dv", "dg_slc", "dg_swa"), leaves, refs):
        _check(name, a.grad, r.grad, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_parallel_nsa_backward_with_repeated_block_ids(dtype):
    """A block listed twice by a row enters that row's softmax twice (tests/test_parallel_nsa.py:133-146): the
    backward sees two (token, block) pairs with the same keys, and the gradients are those of the doubled weight."""
    import nsa_amd
    B, T, H, HQ, D, S, bs, W = 1, 256, 2, 16, 64, 4, 64, 32
    q = randn(B, T, HQ, D, seed=310, dtype=dtype)
    k = randn(B, T, H, D, seed=311, dtype=dtype)
    v = randn(B, T, H, D, seed=312, dtype=dtype)
    g_slc, g_swa = randn(B, T, HQ, seed=313, dtype=dtype), randn(B, T, HQ, seed=314, dtype=dtype)
    d_o = randn(B, T, HQ, D, seed=315, dtype=dtype)
    idx = _random_indices(T, H, S, bs, 316)[None].clone()
    idx[..., 1] = idx[..., 0]
    idx[:, T // 2:, 1, 3] = idx[:, T // 2:, 1, 0]
    leaves = [_leaf(t) for t in (q, k, v, g_slc, g_swa)]
    o = nsa_amd.selection_attention(*leaves, idx.to(DEV), None, bs, W)
    o.backward(d_o.to(DEV))
    scale = D ** -0.5
    refs = [t.double().clone().requires_grad_(True) for t in (q, k, v, g_slc, g_swa)]
    o_slc = O.selected_attention(refs[0][0], refs[1][0], refs[2][0], idx[0], None, bs, scale, math_dtype=torch.float64)
    o_swa = O.sliding_attention(refs[0][0], refs[1][0], refs[2][0], W, scale, math_dtype=torch.float64)
    ref = O.gated_combine(refs[3][0], o_slc, refs[4][0], o_swa)[None]
    ref.backward(d_o.double())
    _check("out", o.detach(), ref.detach(), dtype)
    for name, a, r in zip(("dq", "dk", "dv", "dg_slc", "dg_swa"), leaves, refs):
        _check(name, a.grad, r.grad, dtype)


def test_compress_kv_backward():
    """compress_kv (functional, learned weights) and KVCompressorVarlen: gradients of k, v and the weights."""
    from nsa_amd.compression_kv import KVCompressorVarlen
    dtype, lens, H, D, l, d = torch.bfloat16, [200, 90], 2, 64, 32, 16
    T = sum(lens)
    mod = KVCompressorVarlen(d, l, D, DEV, dtype)
    k, v = randn(T, H, D, seed=210, dtype=dtype), randn(T, H, D, seed=211, dtype=dtype)
    kd, vd = _leaf(k), _leaf(v)
    ck, cv, cu_out = mod(kd, vd, _cu(lens))
    ncs = [O.compressed_len_functional(t, l, d) for t in lens]
    assert cu_out.cpu().tolist() == ragged_cu(ncs)
    d1, d2 = randn(sum(ncs), H, D, seed=212, dtype=dtype), randn(sum(ncs), H, D, seed=213, dtype=dtype)
    (ck.float() * d1.to(DEV).float()).sum().backward(retain_graph=True)
    (cv.float() * d2.to(DEV).float()).sum().backward()
    cuh, cuc = ragged_cu(lens), ragged_cu(ncs)
    for x, xd, w, dd, name in ((k, kd, mod.k_weight, d1, "k"), (v, vd, mod.v_weight, d2, "v")):
        wr = w.detach().cpu().double().requires_grad_(True)
        xr = x.double().clone().requires_grad_(True)
        ref = torch.cat([O.compress_weighted(xr[s:e], wr, None, l, d, n, math_dtype=torch.float64)
                         for s, e, n in zip(cuh[:-1], cuh[1:], ncs)])
        ref.backward(dd.double())
        print("compress_kv_bwd", name)
        _check("dx", xd.grad, xr.grad, dtype)
        _check("dw", w.grad, wr.grad, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,Hq,D,Dv,act", [(300, 16, 64, 64, 1), (257, 6, 192, 128, 0), (64, 4, 128, 128, 1)])
def test_gate_and_combine_kernels(dtype, T, Hq, D, Dv, act):
    """nsa_gate_combine_fwd / _bwd and nsa_gate_bwd against the same arithmetic in torch float64."""
    ops = _ops()
    q = randn(T, Hq, D, seed=220, scale=0.7, dtype=dtype)
    w = randn(3, D, seed=221, scale=0.2, dtype=dtype)
    gl = randn(T, Hq, 3, seed=222, dtype=dtype)
    o = [randn(T, Hq, Dv, seed=223 + i, dtype=dtype) for i in range(3)]
    d_out = randn(T, Hq, Dv, seed=227, dtype=dtype)
    d_gl_in = randn(T, Hq, 3, seed=228, dtype=dtype)
    f = torch.sigmoid if act else (lambda x: x)
    for with_swa, with_cmp in ((True, True), (False, True), (True, False)):
        od = [o[0].to(DEV), o[1].to(DEV) if with_swa else None, o[2].to(DEV) if with_cmp else None]
        out = ops.gate_combine(gl.to(DEV), od[0], od[1], od[2], act)
        d_slc, d_swa, d_cmp, d_gl = ops.gate_combine_bwd(gl.to(DEV), d_out.to(DEV), od[0], od[1], od[2], act)
        glr = gl.double().requires_grad_(True)
        orr = [t.double().requires_grad_(True) for t in o]
        g = f(glr)
        ref = g[..., 0:1] * orr[0]
        if with_swa:
            ref = ref + g[..., 1:2] * orr[1]
        if with_cmp:
            ref = ref + g[..., 2:3] * orr[2]
        ref.backward(d_out.double())
        _check("out", out, ref.detach(), dtype)
        _check("dslc", d_slc, orr[0].grad, dtype)
        if with_swa:
            _check("dswa", d_swa, orr[1].grad, dtype)
        if with_cmp:
            _check("dcmp", d_cmp, orr[2].grad, dtype)
        _check("dgl", d_gl, glr.grad, dtype, floor=float(glr.grad.abs().max()) if dtype == torch.bfloat16 else 1.0)
        # the same call asked for the row sums and gates instead of the scaled copies
        n1, n2, n3, d_gl2, st = ops.gate_combine_bwd(gl.to(DEV), d_out.to(DEV), od[0], od[1], od[2], act,
                                                     want_scaled=False, want_stats=True)
        assert n1 is None and n2 is None and n3 is None and torch.equal(d_gl2, d_gl)
        for b, present in enumerate((True, with_swa, with_cmp)):
            dots = (d_out.double() * o[b].double()).sum(-1) if present else torch.zeros(T, Hq, dtype=torch.float64)
            _check("dot%d" % b, st[b], dots, torch.float32, floor=float(dots.abs().max()) * (64 if dtype == torch.bfloat16 else 1))
            _check("g%d" % b, st[3 + b], f(gl.double()[..., b]), torch.float32)
    dq, dw, db = ops.gate_bwd(q.to(DEV), w.to(DEV), d_gl_in.to(DEV))
    qr, wr = q.double().requires_grad_(True), w.double().requires_grad_(True)
    br = torch.zeros(3, dtype=torch.float64, requires_grad=True)
    (qr @ wr.t() + br).backward(d_gl_in.double())
    _check("dq", dq, qr.grad, dtype)
    _check("dw", dw, wr.grad, dtype)
    _check("db", db, br.grad, dtype)


def test_backward_full_size_cfg4():
    """The benchmark workload at its real size (T=32768, Hq64/Hkv4, Dqk192/Dv128, top-16, window 512): the
    oracle cannot differentiate 2M rows, so dQ is compared on sampled rows (a row's dQ depends on that row's
    output only) and dK / dV through what the mathematics fixes for any size: every softmax row sums to one,
    hence  sum_t dV[t] = sum over rows of (sum of the gates of the branches that see a key) * dO[row]  and
    sum_t dK[t] = 0, per kv head; the mean-pool compressor passes both sums on unchanged."""
    from nsa_amd.nsa import NSAAttention
    dtype, T, Hq, Hkv, Dk, Dv, S, W = torch.bfloat16, 32768, 64, 4, 192, 128, 16, 512
    G = Hq // Hkv
    q, k, v, gl = make_qkv(T, Hq, Hkv, Dk, Dv, 3, dtype, 0.5)
    d_o = randn(T, Hq, Dv, seed=230, dtype=dtype)
    mod = NSAAttention(Dk, causal=True, selected_block_count=S, sliding_window=W, device=DEV, dtype=dtype,
                       compressor_mode="mean", gate_activation="sigmoid")
    qd, kd, vd = _leaf(q), _leaf(k), _leaf(v)
    out, idx = mod(qd, kd, vd, _cu([T]), gates=gl.to(DEV), return_indices=True)
    out.backward(d_o.to(DEV))
    dq, dk, dv = qd.grad.cpu(), kd.grad.double().cpu(), vd.grad.double().cpu()
    idx = idx.cpu().long()
    assert torch.isfinite(dq).all() and torch.isfinite(dk).all() and torch.isfinite(dv).all()

    # checksums of dV and dK
    g = torch.sigmoid(gl.double())                                            # [T,Hq,3]
    t = torch.arange(T)
    has_slc = ((idx >= 0) & (idx * 64 <= t[:, None, None])).any(-1)           # [T,Hkv]
    w = g[..., 0] * has_slc.repeat_interleave(G, 1) + g[..., 1] + g[..., 2] * (t >= 32)[:, None]
    ref_dv = (w[..., None] * d_o.double()).view(T, Hkv, G, Dv).sum((0, 2))    # [Hkv,Dv]
    got_dv, got_dk = dv.sum(0), dk.sum(0)
    tol_v = 4 * 2.0 ** -9 * math.sqrt(T) * float(dv.abs().max())
    tol_k = 4 * 2.0 ** -9 * math.sqrt(T) * float(dk.abs().max())
    err_v, err_k = float((got_dv - ref_dv).abs().max()), float(got_dk.abs().max())
    print("full-size backward: sum dV err %.3f (tol %.3f, |ref| max %.1f), |sum dK| max %.3f (tol %.3f, sum|dK| %.0f)"
          % (err_v, tol_v, float(ref_dv.abs().max()), err_k, tol_k, float(dk.abs().sum(0).max())))
    assert err_v <= tol_v and err_k <= tol_k

    # dQ on sampled rows against the oracle with the module's picks forced
    rows = torch.tensor(sorted({0, 31, 32, 33, 63, 64, 511, 512, 513, 1000, 4097, 16384, 20011, 32700, 32767}))
    p = O.NSAParams(32, 16, 64, S, W, scale=1.0 / math.sqrt(Dk))
    qr = q.double().clone().requires_grad_(True)
    ref = O.nsa_forward_single(qr, k.double(), v.double(), g, p, math_dtype=torch.float64, force_idx=idx, rows=rows)
    ref.backward(d_o.double()[rows])
    _check("out", out.detach()[rows.to(DEV)], ref.detach(), dtype)
    _check("dq", dq[rows], qr.grad[rows], dtype)
