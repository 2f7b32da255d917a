"""Pins the CPU oracle against library routines, closed forms and brute force.

Nothing here repeats the oracle's own formulas: compression is checked against
F.conv1d / unfold().mean() / a flatten-and-matmul loop, pooling against
F.avg_pool1d, the attention branches against F.scaled_dot_product_attention with
explicit boolean masks and against a per-token loop, the packed layout against
per-sequence runs and the decode step against the last prefill row.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import nsa_oracle as O

D64 = torch.float64


def _rand(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


# ---------------------------------------------------------------- counts
@pytest.mark.parametrize("T,l,d", [(1024, 32, 16), (1000, 32, 16), (31, 32, 16), (32, 32, 16),
                                   (1024, 64, 16), (77, 8, 4)])
def test_counts_match_conv1d(T, l, d):
    if T >= l:
        n = F.conv1d(torch.zeros(1, 1, T), torch.zeros(1, 1, l), stride=d).shape[-1]
    else:
        n = 0
    assert O.compressed_len_conv(T, l, d) == n
    assert O.compressed_len_functional(T, l, d) == max(n - 1, 0)


# ---------------------------------------------------------------- compression
@pytest.mark.parametrize("T,H,D,l,d", [(200, 2, 16, 32, 16), (133, 1, 8, 8, 4), (96, 3, 32, 64, 16)])
def test_compress_weighted_is_conv1d(T, H, D, l, d):
    x = _rand(T, H, D, seed=1)
    conv = torch.nn.Conv1d(D, D, l, d)
    w_lin = conv.weight.detach().permute(2, 1, 0).reshape(l * D, D)      # [j*D+i, o] = W[o,i,j]
    n = O.compressed_len_conv(T, l, d)
    got = O.compress_weighted(x, w_lin, conv.bias.detach(), l, d, n, math_dtype=D64, out_dtype=D64)
    ref = conv.double()(x.double().permute(1, 2, 0)).permute(2, 0, 1)    # [H,D,T]->[H,D,n]->[n,H,D]
    torch.testing.assert_close(got, ref.detach(), rtol=1e-10, atol=1e-10)
    brute = O.compress_loop(x, w_lin, conv.bias.detach(), l, d, n)
    torch.testing.assert_close(got, brute, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("T,l,d", [(256, 32, 16), (250, 32, 16), (100, 64, 16)])
def test_compress_meanpool_is_unfold_mean(T, l, d):
    x = _rand(T, 2, 16, seed=2)
    n = O.compressed_len_conv(T, l, d)
    got = O.compress_meanpool(x, l, d, n, math_dtype=D64, out_dtype=D64)
    ref = x.double().unfold(0, l, d).mean(-1)
    torch.testing.assert_close(got, ref, rtol=1e-12, atol=1e-12)
    eye = (torch.eye(16) / l).repeat(l, 1)                               # W[j*D+i,o] = delta_io / l
    via_w = O.compress_weighted(x, eye, None, l, d, n, math_dtype=D64, out_dtype=D64)
    torch.testing.assert_close(got, via_w, rtol=1e-12, atol=1e-12)


def test_functional_count_drops_last_block():
    x = _rand(128, 1, 8, seed=3)
    w = _rand(32 * 8, 8, seed=4)
    n_conv = O.compressed_len_conv(128, 32, 16)
    n_fun = O.compressed_len_functional(128, 32, 16)
    assert n_fun == n_conv - 1
    a = O.compress_weighted(x, w, None, 32, 16, n_conv, D64, D64)
    b = O.compress_weighted(x, w, None, 32, 16, n_fun, D64, D64)
    torch.testing.assert_close(a[:n_fun], b)


# ---------------------------------------------------------------- pooling
@pytest.mark.parametrize("Nc", [5, 6, 7, 8, 9, 15, 16, 17, 61, 62, 63, 64, 65, 511, 2047])
@pytest.mark.parametrize("k,s,p", [(5, 4, 0), (5, 4, 2), (3, 2, 0), (9, 8, 0)])
def test_pool_matches_avg_pool1d(Nc, k, s, p):
    if Nc + 2 * p < k:
        pytest.skip("window larger than input")
    x = _rand(3, Nc, seed=Nc, dtype=D64).abs()
    ref = F.avg_pool1d(x[None], k, s, p, True)[0]
    Ns, _ = O.pool_geometry(Nc, k, s, p)
    assert Ns == ref.shape[-1]
    torch.testing.assert_close(O.pool_scores_direct(x, k, s, p), ref, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(O.pool_scores(x, k, s, p), ref, rtol=1e-9, atol=1e-12)


def test_ns_equals_T_over_64_when_divisible():
    for T in (1024, 8192, 32768):
        Nc = O.compressed_len_conv(T, 32, 16)
        assert O.pool_geometry(Nc, 5, 4, 0)[0] == T // 64
    assert O.pool_geometry(O.compressed_len_conv(1000, 32, 16), 5, 4, 0)[0] == 15
    assert O.pool_geometry(O.compressed_len_conv(1055, 32, 16), 5, 4, 0)[0] == 16


# ---------------------------------------------------------------- importance + top-n
def test_importance_matches_library_pipeline():
    T, Hq, Hkv, Dk = 192, 8, 2, 16
    q = _rand(T, Hq, Dk, seed=5)
    ck = _rand(11, Hkv, Dk, seed=6)
    got = O.importance_scores(q, ck, 5, 4, 0, math_dtype=D64)
    # library route: einsum over repeated heads -> softmax -> reshape/sum -> avg_pool1d
    ckr = ck.double().repeat_interleave(Hq // Hkv, dim=1)
    p = torch.softmax(torch.einsum("thd,shd->hts", q.double(), ckr), -1)      # [Hq,T,Nc]
    p = p.reshape(Hkv, Hq // Hkv, T, -1).sum(1)
    ref = F.avg_pool1d(p, 5, 4, 0, True).transpose(0, 1)                      # [T,Hkv,Ns]
    torch.testing.assert_close(got, ref, rtol=1e-10, atol=1e-12)
    # invariant: un-pooled importance sums to G per (t, h); the pooled sum brackets it
    assert torch.allclose(p.sum(-1), torch.full((Hkv, T), float(Hq // Hkv), dtype=D64))
    idx = O.select_blocks(got, 2)
    ref_idx = torch.topk(ref, 2, dim=-1).indices
    assert torch.equal(idx.sort(-1).values, ref_idx.sort(-1).values)


def test_select_blocks_pads_when_few_bins():
    pooled = torch.tensor([[[0.1, 0.7, 0.2]]])
    idx = O.select_blocks(pooled, 5)
    assert idx[0, 0].tolist() == [1, 2, 0, -1, -1]


# ---------------------------------------------------------------- compressed attention
def test_compressed_attention_is_masked_sdpa():
    T, Hq, Hkv, Dk, Dv, l, d = 160, 4, 2, 16, 8, 32, 16
    q, k, v = _rand(T, Hq, Dk, seed=7), _rand(T, Hkv, Dk, seed=8), _rand(T, Hkv, Dv, seed=9)
    Nc = O.compressed_len_conv(T, l, d)
    ck = O.compress_meanpool(k, l, d, Nc, D64, D64)
    cv = O.compress_meanpool(v, l, d, Nc, D64, D64)
    got = O.compressed_attention(q, ck, cv, l, d, None, D64)
    vis = (torch.arange(Nc)[None] * d + l) <= torch.arange(T)[:, None]        # [T,Nc]
    G = Hq // Hkv
    qq = q.double().transpose(0, 1)[None]                                     # [1,Hq,T,Dk]
    kk = ck.repeat_interleave(G, 1).transpose(0, 1)[None]
    vv = cv.repeat_interleave(G, 1).transpose(0, 1)[None]
    rows = vis.any(-1)
    ref = F.scaled_dot_product_attention(qq[:, :, rows], kk, vv, attn_mask=vis[rows][None, None])
    torch.testing.assert_close(got[rows], ref[0].transpose(0, 1), rtol=1e-9, atol=1e-10)
    assert rows[:l].sum() == 0 and rows[l:].all()
    assert torch.count_nonzero(got[:l]) == 0
    # row t depends only on the first n_c(t) compressed rows
    t = 100
    n_vis = (t - l) // d + 1
    ck2, cv2 = ck.clone(), cv.clone()
    ck2[n_vis:] += 3.0
    cv2[n_vis:] -= 5.0
    got2 = O.compressed_attention(q, ck2, cv2, l, d, None, D64)
    torch.testing.assert_close(got2[t], got[t])


# ---------------------------------------------------------------- selected / sliding
def _sdpa_causal(q, k, v, mask=None):
    G = q.shape[1] // k.shape[1]
    qq = q.double().transpose(0, 1)[None]
    kk = k.double().repeat_interleave(G, 1).transpose(0, 1)[None]
    vv = v.double().repeat_interleave(G, 1).transpose(0, 1)[None]
    if mask is None:
        out = F.scaled_dot_product_attention(qq, kk, vv, is_causal=True)
    else:
        out = F.scaled_dot_product_attention(qq, kk, vv, attn_mask=mask[None, None])
    return out[0].transpose(0, 1)


def test_all_blocks_selected_is_causal_attention():
    T, Hq, Hkv, Dk, Dv, bs = 96, 4, 2, 16, 8, 16
    q, k, v = _rand(T, Hq, Dk, seed=10), _rand(T, Hkv, Dk, seed=11), _rand(T, Hkv, Dv, seed=12)
    nb = T // bs
    idx = torch.arange(nb).flip(0).expand(T, Hkv, nb).contiguous()
    got = O.selected_attention(q, k, v, idx, None, bs, None, D64)
    torch.testing.assert_close(got, _sdpa_causal(q, k, v), rtol=1e-9, atol=1e-10)


@pytest.mark.parametrize("W", [1, 7, 32, 96, 500])
def test_sliding_is_banded_sdpa(W):
    T, Hq, Hkv, Dk, Dv = 96, 4, 2, 16, 8
    q, k, v = _rand(T, Hq, Dk, seed=13), _rand(T, Hkv, Dk, seed=14), _rand(T, Hkv, Dv, seed=15)
    got = O.sliding_attention(q, k, v, W, None, D64, row_chunk=40)
    r, c = torch.arange(T)[:, None], torch.arange(T)[None]
    band = (c <= r) & (c >= r - W + 1)
    torch.testing.assert_close(got, _sdpa_causal(q, k, v, band), rtol=1e-9, atol=1e-10)
    if W >= T:
        torch.testing.assert_close(got, _sdpa_causal(q, k, v), rtol=1e-9, atol=1e-10)


def test_selected_matches_token_loop_with_counts_and_poison():
    # shaped like the reference's own test: B=1,T=64,H=1,HQ=16,D=32,S=2,bs=32, random counts,
    # future/out-of-range ids as padding, two rows forced to an empty selection.
    T, Hq, Hkv, D, S, bs, W = 64, 16, 1, 32, 2, 32, 128
    q, k, v = _rand(T, Hq, D, seed=16), _rand(T, Hkv, D, seed=17), _rand(T, Hkv, D, seed=18)
    g = torch.Generator().manual_seed(19)
    idx = torch.full((T, Hkv, S), T, dtype=torch.int64)
    for t in range(T):
        perm = torch.randperm(max(1, t // bs), generator=g)[:S]
        idx[t, 0, :len(perm)] = perm
    idx = idx.sort(-1).values
    idx[0, 0, 0] = 4
    idx[63, 0, 0] = 7
    idx[63, 0, 1] = -3
    counts = torch.randint(1, S + 1, (T, Hkv), generator=g)
    got_slc = O.selected_attention(q, k, v, idx, counts, bs, None, D64, row_chunk=24)
    got_swa = O.sliding_attention(q, k, v, W, None, D64, row_chunk=24)
    ref_slc, ref_swa = O.selected_sliding_loop(q, k, v, idx, counts, bs, W)
    torch.testing.assert_close(got_slc, ref_slc, rtol=1e-9, atol=1e-10)
    torch.testing.assert_close(got_swa, ref_swa, rtol=1e-9, atol=1e-10)
    assert torch.count_nonzero(got_slc[0]) == 0 and torch.count_nonzero(got_slc[63]) == 0


def test_token_loop_is_itself_sdpa_on_a_dense_case():
    # guards the loop used above: with every past block listed it must be causal attention
    T, Hq, Hkv, D, bs = 48, 2, 1, 8, 16
    q, k, v = _rand(T, Hq, D, seed=20), _rand(T, Hkv, D, seed=21), _rand(T, Hkv, D, seed=22)
    idx = torch.arange(T // bs).expand(T, Hkv, -1).contiguous()
    slc, swa = O.selected_sliding_loop(q, k, v, idx, None, bs, T)
    ref = _sdpa_causal(q, k, v)
    torch.testing.assert_close(slc, ref, rtol=1e-9, atol=1e-10)
    torch.testing.assert_close(swa, ref, rtol=1e-9, atol=1e-10)


def _gather_softmax(q, k, v, idx, bs, scale):
    """Brute force in the shape of the reference's naive loop (tests/test_parallel_nsa.py:118-146): every entry of a
    row's index list is expanded to its bs token positions, keys and values are GATHERED at those positions (so a
    block listed twice is gathered twice), positions < 0 or > t are masked, one softmax over the S*bs gathered keys."""
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    out = torch.zeros(T, Hq, v.shape[-1], dtype=D64)
    pos = (idx[..., None] * bs + torch.arange(bs)).reshape(T, Hkv, -1)          # [T,Hkv,S*bs]
    for t in range(T):
        for h in range(Hq):
            pt = pos[t, h // G]
            kk, vv = k[pt.clamp(0, T - 1), h // G].double(), v[pt.clamp(0, T - 1), h // G].double()
            sc = (kk @ q[t, h].double() * scale).masked_fill((pt < 0) | (pt > t), float("-inf"))
            if torch.isinf(sc).all():
                continue
            out[t, h] = torch.softmax(sc, 0) @ vv
    return out


def test_repeated_block_ids_enter_the_softmax_once_per_occurrence():
    T, Hq, Hkv, D, S, bs = 96, 4, 2, 16, 4, 16
    q, k, v = _rand(T, Hq, D, seed=60), _rand(T, Hkv, D, seed=61), _rand(T, Hkv, D, seed=62)
    g = torch.Generator().manual_seed(63)
    idx = torch.randint(0, T // bs, (T, Hkv, S), generator=g)
    idx[:, :, 1] = idx[:, :, 0]                       # every row lists its first block twice ...
    idx[T // 2:, 0, 3] = idx[T // 2:, 0, 0]           # ... and half of the rows of head 0 three times
    idx[5, :, 2] = -1
    scale = 1.0 / math.sqrt(D)
    ref = _gather_softmax(q, k, v, idx, bs, scale)
    got = O.selected_attention(q, k, v, idx, None, bs, scale, D64, row_chunk=40)
    torch.testing.assert_close(got, ref, rtol=1e-9, atol=1e-10)
    loop, _ = O.selected_sliding_loop(q, k, v, idx, None, bs, 0)
    torch.testing.assert_close(loop, ref, rtol=1e-9, atol=1e-10)
    # and it differs from listing the block once (so the check above can fail)
    once = idx.clone()
    once[:, :, 1] = -1
    once[T // 2:, 0, 3] = -1
    assert (O.selected_attention(q, k, v, once, None, bs, scale, D64) - ref).abs().max() > 1e-3
    # closed form: EVERY usable block listed twice is the same softmax as listing each once
    both = torch.arange(T // bs).repeat(2).expand(T, Hkv, -1).contiguous()
    torch.testing.assert_close(O.selected_attention(q, k, v, both, None, bs, scale, D64), _sdpa_causal(q, k, v),
                               rtol=1e-9, atol=1e-10)
    # decode step: a repeated pick in force_idx counts twice as well (last row of the prefill with the same list)
    p = O.NSAParams(8, 4, bs, S, 0)
    gates = torch.ones(Hq, 3, dtype=D64)
    _, parts = O.nsa_decode_step(q[-1].double(), k.double(), v.double(), gates, p, D64, return_parts=True,
                                 force_idx=idx[-1])
    torch.testing.assert_close(parts["o_slc"], ref[-1], rtol=1e-9, atol=1e-10)


# ---------------------------------------------------------------- combine / full forward
def test_gated_combine_closed_form():
    a, b, c = _rand(5, 3, 4, seed=23), _rand(5, 3, 4, seed=24), _rand(5, 3, 4, seed=25)
    g = torch.sigmoid(_rand(5, 3, 3, seed=26))
    got = O.gated_combine(g[..., 0], a, g[..., 1], b, g[..., 2], c)
    ref = torch.stack([a, b, c], -1) @ g.unsqueeze(-1)
    torch.testing.assert_close(got, ref.squeeze(-1))


def _cfg(T, Hq, Hkv, Dk, Dv, seed, dtype=torch.float32, scale=1.0):
    q = _rand(T, Hq, Dk, seed=seed, scale=scale, dtype=dtype)
    k = _rand(T, Hkv, Dk, seed=seed + 1, scale=scale, dtype=dtype)
    v = _rand(T, Hkv, Dv, seed=seed + 2, scale=scale, dtype=dtype)
    gates = torch.sigmoid(_rand(T, Hq, 3, seed=seed + 3)).to(dtype)
    return q, k, v, gates


def test_forward_is_sum_of_pinned_parts_and_finite():
    p = O.NSAParams(32, 16, 64, 4, 128)
    q, k, v, gates = _cfg(512, 4, 1, 64, 64, 30)
    out, parts = O.nsa_forward_single(q, k, v, gates, p, return_parts=True)
    assert torch.isfinite(out).all()
    assert parts["idx"].shape == (512, 1, 4) and parts["pooled"].shape[-1] == 8
    ref = (torch.stack([parts["o_slc"], parts["o_swa"], parts["o_cmp"]], -1)
           @ gates.unsqueeze(-1)).squeeze(-1)
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-6)
    # a row whose picks are all future blocks has an exactly-zero selected branch
    valid = (parts["idx"] * 64 <= torch.arange(512)[:, None, None]) & (parts["idx"] >= 0)
    empty = ~valid.any(-1)[:, 0]
    assert empty.any()
    assert torch.count_nonzero(parts["o_slc"][empty]) == 0


def test_varlen_is_concatenation():
    p = O.NSAParams(32, 16, 64, 2, 64)
    lens = [130, 64, 257]
    cu = [0, 130, 194, 451]
    q, k, v, gates = _cfg(sum(lens), 4, 2, 16, 16, 40)
    packed = O.nsa_forward_varlen(q, k, v, gates, cu, p)
    for b in range(3):
        s, e = cu[b], cu[b + 1]
        alone = O.nsa_forward_single(q[s:e].clone(), k[s:e].clone(), v[s:e].clone(), gates[s:e].clone(), p)
        assert torch.equal(packed[s:e], alone)


@pytest.mark.parametrize("ctx", [256, 250, 70, 33, 20])
def test_decode_is_last_prefill_row(ctx):
    p = O.NSAParams(32, 16, 64, 2, 48)
    q, k, v, gates = _cfg(ctx, 4, 2, 16, 16, 50)
    full, parts = O.nsa_forward_single(q, k, v, gates, p, math_dtype=D64, return_parts=True)
    step, sp = O.nsa_decode_step(q[-1], k, v, gates[-1], p, math_dtype=D64, return_parts=True)
    torch.testing.assert_close(step, full[-1], rtol=1e-5, atol=1e-6)
    assert torch.equal(sp["idx"].sort(-1).values, parts["idx"][-1].sort(-1).values)


def test_compare_selection_rule():
    pooled = torch.tensor([[[0.5, 0.3, 0.2995, 0.1]]])
    ref = torch.tensor([[[0, 1]]])
    assert O.compare_selection(torch.tensor([[[1, 0]]]), ref, pooled) == (1, 1, 0, 0)
    assert O.compare_selection(torch.tensor([[[0, 2]]]), ref, pooled) == (1, 0, 1, 0)
    assert O.compare_selection(torch.tensor([[[0, 3]]]), ref, pooled) == (1, 0, 0, 1)


def test_row_subset_equals_full_run():
    p = O.NSAParams(32, 16, 64, 3, 100)
    q, k, v, gates = _cfg(700, 8, 2, 32, 16, 60)
    full, fp = O.nsa_forward_single(q, k, v, gates, p, return_parts=True)
    rows = torch.tensor([0, 1, 31, 32, 63, 64, 65, 300, 511, 512, 698, 699])
    sub, sp = O.nsa_forward_single(q, k, v, gates, p, return_parts=True, rows=rows)
    torch.testing.assert_close(sub, full[rows], rtol=1e-5, atol=1e-6)
    for key in ("o_cmp", "o_slc", "o_swa", "pooled"):
        torch.testing.assert_close(sp[key], fp[key][rows], rtol=1e-5, atol=1e-6)
    assert torch.equal(sp["idx"], fp["idx"][rows])


def test_short_sequence_has_compressed_branch_but_no_selection():
    p = O.NSAParams(32, 16, 64, 2, 16)
    q, k, v, gates = _cfg(64, 4, 2, 16, 16, 61)       # Nc = 3 < pool kernel 5
    out, parts = O.nsa_forward_single(q, k, v, gates, p, return_parts=True)
    assert (parts["idx"] == -1).all() and torch.count_nonzero(parts["o_slc"]) == 0
    assert torch.count_nonzero(parts["o_cmp"][32:]) > 0 and torch.count_nonzero(parts["o_cmp"][:32]) == 0


# ----------------------------------------------------------------------------- gradients
# The backward kernels are checked against autograd through the oracle's forward in float64.  These
# pins show that this is the right derivative: finite differences on tiny inputs (a dropped term or a
# wrong sign in any branch fails them) and the library's own attention gradient on the dense cases.

def _tiny(T=7, Hq=4, Hkv=2, Dk=4, Dv=3, seed=0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).requires_grad_(True)
    return mk(T, Hq, Dk), mk(T, Hkv, Dk), mk(T, Hkv, Dv)


def test_oracle_gradients_pass_finite_differences():
    q, k, v = _tiny()
    assert torch.autograd.gradcheck(lambda a, b, c: O.sliding_attention(a, b, c, 3, 0.5, math_dtype=torch.float64),
                                    (q, k, v), eps=1e-6, atol=1e-6)
    idx = torch.tensor([[[0, 1]], [[1, 0]], [[0, 5]], [[1, -1]], [[2, 0]], [[0, 1]], [[3, 1]]]).expand(7, 2, 2)
    assert torch.autograd.gradcheck(
        lambda a, b, c: O.selected_attention(a, b, c, idx, None, 2, 0.5, math_dtype=torch.float64),
        (q, k, v), eps=1e-6, atol=1e-6)
    g = torch.Generator().manual_seed(1)
    ck = torch.randn(3, 2, 4, generator=g, dtype=torch.float64).requires_grad_(True)
    cv = torch.randn(3, 2, 3, generator=g, dtype=torch.float64).requires_grad_(True)
    assert torch.autograd.gradcheck(
        lambda a, b, c: O.compressed_attention(a, b, c, 2, 2, 0.5, math_dtype=torch.float64),
        (q, ck, cv), eps=1e-6, atol=1e-6)
    x = torch.randn(9, 2, 3, generator=g, dtype=torch.float64).requires_grad_(True)
    w = torch.randn(4 * 3, 3, generator=g, dtype=torch.float64).requires_grad_(True)
    b = torch.randn(3, generator=g, dtype=torch.float64).requires_grad_(True)
    assert torch.autograd.gradcheck(lambda a, ww, bb: O.compress_weighted(a, ww, bb, 4, 2, 3, math_dtype=torch.float64),
                                    (x, w, b), eps=1e-6, atol=1e-6)
    assert torch.autograd.gradcheck(lambda a: O.compress_meanpool(a, 4, 2, 3, math_dtype=torch.float64), (x,),
                                    eps=1e-6, atol=1e-6)


def test_oracle_gradients_match_library_attention_on_dense_cases():
    """A window that covers the sequence, and all blocks selected, are plain causal attention: the
    oracle's gradients must equal those of F.scaled_dot_product_attention."""
    T, Hq, Hkv, D = 12, 4, 2, 8
    q, k, v = _tiny(T, Hq, Hkv, D, D, seed=3)
    d_o = torch.randn(T, Hq, D, generator=torch.Generator().manual_seed(4), dtype=torch.float64)

    def grads(fn):
        ins = [t.detach().clone().requires_grad_(True) for t in (q, k, v)]
        fn(*ins).backward(d_o)
        return [t.grad for t in ins]

    def sdpa(a, b, c):
        kk, vv = b.repeat_interleave(Hq // Hkv, 1), c.repeat_interleave(Hq // Hkv, 1)
        o = F.scaled_dot_product_attention(a.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True,
                                           scale=0.3)
        return o.transpose(0, 1)

    ref = grads(sdpa)
    idx = torch.arange(3).expand(T, Hkv, 3)
    for fn in (lambda a, b, c: O.sliding_attention(a, b, c, T, 0.3, math_dtype=torch.float64),
               lambda a, b, c: O.selected_attention(a, b, c, idx, None, 4, 0.3, math_dtype=torch.float64)):
        for got, want in zip(grads(fn), ref):
            assert float((got - want).abs().max()) < 1e-10


# ------------------------------------------------------------------------------ rotary embedding / layer
def _rope_inputs(interleaved, seed=0):
    from oracle import layer_oracle as L
    g = torch.Generator().manual_seed(seed)
    T, H, D, off, rd = 37, 3, 48, 16, 32
    x = torch.randn(T, H, D, generator=g, dtype=torch.float64)
    pos = torch.randint(0, 5000, (T,), generator=g)
    inv = 1.0 / (10000.0 ** (torch.arange(0, rd, 2, dtype=torch.float32) / rd))
    return L, x, pos, inv, off, rd


@pytest.mark.parametrize("interleaved", [False, True])
def test_rope_oracle_is_complex_multiplication(interleaved):
    """Rotation of a channel pair == multiplication of a + ib by exp(i * angle)."""
    L, x, pos, inv, off, rd = _rope_inputs(interleaved)
    y = L.rope_rotate(x, pos, inv, off, rd, interleaved, math_dtype=torch.float64)
    ang = (pos.float()[:, None] * inv[None, :]).double()
    unit = torch.polar(torch.ones_like(ang), ang)[:, None, :]
    r = x[..., off:off + rd]
    z = torch.complex(r[..., 0::2], r[..., 1::2]) if interleaved else torch.complex(r[..., :rd // 2], r[..., rd // 2:])
    z = z * unit
    want = torch.stack([z.real, z.imag], -1).flatten(-2) if interleaved else torch.cat([z.real, z.imag], -1)
    assert torch.allclose(y[..., off:off + rd], want, atol=1e-12)
    assert torch.equal(y[..., :off], x[..., :off])


def test_rope_oracle_invariants():
    L, x, pos, inv, off, rd = _rope_inputs(False, seed=1)
    kw = dict(math_dtype=torch.float64)
    y = L.rope_rotate(x, pos, inv, off, rd, False, **kw)
    # the two pairings are the same rotation up to the channel permutation between them
    perm = torch.arange(rd).view(2, rd // 2).t().reshape(-1)            # half layout -> interleaved layout
    xi = x.clone()
    xi[..., off:off + rd] = x[..., off:off + rd][..., perm]
    yi = L.rope_rotate(xi, pos, inv, off, rd, True, **kw)
    assert torch.allclose(yi[..., off:off + rd], y[..., off:off + rd][..., perm], atol=1e-12)
    # position 0 is the identity, norms are preserved, the inverse undoes it
    assert torch.equal(L.rope_rotate(x, torch.zeros_like(pos), inv, off, rd, False, **kw), x)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-12)
    assert torch.allclose(L.rope_rotate(y, pos, inv, off, rd, False, inverse=True, **kw), x, atol=1e-12)
    # scores depend on the distance only (dyadic inv_freq and small positions: the fp32 angles are exact)
    inv2 = 2.0 ** -torch.arange(rd // 2, dtype=torch.float32)
    q, k = x[:1], x[1:2]
    def score(m, n):
        qm = L.rope_rotate(q, torch.tensor([m]), inv2, off, rd, False, **kw)
        kn = L.rope_rotate(k, torch.tensor([n]), inv2, off, rd, False, **kw)
        return (qm * kn).sum(-1)
    assert torch.allclose(score(70, 50), score(25, 5), atol=1e-10)
    assert not torch.allclose(score(70, 50), score(70, 49), atol=1e-3)


def test_layer_oracle_without_rope_is_the_reference_module_on_projected_inputs():
    """With no rotation the layer oracle is Linear -> (gating on q, NSA forward) -> Linear."""
    from oracle import layer_oracle as L
    g = torch.Generator().manual_seed(3)
    T, hidden, hq, hkv, d = 96, 32, 4, 2, 16
    x = torch.randn(T, hidden, generator=g)
    wq, wk, wv = (torch.randn(n * d, hidden, generator=g) * 0.2 for n in (hq, hkv, hkv))
    wo = torch.randn(hidden, hq * d, generator=g) * 0.2
    gw, gb = torch.randn(3, d, generator=g), torch.randn(3, generator=g)
    p = O.NSAParams(8, 4, 16, 2, 16)
    out = L.layer_forward(x, wq, wk, wv, wo, gw, gb, [0, 60, T], p, hq, hkv, d, d)
    q, k, v = (F.linear(x, w).view(T, -1, d) for w in (wq, wk, wv))
    o = O.nsa_forward_varlen(q, k, v, F.linear(q, gw, gb), [0, 60, T], p)
    assert torch.allclose(out, F.linear(o.reshape(T, -1), wo), atol=1e-5)


def test_reference_signature_adapters_match_library_pipeline():
    """oracle/torch_attention.py (the reference's attention_ref / get_indices / construct_local_mask
    signatures, nsa/torch_attention.py:12,51,66) against library routines on the reference's batched
    layout: masked SDPA for the output, softmax -> group sum -> avg_pool1d(ceil_mode) -> topk for
    the indices, and the decode force_idx switch of the step oracle."""
    from oracle import torch_attention as TA
    B, T, Hq, Hkv, D, l, d, S = 2, 200, 8, 2, 32, 32, 16, 3
    G = Hq // Hkv
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, T, Hq, D, generator=g, dtype=torch.float64)
    Nc = O.compressed_len_conv(T, l, d)
    ck = torch.randn(B, Nc, Hkv, D, generator=g, dtype=torch.float64)
    cv = torch.randn(B, Nc, Hkv, D, generator=g, dtype=torch.float64)
    ckr, cvr = ck.repeat_interleave(G, 2), cv.repeat_interleave(G, 2)          # the "(h g)" repeat of the module
    out, idx = TA.attention_ref(q.float(), ckr.float(), cvr.float(), d, l, causal=True, pool_num_kv_head=Hkv,
                                pool_kernel_size=5, pool_stride=4, pool_padding=0, select_block_count=S)
    assert out.shape == (B, T, Hq, D) and idx.shape == (B, T, Hkv, S) and idx.dtype == torch.int64
    hidden = TA.construct_local_mask(T, Nc, d, l)
    assert hidden.shape == (T, Nc) and bool(hidden[l - 1].all()) and not bool(hidden[l, 0]) and bool(hidden[l, 1])
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), ckr.transpose(1, 2), cvr.transpose(1, 2),
                                         attn_mask=~hidden[None, None]).transpose(1, 2)
    ref = torch.where(hidden.all(-1)[None, :, None, None], torch.zeros_like(ref), ref)   # rows that see nothing
    assert float((out.double() - ref).abs().max()) < 1e-5
    p = torch.softmax(torch.einsum("bthd,bchd->bhtc", q, ckr), -1)
    pooled = F.avg_pool1d(p.reshape(B, Hkv, G, T, Nc).sum(2).reshape(B * Hkv, T, Nc), 5, 4, 0, True)
    lib_idx = torch.topk(pooled.reshape(B, Hkv, T, -1), S, dim=3).indices.transpose(1, 2)
    assert torch.equal(idx.sort(-1).values, lib_idx.sort(-1).values)
    assert torch.equal(TA.get_indices(p.float(), Hkv, 5, 4, 0, S).sort(-1).values, lib_idx.sort(-1).values)
    # non-causal: every compressed row visible
    out_nc, _ = TA.attention_ref(q.float(), ckr.float(), cvr.float(), d, l, causal=False)
    ref_nc = F.scaled_dot_product_attention(q.transpose(1, 2), ckr.transpose(1, 2), cvr.transpose(1, 2)).transpose(1, 2)
    assert float((out_nc.double() - ref_nc).abs().max()) < 1e-5
    with pytest.raises(NotImplementedError):
        TA.attention_ref(q, ckr, cvr, d, l, dropout_p=0.1)


def test_decode_oracle_forced_picks():
    """force_idx replaces the blocks of the selected branch only; the oracle's own picks still come back."""
    ctx, Hq, Hkv, D = 700, 8, 2, 32
    g = torch.Generator().manual_seed(6)
    q = torch.randn(Hq, D, generator=g)
    k = torch.randn(ctx, Hkv, D, generator=g)
    v = torch.randn(ctx, Hkv, D, generator=g)
    gates = torch.rand(Hq, 3, generator=g)
    p = O.NSAParams(32, 16, 64, 3, 64)
    a, pa = O.nsa_decode_step(q, k, v, gates, p, return_parts=True)
    b, pb = O.nsa_decode_step(q, k, v, gates, p, return_parts=True, force_idx=pa["idx"])
    assert torch.equal(a, b) and torch.equal(pa["idx"], pb["idx"])
    other = torch.tensor([[0, 1, 2], [3, 4, 5]])
    c, pc = O.nsa_decode_step(q, k, v, gates, p, return_parts=True, force_idx=other)
    assert torch.equal(pc["idx"], pa["idx"]) and torch.equal(pc["o_cmp"], pa["o_cmp"]) and torch.equal(pc["o_swa"], pa["o_swa"])
    blocks = torch.cat([torch.arange(0, 192), ])
    s0 = (q.view(Hkv, -1, D)[0] @ k[blocks, 0].T) / math.sqrt(D)
    assert torch.allclose(pc["o_slc"].view(Hkv, -1, D)[0], torch.softmax(s0, -1) @ v[blocks, 0], atol=1e-5)
