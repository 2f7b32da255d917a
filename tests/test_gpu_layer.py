"""GPU tests of the model-integration pieces: the packed-row split with rotary embedding (forward and
its transpose), and the attention layer built on it (fused projection with the gating Linear folded
in -> split + rotation -> NSA -> output projection; prefill, decode, backward) against the un-fused
CPU oracle."""
import math

import pytest
import torch

from oracle import layer_oracle as L
from oracle import nsa_oracle as O
from tests.util import max_abs, ragged_cu, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _inv_freq(rd, theta=10000.0):
    return 1.0 / (theta ** (torch.arange(0, rd, 2, dtype=torch.float32) / rd))


def _layout(hq, hkv, dk, dv, lead=0, gap=8):
    """column offsets with gaps between the four ranges, so that strides and offsets are exercised"""
    q_off = lead
    k_off = q_off + hq * dk + gap
    v_off = k_off + hkv * dk
    g_off = v_off + hkv * dv + 3          # gate columns need no alignment
    ld = (g_off + 3 * hq + 7) // 8 * 8 + gap
    return (q_off, k_off, v_off, g_off), ld


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hq,hkv,dk,dv,off,rd,inter,explicit", [
    (64, 4, 192, 128, 128, 64, False, False),
    (8, 2, 64, 64, 0, 64, False, True),
    (5, 1, 48, 40, 16, 32, True, False),
    (4, 4, 128, 64, 120, 8, True, True),
    (3, 1, 64, 64, 0, 0, False, False),
])
def test_qkv_rope_split_matches_oracle(dtype, hq, hkv, dk, dv, off, rd, inter, explicit):
    from nsa_amd import ops
    lens = [300, 1, 77, 129]
    T = sum(lens)
    offsets, ld = _layout(hq, hkv, dk, dv, lead=8)
    packed = randn(T, ld, seed=800, dtype=dtype)
    cu = ragged_cu(lens)
    pos = L.positions_from_cu(cu)
    if explicit:
        pos = (pos * 97 + 31000) % 40000                     # large, unordered positions
    inv = _inv_freq(rd) if rd else None
    q, k, v, g = ops.qkv_rope_split(packed.to(DEV), hq, hkv, dk, dv, offsets, inv,
                                    pos.to(DEV) if explicit else None, torch.tensor(cu, dtype=torch.int32, device=DEV),
                                    off, rd, inter)
    qo, ko, vo, go = offsets
    qs = packed[:, qo:qo + hq * dk].view(T, hq, dk)
    ks = packed[:, ko:ko + hkv * dk].view(T, hkv, dk)
    assert torch.equal(v.cpu(), packed[:, vo:vo + hkv * dv].view(T, hkv, dv))
    assert torch.equal(g.cpu(), packed[:, go:go + 3 * hq].view(T, hq, 3))
    for got, src in ((q, qs), (k, ks)):
        got = got.cpu()
        want = L.rope_rotate(src, pos, inv, off, rd, inter) if rd else src.float()
        keep = torch.ones(dk, dtype=torch.bool)
        keep[off:off + rd] = False
        assert torch.equal(got[..., keep], src[..., keep])                       # content channels: a copy
        err = (got.double() - want.double()).abs()
        ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
        bound = 1e-5 if dtype == torch.float32 else want.double().abs() * ulp + 1e-6        # one rounding
        assert bool((err <= bound).all()), float(err.max())


@pytest.mark.parametrize("inter", [False, True])
def test_qkv_rope_pack_is_the_transpose_of_split(inter):
    """<split(x), g> == <x, pack(g)> for random x and g (fp32), and pack(split(x)) == x on the
    covered columns: the backward pass is the exact adjoint, rotation included."""
    from nsa_amd import ops
    hq, hkv, dk, dv, off, rd = 6, 2, 96, 64, 32, 64
    lens = [100, 37]
    T = sum(lens)
    offsets, ld = _layout(hq, hkv, dk, dv)
    cu = torch.tensor(ragged_cu(lens), dtype=torch.int32, device=DEV)
    inv = _inv_freq(rd)
    x = randn(T, ld, seed=810).to(DEV)
    q, k, v, g = ops.qkv_rope_split(x, hq, hkv, dk, dv, offsets, inv, None, cu, off, rd, inter)
    gq, gk, gv, gg = (randn(*t.shape, seed=811 + i).to(DEV) for i, t in enumerate((q, k, v, g)))
    back = ops.qkv_rope_pack(gq, gk, gv, gg, ld, offsets, inv, None, cu, off, rd, inter)
    lhs = sum(float((a.double() * b.double()).sum()) for a, b in ((q, gq), (k, gk), (v, gv), (g, gg)))
    rhs = float((x.double() * back.double()).sum())
    assert abs(lhs - rhs) <= 1e-4 * max(1.0, abs(lhs)), (lhs, rhs)
    again = ops.qkv_rope_pack(q, k, v, g, ld, offsets, inv, None, cu, off, rd, inter)
    covered = torch.zeros(ld, dtype=torch.bool)
    for o, n in zip(offsets, (hq * dk, hkv * dk, hkv * dv, 3 * hq)):
        covered[o:o + n] = True
    assert max_abs(again[:, covered], x[:, covered]) <= 1e-5
    assert (again[:, ~covered] == 0).all()


def _layer(dtype, hidden, hq, hkv, dk, dv, rd, mode, act, S, W, bias=False, inter=False, seed=0, sel_block=64):
    from nsa_amd.layer import NSAAttentionLayer
    torch.manual_seed(seed)
    layer = NSAAttentionLayer(hidden, hq, hkv, qk_head_dim=dk, v_head_dim=dv, rope_dim=rd, rope_interleaved=inter,
                              bias=bias, selection_block=sel_block, selected_block_count=S, sliding_window=W, compressor_mode=mode,
                              gate_activation=act, dtype=dtype)
    with torch.no_grad():                      # livelier than the default init: gates of both signs
        layer.attn.gating.weight.normal_(0, 0.3)
        layer.attn.gating.bias.normal_(0, 0.5)
    return layer


def _oracle_args(layer, math=None):
    def c(t):
        if t is None:
            return None
        t = t.detach().cpu()
        return t if math is None else t.to(math).requires_grad_(True)

    a = dict(w_q=c(layer.q_proj.weight), w_k=c(layer.k_proj.weight), w_v=c(layer.v_proj.weight),
             w_o=c(layer.o_proj.weight), gating_w=c(layer.attn.gating.weight), gating_b=c(layer.attn.gating.bias),
             b_q=c(layer.q_proj.bias), b_k=c(layer.k_proj.bias), b_v=c(layer.v_proj.bias), b_o=c(layer.o_proj.bias))
    comp = None
    if layer.attn.compressor.mode == "conv":
        def lin(conv):
            w = conv.weight.detach().cpu()
            w = w.permute(2, 1, 0).reshape(-1, w.shape[0])
            return w if math is None else w.to(math).requires_grad_(True)
        ck, cv = layer.attn.compressor.compressor_k, layer.attn.compressor.compressor_v
        comp = {"wk": lin(ck), "wv": lin(cv), "bk": c(ck.bias), "bv": c(cv.bias)}
    return a, comp


def _params(layer):
    a = layer.attn
    return O.NSAParams(a.compression_block, a.compression_stride, a.selection_block_size, a.selected_block_count,
                       a.sliding_window, 1.0 / math.sqrt(layer.dk))


@pytest.mark.parametrize("mode,act,rd,bias,inter,lens", [
    ("mean", "sigmoid", 32, False, False, [300, 129]),
    ("conv", None, 0, True, False, [257]),
    ("mean", None, 16, True, True, [64, 1, 200]),
])
def test_layer_fp32_matches_unfused_oracle(mode, act, rd, bias, inter, lens):
    hidden, hq, hkv, dk, dv = 96, 8, 2, 64, 64
    layer = _layer(torch.float32, hidden, hq, hkv, dk, dv, rd, mode, act, 3, 48, bias, inter).to(DEV)
    T = sum(lens)
    x = randn(T, hidden, seed=820, scale=1.0)
    cu = ragged_cu(lens)
    with torch.no_grad():
        out, idx = layer(x.to(DEV), cu_seqlens=torch.tensor(cu, dtype=torch.int32, device=DEV), return_indices=True)
    a, comp = _oracle_args(layer)
    ref = L.layer_forward(x, cu_seqlens=cu, p=_params(layer), hq=hq, hkv=hkv, dk=dk, dv=dv,
                          inv_freq=None if rd == 0 else layer.inv_freq.cpu(), rope_off=dk - rd, rope_dim=rd,
                          interleaved=inter, gate_activation=act, compressor=comp, force_idx=idx.cpu().long(), **a)
    err = max_abs(out, ref)
    print("layer fp32", mode, act, rd, lens, "max_abs", err, "max|ref|", float(ref.abs().max()))
    assert err <= 2e-4 * max(1.0, float(ref.abs().max()))


def test_layer_bf16_projections_match_unfused_oracle_and_equal_lengths_batch():
    """bf16: q, k, v and the folded gate logits against the un-fused oracle (one rounding each), and
    the [B, T, hidden] calling convention against the packed one."""
    from nsa_amd import ops
    hidden, hq, hkv, dk, dv, rd = 256, 16, 2, 192, 128, 64
    layer = _layer(torch.bfloat16, hidden, hq, hkv, dk, dv, rd, "mean", "sigmoid", 4, 64).to(DEV)
    B, T = 2, 320
    x = randn(B, T, hidden, seed=830, dtype=torch.bfloat16)
    with torch.no_grad():
        w, b = layer.fused_projection()
        packed = torch.nn.functional.linear(x.view(B * T, hidden).to(DEV), w, b)
        cu = ops.uniform_cu(B, T, DEV)
        q, k, v, g = ops.qkv_rope_split(packed, hq, hkv, dk, dv, layer.offsets, layer.inv_freq, None, cu, dk - rd, rd)
        out_b, _ = layer(x.to(DEV))
        out_p, _ = layer(x.view(B * T, hidden).to(DEV), cu_seqlens=cu)
    assert out_b.shape == (B, T, hidden) and torch.equal(out_b.view(B * T, hidden), out_p)
    assert torch.isfinite(out_b.float()).all()
    a, _ = _oracle_args(layer)
    _, parts = L.layer_forward(x.view(B * T, hidden), cu_seqlens=[0, T, 2 * T], p=_params(layer), hq=hq, hkv=hkv,
                               dk=dk, dv=dv, inv_freq=layer.inv_freq.cpu(), rope_off=dk - rd, rope_dim=rd,
                               gate_activation="sigmoid", return_parts=True, **a)
    for name, got, want in (("q", q, parts["q"]), ("k", k, parts["k"]), ("v", v, parts["v"]),
                            ("gate logits", g, parts["logits"])):
        err = max_abs(got, want)
        print("layer bf16", name, "max_abs", err, "max|ref|", float(want.float().abs().max()))
        assert err <= 2e-2 * max(1.0, float(want.float().abs().max()))


@pytest.mark.parametrize("hq,hkv,sel_block", [(16, 2, 64), (64, 2, 64), (16, 2, 32)])
@pytest.mark.parametrize("paged", [False, True])
def test_layer_decode_continues_prefill(paged, hq, hkv, sel_block):
    """Prompt through the layer with a cache, then single-token calls: every decoded row equals the
    corresponding row of one prefill over the whole sequence (also for a GQA group of 32 heads).  With selection
    blocks of 32 keys the picks are a real choice (8 blocks, 4 picks), and a prefill row's picks depend on the
    compressed rows after it (the importance softmax is normalised over all of them, per head, before the head
    sum): there a decoded row is compared with the last row of a prefill over exactly the cached tokens."""
    from nsa_amd.decode import NSADecodeCache, NSAPagedDecodeCache
    hidden, dk, dv, rd = 256, 192, 128, 64
    layer = _layer(torch.bfloat16, hidden, hq, hkv, dk, dv, rd, "mean", "sigmoid", 4, 64, sel_block=sel_block).to(DEV)
    B, T0, steps = 2, 250, 20
    x = randn(B, T0 + steps, hidden, seed=840, dtype=torch.bfloat16).to(DEV)
    with torch.no_grad():
        full, _ = layer(x)
        if paged:
            cache = NSAPagedDecodeCache(B, 12, 320, hkv, dk, dv, dtype=torch.bfloat16, device=DEV)
        else:
            cache = NSADecodeCache(B, 320, hkv, dk, dv, dtype=torch.bfloat16, device=DEV)
        first, _ = layer(x[:, :T0], past_key_value=cache, use_cache=True)
        assert max_abs(first, full[:, :T0] if sel_block == 64 else layer(x[:, :T0])[0]) <= 2e-2
        worst = 0.0
        for s in range(steps):
            out, _ = layer(x[:, T0 + s:T0 + s + 1], past_key_value=cache, use_cache=True)
            assert out.shape == (B, 1, hidden)
            row = full[:, T0 + s] if sel_block == 64 else layer(x[:, :T0 + s + 1])[0][:, -1]
            worst = max(worst, max_abs(out[:, 0], row))
    print("layer decode vs prefill rows max_abs", worst)
    assert int(cache.ctx_lens[0]) == T0 + steps
    assert worst <= 3e-2


@pytest.mark.parametrize("mode,act,rd,lens", [("mean", "sigmoid", 32, [300, 150]), ("conv", None, 64, [260])])
def test_layer_backward_matches_oracle_autograd(mode, act, rd, lens):
    """Gradients of the input and of every parameter (projections through the fused GEMM, the gating
    Linear through the fold, compressor, output projection) against float64 autograd through the
    un-fused oracle with the layer's own block picks."""
    hidden, hq, hkv, dk, dv = 128, 16, 1, 64, 64
    dtype = torch.bfloat16
    layer = _layer(dtype, hidden, hq, hkv, dk, dv, rd, mode, act, 3, 48, bias=True).to(DEV)
    T = sum(lens)
    x = randn(T, hidden, seed=850, dtype=dtype)
    d_out = randn(T, hidden, seed=851, dtype=dtype)
    cu = ragged_cu(lens)
    xd = x.to(DEV).requires_grad_(True)
    out, idx = layer(xd, cu_seqlens=torch.tensor(cu, dtype=torch.int32, device=DEV), return_indices=True)
    out.backward(d_out.to(DEV))
    a, comp = _oracle_args(layer, math=torch.float64)
    xr = x.double().requires_grad_(True)
    ref = L.layer_forward(xr, cu_seqlens=cu, p=_params(layer), hq=hq, hkv=hkv, dk=dk, dv=dv,
                          inv_freq=layer.inv_freq.cpu() if rd else None, rope_off=dk - rd, rope_dim=rd,
                          gate_activation=act, compressor=comp, force_idx=idx.cpu().long(),
                          math_dtype=torch.float64, **a)
    ref.backward(d_out.double())

    def check(name, got, want, tol=3e-2):
        err = max_abs(got, want)
        mag = max(1.0, float(want.abs().max()))
        print("   %-12s max_abs %.3e  (max|ref| %.3f)" % (name, err, mag))
        assert torch.isfinite(got.float()).all() and err <= tol * mag, name

    print("layer_bwd", mode, act, rd, lens)
    check("out", out.detach(), ref.detach())
    check("dx", xd.grad, xr.grad)
    check("dWq", layer.q_proj.weight.grad, a["w_q"].grad)
    check("dWk", layer.k_proj.weight.grad, a["w_k"].grad)
    check("dWv", layer.v_proj.weight.grad, a["w_v"].grad)
    check("dWo", layer.o_proj.weight.grad, a["w_o"].grad)
    check("dbq", layer.q_proj.bias.grad, a["b_q"].grad)
    check("dbv", layer.v_proj.bias.grad, a["b_v"].grad)
    check("dgating.w", layer.attn.gating.weight.grad, a["gating_w"].grad)
    check("dgating.b", layer.attn.gating.bias.grad, a["gating_b"].grad)
    if mode == "conv":
        conv = layer.attn.compressor.compressor_k
        w = comp["wk"].grad
        check("dconv_k.w", conv.weight.grad, w.reshape(-1, dk, dk).permute(2, 1, 0))


def test_layer_explicit_position_ids_equal_derived_positions():
    hidden, hq, hkv, dk, dv, rd = 128, 8, 2, 64, 64, 32
    layer = _layer(torch.bfloat16, hidden, hq, hkv, dk, dv, rd, "mean", "sigmoid", 2, 32).to(DEV)
    lens = [200, 1, 90]
    cu = ragged_cu(lens)
    x = randn(sum(lens), hidden, seed=860, dtype=torch.bfloat16).to(DEV)
    cud = torch.tensor(cu, dtype=torch.int32, device=DEV)
    with torch.no_grad():
        a, _ = layer(x, cu_seqlens=cud, max_seqlen=max(lens))
        b, _ = layer(x, cu_seqlens=cud, position_ids=L.positions_from_cu(cu).to(DEV))
        c, _ = layer(x, cu_seqlens=cud, position_ids=L.positions_from_cu(cu).to(DEV) + 7)
    assert torch.equal(a, b)
    assert not torch.equal(a, c)      # content channels make absolute positions matter (rope_dim < head dim)
