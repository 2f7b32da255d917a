"""CPU-side checks of the boundary: the shared library loads, exports every symbol the header
declares, and the host-only helpers and error paths behave (no kernel is launched here)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
    src = open(os.path.join(ROOT, "include", "nsa_hip.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(nsa_[a-z0-9_]+)\s*\(", src)))


@pytest.fixture(scope="module")
def lib():
    from nsa_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from nsa_amd import build
        build.build()
    return _lib.load()


def test_every_declared_symbol_is_exported_and_bound(lib):
    from nsa_amd import _lib
    names = _header_symbols()
    assert "nsa_compress_fwd" in names and "nsa_slc_combine_fwd" in names
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), "header declares %s but the library does not export it" % n
        assert n in _lib.SIGNATURES, "%s has no ctypes signature" % n
    for n in _lib.SIGNATURES:
        assert n in names, "%s is bound but not declared in include/nsa_hip.h" % n


def test_signature_arity_matches_header(lib):
    from nsa_amd import _lib
    src = open(os.path.join(ROOT, "include", "nsa_hip.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    for name, (_, args) in _lib.SIGNATURES.items():
        m = re.search(r"\b%s\s*\(([^)]*)\)" % name, src)
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else params.count(",") + 1
        assert n == len(args), "%s: header has %d parameters, binding has %d" % (name, n, len(args))


def test_host_helpers(lib):
    assert lib.nsa_version() >= 100
    for cu_b, b in [(0, 0), (1, 1), (8, 1), (1000, 3), (32768, 1)]:
        off = lib.nsa_transposed_offset(cu_b, b)
        assert off % 8 == 0 and off >= cu_b
    # offsets never overlap: next sequence starts after the previous one ends
    cu = [0, 5, 5, 77, 1024, 1031]
    offs = [lib.nsa_transposed_offset(c, b) for b, c in enumerate(cu)]
    for b in range(len(cu) - 1):
        assert offs[b] + (cu[b + 1] - cu[b]) <= offs[b + 1]
    cols = lib.nsa_transposed_cols(cu[-1], len(cu) - 1)
    assert cols % 64 == 0 and cols >= offs[-1] + 64


def test_argument_errors_do_not_launch(lib):
    # null pointers / bad sizes are rejected before any HIP call, so this runs without a GPU
    rc = lib.nsa_swa_fwd(None, None, None, None, None, None, 1, 64, 4, 1, 64, 64, 128, 16, 0.1, 0, None)
    assert rc == -1 and b"null" in lib.nsa_last_error_string()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.c_void_p((ctypes.addressof(buf) + 15) & ~15)
    rc = lib.nsa_swa_fwd(p, p, p, p, None, p, 1, 64, 48, 2, 64, 64, 128, 16, 0.1, 0, None)      # GQA group of 24
    assert rc == -2 and b"group size" in lib.nsa_last_error_string()
    rc = lib.nsa_decode_step(p, p, p, p, p, p, None, p, None, 1, 64, 2, 64, 64, 64, 64, 32, 16, 64, 5, 4, 0, 4, 16, 0.1,
                             0, 0, None)                                        # group of 32: the split schedule only
    assert rc == -2 and b"nsa_decode_step_split" in lib.nsa_last_error_string()
    rc = lib.nsa_decode_step(p, p, p, p, p, p, None, p, None, 1, 48, 2, 64, 64, 64, 64, 32, 16, 64, 5, 4, 0, 4, 16, 0.1,
                             0, 0, None)                                                             # group of 24
    assert rc == -2 and b"group size" in lib.nsa_last_error_string()
    rc = lib.nsa_decode_step(p, p, p, p, p, p, None, p, None, 1, 4, 1, 64, 64, 4096, 256, 32, 16, 32, 2, 1, 0, 4, 16,
                             0.1, 0, 0, None)                                                        # 255 bins > 132
    assert rc == -2 and b"pooled bins" in lib.nsa_last_error_string()
    rc = lib.nsa_decode_step(p, p, p, p, p, p, None, p, None, 1, 4, 1, 64, 64, 65536, 4096, 32, 16, 64, 5, 4, 0, 4, 16,
                             0.1, 0, 0, None)                                                        # one workgroup: 2304 rows
    assert rc == -2 and b"nsa_decode_step_split" in lib.nsa_last_error_string()
    rc = lib.nsa_decode_step_split_static(p, p, p, None, 0, p, p, p, None, p, None, 160, 64, 4, 128, 128, 32768, 2048, 32,
                                          16, 64, 5, 4, 0, 16, 512, 0.1, 0, 0, 8, None)
    assert rc == -3 and b"fixed array" in lib.nsa_last_error_string()
    rc = lib.nsa_swa_fwd(p, p, p, p, None, p, 1, 64, 4, 1, 48, 64, 128, 16, 0.1, 0, None)
    assert rc == -2
    rc = lib.nsa_swa_fwd(p, p, p, p, None, p, 1, 64, 4, 1, 64, 64, 128, 16, 0.1, 7, None)
    assert rc == -1
    rc = lib.nsa_slc_combine_fwd(p, p, p, p, None, None, None, None, 1, None, None, p, None, p, 1, 64, 4, 1, 64, 64, 128,
                                 4, 60, 0.1, 1, 0, 0, None, 0, None)
    assert rc == -2 and b"block_size" in lib.nsa_last_error_string()
    # the slab schedule: null pointers, a selection block the 64-key schedule cannot express, a workspace below one tile
    fused = lambda ws, ws_bytes, block=64, q=p: lib.nsa_slc_swa_fused_fwd(      # noqa: E731
        q, p, p, p, None, None, None, None, 1, None, p, p, 1, 4096, 16, 1, 64, 64, 4224, 128, 4, block, 0.1, 0, 0, 0, None,
        None, None, None, ws, ws_bytes, None)
    assert fused(p, 1 << 30, q=None) == -1 and b"null" in lib.nsa_last_error_string()
    assert fused(None, 1 << 30) == -1
    assert fused(p, 1 << 30, block=48) == -2 and b"multiple of 64" in lib.nsa_last_error_string()
    assert fused(p, 1024) == -1 and b"one tile" in lib.nsa_last_error_string()
    one_tile = lib.nsa_slc_swa_fused_workspace_bytes(4096, 1, 16, 1, 64, 64, 4, 64, 0, 1)
    assert 0 < one_tile < lib.nsa_slc_swa_fused_workspace_bytes(4096, 1, 16, 1, 64, 64, 4, 64, 0, 1024) \
        < lib.nsa_slc_swa_fused_workspace_bytes(4096, 1, 16, 1, 64, 64, 4, 64, 0, 0) \
        == lib.nsa_slc_workspace_bytes(4096, 1, 1, 64, 64, 4, 64, 0)
    assert lib.nsa_slc_swa_fused_workspace_bytes(4096, 1, 16, 1, 64, 64, 4, 64, 1, 0) == 0      # fp32: no block-major schedule
    rc = lib.nsa_compress_fwd(p, None, None, p, p, p, 1, 10, 2, 60, 32, 16, 0, None)
    assert rc == -2
    # K and V in one call: both weights or neither, dims in pieces of 8, known dtypes (0, 1, 2)
    rc = lib.nsa_compress_kv_fwd(p, p, p, None, None, None, p, p, p, p, 1, 10, 2, 64, 64, 32, 16, 0, None)
    assert rc == -1 and b"both weights" in lib.nsa_last_error_string()
    rc = lib.nsa_compress_kv_fwd(p, p, None, None, None, None, p, None, p, p, 1, 10, 2, 64, 64, 32, 16, 0, None)
    assert rc == -1 and b"null" in lib.nsa_last_error_string()
    rc = lib.nsa_compress_kv_fwd(p, p, None, None, None, None, p, p, p, p, 1, 10, 2, 64, 60, 32, 16, 0, None)
    assert rc == -2
    rc = lib.nsa_compress_kv_fwd(p, p, None, None, None, None, p, p, p, p, 1, 10, 2, 64, 64, 32, 16, 3, None)
    assert rc == -1 and b"dtype" in lib.nsa_last_error_string()
    rc = lib.nsa_compress_bwd(None, None, p, p, None, None, p, p, 1, 64, 3, 1, 64, 32, 16, 3, None)
    assert rc == -1 and b"dtype" in lib.nsa_last_error_string()


def test_python_wrappers_refuse_cpu_tensors_and_missing_library(monkeypatch):
    from nsa_amd import _lib, ops
    x = torch.zeros(64, 1, 64, dtype=torch.bfloat16)
    cu = torch.tensor([0, 64], dtype=torch.int32)
    with pytest.raises(RuntimeError):
        ops.transpose(x, cu, 1)
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libnsa_hip.so")
    with pytest.raises(_lib.NSALibraryError):
        _lib.load()


def test_host_side_shapes_and_counts():
    from nsa_amd import ops
    from nsa_amd.compression_kv import calc_compressed_len, conv_compressed_len
    from oracle import nsa_oracle as O
    for T in (31, 32, 64, 1000, 1024, 32768):
        assert conv_compressed_len(T, 16, 32) == O.compressed_len_conv(T, 32, 16)
    assert calc_compressed_len(1024, 16, 64) == (1024 - 64) // 16
    for nc in (0, 3, 5, 63, 511, 2047):
        for k, s, p in ((5, 4, 0), (5, 4, 2)):
            assert ops.pool_bins(nc, k, s, p) == (O.pool_geometry(nc, k, s, p)[0] if nc > 0 else 0)
    cu = torch.tensor([0, 100, 131, 1131], dtype=torch.int32)
    assert ops.compressed_offsets(cu, 32, 16, 1).tolist() == [0, 5, 5, 66]
    assert ops.compressed_offsets(cu, 32, 16, 0).tolist() == [0, 4, 4, 64]


def test_module_keeps_reference_parameter_names():
    from nsa_amd.nsa import NSAAttention
    m = NSAAttention(64, True)
    names = set(dict(m.named_parameters()))
    assert names == {"compressor.compressor_k.weight", "compressor.compressor_k.bias",
                     "compressor.compressor_v.weight", "compressor.compressor_v.bias",
                     "gating.weight", "gating.bias"}
    assert m.compressor.compressor_k.weight.shape == (64, 64, 32) and m.gating.weight.shape == (3, 64)
    assert (m.pool_kernel_size, m.pool_stride, m.pool_padding) == (5, 4, 0)


def test_uniform_cu_of_empty_sequences():
    """A batch whose sequences have no compressed rows still gets a valid offsets tensor."""
    import torch
    from nsa_amd import ops
    assert ops.uniform_cu(3, 0, "cpu").tolist() == [0, 0, 0, 0]
    assert ops.uniform_cu(2, 5, "cpu").tolist() == [0, 5, 10]


def test_backward_argument_errors_do_not_launch(lib):
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.c_void_p((ctypes.addressof(buf) + 15) & ~15)
    # compressed attention backward
    rc = lib.nsa_cmp_attn_bwd(None, p, p, p, p, p, None, None, p, p, 1, 64, 2, 16, 1, 64, 64, 32, 16, 0.1, 1, 0, p, p, p, p, 1 << 20, None)
    assert rc == -1 and b"null" in lib.nsa_last_error_string()
    rc = lib.nsa_cmp_attn_bwd(p, p, p, p, p, p, None, None, p, p, 1, 64, 2, 16, 1, 64, 64, 32, 16, 0.1, 1, 0, p, p, p, p, 8, None)
    assert rc == -1 and b"workspace" in lib.nsa_last_error_string()
    assert lib.nsa_cmp_attn_bwd_workspace_bytes(64, 2, 16, 1, 64, 64) >= 64 * 16 * 4 + 2 * 2 * 64 * 4
    # selected + sliding backward: a branch needs its saved tensors
    rc = lib.nsa_slc_swa_bwd(p, p, p, None, None, p, None, None, None, None, None, None, None, None, None, p, 1, 64, 16, 1, 64, 64, 4, 64, 0, 0.1, 1,
                             0, None, p, p, p, p, 1 << 30, None)
    assert rc == -1 and b"selected branch" in lib.nsa_last_error_string()
    # selection blocks: 8, 16, 32 or a multiple of 64 keys, at most 64 slots of 64 keys per (token, head)
    for block, top_n in ((48, 4), (24, 4), (128, 40)):
        rc = lib.nsa_slc_swa_bwd(p, p, p, p, None, p, None, p, None, None, None, None, None, p, None, p, 1, 64, 16, 1, 64, 64, top_n, block, 0, 0.1, 1, 0,
                                 None, p, p, p, p, 1 << 30, None)
        assert rc == -2 and b"multiple of 64" in lib.nsa_last_error_string()
    assert lib.nsa_slc_workspace_bytes(64, 1, 1, 64, 64, 4, 48, 0) == 0
    assert lib.nsa_slc_workspace_bytes(64, 1, 1, 64, 64, 40, 128, 0) == 0
    assert lib.nsa_slc_workspace_bytes(64, 1, 1, 64, 64, 4, 128, 0) > lib.nsa_slc_workspace_bytes(64, 1, 1, 64, 64, 4, 32, 0) > 0
    rc = lib.nsa_slc_swa_bwd(p, p, p, None, p, None, p, None, p, None, None, None, None, None, None, p, 1, 64, 16, 1, 64, 64, 0, 64, 0, 0.1, 1, 0, None, p, p,
                             p, p, 1 << 30, None)
    assert rc == -1 and b"sliding branch" in lib.nsa_last_error_string()
    # dq_add must not be the output itself
    rc = lib.nsa_slc_swa_bwd(p, p, p, None, p, None, p, None, p, None, None, None, None, None, None, p, 1, 64, 16, 1, 64, 64, 0, 64, 64, 0.1, 1, 0, p, p,
                             p, p, p, 1 << 30, None)
    assert rc == -1 and b"dq_add" in lib.nsa_last_error_string()
    need = lib.nsa_slc_swa_bwd_workspace_bytes(64, 1, 16, 1, 64, 64, 4, 64, 0)
    assert need > lib.nsa_slc_swa_bwd_workspace_bytes(64, 1, 16, 1, 64, 64, 0, 64, 0) > 0
    # compression, gates
    rc = lib.nsa_compress_bwd(None, None, p, p, p, None, p, p, 1, 64, 2, 1, 64, 32, 16, 0, None)
    assert rc == -1 and b"weight" in lib.nsa_last_error_string()
    rc = lib.nsa_gate_bwd(p, p, p, p, None, None, 64, 64, 0, None)
    assert rc == -1
    rc = lib.nsa_gate_combine_fwd(p, p, None, None, p, 64, 60, 0, 0, None)
    assert rc == -1 and b"multiple of 8" in lib.nsa_last_error_string()
    rc = lib.nsa_gate_combine_bwd(p, p, p, p, None, p, None, None, p, None, 64, 64, 0, 0, None)
    assert rc == -1 and b"null" in lib.nsa_last_error_string()


def test_needs_grad_follows_the_grad_mode():
    from nsa_amd.autograd import needs_grad
    for dtype in (torch.float16, torch.bfloat16, torch.float32):
        x = torch.zeros(2, 2, dtype=dtype, requires_grad=True)
        assert needs_grad(None, x)
        with torch.no_grad():
            assert not needs_grad(x)
        assert not needs_grad(x.detach(), None)


def test_training_path_is_taken_only_when_something_requires_grad():
    from nsa_amd.autograd import needs_grad
    a, b = torch.zeros(2), torch.zeros(2, requires_grad=True)
    assert not needs_grad(a, None) and needs_grad(a, b)
    with torch.no_grad():
        assert not needs_grad(a, b)


def test_paged_cache_bookkeeping_on_host():
    """Free list, growth, release and capacity errors of the paged cache need no GPU."""
    from nsa_amd.decode import NSAPagedDecodeCache
    c = NSAPagedDecodeCache(2, 5, 200, 1, 64, 64, dtype=torch.float32, device="cpu")
    assert (c.max_pages, c.ctx_cap, c.free_pages) == (4, 256, 5)
    assert c._grow(0, 65) == [(0, 1), (1, 2)]
    assert c._grow(0, 128) == []
    assert c._grow(1, 1) == [(0, 3)]
    c._publish([(0, 0, 1), (0, 1, 2), (1, 0, 3)])
    assert c.block_table.tolist() == [[1, 2, 0, 0], [3, 0, 0, 0]]
    with pytest.raises(RuntimeError, match="capacity"):
        c._grow(0, 257)
    c._grow(1, 192)
    with pytest.raises(RuntimeError, match="exhausted"):
        c._grow(0, 192)
    assert len(c._pages[0]) == 2 and c.free_pages == 0          # a failed growth takes nothing
    c.release(1)
    assert c.free_pages == 3 and c.block_table[1].tolist() == [0, 0, 0, 0]
    with pytest.raises(ValueError):
        NSAPagedDecodeCache(1, 4, 256, 1, 64, 64, block=128, device="cpu")


def test_qkv_rope_argument_errors_do_not_launch(lib):
    buf = ctypes.create_string_buffer(4096)
    p = (ctypes.addressof(buf) + 63) // 64 * 64
    base = dict(packed=p, q=p, k=p, v=p, gates=p, inv_freq=p, positions=None, cu=p, batch=1, total=4, ld=120,
                q_off=0, k_off=64, v_off=80, g_off=96, hq=4, hkv=1, dk=16, dv=16, rope_off=0, rope_dim=16,
                interleaved=0, pack=0, dtype=0)

    def call(**kw):
        a = dict(base, **kw)
        return lib.nsa_qkv_rope(a["packed"], a["q"], a["k"], a["v"], a["gates"], a["inv_freq"], a["positions"],
                                a["cu"], a["batch"], a["total"], a["ld"], a["q_off"], a["k_off"], a["v_off"],
                                a["g_off"], a["hq"], a["hkv"], a["dk"], a["dv"], a["rope_off"], a["rope_dim"],
                                a["interleaved"], a["pack"], a["dtype"], None)

    for bad in (dict(packed=None), dict(dtype=7), dict(total=0), dict(dk=12), dict(ld=100), dict(k_off=60),
                dict(v_off=112), dict(g_off=110), dict(rope_dim=8), dict(rope_dim=24, interleaved=1),
                dict(rope_off=4), dict(rope_off=8, rope_dim=16), dict(cu=None), dict(q=p + 4)):
        assert call(**bad) == -1, bad
        assert b"qkv_rope" in lib.nsa_last_error_string()


def test_layer_folds_the_gating_linear_into_the_projection():
    """Pure host arithmetic: the gate columns of the fused GEMM equal gating(q_proj(x)), and the
    q / k / v columns are the three projections, with and without biases."""
    from nsa_amd.layer import NSAAttentionLayer
    torch.manual_seed(0)
    for bias in (False, True):
        layer = NSAAttentionLayer(40, 6, 2, qk_head_dim=24, v_head_dim=16, rope_dim=16, bias=bias,
                                  dtype=torch.float64)
        w, b = layer.fused_projection()
        assert w.shape == (layer.ld, 40) and layer.ld % 8 == 0 and layer.ld >= 6 * 24 + 2 * 24 + 2 * 16 + 18
        x = torch.randn(11, 40, dtype=torch.float64)
        packed = torch.nn.functional.linear(x, w, b)
        q = layer.q_proj(x)
        o = layer.offsets
        assert torch.allclose(packed[:, :o[1]], q)
        assert torch.allclose(packed[:, o[1]:o[2]], layer.k_proj(x))
        assert torch.allclose(packed[:, o[2]:o[3]], layer.v_proj(x))
        gates = layer.attn.gating(q.view(11, 6, 24))
        assert torch.allclose(packed[:, o[3]:o[3] + 18].view(11, 6, 3), gates, atol=1e-12)
        assert (packed[:, o[3] + 18:] == 0).all()
    names = set(layer.state_dict())
    assert {"q_proj.weight", "o_proj.weight", "attn.gating.weight", "attn.compressor.compressor_k.weight"} <= names
    assert layer.attn.compressor.compressor_v.weight.shape[0] == 16
    with pytest.raises(ValueError):
        NSAAttentionLayer(40, 6, 4)
    with pytest.raises(ValueError):
        NSAAttentionLayer(40, 6, 2, qk_head_dim=24, rope_dim=12)
    with pytest.raises(NotImplementedError):
        layer(torch.zeros(1, 4, 40, dtype=torch.float64), attention_mask=torch.ones(1, 4))


def test_split_decode_argument_errors_do_not_launch(lib):
    assert lib.nsa_decode_split_workspace_bytes(0, 4, 128, 2048, 8) == 0
    need = lib.nsa_decode_split_workspace_bytes(2, 4, 128, 2048, 8)
    assert need > 0 and need % 4 == 0
    assert lib.nsa_decode_split_workspace_bytes(2, 4, 128, 2048, 2) <= need      # fewer splits never need more
    buf = ctypes.create_string_buffer(4096)
    p = (ctypes.addressof(buf) + 63) // 64 * 64

    def call(splits=8, pool=(5, 4, 0), ws=p, ws_bytes=1 << 40, top_n=16):
        return lib.nsa_decode_step_split(p, p, p, None, 0, p, p, p, None, p, None, 2, 64, 4, 128, 128, 2048, 2048, 32,
                                         16, 64, pool[0], pool[1], pool[2], top_n, 512, 0.1, 0, 0, splits, ws,
                                         ws_bytes, None)

    assert call(splits=0) == -1
    assert call(splits=17) == -1
    # other pooling geometries are served; their workspace is sized by the pooled variant (windows every 2 rows
    # make twice the bins of the default, which the plain size function assumes)
    pooled = lib.nsa_decode_split_pooled_workspace_bytes
    assert pooled(2, 4, 128, 2048, 8, 5, 4, 0) == need
    assert pooled(2, 4, 128, 2048, 8, 3, 2, 0) > need >= pooled(2, 4, 128, 2048, 8, 9, 8, 0)
    assert pooled(2, 4, 128, 2048, 8, 0, 2, 0) == 0
    assert call(pool=(3, 2, 0), ws_bytes=need) == -1 and b"workspace" in lib.nsa_last_error_string()
    assert call(ws=None) == -1
    assert call(ws_bytes=16) == -1 and b"workspace" in lib.nsa_last_error_string()
    assert call(top_n=65) == -2


def test_sequence_lengths_are_read_on_the_host_once_per_cu_seqlens_tensor(monkeypatch):
    """NSAAttention.forward with max_seqlen 0 and a batch checks that the batch really is uniform.  The check reads
    cu_seqlens once per tensor object and version; the second forward with the same tensor reads nothing."""
    from nsa_amd import nsa as nsa_mod
    cu = torch.tensor([0, 40, 80, 120], dtype=torch.int32)
    reads = []
    real = torch.Tensor.tolist
    monkeypatch.setattr(torch.Tensor, "tolist", lambda self: (reads.append(1), real(self))[1])
    assert nsa_mod._sequence_lengths_once(cu) == (True, 40)
    assert nsa_mod._sequence_lengths_once(cu) == (True, 40)
    assert len(reads) == 1
    cu[2] = 90                                        # in-place change: version counter moves, lengths are re-read
    assert nsa_mod._sequence_lengths_once(cu) == (False, 50)
    assert len(reads) == 2
    other = torch.tensor([0, 40, 80, 120], dtype=torch.int32)
    assert nsa_mod._sequence_lengths_once(other) == (True, 40) and len(reads) == 3
    for _ in range(40):                               # the table stays small
        nsa_mod._sequence_lengths_once(torch.tensor([0, 3, 7]))
    assert len(nsa_mod._LENGTHS_SEEN) <= 16


def test_single_pass_eligibility_and_pack_errors_on_the_host(lib):
    # which shapes the one-kernel compressed attention + selection takes: answered without a GPU
    base = dict(hq=64, hkv=4, dk=192, dv=128, pk=5, ps=4, pp=0, top_n=16, max_nc=2047, dtype=0)

    def ok(**kw):
        return lib.nsa_cmp_select_single_pass(*{**base, **kw}.values())

    assert ok() == 1 and ok(dtype=2) == 1 and ok(dk=128) == 1 and ok(dk=64, dv=64) == 1 and ok(hq=36) == 1
    assert ok(max_nc=2048) == 1 and ok(max_nc=2049) == 0                       # 2048 compressed rows per sequence
    assert ok(dtype=1) == 0                                                    # fp32 stays on the three launches
    assert ok(hq=32) == 0 and ok(hq=128) == 0 and ok(hq=0) == 0 and ok(hq=65) == 0   # groups of 9..16 heads
    assert ok(dk=192, dv=192) == 0 and ok(dk=32, dv=32) == 0
    assert ok(pk=3, ps=2) == 0 and ok(pp=1) == 0 and ok(top_n=65) == 0
    # chunk slots of the fragment-major copy: room for every sequence's partial last chunk
    for rows, batch in [(0, 1), (63, 1), (64, 1), (2047, 1), (5000, 7)]:
        assert lib.nsa_cmp_pack_chunks(rows, batch) >= (rows + 63) // 64 + batch - (1 if rows else 0)
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.c_void_p((ctypes.addressof(buf) + 15) & ~15)
    pack = lambda ck=p, chunks=40, dtype=0, stride=768, dk=192: lib.nsa_cmp_pack_fwd(      # noqa: E731
        ck, p, p, p, 1, 2047, 4, dk, 128, stride, dk, 512, 128, chunks, dtype, None)
    assert pack(ck=None) == -1 and b"null" in lib.nsa_last_error_string()
    assert pack(dtype=1) == -2 and b"16-bit" in lib.nsa_last_error_string()
    assert pack(stride=772) == -1 and b"multiples of 8" in lib.nsa_last_error_string()
    assert pack(chunks=8) == -1 and b"nsa_cmp_pack_chunks" in lib.nsa_last_error_string()
    # the selection entry point: indices are not optional, single_pass is -1 / 0 / 1
    sel = lambda indices=p, single_pass=-1: lib.nsa_cmp_select_fwd(      # noqa: E731
        p, p, p, p, 40, p, indices, None, p, None, None, None, None, p, p, 1, 4096, 64, 4, 192, 128, 768, 192, 4160, 32,
        16, 5, 4, 0, 16, 255, 64, 0, 0, 0.1, 1, 0, 0, single_pass, None)
    assert sel(indices=None) == -1 and b"null" in lib.nsa_last_error_string()
    assert sel(single_pass=2) == -1 and b"single_pass" in lib.nsa_last_error_string()


def test_module_inference_takes_the_single_pass_kernel_exactly_when_the_library_says_so(monkeypatch):
    """The module's no-grad forward asks the library whether the shape runs as one kernel and stages the matching
    operands: the fragment-major copy for the single pass, the transposed compressed values otherwise."""
    from nsa_amd import nsa as nsa_mod, ops
    calls = []

    def fake(name, ret):
        def f(*a, **kw):
            calls.append((name, kw))
            return ret(*a, **kw) if callable(ret) else ret
        return f

    def run(hq, dtype, T=640):
        del calls[:]
        hkv, d = 4, 128
        m = nsa_mod.NSAAttention(d, causal=True, device="cpu", dtype=dtype, compressor_mode="mean")
        q = torch.zeros(T, hq, d, dtype=dtype)
        k = torch.zeros(T, hkv, d, dtype=dtype)
        nc = (T - 32) // 16 + 1
        o = torch.zeros(T, hq, d, dtype=dtype)
        idx = torch.zeros(T, hkv, 16, dtype=torch.int32)
        gates = torch.zeros(T, hq, 3, dtype=dtype)
        monkeypatch.setattr(m.compressor, "compress_packed", fake("compress", (k[:nc], k[:nc], torch.tensor([0, nc]), nc)))
        monkeypatch.setattr(ops, "cmp_pack", fake("cmp_pack", ("frag", 1)))
        monkeypatch.setattr(ops, "transpose", fake("transpose", "t"))
        monkeypatch.setattr(ops, "cmp_select", fake("cmp_select", dict(o=o, indices=idx, gates=gates)))
        monkeypatch.setattr(ops, "cmp_attn", fake("cmp_attn", (o, "lse", gates)))
        monkeypatch.setattr(ops, "block_select", fake("block_select", (idx, None)))
        monkeypatch.setattr(ops, "slc_workspace", fake("slc_workspace", "ws"))
        monkeypatch.setattr(ops, "slc_partials", fake("slc_partials", None))
        monkeypatch.setattr(ops, "swa_merge", fake("swa_merge", o))
        with torch.no_grad():
            out = m._forward_infer(q, k, k, torch.tensor([0, T], dtype=torch.int32), 1, 0.1, True, T, True, None, None,
                                   False)
        assert out is o
        return [c[0] for c in calls]

    one = run(64, torch.bfloat16)                                  # group of 16, 16-bit: the single pass
    assert one == ["compress", "cmp_pack", "transpose", "cmp_select", "slc_workspace", "slc_partials", "swa_merge"]
    assert calls[3][1]["single_pass"] is True and calls[3][1]["frag"] == ("frag", 1)
    three = run(32, torch.bfloat16)                                # group of 8: compressed attention, then selection
    assert three == ["compress", "transpose", "transpose", "cmp_attn", "block_select", "slc_workspace", "slc_partials",
                     "swa_merge"]
    assert run(64, torch.float32)[3] == "cmp_attn"                 # fp32: three launches


def test_conv_compressor_keeps_its_kernel_layout_weight_until_the_parameter_changes():
    from nsa_amd.compression_kv import KVCompressor
    c = KVCompressor(16, 32, 8, device="cpu", dtype=torch.float32)
    w0 = c._wt(c.compressor_k)
    assert w0.shape == (8, 32 * 8)
    assert torch.equal(w0, c.compressor_k.weight.detach().permute(0, 2, 1).reshape(8, -1))
    assert c._wt(c.compressor_k) is w0 and c._wt(c.compressor_v) is not w0       # per convolution
    with torch.no_grad():
        c.compressor_k.weight.mul_(2.0)                                          # an optimizer step
    w1 = c._wt(c.compressor_k)
    assert w1 is not w0 and torch.equal(w1, 2.0 * w0)
    c.load_state_dict({k: torch.ones_like(v) for k, v in c.state_dict().items()})   # copy_ bumps the version too
    assert torch.equal(c._wt(c.compressor_k), torch.ones(8, 32 * 8))
    c.compressor_k.weight = torch.nn.Parameter(torch.zeros(8, 8, 32))            # a new parameter object
    assert torch.equal(c._wt(c.compressor_k), torch.zeros(8, 32 * 8))
    assert "_wt_cache" not in c.state_dict()
