"""GPU test of nsa_decode_step_split_static, the decode entry point that allocates nothing: called through the
C ABI (ctypes, caller-owned output buffers) it must return exactly what nsa_decode_step_split returns with a
caller workspace (same kernels, same order: bit for bit), on two calls in a row that share the library's
fixed scratch array, the second on a smaller input, and it must refuse what does not fit the array."""
import ctypes as C

import pytest
import torch

from tests.util import randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _call(lib, static, q, cache, gl, out, idx, S, W, splits, ws=None):
    from nsa_amd import _lib
    from nsa_amd.ops import _dtype_code, _ptr, _stream
    B, hq, dk = q.shape
    common = [_ptr(q), _ptr(cache.k), _ptr(cache.vt), None, 0, _ptr(cache.ck), _ptr(cache.cvt), _ptr(cache.ctx_lens),
              _ptr(gl), _ptr(out), _ptr(idx), B, hq, cache.hkv, dk, cache.dv, cache.ctx_cap, cache.nc_cap,
              cache.block, cache.stride, 64, 5, 4, 0, S, W, float(dk ** -0.5), _lib.GATE_SIGMOID, _dtype_code(q), splits]
    if static:
        return lib.nsa_decode_step_split_static(*common, _stream())
    return lib.nsa_decode_step_split(*common, _ptr(ws), ws.numel(), _stream())


def _case(lib, dtype, ctxs, Hq, Hkv, D, S, W, splits, seed):
    from nsa_amd.decode import NSADecodeCache
    B, T = len(ctxs), max(ctxs)
    q = randn(B, Hq, D, seed=seed, scale=0.5, dtype=dtype).to(DEV)
    k = randn(B, T, Hkv, D, seed=seed + 1, scale=0.5, dtype=dtype).to(DEV)
    v = randn(B, T, Hkv, D, seed=seed + 2, scale=0.5, dtype=dtype).to(DEV)
    gl = randn(B, Hq, 3, seed=seed + 3, dtype=dtype).to(DEV)
    cache = NSADecodeCache(B, T, Hkv, D, D, dtype=dtype, device=DEV)
    cache.fill(k, v)
    cache.ctx_lens.copy_(torch.tensor(ctxs, dtype=torch.int32))
    need = lib.nsa_decode_split_workspace_bytes(B, Hkv, D, cache.nc_cap, splits)
    assert 0 < need <= lib.nsa_decode_split_static_bytes()
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    ref, ref_idx = torch.empty(B, Hq, D, dtype=dtype, device=DEV), torch.empty(B, Hkv, S, dtype=torch.int32, device=DEV)
    out, idx = torch.full_like(ref, float("nan")), torch.full_like(ref_idx, -7)
    assert _call(lib, False, q, cache, gl, ref, ref_idx, S, W, splits, ws) == 0
    # one call beforehand: the first call on a device looks the array's address up and sets kernel attributes
    warm, warm_idx = torch.empty_like(ref), torch.empty_like(ref_idx)
    assert _call(lib, True, q, cache, gl, warm, warm_idx, S, W, splits) == 0, lib.nsa_last_error_string()
    torch.cuda.synchronize()
    # free device memory as the driver counts it: an allocation inside the library (which PyTorch's own counters
    # would not see) lowers it.  Nothing else allocates in between: no tensor is created, the stream exists.
    free_before = torch.cuda.mem_get_info()[0]
    torch_before = torch.cuda.memory_allocated()
    assert _call(lib, True, q, cache, gl, out, idx, S, W, splits) == 0, lib.nsa_last_error_string()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.cuda.memory_allocated() == torch_before
    assert torch.equal(idx, ref_idx)
    assert torch.equal(out, ref) and torch.isfinite(out.float()).all()
    return cache, q, gl


def test_static_scratch_step_equals_workspace_step_twice_then_smaller():
    from nsa_amd import _lib
    lib = _lib.load()
    # first call: 16 pairs of up to 4096 tokens, 8 splits; second call right after it: fewer, shorter sequences and
    # fewer splits, so most of the array still holds the first call's partial results
    _case(lib, torch.bfloat16, [4096, 4000, 2049, 777], 64, 4, 128, 16, 512, 8, seed=800)
    cache, q, gl = _case(lib, torch.bfloat16, [300, 33], 32, 2, 128, 4, 128, 3, seed=810)
    _case(lib, torch.float32, [1000, 64, 5], 8, 2, 64, 4, 64, 8, seed=820)
    # through the Python wrapper as well, into caller buffers
    from nsa_amd.decode import nsa_decode_step
    out = torch.empty(2, 32, 128, dtype=torch.bfloat16, device=DEV)
    idx = torch.empty(2, 2, 4, dtype=torch.int32, device=DEV)
    r, ri = nsa_decode_step(q, cache, gl, 64, 4, 128, gate_activation="sigmoid", return_indices=True, splits=3,
                            out=out, indices=idx, static_scratch=True)
    assert r.data_ptr() == out.data_ptr() and ri.data_ptr() == idx.data_ptr()
    ref, ref_idx = nsa_decode_step(q, cache, gl, 64, 4, 128, gate_activation="sigmoid", return_indices=True, splits=3)
    assert torch.equal(out, ref) and torch.equal(idx, ref_idx)
    with pytest.raises(ValueError):          # splits=0 names the one-workgroup step, which has no scratch buffer
        nsa_decode_step(q, cache, gl, 64, 4, 128, gate_activation="sigmoid", splits=0, static_scratch=True)


def test_static_scratch_step_refuses_what_does_not_fit():
    from nsa_amd import _lib
    from nsa_amd.decode import NSADecodeCache
    lib = _lib.load()
    B, Hq, Hkv, D = 40, 64, 4, 128                      # 160 pairs of 32k context: ~37 MB of partial results
    cache = NSADecodeCache(B, 32768, Hkv, D, D, dtype=torch.bfloat16, device=DEV)
    assert lib.nsa_decode_split_workspace_bytes(B, Hkv, D, cache.nc_cap, 8) > lib.nsa_decode_split_static_bytes()
    q = torch.zeros(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    out = torch.zeros(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    rc = _call(lib, True, q, cache, None, out, None, 16, 512, 8)
    assert rc == -3 and b"fixed array" in lib.nsa_last_error_string()
