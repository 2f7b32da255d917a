"""Seeded inputs shared by the GPU parity tests (generated on the CPU so oracle and kernels see the same bits)."""
import torch

from oracle import nsa_oracle as O

TOL = {torch.bfloat16: 2e-2, torch.float16: 3e-3, torch.float32: 1e-4}   # max-abs bound per dtype
ROW_TOL = {torch.bfloat16: 4e-3, torch.float16: 5e-4, torch.float32: 1e-6}   # a mean / a sum of a few rows


def randn(*shape, seed, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def make_qkv(T, Hq, Hkv, Dk, Dv, seed, dtype, scale=1.0):
    q = randn(T, Hq, Dk, seed=seed, scale=scale, dtype=dtype)
    k = randn(T, Hkv, Dk, seed=seed + 1, scale=scale, dtype=dtype)
    v = randn(T, Hkv, Dv, seed=seed + 2, scale=scale, dtype=dtype)
    gl = randn(T, Hq, 3, seed=seed + 3, dtype=dtype)          # gate logits
    return q, k, v, gl


def max_abs(a, b):
    return float((a.detach().double().cpu() - b.detach().double().cpu()).abs().max()) if a.numel() else 0.0


def ragged_cu(lens):
    cu = [0]
    for x in lens:
        cu.append(cu[-1] + x)
    return cu


def within(out, ref, dtype, large_values=False):
    """max-abs bar of the dtype; with large_values (raw, un-activated gates make |out| > 4) one bf16
    unit in the last place of the reference is allowed on top, since both sides round once to bf16."""
    a, b = out.double().cpu(), ref.double().cpu()
    bound = torch.full_like(b, TOL[dtype])
    if large_values and dtype == torch.bfloat16:
        bound = bound + b.abs() * 2.0 ** -7
    if large_values and dtype == torch.float16:
        bound = bound + b.abs() * 2.0 ** -10
    return bool(((a - b).abs() <= bound).all())


def sample_rows(T, n, seed, edges=(0, 1, 31, 32, 33, 63, 64, 65, 511, 512, 513)):
    g = torch.Generator().manual_seed(seed)
    r = set(int(x) for x in torch.randint(0, T, (n,), generator=g))
    r.update(e for e in edges if e < T)
    r.update((T - 1, max(T - 2, 0), max(T - 65, 0)))
    return torch.tensor(sorted(r))
