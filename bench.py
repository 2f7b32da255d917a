#!/usr/bin/env python3
"""NSA forward benchmark on one MI355X.

One "step" is one pass of the NSA forward path (compress -> compressed attention + block selection
-> sliding window -> selected blocks + gated combine) over one batch of synthetic input that is
already resident in HBM.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload prefill_cfg4|prefill_cfg2|prefill_32k_d128]
                  [--no-cpu-baseline] [--no-decode] [--no-backward] [--no-layer]

roofline: taken for the kernel stage with the largest share of the step; its algorithmic flops
(causal compressed rows, whole valid selected blocks, exact window; nothing for exp / pooling /
top-n or for the non-causal part of the importance scores) divided by its mean duration measured
with events on the launch stream; `executed` (extra) is the same with the uncredited QK^T of the keys
a token cannot see, which the kernel multiplies for the importance normaliser.  cpu_baseline: the CPU oracle (a port of the reference's naive
torch path) on a bounded sample of query rows of the same workload, on this host's cores.
train_step (extra, not the headline metric): forward + backward of the same workload through the
module's autograd path.  decode / decode_small_batch (extra): the decode step of benchmark config 5 at
batch 64 and at batch 8.  layer (extra): the attention layer (projections, rotary embedding, NSA,
output projection) around the same workload.  compress (extra): the mean-pooling and the learned compressor alone.
roofline.traffic is read from the committed counter summary under profiles/ and only when the kernel sources
still hash to the build it was measured on (roofline.traffic_source says which, or why not).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # name: (lens, Hq, Hkv, Dqk, Dv, top_n, window, seed)
    "prefill_cfg4": ([32768], 64, 4, 192, 128, 16, 512, 3),
    "prefill_32k_d128": ([32768], 64, 4, 128, 128, 16, 512, 3),
    "prefill_cfg2": ([8192], 64, 4, 128, 128, 16, 512, 1),
}
BLOCK, STRIDE, SEL_BLOCK = 32, 16, 64
TRAFFIC_PROFILE = "profiles/prefill_cfg4_hbm_traffic.md"


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` as the committed counter summary states them, and where they come from.
    The summary carries a line `roofline.traffic: workload=<w> kernel=<k> bytes=<n> csrc_sha256=<digest>`; the
    figure is only passed on when the kernel sources are still the ones it was measured on."""
    import re
    from nsa_amd.build import sources_digest
    try:
        text = open(os.path.join(ROOT, TRAFFIC_PROFILE)).read()
    except OSError:
        return None, "%s not found" % TRAFFIC_PROFILE
    for m in re.finditer(r"roofline\.traffic:\s*workload=(\S+)\s+kernel=(\S+)\s+bytes=(\d+)\s+csrc_sha256=([0-9a-f]+)", text):
        if m.group(1) == workload and m.group(2) == kernel:
            now = sources_digest()
            if m.group(4) != now:
                return None, "%s was measured on other kernel sources (%s, this build %s)" % (TRAFFIC_PROFILE, m.group(4), now)
            return int(m.group(3)), "%s (rocprofv3 FETCH_SIZE + WRITE_SIZE, kernel sources %s)" % (TRAFFIC_PROFILE, now)
    return None, "%s has no figure for %s / %s" % (TRAFFIC_PROFILE, workload, kernel)


def flops_model(lens, hq, hkv, dqk, dv, window, valid_blocks_total):
    """Effective sparse flops of one forward, split per branch."""
    per = 2.0 * (dqk + dv)
    cmp_f = swa_f = 0.0
    for T in lens:
        nc = (T - BLOCK) // STRIDE + 1 if T >= BLOCK else 0
        # n_c(t) = clamp((t-32)//16 + 1, 0, Nc)
        n_vis = 0
        for t0 in range(0, T, STRIDE):          # n_c is constant over runs of STRIDE tokens
            t = t0
            cnt = min(max((t - BLOCK) // STRIDE + 1, 0), nc) if t >= BLOCK else 0
            n_vis += cnt * min(STRIDE, T - t0)
        cmp_f += hq * per * n_vis
        w = sum(min(t + 1, window) for t in range(min(T, window))) + max(T - window, 0) * window
        swa_f += hq * per * w
    g = hq // hkv
    slc_f = g * per * SEL_BLOCK * valid_blocks_total
    return dict(cmp=cmp_f, slc=slc_f, swa=swa_f)


def cpu_baseline(q, k, v, gl, top_n, window, budget_s=20.0):
    """Oracle on a sample of query rows of the same workload; compression cost added pro rata."""
    import torch
    from oracle import nsa_oracle as O
    T = q.shape[0]
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    p = O.NSAParams(BLOCK, STRIDE, SEL_BLOCK, top_n, window)
    gates = torch.sigmoid(gl.float()).to(q.dtype)
    nc = O.compressed_len_conv(T, BLOCK, STRIDE)
    t0 = time.perf_counter()
    ckcv = (O.compress_meanpool(k, BLOCK, STRIDE, nc), O.compress_meanpool(v, BLOCK, STRIDE, nc))
    t_comp = time.perf_counter() - t0
    g = torch.Generator().manual_seed(123)
    n = 8
    done_rows, spent = 0, 0.0
    while True:
        rows = torch.sort(torch.randint(0, T, (n,), generator=g)).values.unique()
        t0 = time.perf_counter()
        O.nsa_forward_single(q, k, v, gates, p, rows=rows, compressed=ckcv)
        dt = time.perf_counter() - t0
        done_rows += len(rows)
        spent += dt
        if spent > budget_s or n >= 512:
            break
        n *= 2
    per_row = spent / done_rows + t_comp / T
    return dict(value=1.0 / per_row, unit="tokens/s", cores=cores, kind="port",
                sample="CPU oracle (torch fp32 port of the reference's naive path) on %d sampled query rows "
                       "of the same workload in %.1f s; compression of the whole K/V (%.2f s) charged pro rata"
                       % (done_rows, spent, t_comp))


def cpu_baseline_cfg1():
    """Benchmark configuration 1 as it is defined: batch 1, 1024 tokens, Hq 4 / Hkv 1, head dim 64, fp32, q / k / v ~
    N(0, 1) and gate logits ~ N(0, 1) from seed 0, compression 32 / 16 (mean), selection blocks of 64, top 4, window
    128; the whole sequence through the CPU oracle on all host cores, one warm-up run and the median of three."""
    import torch
    from oracle import nsa_oracle as O
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    T, hq, hkv, d = 1024, 4, 1, 64
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(T, h, d, generator=g) for h in (hq, hkv, hkv))
    gates = torch.sigmoid(torch.randn(T, hq, 3, generator=g))
    p = O.NSAParams(BLOCK, STRIDE, SEL_BLOCK, 4, 128)
    times = []
    for i in range(4):
        t0 = time.perf_counter()
        out = O.nsa_forward_single(q, k, v, gates, p)
        times.append(time.perf_counter() - t0)
    assert torch.isfinite(out).all()
    med = sorted(times[1:])[1]
    return dict(value=T / med, unit="tokens/s", cores=cores, kind="port", seconds_per_forward=med,
                sample="CPU oracle, whole sequence of benchmark configuration 1 (1024 tokens, Hq4/Hkv1, D64, fp32), "
                       "1 warm-up + 3 runs, median")


def decode_bench(steps, warmup):
    """benchmark config 5: batch 64, one query token per sequence, 32768 cached tokens each (+ the
    compressed caches), Hq64/Hkv4, D128, top-16 blocks of 64, window 512, bf16."""
    import torch
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    dev = "cuda:0"
    B, ctx, hq, hkv, d, top_n, window = 64, 32768, 64, 4, 128, 16, 512
    g = torch.Generator(device=dev).manual_seed(4)
    cache = NSADecodeCache(B, ctx, hkv, d, d, dtype=torch.bfloat16, device=dev)
    for b0 in range(0, B, 8):                                  # fill in slices to bound the temporaries
        k = (torch.randn(8, ctx, hkv, d, device=dev, generator=g) * 0.5).bfloat16()
        v = (torch.randn(8, ctx, hkv, d, device=dev, generator=g) * 0.5).bfloat16()
        sub = NSADecodeCache(8, ctx, hkv, d, d, dtype=torch.bfloat16, device=dev)
        sub.fill(k, v)
        cache.k[b0:b0 + 8], cache.vt[b0:b0 + 8] = sub.k, sub.vt
        cache.ck[b0:b0 + 8], cache.cvt[b0:b0 + 8] = sub.ck, sub.cvt
        del sub, k, v
    cache.ctx_lens.fill_(ctx)
    q = (torch.randn(B, hq, d, device=dev, generator=g) * 0.5).bfloat16()
    gl = torch.randn(B, hq, 3, device=dev, generator=g).bfloat16()
    run = lambda: nsa_decode_step(q, cache, gl, SEL_BLOCK, top_n, window, gate_activation="sigmoid",
                                  return_indices=True)
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    beg.record()
    for _ in range(steps):
        out, idx = run()
    end.record()
    torch.cuda.synchronize()
    us = beg.elapsed_time(end) / steps * 1e3
    assert torch.isfinite(out).all()
    # algorithmic bytes: all compressed keys, visible compressed values, distinct selected/window rows, q/o/gates
    nc = (ctx - BLOCK) // STRIDE + 1
    n_vis = min((ctx - 1 - BLOCK) // STRIDE + 1, nc)
    t = ctx - 1
    blk_lo = (t - window + 1) // SEL_BLOCK                      # blocks that the window fully or partly covers
    idx = idx.long()
    valid = (idx >= 0) & (idx * SEL_BLOCK <= t)
    outside = valid & (idx < blk_lo)                           # rows not already counted with the window
    rows = outside.sum().item() * SEL_BLOCK + B * hkv * (t + 1 - blk_lo * SEL_BLOCK)
    nbytes = B * hkv * (nc * d * 2 + n_vis * d * 2) + rows * (d + d) * 2 + B * hq * (d + d + 3) * 2
    return {"us_per_step": us, "batch": B, "context": ctx, "algorithmic_bytes": nbytes,
            "achieved_GBps": nbytes / (us * 1e-6) / 1e9, "hbm_peak_GBps": PEAK_HBM_GBS,
            "hbm_frac": nbytes / (us * 1e-6) / 1e9 / PEAK_HBM_GBS,
            "workload": "decode_cfg5: batch 64 x 1 token, ctx 32768, Hq64/Hkv4, D128, top-16 x 64, window 512, bf16"}


def compress_bench(k, v, cu, steps=20):
    """The two compressors alone on the workload's K / V (extra): mean pooling is a pure HBM stream (algorithmic
    bytes: K and V read once, the compressed rows written), the learned (Conv1d-equivalent) compressor a GEMM of
    [rows x block*D] by [block*D x D] per head and tensor."""
    import torch
    from nsa_amd import ops
    total, h, dk = k.shape
    dv = v.shape[2]
    batch = cu.numel() - 1
    cu_out = ops.compressed_offsets(cu, BLOCK, STRIDE, extra=1)
    rows = int(cu_out[-1].item())
    gen = torch.Generator(device=k.device).manual_seed(11)
    wk = (torch.randn(dk, BLOCK * dk, device=k.device, generator=gen) * 0.02).bfloat16()
    wv = (torch.randn(dv, BLOCK * dv, device=k.device, generator=gen) * 0.02).bfloat16()

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        beg.record()
        for _ in range(steps):
            fn()
        end.record()
        torch.cuda.synchronize()
        return beg.elapsed_time(end) / steps * 1e3

    us_mean = timed(lambda: ops.compress_kv(k, v, cu, cu_out, rows, BLOCK, STRIDE))
    us_w = timed(lambda: ops.compress_kv(k, v, cu, cu_out, rows, BLOCK, STRIDE, wk, wv))
    nbytes = (total + rows) * h * (dk + dv) * 2
    flops = 2.0 * rows * h * BLOCK * (dk * dk + dv * dv)
    return {"mean": {"us": us_mean, "algorithmic_bytes": nbytes, "achieved_GBps": nbytes / (us_mean * 1e-6) / 1e9,
                     "hbm_frac": nbytes / (us_mean * 1e-6) / 1e9 / PEAK_HBM_GBS,
                     "note": "back-to-back launches through the Python wrapper, host launch cost included"},
            "learned": {"us": us_w, "flops": flops, "tflops": flops / (us_w * 1e-6) / 1e12,
                        "mfma_peak_frac": flops / (us_w * 1e-6) / 1e12 / PEAK_BF16_TFLOPS},
            "rows": rows, "batch": batch}


def train_bench(m, q, k, v, gl, cu, max_len, total, f_eff, steps, warmup):
    """Forward + backward through the module's training path (un-fused forward that keeps the
    per-branch outputs and log-sum-exps, hand-written backward kernels) on the same workload.
    Model flops of the step: 3.5 x the forward's effective flops (two GEMMs forward, five backward)."""
    import torch
    qg, kg, vg, gg = (t.detach().clone().requires_grad_(True) for t in (q, k, v, gl))
    d_o = torch.randn(total, q.shape[1], v.shape[2], device=q.device, generator=torch.Generator(q.device).manual_seed(9))
    d_o = d_o.bfloat16()

    def fwd():
        return m(qg, kg, vg, cu, max_len, gates=gg)

    def timed(fn, n):
        beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        beg.record()
        for _ in range(n):
            fn()
        end.record()
        torch.cuda.synchronize()
        return beg.elapsed_time(end) / n

    def both():
        for t in (qg, kg, vg, gg):
            t.grad = None
        fwd().backward(d_o)

    for _ in range(warmup):
        both()
    ms_both = timed(both, steps)
    ms_fwd = timed(fwd, steps)
    assert all(torch.isfinite(t.grad).all() for t in (qg, kg, vg, gg))
    return {"ms_fwd_bwd": ms_both, "ms_fwd_training_path": ms_fwd, "ms_bwd": ms_both - ms_fwd,
            "tokens_per_s": total / (ms_both * 1e-3), "model_tflops": 3.5 * f_eff / (ms_both * 1e-3) / 1e12,
            "mfma_peak_frac": 3.5 * f_eff / (ms_both * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}


def decode_small_bench(batch=8, steps=200, warmup=10):
    """The same decode step at a small batch (extra): 32 (sequence, kv head) pairs cannot fill 256 CUs with
    one workgroup each, so the step is spread over 8 workgroups per pair; both schedules are timed."""
    import torch
    from nsa_amd.decode import NSADecodeCache, nsa_decode_step
    dev = "cuda:0"
    ctx, hq, hkv, d, top_n, window = 32768, 64, 4, 128, 16, 512
    g = torch.Generator(device=dev).manual_seed(5)
    cache = NSADecodeCache(batch, ctx, hkv, d, d, dtype=torch.bfloat16, device=dev)
    k = (torch.randn(batch, ctx, hkv, d, device=dev, generator=g) * 0.5).bfloat16()
    v = (torch.randn(batch, ctx, hkv, d, device=dev, generator=g) * 0.5).bfloat16()
    cache.fill(k, v)
    del k, v
    q = (torch.randn(batch, hq, d, device=dev, generator=g) * 0.5).bfloat16()
    gl = torch.randn(batch, hq, 3, device=dev, generator=g).bfloat16()
    res = {"batch": batch, "context": ctx}
    for name, splits in (("us_per_step", None), ("us_per_step_one_workgroup_per_pair", 0)):
        run = lambda: nsa_decode_step(q, cache, gl, SEL_BLOCK, top_n, window, gate_activation="sigmoid", splits=splits)
        for _ in range(warmup):
            run()
        torch.cuda.synchronize()
        beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        beg.record()
        for _ in range(steps):
            out = run()
        end.record()
        torch.cuda.synchronize()
        assert torch.isfinite(out).all()
        res[name] = beg.elapsed_time(end) / steps * 1e3
    return res


def layer_bench(total, hq, hkv, dqk, dv, top_n, window, steps, warmup, hidden=4096, rope_dim=64):
    """The attention layer around the same workload (extra, not the headline metric): fused q/k/v/gate
    projection GEMM (hipBLASLt through torch), split + rotary embedding in one HIP pass, NSA forward,
    output projection.  The split kernel is HBM-bound: bytes = one read and one write of the packed row."""
    import torch
    from nsa_amd import ops
    from nsa_amd.layer import NSAAttentionLayer
    layer = NSAAttentionLayer(hidden, hq, hkv, dqk, dv, rope_dim=rope_dim, selected_block_count=top_n,
                              sliding_window=window, compressor_mode="mean", gate_activation="sigmoid",
                              dtype=torch.bfloat16).cuda()
    x = torch.randn(1, total, hidden, device="cuda", dtype=torch.bfloat16,
                    generator=torch.Generator("cuda").manual_seed(11))

    def timed(fn, n):
        for _ in range(warmup):
            fn()
        beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        beg.record()
        for _ in range(n):
            fn()
        end.record()
        torch.cuda.synchronize()
        return beg.elapsed_time(end) / n

    with torch.no_grad():
        w, b = layer._fused_cached()
        packed = torch.nn.functional.linear(x.view(total, hidden), w, b)
        cu = ops.uniform_cu(1, total, "cuda")
        ms_split = timed(lambda: ops.qkv_rope_split(packed, hq, hkv, dqk, dv, layer.offsets, layer.inv_freq, None,
                                                    cu, dqk - rope_dim, rope_dim), steps)
        ms_layer = timed(lambda: layer(x), steps)
    nbytes = 2 * 2 * total * (hq * dqk + hkv * dqk + hkv * dv + 3 * hq)
    return {"hidden": hidden, "rope_dim": rope_dim, "ms_layer_fwd": ms_layer, "tokens_per_s": total / (ms_layer * 1e-3),
            "ms_split_rope": ms_split, "split_rope_GBps": nbytes / (ms_split * 1e-3) / 1e9,
            "split_rope_hbm_frac": nbytes / (ms_split * 1e-3) / 1e9 / PEAK_HBM_GBS}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="prefill_cfg4", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-budget", type=float, default=20.0)
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--no-backward", action="store_true")
    ap.add_argument("--no-layer", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy (reference point for FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the one-GPU NSA forward path; --gpus %d is not supported (this build has no "
              "multi-GPU path)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from nsa_amd.nsa import NSAAttention
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    # The decode step is an HBM benchmark of 0.1 ms per step: it runs first, before seconds of MFMA-heavy
    # prefill work, after which the same 200 steps measure 3-4 % slower.
    decode_res = None
    if not args.no_decode:
        decode_res = decode_bench(max(args.steps, 200), max(args.warmup, 10))
        torch.cuda.empty_cache()
        decode_small = decode_small_bench()
        torch.cuda.empty_cache()
    lens, hq, hkv, dqk, dv, top_n, window, seed = WORKLOADS[args.workload]
    total = sum(lens)
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(total, hq, dqk, generator=g) * 0.5).bfloat16()
    k = (torch.randn(total, hkv, dqk, generator=g) * 0.5).bfloat16()
    v = (torch.randn(total, hkv, dv, generator=g) * 0.5).bfloat16()
    cu_list = [0]
    for x in lens:
        cu_list.append(cu_list[-1] + x)
    cu = torch.tensor(cu_list, dtype=torch.int32, device=dev)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    m = NSAAttention(dqk, True, compression_stride=STRIDE, compression_block=BLOCK, selection_block=SEL_BLOCK,
                     selected_block_count=top_n, sliding_window=window, dtype=torch.bfloat16,
                     compressor_mode="mean", gate_activation="sigmoid").to(dev)
    max_len = 0 if len(set(lens)) == 1 else max(lens)

    # The step is the module's whole forward, its gating Linear on q included (it is evaluated inside the
    # compressed-attention kernel); the gate logits the CPU baseline and the training step use are the same Linear's.
    gl = torch.nn.functional.linear(q.float(), m.gating.weight.detach().float().cpu(),
                                    m.gating.bias.detach().float().cpu()).bfloat16()
    gd = gl.to(dev)

    def step():                       # inference: the fused schedule (the gating parameters require grad)
        with torch.no_grad():
            return m(qd, kd, vd, cu, max_len)

    if args.copy_calibration:
        src = torch.zeros(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(2):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms = dt / args.steps * 1e3

    # per-stage durations (events on the launch stream), separate from the timed region
    acc = {}
    reps = max(3, min(args.steps, 10))
    idx = None
    for _ in range(reps):
        st = []
        with torch.no_grad():
            out, idx = m(qd, kd, vd, cu, max_len, stage_times=st, return_indices=True)
        torch.cuda.synchronize()
        for name, beg, end in st:
            acc[name] = acc.get(name, 0.0) + beg.elapsed_time(end)
    stage_ms = {n: t / reps for n, t in acc.items()}
    assert torch.isfinite(out).all()

    tok = torch.cat([torch.arange(x) for x in lens]).to(dev)
    valid = ((idx >= 0) & (idx.long() * SEL_BLOCK <= tok[:, None, None])).sum().item()
    fl = flops_model(lens, hq, hkv, dqk, dv, window, valid)
    f_eff = fl["cmp"] + fl["slc"] + fl["swa"]
    # Per-stage credited flops.  block_select carries none (its score tiles are the uncredited
    # non-causal importance pass); slc_combine is a chain of kernels (bucket, block, merge), the other
    # stages are one kernel each, so the single dominant kernel is the longest of cmp_attn / swa.
    # With the fused schedule the selected branch is "slc_blocks" (bucket + per-block partials) and the
    # window branch "swa_combine" (window attention + merge of the partials + gated sum).
    # "cmp_select" is the one-pass kernel that does the work of cmp_attn + block_select (attention over the visible
    # compressed rows, importance over all of them, top-n); it is credited with the attention flops only.
    stage_flops = {"cmp_attn": fl["cmp"], "cmp_select": fl["cmp"], "swa": fl["swa"], "slc_combine": fl["slc"],
                   "swa_combine": fl["swa"], "slc_blocks": fl["slc"]}
    stage_tflops = {n: stage_flops[n] / (stage_ms[n] * 1e-3) / 1e12 for n in stage_flops if n in stage_ms}
    dom = max(("cmp_attn", "cmp_select", "swa", "swa_combine"), key=lambda n: stage_ms.get(n, 0.0))
    dom_tflops = stage_tflops[dom]
    # HBM bytes per launch of that kernel from rocprofv3 FETCH_SIZE / WRITE_SIZE (profiles/), only
    # recorded for the default workload
    traffic, traffic_source = measured_traffic(args.workload, dom)
    # The compressed-attention kernel also multiplies q with the compressed keys a token cannot see: the
    # importance softmax is normalised over all of them.  `executed` adds that uncredited part of QK^T.
    executed = None
    qk_all = sum(2.0 * hq * dqk * x * max((x - BLOCK) // STRIDE + 1, 0) for x in lens)
    qk_seen = fl["cmp"] * dqk / (dqk + dv)
    if dom in ("cmp_attn", "cmp_select"):
        executed = (fl["cmp"] + max(qk_all - qk_seen, 0.0)) / (stage_ms[dom] * 1e-3) / 1e12
    # flops the whole step executes on the matrix unit: the credited ones plus the non-causal part of QK^T, once
    # in the one-pass kernel, twice (compressed attention, then the importance kernel) on the three-launch schedule
    qk_passes = 1 if "cmp_select" in stage_ms else 2
    executed_step = f_eff + max(qk_all - qk_seen, 0.0) + (qk_passes - 1) * qk_all
    # The two HBM-bound stages of the step against 8 TB/s: bytes per launch from the committed counter summary
    # (same source-digest rule as roofline.traffic), divided by the stage time measured here
    roofline_hbm = {}
    for stage_name, kernel in (("slc_blocks", "slc_blocks"), ("swa_combine", "swa_combine")):
        if stage_name in stage_ms:
            nbytes, src = measured_traffic(args.workload, kernel)
            gbs = None if nbytes is None else nbytes / (stage_ms[stage_name] * 1e-3) / 1e9
            roofline_hbm[stage_name] = {"bound": "hbm", "traffic": nbytes, "traffic_source": src, "achieved": gbs,
                                        "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                        "frac": None if gbs is None else gbs / PEAK_HBM_GBS}

    res = {
        "metric": "nsa_prefill_fwd_tokens_per_s", "value": total / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "seq_lens": lens if len(lens) > 1 else lens[0], "hq": hq, "hkv": hkv,
                   "dqk": dqk, "dv": dv, "compress": "mean %d/%d" % (BLOCK, STRIDE), "sel_block": SEL_BLOCK,
                   "top_n": top_n, "window": window, "gates": "sigmoid(Linear(q)), inside the step"},
        "effective_tflops": f_eff / (ms * 1e-3) / 1e12,
        "effective_flops": {"total": f_eff, **fl, "valid_selected_blocks": valid},
        "mfma_peak_frac_whole_step": f_eff / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
        "stage_ms": stage_ms,
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": dom_tflops, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": dom_tflops / PEAK_BF16_TFLOPS, "traffic": traffic,
                     "traffic_source": traffic_source, "executed": executed},
        "stage_effective_tflops": stage_tflops,
        "roofline_hbm": roofline_hbm,
        "executed_tflops_whole_step": executed_step / (ms * 1e-3) / 1e12,
        "executed_mfma_peak_frac_whole_step": executed_step / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
    }
    res["compress"] = compress_bench(kd, vd, cu)
    if not args.no_backward:
        res["train_step"] = train_bench(m, qd, kd, vd, gd, cu, max_len, total, f_eff, max(2, min(args.steps, 5)), 2)
    if not args.no_layer and len(lens) == 1:
        res["layer"] = layer_bench(total, hq, hkv, dqk, dv, top_n, window, max(2, min(args.steps, 10)), 2)
    if decode_res is not None:
        res["decode"] = decode_res
        res["decode_small_batch"] = decode_small
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(q, k, v, gl, top_n, window, args.cpu_budget)
        res["cpu_baseline_cfg1"] = cpu_baseline_cfg1()
    print(json.dumps(res))


if __name__ == "__main__":
    main()
