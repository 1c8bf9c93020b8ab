#!/usr/bin/env python3
"""Benchmark of the sparse-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only decode,vecmat,topk,prefill,prefill_rows,copy,next]

Prints ONE JSON line.  The headline (`metric`/`value`) is sparse-MLA decode
throughput on the B=32, H=128, topk=2048, 64K-token FP8 latent-cache
configuration; `vecmat` and `topk` carry the two HBM-bound kernels of the same
path with their own roofline objects, `prefill` the causal prefill
configuration when asked for.

A "step" is one pass of the kernel(s) over one synthetic batch that is already
resident in HBM.  Steps are captured into a HIP graph (launch-bound at these
kernel lengths otherwise) and the K timed steps are one graph replay bracketed
by HIP events on the launch stream and host synchronisation.  Input sets
rotate between steps so the HBM-bound kernels cannot be served by the 256 MB
Infinity Cache.

`cpu_baseline` times the NumPy oracle (a port of the reference's pure-MLX
fallback, which cannot be installed here) on a bounded sample of the same
workload on this machine's host cores.  It is a reported baseline only.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


# --------------------------------------------------------------------------- inputs (device side, torch only)

def quantize_block_pow2(x: torch.Tensor, block: int = 128):
    """x [..., K] fp32 -> (e4m3 bytes [..., K], fp32 scale [..., K/block]), scale = 2^ceil(log2(amax/448))."""
    shp = x.shape
    xb = x.reshape(*shp[:-1], shp[-1] // block, block)
    amax = xb.abs().amax(dim=-1)
    scale = torch.where(amax > 0, torch.exp2(torch.ceil(torch.log2(amax / 448.0))), torch.ones_like(amax))
    codes = (xb / scale[..., None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    return codes.reshape(shp).contiguous(), scale.contiguous()


def quantize_block_amax(x: torch.Tensor, block: int = 128):
    """x [..., K] fp32 -> (e4m3 bytes, fp32 scale [..., K/block]), scale = amax/448: the general fp32 block
    scale of the FP8 producers (cppmega_v4/nn/moe_fp8.py:36-58), not a power of two."""
    shp = x.shape
    xb = x.reshape(*shp[:-1], shp[-1] // block, block)
    amax = xb.abs().amax(dim=-1)
    scale = torch.where(amax > 0, amax / 448.0, torch.ones_like(amax))
    codes = (xb / scale[..., None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    return codes.reshape(shp).contiguous(), scale.contiguous()


def make_latent_cache(gen, B, Skv, device, pow2: bool = True):
    codes = torch.empty((B, Skv, 1, 512), dtype=torch.uint8, device=device)
    scale = torch.empty((B, Skv, 1, 4), dtype=torch.float32, device=device)
    rope = torch.empty((B, Skv, 1, 64), dtype=torch.bfloat16, device=device)
    for b in range(B):
        lat = torch.randn((Skv, 1, 512), generator=gen, device=device, dtype=torch.float32)
        c, s = quantize_block_pow2(lat) if pow2 else quantize_block_amax(lat)
        codes[b], scale[b] = c, s
        rope[b] = torch.randn((Skv, 1, 64), generator=gen, device=device, dtype=torch.float32).to(torch.bfloat16)
    return codes, scale, rope


def uniform_indices(gen, B, S, Skv, topk, device):
    """Uniform without replacement per (b, s): top-k of random keys."""
    out = torch.empty((B, S, 1, topk), dtype=torch.int32, device=device)
    for b in range(B):
        for s0 in range(0, S, 256):
            s1 = min(S, s0 + 256)
            r = torch.rand((s1 - s0, Skv), generator=gen, device=device)
            out[b, s0:s1, 0] = r.topk(topk, dim=-1).indices.to(torch.int32)
    return out


def timed_graph(step_fns, steps: int, warmup: int):
    """Run `warmup` eager steps, capture `steps` steps into a HIP graph, replay once timed.

    step_fns: list of zero-argument callables (rotated).  Returns (seconds for
    the K steps by HIP events, seconds by host clock)."""
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        for i in range(max(warmup, 1)):
            step_fns[i % len(step_fns)]()
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for i in range(steps):
            step_fns[i % len(step_fns)]()
    graph.replay()                      # untimed replay: first replay pays upload costs
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    graph.replay()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return e0.elapsed_time(e1) * 1e-3, t1 - t0


# --------------------------------------------------------------------------- workloads

def bench_decode(args, device, pow2: bool = False):
    from cppmega_mlx_amd import ops
    from cppmega_mlx_amd.nn._tilelang import sparse_mla_blockscaled_path_c as bs

    B, H, Skv, topk, d_qk, d_v = 32, 128, 65536, 2048, 576, 512
    gen = torch.Generator(device=device).manual_seed(1234)
    codes, scale, rope = make_latent_cache(gen, B, Skv, device, pow2=pow2)
    n_sets = 3
    qs = [torch.randn((B, 1, H, d_qk), generator=gen, device=device).to(torch.bfloat16) for _ in range(n_sets)]
    idxs = [uniform_indices(gen, B, 1, Skv, topk, device) for _ in range(n_sets)]
    outs = [torch.empty((B, 1, H, d_v), dtype=torch.bfloat16, device=device) for _ in range(n_sets)]
    lses = [torch.empty((B, 1, H), dtype=torch.float32, device=device) for _ in range(n_sets)]
    sm_scale = d_qk ** -0.5
    kernel = ops.sparse_mla_selected_kernel(qs[0], codes, idxs[0], d_v=d_v, kv_rope=rope,
                                            kv_spec=ops.QuantSpec(3, scale, 128))

    def make(i):
        return lambda: bs.sparse_mla_blockscaled_path_c_apply_direct(
            qs[i], None, codes, scale, idxs[i], sm_scale=sm_scale, out=outs[i], lse=lses[i], d_v=d_v, kv_rope=rope)

    steps = args.steps
    secs, host_secs = timed_graph([make(i) for i in range(n_sets)], steps, args.warmup)
    flops = 2.0 * B * H * topk * (d_qk + d_v)
    bytes_alg = B * topk * 656 + B * H * d_qk * 2 + B * H * d_v * 2 + B * topk * 4 + B * H * 4
    per_step = secs / steps
    res = {
        "workload": "sparse_mla_decode B=32 S_q=1 H=128 topk=2048 Skv=65536 latent e4m3[512]+fp32/128 +bf16 rope[64], "
                    + ("power-of-two block scales" if pow2 else "general fp32 block scales (amax/448)"),
        "kernel": kernel,
        "ms_per_step": per_step * 1e3,
        "host_ms_per_step": host_secs / steps * 1e3,
        "tflops": flops / per_step / 1e12,
        "flops_per_step": flops,
        "algorithmic_bytes_per_step": bytes_alg,
        "hbm_gbs": bytes_alg / per_step / 1e9,
    }
    sample = (qs[0], codes, scale, rope, idxs[0], outs[0], lses[0], sm_scale)
    return res, sample


def host_description(threads: int) -> str:
    model = "unknown CPU"
    try:
        with open("/proc/cpuinfo") as fh:
            for ln in fh:
                if ln.startswith("model name"):
                    model = ln.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return f"{model}, {threads} torch threads of {os.cpu_count()} logical CPUs"


def repeat_timed(fn, min_seconds: float = 8.0, max_reps: int = 1000):
    """Repeats fn() until min_seconds of host time have gone by (one untimed call first); returns
    (seconds per call, calls)."""
    fn()
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds or reps >= max_reps:
            return dt / reps, reps


def host_threads() -> int:
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    return torch.get_num_threads()


def cpu_baseline_decode(sample, budget_s: float = 10.0):
    """The reference's CPU fallback (gather -> fp32 matmul -> mask -> softmax -> matmul, restated in
    float32 torch on all host cores) timed on the first sequences of the decode batch; the GPU
    result of the same sequences is checked against the float64 oracle."""
    from oracle import sparse_mla as om, torch_cpu

    q, codes, scale, rope, idx, out, lse, sm_scale = sample
    H, topk = q.shape[2], idx.shape[-1]
    errs = []
    threads = host_threads()
    nseq = q.shape[0]
    rows_all = np.empty((nseq, topk, 1, 576), dtype=np.float32)
    for b in range(nseq):
        ids = idx[b, 0, 0].long()
        rows_all[b] = om.dequant_block_latent(codes[b, ids, 0].cpu().numpy(), scale[b, ids, 0].cpu().numpy(),
                                              rope[b, ids, 0].float().cpu().numpy())[:, None, :]
    q_t = q.float().cpu()
    rows_t = torch.from_numpy(rows_all)
    ar = np.arange(topk, dtype=np.int64)[None, None, None, :]
    ar_t = torch.from_numpy(np.broadcast_to(ar, (nseq, 1, 1, topk)).copy())
    per_pass, reps = repeat_timed(lambda: torch_cpu.sparse_mla_fallback(q_t, rows_t, ar_t, sm_scale=sm_scale, d_v=512), budget_s)
    for b in range(2):
        want, _ = om.sparse_mla_oracle(q_t[b:b + 1].numpy(), rows_all[b:b + 1], ar, sm_scale=sm_scale, d_v=512)
        got = out[b:b + 1].float().cpu().numpy()
        errs.append(float(np.abs(got - want).max() / np.abs(want).max()))
    flops = 2.0 * nseq * H * topk * (576 + 512)
    return {
        "value": flops / per_pass / 1e12,
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"float32 torch restatement of the reference fallback on all {nseq} sequences (H=128, topk=2048, "
                  f"rows already gathered), {reps} passes of {per_pass:.3f} s; {host_description(threads)}",
    }, max(errs)


def bench_vecmat(args, device, M: int):
    from cppmega_mlx_amd.nn._tilelang import fp8_vecmat_path_c as vm

    N, K = 7168, 16384
    gen = torch.Generator(device=device).manual_seed(77 + M)
    n_sets = 3
    ws, ss = [], []
    for _ in range(n_sets):
        w = torch.randn((N, K), generator=gen, device=device, dtype=torch.float32)
        c, s = quantize_block_pow2(w)
        ws.append(c)
        ss.append(s)
        del w
    xs = [torch.randn((M, K), generator=gen, device=device).to(torch.bfloat16) for _ in range(n_sets)]
    outs = [torch.empty((M, N), dtype=torch.bfloat16, device=device) for _ in range(n_sets)]

    def make(i):
        return lambda: vm.fp8_scaled_vecmat_path_c_direct(xs[i], ws[i], scale_x=None, scale_w=ss[i], out=outs[i])

    steps = max(args.steps, 30)
    secs, _ = timed_graph([make(i) for i in range(n_sets)], steps, args.warmup)
    per = secs / steps
    bytes_alg = N * K + N * (K // 128) * 4 + M * K * 2 + M * N * 2
    res = {
        "workload": f"fp8_vecmat W e4m3[7168,16384] + fp32 scale/1x128, x bf16[{M},16384] -> bf16[{M},7168]",
        "us_per_launch": per * 1e6,
        "algorithmic_bytes": bytes_alg,
        "roofline": {"bound": "hbm", "achieved": bytes_alg / per / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": bytes_alg / per / 1e9 / HBM_PEAK_GBS,
                     "traffic": measured_traffic({1: "fp8_vecmat", 4: "fp8_vecmat_m4", 16: "fp8_vecmat_m16", 32: "fp8_vecmat_m32"}.get(M, ""))},
    }
    return res, (xs[0], ws[0], ss[0], outs[0])


def bench_vecmat_fp8x(args, device):
    """The reference's own vecmat form (fp8_vecmat_path_c.py:790-813): e4m3 activation vector with one
    fp32 scale, e4m3 weights with one fp32 scale per output row, fp32 out."""
    from cppmega_mlx_amd.nn._tilelang import fp8_vecmat_path_c as vm

    N, K = 7168, 16384
    gen = torch.Generator(device=device).manual_seed(177)
    sets = []
    for _ in range(3):
        w = torch.randn((N, K), generator=gen, device=device).clamp(-3.5, 3.5).to(torch.float8_e4m3fn).view(torch.uint8)
        x = torch.randn((K,), generator=gen, device=device).clamp(-3.5, 3.5).to(torch.float8_e4m3fn).view(torch.uint8)
        sw = torch.rand((N,), generator=gen, device=device) + 0.5
        sx = torch.full((1,), 0.37, device=device)
        sets.append((x, w, sx, sw, torch.empty((N,), dtype=torch.float32, device=device)))
    fns = [(lambda t=t: vm.fp8_scaled_vecmat_path_c_direct(t[0], t[1], scale_x=t[2], scale_w=t[3], out=t[4])) for t in sets]
    steps = max(args.steps, 30)
    secs, _ = timed_graph(fns, steps, args.warmup)
    per = secs / steps
    bytes_alg = N * K + N * 4 + K + N * 4
    return {
        "workload": "fp8_vecmat W e4m3[7168,16384] + fp32 scale per row, x e4m3[16384] + fp32 scale -> f32[7168]",
        "us_per_launch": per * 1e6,
        "algorithmic_bytes": bytes_alg,
        "roofline": {"bound": "hbm", "achieved": bytes_alg / per / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": bytes_alg / per / 1e9 / HBM_PEAK_GBS, "traffic": measured_traffic("fp8_vecmat_e4m3_activation")},
    }


def cpu_baseline_vecmat(sample, rows: int = 7168):
    from oracle import fp8, torch_cpu, vecmat as ov

    x, w, s, out = sample
    threads = host_threads()
    wf = torch.from_numpy(fp8.e4m3_decode(w[:rows].cpu().numpy()))
    sn, xn = s[:rows].cpu(), x.float().cpu()
    dt, reps = repeat_timed(lambda: torch_cpu.fused_fp8_gemm_fallback(wf, sn, xn), 8.0)
    check = 256
    want = ov.fused_fp8_gemm_oracle(w[:check].cpu().numpy(), s[:check].cpu().numpy(), xn.numpy())
    err = float(np.abs(out[:, :check].float().cpu().numpy() - want).max() / np.abs(want).max())
    nbytes = rows * w.shape[1] * (1 + 4 / 128)
    return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"float32 torch dequantise + matmul (the reference's fallback) on {rows} of 7168 weight rows, "
                      f"byte decode not timed, {reps} passes of {dt:.3f} s; {host_description(threads)}"}, err


def bench_topk(args, device):
    from cppmega_mlx_amd.nn._tilelang import topk_selector as tk

    B, S, T, k = 4, 1024, 8192, 2048
    gen = torch.Generator(device=device).manual_seed(99)
    n_sets = 3
    ends = (T - S + torch.arange(S, device=device, dtype=torch.int32) + 1).repeat(B)
    col = torch.arange(T, device=device)[None, :]
    scores, outs = [], []
    for _ in range(n_sets):
        s = torch.randn((B * S, T), generator=gen, device=device)
        n_dup = T // 20
        dst = torch.randint(0, T, (B * S, n_dup), generator=gen, device=device)
        src = torch.randint(0, T, (B * S, n_dup), generator=gen, device=device)
        s.scatter_(1, dst, s.gather(1, src))
        s.masked_fill_(col >= ends[:, None], float("-inf"))
        scores.append(s)
        outs.append(torch.empty((B * S, k), dtype=torch.int32, device=device))

    def make(i):
        return lambda: tk.topk_selector_tilelang_direct(scores[i], k, out=outs[i], ends=ends, order="index")

    steps = max(args.steps, 30)
    secs, _ = timed_graph([make(i) for i in range(n_sets)], steps, args.warmup)
    per = secs / steps
    bytes_alg = B * S * T * 4 + B * S * k * 4
    res = {
        "workload": "topk_selector scores fp32[4,1024,8192] (5% ties, causal bounds) -> int32[4,1024,2048]",
        "us_per_launch": per * 1e6,
        "algorithmic_bytes": bytes_alg,
        "roofline": {"bound": "hbm", "achieved": bytes_alg / per / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": bytes_alg / per / 1e9 / HBM_PEAK_GBS, "traffic": measured_traffic("topk_selector")},
    }
    # the same rows with the selection ordered by value (the order of the reference's kernel; the attention path takes index order)
    secs_v, _ = timed_graph([lambda i=i: tk.topk_selector_tilelang_direct(scores[i], k, out=outs[i], ends=ends, order="value")
                             for i in range(n_sets)], steps, args.warmup)
    res["value_order"] = {"workload": res["workload"] + ", value-descending output", "us_per_launch": secs_v / steps * 1e6,
                          "algorithmic_bytes": bytes_alg,
                          "roofline": {"bound": "hbm", "achieved": bytes_alg / (secs_v / steps) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                       "frac": bytes_alg / (secs_v / steps) / 1e9 / HBM_PEAK_GBS, "traffic": None}}
    # the decode-time shape: one row per sequence over the whole cache, two-stage selection
    from cppmega_mlx_amd import ops
    wide = [torch.randn((32, 65536), generator=gen, device=device) for _ in range(n_sets)]
    wide_out = torch.empty((32, k), dtype=torch.int32, device=device)
    for name, two_stage in (("decode_shape", True), ("decode_shape_one_workgroup_per_row", False)):
        secs, _ = timed_graph([lambda i=i: ops.topk_select(wide[i], k, out=wide_out, two_stage=two_stage) for i in range(n_sets)],
                              steps, args.warmup)
        nbytes = 32 * 65536 * 4 + 32 * k * 4
        res[name] = {"workload": "topk_selector scores fp32[32,65536] -> int32[32,2048]", "us_per_launch": secs / steps * 1e6,
                     "algorithmic_bytes": nbytes,
                     "roofline": {"bound": "hbm", "achieved": nbytes / (secs / steps) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                  "frac": nbytes / (secs / steps) / 1e9 / HBM_PEAK_GBS, "traffic": None}}
    return res, (scores[0], ends, outs[0], k)


def cpu_baseline_topk(sample, rows: int = 4096):
    from oracle import topk as ot, torch_cpu

    scores, ends, out, k = sample
    threads = host_threads()
    st, et = scores[:rows].cpu(), ends[:rows].cpu()
    dt, reps = repeat_timed(lambda: torch_cpu.topk_fallback(st, k, ends=et), 8.0)
    check = 256
    want = ot.topk_selector_oracle(st[:check].numpy(), k, ends=et[:check].numpy())
    exact = bool(np.array_equal(out[:check].cpu().numpy(), want))
    nbytes = rows * (scores.shape[1] * 4 + k * 4)
    return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"float32 torch stable-sort selection (the reference's argsort fallback) on {rows} of 4096 rows, "
                      f"{reps} passes of {dt:.3f} s; {host_description(threads)}"}, exact


def bench_prefill(args, device):
    from cppmega_mlx_amd.nn._tilelang import sparse_mla_blockscaled_path_c as bs, topk_selector as tk

    S, H, topk = 8192, 128, 2048
    gen = torch.Generator(device=device).manual_seed(555)
    codes, scale, rope = make_latent_cache(gen, 1, S, device)
    q = torch.randn((1, S, H, 576), generator=gen, device=device).to(torch.bfloat16)
    idx_scores = torch.randn((S, S), generator=gen, device=device)
    ends = torch.arange(1, S + 1, device=device, dtype=torch.int32)
    idx = torch.empty((S, topk), dtype=torch.int32, device=device)
    tk.topk_selector_tilelang_direct(idx_scores, topk, out=idx, ends=ends, order="index")
    idx = idx.view(1, S, 1, topk)
    out = torch.empty((1, S, H, 512), dtype=torch.bfloat16, device=device)
    lse = torch.empty((1, S, H), dtype=torch.float32, device=device)
    fn = lambda: bs.sparse_mla_blockscaled_path_c_apply_direct(q, None, codes, scale, idx, sm_scale=576 ** -0.5, out=out,
                                                               lse=lse, d_v=512, kv_rope=rope)
    steps = max(1, min(args.steps, 5))
    secs, _ = timed_graph([fn], steps, 1)
    per = secs / steps
    pairs = int(torch.minimum(ends.long(), torch.tensor(topk, device=device)).sum().item())
    flops = 2.0 * H * pairs * (576 + 512)
    return {"workload": "sparse_mla_prefill B=1 S=8192 H=128 topk=2048 causal", "ms_per_step": per * 1e3,
            "tflops_valid_pairs": flops / per / 1e12, "frac_of_bf16_mfma_peak": flops / per / 1e12 / MFMA_BF16_PEAK_TFLOPS,
            "roofline": {"bound": "mfma", "achieved": flops / per / 1e12, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": flops / per / 1e12 / MFMA_BF16_PEAK_TFLOPS, "traffic": None}}


def bench_prefill_rows(args, device):
    """The same prefill on the other row layouts the reference's Path C kernels take, all rows of 576
    channels without a separate rope part: unquantised float16 rows (float Path C), e4m3 codes with
    one fp32 scale per row and per (query, head) (FP8 Path C), e4m3 codes with one E8M0 byte per 32
    channels (block-scaled Path C).  The 32-head tile kernel, four wavefronts sharing one key stream."""
    from cppmega_mlx_amd import ops
    from cppmega_mlx_amd.nn._tilelang import (sparse_mla_blockscaled_path_c as bs, sparse_mla_fp8_path_c as f8,
                                              topk_selector as tk)

    S, H, topk = 8192, 128, 2048
    gen = torch.Generator(device=device).manual_seed(556)
    idx_scores = torch.randn((S, S), generator=gen, device=device)
    ends = torch.arange(1, S + 1, device=device, dtype=torch.int32)
    idx = torch.empty((S, topk), dtype=torch.int32, device=device)
    tk.topk_selector_tilelang_direct(idx_scores, topk, out=idx, ends=ends, order="index")
    idx = idx.view(1, S, 1, topk)
    del idx_scores
    lse = torch.empty((1, S, H), dtype=torch.float32, device=device)
    pairs = int(torch.minimum(ends.long(), torch.tensor(topk, device=device)).sum().item())
    flops = 2.0 * H * pairs * (576 + 512)
    steps = max(1, min(args.steps, 5))
    res = {}

    def timed(name, fn, what):
        secs, _ = timed_graph([fn], steps, 1)
        per = secs / steps
        res[name] = {"workload": f"sparse_mla_prefill {what} B=1 S=8192 H=128 topk=2048 causal", "ms_per_step": per * 1e3,
                     "tflops_valid_pairs": flops / per / 1e12, "frac_of_bf16_mfma_peak": flops / per / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                     "roofline": {"bound": "mfma", "achieved": flops / per / 1e12, "peak": MFMA_BF16_PEAK_TFLOPS,
                                  "unit": "TFLOP/s", "frac": flops / per / 1e12 / MFMA_BF16_PEAK_TFLOPS, "traffic": None}}

    kv = torch.randn((1, S, 1, 576), generator=gen, device=device).to(torch.float16)
    q = torch.randn((1, S, H, 576), generator=gen, device=device).to(torch.float16)
    out = torch.empty((1, S, H, 512), dtype=torch.float16, device=device)
    timed("float16_rows", lambda: ops.sparse_mla_forward(q, kv, idx, sm_scale=576 ** -0.5, d_v=512, out=out, lse=lse),
          "float16 rows")
    qc = torch.randn((1, S, H, 576), generator=gen, device=device).to(torch.float8_e4m3fn).view(torch.uint8)
    kc = torch.randn((1, S, 1, 576), generator=gen, device=device).to(torch.float8_e4m3fn).view(torch.uint8)
    out = torch.empty((1, S, H, 512), dtype=torch.bfloat16, device=device)
    qs = torch.rand((1, S, H), generator=gen, device=device) + 0.5
    ks = torch.rand((1, S, 1), generator=gen, device=device) + 0.5
    timed("fp8_per_token", lambda: f8.sparse_mla_fp8_path_c_apply_direct(qc, qs, kc, ks, idx, sm_scale=576 ** -0.5, out=out,
                                                                         lse=lse, d_v=512),
          "e4m3 rows + fp32 scale per row, e4m3 q + fp32 scale per head")
    qe = torch.randint(120, 130, (1, S, H, 18), generator=gen, device=device, dtype=torch.uint8)
    ke = torch.randint(120, 130, (1, S, 1, 18), generator=gen, device=device, dtype=torch.uint8)
    timed("fp8_e8m0", lambda: bs.sparse_mla_blockscaled_path_c_apply_direct(qc, qe, kc, ke, idx, sm_scale=576 ** -0.5, out=out,
                                                                           lse=lse, d_v=512),
          "e4m3 rows and q + one E8M0 byte per 32 channels")
    return res


def bench_copy(args, device):
    """A plain device copy of known size: the yardstick the FETCH_SIZE / WRITE_SIZE
    counters of the other kernels are scaled by."""
    n = 256 << 20
    src = torch.full((n,), 7, dtype=torch.uint8, device=device)
    dst = torch.empty_like(src)
    secs, _ = timed_graph([lambda: dst.copy_(src)], args.steps, args.warmup)
    per = secs / args.steps
    return {"workload": "torch copy_ of 256 MiB (u8)", "bytes_read": n, "bytes_written": n, "us_per_launch": per * 1e6,
            "gbs": 2.0 * n / per / 1e9}


def bench_next_rows(args, device):
    """The rows either side of the attention call: the fused producer + cache append for a
    prefill chunk (8192 latent rows of 512 + 64 rope channels) and for one decode step (32 rows),
    and the two index producers at prefill size.  HBM-bound; bytes are algorithmic."""
    from cppmega_mlx_amd import ops
    gen = torch.Generator(device=device).manual_seed(99)
    res = {}
    steps = max(args.steps, 30)

    def hbm(name, fn, nbytes, workload):
        secs, _ = timed_graph([fn], steps, args.warmup)
        per = secs / steps
        res[name] = {"workload": workload, "us_per_launch": per * 1e6, "algorithmic_bytes": nbytes,
                     "roofline": {"bound": "hbm", "achieved": nbytes / per / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                  "frac": nbytes / per / 1e9 / HBM_PEAK_GBS, "traffic": None}}

    for tag, B, S, cap in (("append_prefill", 1, 8192, 8192), ("append_decode", 32, 1, 4096)):
        lat = torch.randn((B, S, 1, 512), generator=gen, device=device).to(torch.bfloat16)
        rope = torch.randn((B, S, 1, 64), generator=gen, device=device).to(torch.bfloat16)
        kv = torch.zeros((B, cap, 1, 512), dtype=torch.uint8, device=device)
        sc = torch.zeros((B, cap, 1, 4), dtype=torch.float32, device=device)
        rp = torch.zeros((B, cap, 1, 64), dtype=torch.bfloat16, device=device)
        hbm(tag, lambda lat=lat, rope=rope, kv=kv, sc=sc, rp=rp: ops.kv_cache_append(
                lat, kv_cache=kv, scale_cache=sc, position=0, rope=rope, rope_cache=rp, scale_block=128, pow2_scales=True),
            B * S * (512 * 2 + 64 * 2 + 656),
            f"bf16 latent[{B},{S},1,512] + rope[..,64] -> e4m3 + fp32/128 scales + bf16 rope at the cache position")
    S = K = 8192
    out = torch.empty((1, S, 1, 2048), dtype=torch.int32, device=device)
    hbm("causal_indices", lambda: ops.causal_sparse_indices(out, query_offset=0, key_length=K), out.numel() * 4,
        "causal_sparse_indices(1, 8192, 1, 2048) int32")
    mask = (torch.arange(K, device=device)[None, :] <= torch.arange(S, device=device)[:, None]).contiguous()
    hbm("mask_indices", lambda: ops.mask_sparse_indices(mask[None, None], out, topk=2048), mask.numel() + out.numel() * 4,
        "sparse_indices_from_attention_mask: bool mask [8192, 8192] -> int32 [1,8192,1,2048]")
    # indexer scores -> top-k: prefill (causal bounds, no mask read) and one decode step
    for tag, B, Sq, Skv in (("indexer_prefill", 1, 8192, 8192), ("indexer_decode", 32, 1, 65536)):
        H, D, topk = 64, 128, 2048
        q = torch.randn((B, Sq, H, D), generator=gen, device=device).to(torch.bfloat16)
        kk = torch.randn((B, Skv, D), generator=gen, device=device).to(torch.bfloat16)
        w = (torch.randn((B, Sq, H), generator=gen, device=device) * H ** -0.5).to(torch.bfloat16)
        ends = (torch.arange(1, Sq + 1, device=device, dtype=torch.int32) + (Skv - Sq)).repeat(B).contiguous()
        idx = torch.empty((B, Sq, topk), dtype=torch.int32, device=device)
        nbytes = (q.numel() + kk.numel() + w.numel()) * 2 + ends.numel() * 4 + idx.numel() * 4
        hbm(tag, lambda q=q, kk=kk, w=w, ends=ends, idx=idx: ops.indexer_topk(q, kk, w, sm_scale=D ** -0.5, topk=topk, out=idx, ends=ends),
            nbytes, f"indexer_topk q bf16[{B},{Sq},{H},{D}] k bf16[{B},{Skv},{D}] -> int32[{B},{Sq},{topk}] "
                    f"(scores stay in a {ops.indexer_topk_workspace_bytes(q, kk, w, topk=topk) >> 20} MiB chunk buffer)")
    # the per-head projections either side of the decode attention call (bf16 weights, 32 sequences)
    B, H, D_k, D_kv, D_v = 32, 128, 128, 512, 128
    for tag, K, N in (("absorb_query", D_k, D_kv), ("unabsorb_output", D_kv, D_v)):
        x = torch.randn((B, H, K), generator=gen, device=device).to(torch.bfloat16)
        w = (torch.randn((H, N, K), generator=gen, device=device) * K ** -0.5).to(torch.bfloat16)
        y = torch.empty((B, H, N), dtype=torch.bfloat16, device=device)
        hbm(tag, lambda x=x, w=w, y=y: ops.head_gemm(x, w, out=y), (x.numel() + w.numel() + y.numel()) * 2,
            f"head_gemm x bf16[{B},{H},{K}] . W bf16[{H},{N},{K}] -> bf16[{B},{H},{N}]")
    # training side: sparse-MLA backward on the matrix cores (bound by the float32 atomic adds into dkv)
    B, S, H, D, d_v, Skv, topk = 1, 1024, 16, 576, 512, 4096, 256
    q = torch.randn((B, S, H, D), generator=gen, device=device).to(torch.bfloat16)
    kv = torch.randn((B, Skv, 1, D), generator=gen, device=device).to(torch.bfloat16)
    d_out = torch.randn((B, S, H, d_v), generator=gen, device=device).to(torch.bfloat16)
    idx = torch.stack([torch.randperm(Skv, generator=gen, device=device)[:topk] for _ in range(S)]).to(torch.int32).view(B, S, 1, topk)
    dq = torch.empty_like(q)
    dkv = torch.empty((B, Skv, 1, D), dtype=torch.float32, device=device)
    secs, _ = timed_graph([lambda: ops.sparse_mla_backward(q, kv, d_out, idx, sm_scale=D ** -0.5, d_v=d_v, dq=dq, dkv=dkv)], steps, args.warmup)
    flops = 2.0 * B * S * H * topk * (3 * D + 2 * d_v)
    res["sparse_mla_backward"] = {
        "workload": f"sparse_mla_bwd q bf16[{B},{S},{H},{D}] kv bf16[{B},{Skv},1,{D}] topk {topk} -> dq bf16, dkv f32 (atomic adds)",
        "us_per_launch": secs / steps * 1e6, "algorithmic_flops": flops,
        "roofline": {"bound": "mfma", "achieved": flops / (secs / steps) / 1e12, "peak": 2500.0, "unit": "TFLOP/s",
                     "frac": flops / (secs / steps) / 1e12 / 2500.0, "traffic": None},
        "float32_atomic_adds": B * S * topk * D, "atomic_add_floor_us": B * S * topk * D / (128 * 2.4e9) * 1e6}

    # the same backward over per-token FP8 operands (e4m3 code values + float32 scale per token)
    q8 = (torch.randn((B, S, H, D), generator=gen, device=device) * 64).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    kv8 = (torch.randn((B, Skv, 1, D), generator=gen, device=device) * 64).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    qs = torch.rand((B, S, H), generator=gen, device=device) * 0.02 + 0.005
    kvs = torch.rand((B, Skv, 1), generator=gen, device=device) * 0.02 + 0.005
    dq32 = torch.empty((B, S, H, D), dtype=torch.float32, device=device)
    secs, _ = timed_graph([lambda: ops.sparse_mla_backward(q8, kv8, d_out, idx, sm_scale=D ** -0.5, d_v=d_v, dq=dq32, dkv=dkv,
                                                           q_scale=qs, kv_scale=kvs)], steps, args.warmup)
    res["sparse_mla_backward_fp8"] = {
        "workload": f"sparse_mla_bwd q e4m3[{B},{S},{H},{D}] + f32 scale per token, kv e4m3[{B},{Skv},1,{D}] + f32 scale per token, "
                    f"d_out bf16, topk {topk} -> dq f32, dkv f32 (atomic adds)",
        "us_per_launch": secs / steps * 1e6, "algorithmic_flops": flops,
        "roofline": {"bound": "mfma", "achieved": flops / (secs / steps) / 1e12, "peak": 2500.0, "unit": "TFLOP/s",
                     "frac": flops / (secs / steps) / 1e12 / 2500.0, "traffic": None}}

    # DSA indexer KL loss (training side): one launch over every (batch, query position)
    ASq = Sk = 4096; AB, AH, AD, topk = 1, 8, 64, 1024
    qq = torch.randn((ASq, AB, AH, AD), generator=gen, device=device).to(torch.bfloat16)
    kk = torch.randn((Sk, AB, AH, AD), generator=gen, device=device).to(torch.bfloat16)
    isc = torch.randn((AB, ASq, Sk), generator=gen, device=device)
    top = torch.topk(isc, topk, dim=-1).indices.to(torch.int32).contiguous()
    loss = torch.empty((AB, ASq), dtype=torch.float32, device=device)
    for name, lst in (("dsa_indexer_loss_dense", None), ("dsa_indexer_loss_sparse", top)):
        secs, _ = timed_graph([lambda: ops.dsa_indexer_loss(qq, kk, isc, softmax_scale=AD ** -0.5, out=loss, topk_indices=lst)], steps, args.warmup)
        flops = 2.0 * AB * AH * AD * (ASq * (ASq + 1) / 2)
        res[name] = {
            "workload": f"dsa_indexer_loss query/key bf16[{ASq},{AB},{AH},{AD}] index_scores f32[{AB},{ASq},{Sk}]"
                        + (f" topk_indices i32[{AB},{ASq},{topk}]" if lst is not None else "") + " -> loss f32",
            "us_per_launch": secs / steps * 1e6, "algorithmic_flops": flops,
            "roofline": {"bound": "mfma", "achieved": flops / (secs / steps) / 1e12, "peak": 2500.0, "unit": "TFLOP/s",
                         "frac": flops / (secs / steps) / 1e12 / 2500.0, "traffic": None}}
    return res


def measured_traffic(name):
    """HBM bytes per launch from the committed rocprofv3 counter runs, or None."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "traffic.json")
    try:
        with open(path) as fh:
            return json.load(fh)["workloads"][name]["hbm_bytes_per_launch"]
    except (OSError, KeyError, ValueError):
        return None


# --------------------------------------------------------------------------- rocprofv3 summaries
# The three profiler runs whose CSV output `--summarise-profiles DIR` turns into profiles/*.md and
# profiles/traffic.json.  Each is run from /tmp (`cd /tmp && export TMPDIR=/tmp`) with DIR as below.
PROFILE_RUNS = {
    "prof_all": "rocprofv3 --kernel-trace --stats --output-format csv -d DIR/prof_all -o all -- python3 bench.py "
                "--only decode,vecmat,topk,copy,next,prefill_rows --steps 20 --no-cpu-baseline",
    "pmc_fetch": "rocprofv3 --pmc FETCH_SIZE --output-format csv -d DIR/pmc_fetch -o f -- python3 bench.py "
                 "--only decode,vecmat,topk,copy,next,prefill_rows --steps 3 --warmup 1 --no-cpu-baseline",
    "pmc_write": "rocprofv3 --pmc WRITE_SIZE --output-format csv -d DIR/pmc_write -o w -- python3 bench.py "
                 "--only decode,vecmat,topk,copy,next,prefill_rows --steps 3 --warmup 1 --no-cpu-baseline",
    "pmc_sq": "rocprofv3 --pmc SQ_WAVE_CYCLES SQ_BUSY_CYCLES SQ_INSTS_VALU SQ_INSTS_MFMA SQ_VALU_MFMA_BUSY_CYCLES "
              "SQ_ACTIVE_INST_VALU SQ_WAIT_INST_ANY SQ_ACTIVE_INST_LDS --output-format csv -d DIR/pmc_sq -o s -- python3 bench.py "
              "--only decode --steps 3 --warmup 1 --no-cpu-baseline",
}
# summary file -> (kernel-name fragments, workload text)
PROFILE_WORKLOADS = [
    ("sparse_mla_decode", ("sparse_mla_latent",),
     "decode B=32 S_q=1 H=128 topk=2048 Skv=65536 (e4m3 latent + fp32/128 scales + bf16 rope); the run times the "
     "power-of-two-scale cache and the general-scale cache, so each row averages both"),
    ("fp8_vecmat", ("gemv_stream_kernel<1, 4, 4, 0>",), "W e4m3[7168,16384] + fp32 scale/128, x bf16[1,16384]"),
    ("fp8_vecmat_e4m3_activation", ("gemv_stream_kernel<1, 4, 4, 1>",),
     "W e4m3[7168,16384] + fp32 scale per row, x e4m3[16384] + fp32 scale -> f32[7168] (the reference's own vecmat form)"),
    ("fp8_vecmat_m4", ("gemv_stream_kernel<4",), "W e4m3[7168,16384] + fp32 scale/128, x bf16[4,16384]"),
    ("fp8_vecmat_m16", ("skinny_rows_kernel<1>",),
     "W e4m3[7168,16384] + fp32 scale/128, x bf16[16,16384] (one kernel, no K split, no workspace)"),
    ("fp8_vecmat_m32", ("skinny_mfma_kernel<2>", "skinny_reduce"),
     "W e4m3[7168,16384] + fp32 scale/128, x bf16[32,16384] (split-K kernel + reduce kernel)"),
    ("topk_selector", ("topk_tile_kernel<float, 16, 4, 512, 0>",), "scores fp32[4096 rows,8192] -> int32[4096,2048]"),
    ("topk_selector_decode_shape", ("topk_tile_kernel<float, 16, 4, 512, 1>", "topk_tile_kernel<float, 16, 4, 1024, 2>", "topk_wide_kernel"),
     "scores fp32[32,65536] -> int32[32,2048]: the two-stage path (segment kernel, then candidate kernel) and, for "
     "comparison, the one-workgroup-per-row kernel; the indexer's decode row runs the two-stage kernels as well"),
    ("indexer_scores_topk", ("indexer_scores_kernel", "indexer_qw_kernel"),
     "indexer_topk q bf16[B,Sq,64,128], k bf16[B,Skv,128]: prefill (1, 8192, 8192) and decode (32, 1, 65536) dispatches"),
    ("mla_absorb_head_gemm", ("head_gemm_kernel",),
     "head_gemm x bf16[32,128,128] . W bf16[128,512,128] and x bf16[32,128,512] . W bf16[128,128,512]"),
    ("kv_cache_append", ("cache_append_kernel",),
     "bf16 latent[B,S,1,512] + rope[..,64] -> e4m3 + fp32/128 scales + bf16 rope in the cache: one dispatch of 8192 rows "
     "(prefill chunk) and one of 32 rows (decode step) per step"),
    ("sparse_mla_prefill_row_layouts", ("sparse_mla_mfma_kernel<",),
     "sparse_mla_fwd q [1,8192,128,576], kv [1,8192,1,576], causal top-2048 indices -> [1,8192,128,512] on the 32-head tile kernel, "
     "four wavefronts sharing one key stream: <false, true, true, 0> unquantised float16 rows, <true, false, true, 1> e4m3 rows "
     "with per-token fp32 scales, <true, false, true, 2> e4m3 rows with E8M0 bytes per 32 channels"),
    ("sparse_mla_backward", ("sparse_mla_bwd", "fill_zero_kernel"),
     "sparse_mla_bwd q bf16[1,1024,16,576], kv bf16[1,4096,1,576], d_out bf16[1,1024,16,512], topk 256 -> dq bf16, dkv f32 "
     "(the dkv clear, then the matrix-core kernel with its float32 atomic adds)"),
    ("dsa_indexer_loss", ("dsa_indexer_loss",),
     "dsa_indexer_loss query / key bf16[4096,1,8,64], index_scores f32[1,4096,4096]: one dense and one sparse "
     "(topk_indices i32[1,4096,1024]) dispatch per step"),
    ("sparse_index_producers", ("_indices_",),
     "causal_sparse_indices(1,8192,1,2048) and sparse_indices_from_attention_mask(bool [8192,8192], topk 2048)"),
]


def summarise_profiles(src: str) -> int:
    """Write profiles/*.md and profiles/traffic.json from the CSV output of PROFILE_RUNS under `src`."""
    import collections
    import csv

    here = os.path.dirname(os.path.abspath(__file__))
    out_dir = os.path.join(here, "profiles")
    os.makedirs(out_dir, exist_ok=True)

    def rows(rel):
        with open(os.path.join(src, rel)) as fh:
            return list(csv.DictReader(fh))

    stats = {r["Name"]: r for r in rows("prof_all/all_kernel_stats.csv")}

    def counters(rel):
        agg = collections.defaultdict(list)
        for r in rows(rel):
            agg[r["Kernel_Name"]].append(float(r["Counter_Value"]))
        return agg

    fetch, write = counters("pmc_fetch/f_counter_collection.csv"), counters("pmc_write/w_counter_collection.csv")
    copy_kib = 262144.0                                    # the 256 MiB device copy of bench_copy, each way
    copy_f, copy_w = max(fetch["__amd_rocclr_copyBuffer"]), max(write["__amd_rocclr_copyBuffer"])
    scale_f, scale_w = copy_kib / copy_f, copy_kib / copy_w

    def cmd(key):
        return "`cd /tmp && export TMPDIR=/tmp && " + PROFILE_RUNS[key].replace("DIR", "$GRAFT_REPO_ROOT/gpurun_out").replace(
            "bench.py", "$GRAFT_REPO_ROOT/bench.py") + "`"

    def short(name):
        return name.replace("(anonymous namespace)::", "")

    traffic = {}
    for fname, frags, workload in PROFILE_WORKLOADS:
        names = [n for n in stats if "cm::" in n and any(f in n for f in frags)]
        text = [f"# rocprofv3 summary: {fname}", "", f"Workload: {workload} (one MI355X, synthetic inputs resident in HBM).", "",
                "## Kernel durations (`--kernel-trace --stats`)", "", "Command: " + cmd("prof_all"), "",
                "| kernel | calls | avg us | min us | max us |", "|---|---|---|---|---|"]
        for n in names:
            r = stats[n]
            text.append("| `%s` | %s | %.2f | %.2f | %.2f |" % (short(n), r["Calls"], float(r["AverageNs"]) / 1e3,
                                                              float(r["MinNs"]) / 1e3, float(r["MaxNs"]) / 1e3))
        text += ["", "## HBM traffic per dispatch (`--pmc FETCH_SIZE`, then `--pmc WRITE_SIZE`, KiB)", "",
                 "Commands: " + cmd("pmc_fetch") + " and " + cmd("pmc_write") + ".", "",
                 "Scale factors from the 256 MiB device copy in the same runs (`__amd_rocclr_copyBuffer`, 262144 KiB each way): "
                 "FETCH_SIZE read %.1f KiB -> x%.3f, WRITE_SIZE read %.1f KiB -> x%.3f." % (copy_f, scale_f, copy_w, scale_w), "",
                 "| kernel | FETCH_SIZE KiB | WRITE_SIZE KiB | scaled read MiB | scaled write MiB |", "|---|---|---|---|---|"]
        total = 0.0
        for n in names:
            f = sum(fetch[n]) / len(fetch[n]) if fetch.get(n) else 0.0
            w = sum(write[n]) / len(write[n]) if write.get(n) else 0.0
            text.append("| `%s` | %.1f | %.1f | %.1f | %.1f |" % (short(n), f, w, f * scale_f / 1024, w * scale_w / 1024))
            total += (f * scale_f + w * scale_w) * 1024
        traffic[fname] = {"hbm_bytes_per_launch": int(total), "kernels": names}
        if fname == "sparse_mla_decode" and os.path.exists(os.path.join(src, "pmc_sq/s_counter_collection.csv")):
            sq = collections.defaultdict(list)
            for r in rows("pmc_sq/s_counter_collection.csv"):
                if "sparse_mla_latent_kernel" in r["Kernel_Name"]:
                    sq[r["Counter_Name"]].append(float(r["Counter_Value"]))
            text += ["", "## SQ counters of the main kernel (one `--pmc` pass, average per dispatch, summed over its wavefronts)", "",
                     "Command: " + cmd("pmc_sq"), "", "| counter | value |", "|---|---|"]
            avg = {k: sum(v) / len(v) for k, v in sq.items()}
            for k in sorted(avg):
                text.append("| %s | %.0f |" % (k, avg[k]))
            if avg.get("SQ_WAVE_CYCLES"):
                text += ["", "SQ_VALU_MFMA_BUSY_CYCLES / (4 x SQ_WAVE_CYCLES) = %.3f: the matrix-core busy fraction of the wavefronts' "
                         "lifetime (wave cycles count in units of 4 clocks)." % (avg.get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0) / (4 * avg["SQ_WAVE_CYCLES"]))]
        with open(os.path.join(out_dir, fname + ".md"), "w") as fh:
            fh.write("\n".join(text) + "\n")
    with open(os.path.join(out_dir, "traffic.json"), "w") as fh:
        json.dump({"fetch_scale": scale_f, "write_scale": scale_w, "workloads": traffic}, fh, indent=1)
    print(f"wrote {len(PROFILE_WORKLOADS)} summaries and traffic.json to {out_dir}")
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--summarise-profiles", metavar="DIR", default=None,
                    help="no GPU work: turn the rocprofv3 CSVs under DIR (see PROFILE_RUNS) into profiles/*.md and profiles/traffic.json")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--only", type=str, default="decode,vecmat,topk,next,prefill")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.summarise_profiles:
        return summarise_profiles(args.summarise_profiles)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU; the path shards without communication "
              "(rows / sequences / queries per GPU), so --gpus N>1 is not run here.", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP kernels have no CPU path.", file=sys.stderr)
        return 3
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    from cppmega_mlx_amd import native_status
    native_status()
    parts = set(args.only.split(","))

    line = {
        "metric": "sparse_mla_decode_tflops",
        "value": None,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": None,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {},
    }
    if "decode" in parts:
        res_pow2, sample = bench_decode(args, device, pow2=True)
        del sample
        torch.cuda.empty_cache()
        res, sample = bench_decode(args, device, pow2=False)
        line["value"] = res["tflops"]
        line["ms_per_step"] = res["ms_per_step"]
        line["config"] = {"workload": res["workload"], "kernel": res["kernel"],
                          "flops_per_step": res["flops_per_step"],
                          "algorithmic_bytes_per_step": res["algorithmic_bytes_per_step"],
                          "host_ms_per_step": res["host_ms_per_step"], "hbm_gbs": res["hbm_gbs"],
                          "power_of_two_block_scales": {"ms_per_step": res_pow2["ms_per_step"], "tflops": res_pow2["tflops"],
                                                        "frac": res_pow2["tflops"] / MFMA_BF16_PEAK_TFLOPS}}
        line["roofline"] = {"bound": "mfma", "achieved": res["tflops"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                            "frac": res["tflops"] / MFMA_BF16_PEAK_TFLOPS, "traffic": measured_traffic("sparse_mla_decode")}
        if not args.no_cpu_baseline:
            cpu, rel_err = cpu_baseline_decode(sample)
            line["cpu_baseline"] = cpu
            line["config"]["max_rel_err_vs_oracle_on_sample"] = rel_err
        del sample
        torch.cuda.empty_cache()
    if "vecmat" in parts:
        line["vecmat"] = {}
        for M in (1, 4, 16, 32):
            res, sample = bench_vecmat(args, device, M)
            if not args.no_cpu_baseline and M == 1:
                res["cpu_baseline"], res["max_rel_err_vs_oracle_on_sample"] = cpu_baseline_vecmat(sample)
            line["vecmat"][f"M{M}"] = res
            del sample
            torch.cuda.empty_cache()
        line["vecmat"]["M1_fp8x"] = bench_vecmat_fp8x(args, device)
        torch.cuda.empty_cache()
    if "topk" in parts:
        res, sample = bench_topk(args, device)
        if not args.no_cpu_baseline:
            res["cpu_baseline"], res["bit_exact_vs_oracle_on_sample"] = cpu_baseline_topk(sample)
        line["topk"] = res
        del sample
        torch.cuda.empty_cache()
    if "prefill" in parts:
        line["prefill"] = bench_prefill(args, device)
    if "prefill" in parts or "prefill_rows" in parts:
        line["prefill_row_layouts"] = bench_prefill_rows(args, device)
    if "copy" in parts:
        line["copy"] = bench_copy(args, device)
    if "next" in parts:
        line["next_rows"] = bench_next_rows(args, device)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
