#!/usr/bin/env python3
"""Benchmark of the sparse-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--replays R] [--only PARTS]

Prints ONE JSON line.  The headline (`metric`/`value`) is sparse-MLA decode
throughput on the B=32, H=128, topk=2048, 64K-token FP8 latent-cache
configuration with general fp32 block scales; `vecmat` (M = 1, 4, 16), `topk`
and `prefill` carry the other configurations of the same path with their own
roofline objects.  The default run prints these four and nothing else; the
remaining rows are asked for by name with `--only` (comma separated):
decode, decode_general, decode_pow2, vecmat, vecmat_m32, vecmat_fp8x, topk,
topk_value, topk_wide, prefill, prefill_general, prefill_pow2, prefill_rows,
copy, next.

A "step" is one pass of the kernel(s) over one synthetic batch that is already
resident in HBM.  K steps are captured into a HIP graph (launch-bound at these
kernel lengths otherwise); the graph is replayed R times, each replay
bracketed by HIP events on the launch stream, and a row reports the median
replay (`us` / `ms_per_step`) with the fastest one beside it (`min_*`).
Input sets rotate between steps so the HBM-bound kernels cannot be served by
the 256 MB Infinity Cache.

Every row that has a checker is compared with the oracle on a sample inside
the run; a failed check is reported in the line and makes the exit status 4.

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


REPLAYS = 7


def timed_graph(step_fns, steps: int, warmup: int, replays: int | None = None):
    """Run `warmup` eager steps, capture `steps` steps into a HIP graph, replay it `replays` times,
    each replay timed by HIP events on the launch stream.

    step_fns: list of zero-argument callables (rotated).  Returns a dict of seconds per step:
    median / min / max over the replays, and the host-clock time of the median replay."""
    replays = replays or REPLAYS
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
    graph.replay()                      # untimed replay: the first replay pays upload costs
    torch.cuda.synchronize()
    dev, host = [], []
    for _ in range(replays):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        host.append((time.perf_counter() - t0) / steps)
        dev.append(e0.elapsed_time(e1) * 1e-3 / steps)
    order = sorted(range(replays), key=lambda i: dev[i])
    mid = order[replays // 2]
    return {"median": dev[mid], "min": dev[order[0]], "max": dev[order[-1]], "host": host[mid], "replays": replays}


def sig(x, digits: int = 4):
    """Round to `digits` significant digits (keeps the printed line short)."""
    if x is None or x == 0 or not math.isfinite(x):
        return x
    return round(x, digits - 1 - int(math.floor(math.log10(abs(x)))))


def hbm_row(workload, t, nbytes, traffic_key=None):
    per = t["median"]
    return {"workload": workload, "us": sig(per * 1e6), "min_us": sig(t["min"] * 1e6), "bytes": nbytes,
            "roofline": {"bound": "hbm", "achieved": sig(nbytes / per / 1e9), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": sig(nbytes / per / 1e9 / HBM_PEAK_GBS), "traffic": measured_traffic(traffic_key) if traffic_key else None}}


def mfma_row(workload, t, flops, traffic_key=None, unit_ms=True):
    per = t["median"]
    row = {"workload": workload}
    if unit_ms:
        row.update({"ms_per_step": sig(per * 1e3), "min_ms_per_step": sig(t["min"] * 1e3)})
    else:
        row.update({"us": sig(per * 1e6), "min_us": sig(t["min"] * 1e6)})
    row.update({"flops": flops,
                "roofline": {"bound": "mfma", "achieved": sig(flops / per / 1e12), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                             "frac": sig(flops / per / 1e12 / MFMA_BF16_PEAK_TFLOPS),
                             "traffic": measured_traffic(traffic_key) if traffic_key else None}})
    return row


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

    t = timed_graph([make(i) for i in range(n_sets)], args.steps, args.warmup)
    flops = 2.0 * B * H * topk * (d_qk + d_v)
    bytes_alg = B * topk * 656 + B * H * d_qk * 2 + B * H * d_v * 2 + B * topk * 4 + B * H * 4
    res = {
        "workload": "sparse_mla_decode B=32 S_q=1 H=128 topk=2048 Skv=65536 latent e4m3[512]+fp32/128 +bf16 rope[64], "
                    + ("power-of-two block scales" if pow2 else "general fp32 block scales (amax/448)"),
        "kernel": kernel, "t": t, "flops": flops, "bytes": bytes_alg,
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


def decode_sample_error(sample, seqs=(0, 1)):
    """max |GPU - float64 oracle| / max |oracle| over the given sequences of a decode sample."""
    from oracle import sparse_mla as om

    q, codes, scale, rope, idx, out, lse, sm_scale = sample
    topk = idx.shape[-1]
    ar = np.arange(topk, dtype=np.int64)[None, None, None, :]
    errs = []
    for b in seqs:
        ids = idx[b, 0, 0].long()
        rows = om.dequant_block_latent(codes[b, ids, 0].cpu().numpy(), scale[b, ids, 0].cpu().numpy(),
                                       rope[b, ids, 0].float().cpu().numpy())[None, :, None, :]
        want, _ = om.sparse_mla_oracle(q[b:b + 1].float().cpu().numpy(), rows, ar, sm_scale=sm_scale, d_v=512)
        got = out[b:b + 1].float().cpu().numpy()
        errs.append(float(np.abs(got - want).max() / np.abs(want).max()))
    return max(errs)


def cpu_baseline_decode(sample, budget_s: float = 10.0):
    """The reference's CPU fallback (gather -> fp32 matmul -> mask -> softmax -> matmul, restated in
    float32 torch on all host cores) timed on the whole decode batch with the rows already gathered
    and dequantised (the gather and the byte decode are not timed, which favours the CPU)."""
    from oracle import sparse_mla as om, torch_cpu

    q, codes, scale, rope, idx, out, lse, sm_scale = sample
    H, topk = q.shape[2], idx.shape[-1]
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
    flops = 2.0 * nseq * H * topk * (576 + 512)
    return {
        "value": sig(flops / per_pass / 1e12),
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"fp32 torch restatement of the reference fallback, all {nseq} sequences, gather and byte decode "
                  f"not timed, {reps} passes of {per_pass:.3f} s; {host_description(threads)}",
    }


VECMAT_TRAFFIC = {1: "fp8_vecmat", 4: "fp8_vecmat_m4", 16: "fp8_vecmat_m16", 32: "fp8_vecmat_m32"}


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

    t = timed_graph([make(i) for i in range(n_sets)], max(args.steps, 30), args.warmup)
    bytes_alg = N * K + N * (K // 128) * 4 + M * K * 2 + M * N * 2
    res = hbm_row(f"fp8_vecmat W e4m3[7168,16384]+fp32 scale/1x128, x bf16[{M},16384] -> bf16[{M},7168]", t, bytes_alg,
                  VECMAT_TRAFFIC.get(M))
    return res, (xs[0], ws[0], ss[0], outs[0])


def vecmat_sample_error(sample, check: int = 256):
    from oracle import vecmat as ov

    x, w, s, out = sample
    want = ov.fused_fp8_gemm_oracle(w[:check].cpu().numpy(), s[:check].cpu().numpy(), x.float().cpu().numpy())
    return float(np.abs(out[:, :check].float().cpu().numpy() - want).max() / np.abs(want).max())


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
    t = timed_graph(fns, max(args.steps, 30), args.warmup)
    return hbm_row("fp8_vecmat W e4m3[7168,16384]+fp32 scale per row, x e4m3[16384]+fp32 scale -> f32[7168]", t,
                   N * K + N * 4 + K + N * 4, "fp8_vecmat_e4m3_activation")


def cpu_baseline_vecmat(sample, rows: int = 7168):
    from oracle import fp8, torch_cpu

    x, w, s, out = sample
    threads = host_threads()
    wf = torch.from_numpy(fp8.e4m3_decode(w[:rows].cpu().numpy()))
    sn, xn = s[:rows].cpu(), x.float().cpu()
    dt, reps = repeat_timed(lambda: torch_cpu.fused_fp8_gemm_fallback(wf, sn, xn), 8.0)
    nbytes = rows * w.shape[1] * (1 + 4 / 128)
    return {"value": sig(nbytes / dt / 1e9), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"fp32 torch dequantise + matmul (the reference's fallback) on {rows} of 7168 weight rows, "
                      f"byte decode not timed, {reps} passes of {dt:.3f} s; {host_description(threads)}"}


def topk_inputs(device, n_sets: int = 3):
    B, S, T, k = 4, 1024, 8192, 2048
    gen = torch.Generator(device=device).manual_seed(99)
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
    return scores, ends, outs, k, B * S * T * 4 + B * S * k * 4


def bench_topk(args, device, order: str = "index"):
    from cppmega_mlx_amd.nn._tilelang import topk_selector as tk

    scores, ends, outs, k, bytes_alg = topk_inputs(device)
    t = timed_graph([lambda i=i: tk.topk_selector_tilelang_direct(scores[i], k, out=outs[i], ends=ends, order=order)
                     for i in range(len(scores))], max(args.steps, 30), args.warmup)
    what = "topk_selector scores fp32[4,1024,8192] (5% ties, causal bounds) -> int32[4,1024,2048]"
    if order == "value":
        what += ", value-descending output"
    res = hbm_row(what, t, bytes_alg, "topk_selector" if order == "index" else "topk_selector_value_order")
    return res, (scores[0], ends, outs[0], k)


def topk_sample_exact(sample, order: str = "index", check: int = 256) -> bool:
    """The first `check` rows of the GPU selection against the oracle: the same indices in the same
    order (index order), or the same set (value order: ties among equal values may be listed in either order)."""
    from oracle import topk as ot

    scores, ends, out, k = sample
    want = ot.topk_selector_oracle(scores[:check].cpu().numpy(), k, ends=ends[:check].cpu().numpy())
    got = out[:check].cpu().numpy()
    if order == "index":
        return bool(np.array_equal(got, want))
    return bool(np.array_equal(np.sort(got, axis=-1), np.sort(want, axis=-1)))


def bench_topk_wide(args, device):
    """The decode-time shape: one row per sequence over the whole cache (two-stage selection, and one
    workgroup per row for comparison)."""
    from cppmega_mlx_amd import ops
    gen = torch.Generator(device=device).manual_seed(199)
    k = 2048
    wide = [torch.randn((32, 65536), generator=gen, device=device) for _ in range(3)]
    wide_out = torch.empty((32, k), dtype=torch.int32, device=device)
    res = {}
    for name, two_stage in (("two_stage", True), ("one_workgroup_per_row", False)):
        t = timed_graph([lambda i=i: ops.topk_select(wide[i], k, out=wide_out, two_stage=two_stage) for i in range(3)],
                        max(args.steps, 30), args.warmup)
        res[name] = hbm_row("topk_selector scores fp32[32,65536] -> int32[32,2048]", t, 32 * 65536 * 4 + 32 * k * 4)
    return res


def cpu_baseline_topk(sample, rows: int = 4096):
    from oracle import torch_cpu

    scores, ends, out, k = sample
    threads = host_threads()
    st, et = scores[:rows].cpu(), ends[:rows].cpu()
    dt, reps = repeat_timed(lambda: torch_cpu.topk_fallback(st, k, ends=et), 8.0)
    nbytes = rows * (scores.shape[1] * 4 + k * 4)
    return {"value": sig(nbytes / dt / 1e9), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"fp32 torch stable-sort selection (the reference's argsort fallback) on {rows} of 4096 rows, "
                      f"{reps} passes of {dt:.3f} s; {host_description(threads)}"}


def bench_prefill(args, device, pow2: bool):
    """C5: causal prefill over the FP8 latent cache; sampled queries are checked against the oracle."""
    from cppmega_mlx_amd.nn._tilelang import sparse_mla_blockscaled_path_c as bs, topk_selector as tk
    from oracle import sparse_mla as om

    S, H, topk = 8192, 128, 2048
    gen = torch.Generator(device=device).manual_seed(555)
    codes, scale, rope = make_latent_cache(gen, 1, S, device, pow2=pow2)
    q = torch.randn((1, S, H, 576), generator=gen, device=device).to(torch.bfloat16)
    idx_scores = torch.randn((S, S), generator=gen, device=device)
    ends = torch.arange(1, S + 1, device=device, dtype=torch.int32)
    idx = torch.empty((S, topk), dtype=torch.int32, device=device)
    tk.topk_selector_tilelang_direct(idx_scores, topk, out=idx, ends=ends, order="index")
    del idx_scores
    idx = idx.view(1, S, 1, topk)
    out = torch.empty((1, S, H, 512), dtype=torch.bfloat16, device=device)
    lse = torch.empty((1, S, H), dtype=torch.float32, device=device)
    fn = lambda: bs.sparse_mla_blockscaled_path_c_apply_direct(q, None, codes, scale, idx, sm_scale=576 ** -0.5, out=out,
                                                               lse=lse, d_v=512, kv_rope=rope)
    t = timed_graph([fn], max(1, min(args.steps, 5)), 1, replays=5)
    pairs = int(torch.minimum(ends.long(), torch.tensor(topk, device=device)).sum().item())
    flops = 2.0 * H * pairs * (576 + 512)
    row = mfma_row("sparse_mla_prefill B=1 S=8192 H=128 topk=2048 causal, latent e4m3+fp32/128+bf16 rope, "
                   + ("power-of-two block scales" if pow2 else "general fp32 block scales (amax/448)") + "; FLOPs of valid pairs",
                   t, flops, "sparse_mla_prefill" if not pow2 else "sparse_mla_prefill_pow2_scales")
    rows_all = om.dequant_block_latent(codes.cpu().numpy(), scale.cpu().numpy(), rope.float().cpu().numpy(), 128)
    idx_np = idx.cpu().numpy().astype(np.int64)
    err = 0.0
    for s in (0, 33, 2047, 5000, S - 1):
        want, _ = om.sparse_mla_oracle(q[:, s:s + 1].float().cpu().numpy(), rows_all, idx_np[:, s:s + 1], sm_scale=576 ** -0.5, d_v=512)
        err = max(err, float(np.abs(out[:, s:s + 1].float().cpu().numpy() - want).max() / np.abs(want).max()))
    row["max_rel_err_vs_oracle_on_sample"] = sig(err)
    return row


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
        t = timed_graph([fn], steps, 1, replays=5)
        res[name] = mfma_row(f"sparse_mla_prefill {what} B=1 S=8192 H=128 topk=2048 causal; FLOPs of valid pairs", t, flops)

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
    t = timed_graph([lambda: dst.copy_(src)], args.steps, args.warmup)
    per = t["median"]
    return {"workload": "torch copy_ of 256 MiB (u8)", "bytes_read": n, "bytes_written": n, "us": sig(per * 1e6),
            "gbs": sig(2.0 * n / per / 1e9)}


def bench_next_rows(args, device):
    """The rows either side of the attention call: the fused producer + cache append for a
    prefill chunk (8192 latent rows of 512 + 64 rope channels) and for one decode step (32 rows),
    and the two index producers at prefill size.  HBM-bound; bytes are algorithmic."""
    from cppmega_mlx_amd import ops
    gen = torch.Generator(device=device).manual_seed(99)
    res = {}
    steps = max(args.steps, 30)

    def hbm(name, fn, nbytes, workload):
        res[name] = hbm_row(workload, timed_graph([fn], steps, args.warmup), nbytes)

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
    t = timed_graph([lambda: ops.sparse_mla_backward(q, kv, d_out, idx, sm_scale=D ** -0.5, d_v=d_v, dq=dq, dkv=dkv)], steps, args.warmup)
    flops = 2.0 * B * S * H * topk * (3 * D + 2 * d_v)
    res["sparse_mla_backward"] = mfma_row(
        f"sparse_mla_bwd q bf16[{B},{S},{H},{D}] kv bf16[{B},{Skv},1,{D}] topk {topk} -> dq bf16, dkv f32 (atomic adds)", t, flops, unit_ms=False)
    res["sparse_mla_backward"].update({"float32_atomic_adds": B * S * topk * D,
                                       "atomic_add_floor_us": sig(B * S * topk * D / (128 * 2.4e9) * 1e6)})

    # the same backward over per-token FP8 operands (e4m3 code values + float32 scale per token)
    q8 = (torch.randn((B, S, H, D), generator=gen, device=device) * 64).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    kv8 = (torch.randn((B, Skv, 1, D), generator=gen, device=device) * 64).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    qs = torch.rand((B, S, H), generator=gen, device=device) * 0.02 + 0.005
    kvs = torch.rand((B, Skv, 1), generator=gen, device=device) * 0.02 + 0.005
    dq32 = torch.empty((B, S, H, D), dtype=torch.float32, device=device)
    t = timed_graph([lambda: ops.sparse_mla_backward(q8, kv8, d_out, idx, sm_scale=D ** -0.5, d_v=d_v, dq=dq32, dkv=dkv,
                                                     q_scale=qs, kv_scale=kvs)], steps, args.warmup)
    res["sparse_mla_backward_fp8"] = mfma_row(
        f"sparse_mla_bwd q e4m3[{B},{S},{H},{D}] + f32 scale per token, kv e4m3[{B},{Skv},1,{D}] + f32 scale per token, "
        f"d_out bf16, topk {topk} -> dq f32, dkv f32 (atomic adds)", t, flops, unit_ms=False)

    # DSA indexer KL loss (training side): one launch over every (batch, query position)
    ASq = Sk = 4096; AB, AH, AD, topk = 1, 8, 64, 1024
    qq = torch.randn((ASq, AB, AH, AD), generator=gen, device=device).to(torch.bfloat16)
    kk = torch.randn((Sk, AB, AH, AD), generator=gen, device=device).to(torch.bfloat16)
    isc = torch.randn((AB, ASq, Sk), generator=gen, device=device)
    top = torch.topk(isc, topk, dim=-1).indices.to(torch.int32).contiguous()
    loss = torch.empty((AB, ASq), dtype=torch.float32, device=device)
    for name, lst in (("dsa_indexer_loss_dense", None), ("dsa_indexer_loss_sparse", top)):
        t = timed_graph([lambda: ops.dsa_indexer_loss(qq, kk, isc, softmax_scale=AD ** -0.5, out=loss, topk_indices=lst)], steps, args.warmup)
        flops = 2.0 * AB * AH * AD * (ASq * (ASq + 1) / 2)
        res[name] = mfma_row(
            f"dsa_indexer_loss query/key bf16[{ASq},{AB},{AH},{AD}] index_scores f32[{AB},{ASq},{Sk}]"
            + (f" topk_indices i32[{AB},{ASq},{topk}]" if lst is not None else "") + " -> loss f32", t, flops, unit_ms=False)
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
# The profiler runs whose CSV output `--summarise-profiles DIR` turns into profiles/*.md and
# profiles/traffic.json.  Each is run from /tmp (`cd /tmp && export TMPDIR=/tmp`) with DIR as below.
# Kernels that serve several configurations under one name (the latent kernel: decode and prefill,
# either scale kind; the selector: either output order) get a run per configuration.
_MAIN = "decode_general,vecmat,vecmat_m32,vecmat_fp8x,topk,topk_wide,copy,next,prefill_rows"
_TRACE = "rocprofv3 --kernel-trace --stats --output-format csv -d DIR/{0} -o t -- python3 bench.py --only {1} --steps {2} --replays 3 --no-cpu-baseline"
_PMC = "rocprofv3 --pmc {3} --output-format csv -d DIR/{0} -o c -- python3 bench.py --only {1} --steps {2} --warmup 1 --replays 1 --no-cpu-baseline"
_SQ = ("SQ_WAVE_CYCLES SQ_BUSY_CYCLES SQ_INSTS_VALU SQ_INSTS_MFMA SQ_VALU_MFMA_BUSY_CYCLES SQ_ACTIVE_INST_VALU "
       "SQ_WAIT_INST_ANY SQ_ACTIVE_INST_LDS")
PROFILE_RUNS = {
    "trace_main": _TRACE.format("trace_main", _MAIN, 20),
    "trace_alt": _TRACE.format("trace_alt", "decode_pow2,topk_value", 20),
    "trace_prefill": _TRACE.format("trace_prefill", "prefill_general", 3),
    "trace_prefill_pow2": _TRACE.format("trace_prefill_pow2", "prefill_pow2", 3),
    "fetch_main": _PMC.format("fetch_main", _MAIN, 3, "FETCH_SIZE"),
    "write_main": _PMC.format("write_main", _MAIN, 3, "WRITE_SIZE"),
    "fetch_prefill": _PMC.format("fetch_prefill", "prefill_general,copy", 2, "FETCH_SIZE"),
    "write_prefill": _PMC.format("write_prefill", "prefill_general,copy", 2, "WRITE_SIZE"),
    "sq_decode": _PMC.format("sq_decode", "decode_general", 3, _SQ),
    "sq_prefill": _PMC.format("sq_prefill", "prefill_general", 2, _SQ),
}
# summary file -> (trace run, (fetch run, write run) or None, SQ run or None, kernel-name fragments, workload text
#                  [, grid size in threads: only dispatches of that size count])
PROFILE_WORKLOADS = [
    ("sparse_mla_decode", "trace_main", ("fetch_main", "write_main"), "sq_decode", ("sparse_mla_latent",),
     "decode B=32 S_q=1 H=128 topk=2048 Skv=65536 (e4m3 latent + general fp32/128 scales (amax/448) + bf16 rope)"),
    ("sparse_mla_decode_pow2_scales", "trace_alt", None, None, ("sparse_mla_latent",),
     "decode B=32 S_q=1 H=128 topk=2048 Skv=65536 (e4m3 latent + power-of-two fp32/128 scales + bf16 rope)"),
    ("sparse_mla_prefill", "trace_prefill", ("fetch_prefill", "write_prefill"), "sq_prefill", ("sparse_mla_latent",),
     "causal prefill B=1 S=8192 H=128 topk=2048 (e4m3 latent + general fp32/128 scales (amax/448) + bf16 rope)"),
    ("sparse_mla_prefill_pow2_scales", "trace_prefill_pow2", None, None, ("sparse_mla_latent",),
     "causal prefill B=1 S=8192 H=128 topk=2048 (e4m3 latent + power-of-two fp32/128 scales + bf16 rope)"),
    ("fp8_vecmat", "trace_main", ("fetch_main", "write_main"), None, ("gemv_stream_kernel<1, 4, 4, 0>",),
     "W e4m3[7168,16384] + fp32 scale/128, x bf16[1,16384]"),
    ("fp8_vecmat_e4m3_activation", "trace_main", ("fetch_main", "write_main"), None, ("gemv_stream_kernel<1, 4, 4, 1>",),
     "W e4m3[7168,16384] + fp32 scale per row, x e4m3[16384] + fp32 scale -> f32[7168] (the reference's own vecmat form)"),
    ("fp8_vecmat_m4", "trace_main", ("fetch_main", "write_main"), None, ("gemv_stream_kernel<4",),
     "W e4m3[7168,16384] + fp32 scale/128, x bf16[4,16384]"),
    ("fp8_vecmat_m16", "trace_main", ("fetch_main", "write_main"), None, ("skinny_rows_kernel<1",),
     "W e4m3[7168,16384] + fp32 scale/128, x bf16[16,16384] (one kernel, no K split, no workspace)"),
    ("fp8_vecmat_m32", "trace_main", ("fetch_main", "write_main"), None, ("skinny_mfma_kernel<2>", "skinny_reduce"),
     "W e4m3[7168,16384] + fp32 scale/128, x bf16[32,16384] (split-K kernel + reduce kernel)"),
    ("topk_selector", "trace_main", ("fetch_main", "write_main"), None, ("topk_tile_kernel<float, 16, 4, 512, 0,",),
     "scores fp32[4096 rows,8192] -> int32[4096,2048], indices in ascending order (the dispatches of 4096 workgroups only: "
     "the same kernel also selects for the indexer and for the prefill rows of the same run)", 4096 * 512),
    ("topk_selector_value_order", "trace_alt", None, None, ("topk_tile_kernel<float, 16, 4, 512, 0,",),
     "scores fp32[4096 rows,8192] -> int32[4096,2048], indices by descending value (same kernel, sorted in LDS)", 4096 * 512),
    ("topk_selector_decode_shape", "trace_main", ("fetch_main", "write_main"), None,
     ("topk_tile_kernel<float, 16, 4, 512, 1,", "topk_tile_kernel<float, 16, 4, 1024, 2,", "topk_wide_kernel"),
     "scores fp32[32,65536] -> int32[32,2048]: the two-stage path (segment kernel, then candidate kernel) and, for "
     "comparison, the one-workgroup-per-row kernel; the indexer's decode row runs the two-stage kernels as well"),
    ("indexer_scores_topk", "trace_main", ("fetch_main", "write_main"), None, ("indexer_scores_kernel", "indexer_qw_"),
     "indexer_topk q bf16[B,Sq,64,128], k bf16[B,Skv,128]: prefill (1, 8192, 8192) and decode (32, 1, 65536) dispatches"),
    ("mla_absorb_head_gemm", "trace_main", ("fetch_main", "write_main"), None, ("head_gemm_kernel",),
     "head_gemm x bf16[32,128,128] . W bf16[128,512,128] and x bf16[32,128,512] . W bf16[128,128,512]"),
    ("kv_cache_append", "trace_main", ("fetch_main", "write_main"), None, ("cache_append_kernel",),
     "bf16 latent[B,S,1,512] + rope[..,64] -> e4m3 + fp32/128 scales + bf16 rope in the cache: one dispatch of 8192 rows "
     "(prefill chunk) and one of 32 rows (decode step) per step"),
    ("sparse_mla_prefill_row_layouts", "trace_main", ("fetch_main", "write_main"), None, ("sparse_mla_mfma_kernel<",),
     "sparse_mla_fwd q [1,8192,128,576], kv [1,8192,1,576], causal top-2048 indices -> [1,8192,128,512] on the 32-head tile kernel, "
     "four wavefronts sharing one key stream: <false, true, true, 0> unquantised float16 rows, <true, false, true, 1> e4m3 rows "
     "with per-token fp32 scales, <true, false, true, 2> e4m3 rows with E8M0 bytes per 32 channels"),
    ("sparse_mla_backward", "trace_main", ("fetch_main", "write_main"), None, ("sparse_mla_bwd", "fill_zero_kernel"),
     "sparse_mla_bwd q bf16[1,1024,16,576], kv bf16[1,4096,1,576], d_out bf16[1,1024,16,512], topk 256 -> dq bf16, dkv f32 "
     "(the dkv clear, then the matrix-core kernel with its float32 atomic adds)"),
    ("dsa_indexer_loss", "trace_main", ("fetch_main", "write_main"), None, ("dsa_indexer_loss",),
     "dsa_indexer_loss query / key bf16[4096,1,8,64], index_scores f32[1,4096,4096]: one dense and one sparse "
     "(topk_indices i32[1,4096,1024]) dispatch per step"),
    ("sparse_index_producers", "trace_main", ("fetch_main", "write_main"), None, ("_indices_",),
     "causal_sparse_indices(1,8192,1,2048) and sparse_indices_from_attention_mask(bool [8192,8192], topk 2048)"),
]


def summarise_profiles(src: str) -> int:
    """Write profiles/*.md and profiles/traffic.json from the CSV output of PROFILE_RUNS under `src`.
    Fails (exit status 5) when a listed workload matches no kernel of its trace run."""
    import collections
    import csv

    here = os.path.dirname(os.path.abspath(__file__))
    out_dir = os.path.join(here, "profiles")
    os.makedirs(out_dir, exist_ok=True)

    def rows(rel):
        with open(os.path.join(src, rel)) as fh:
            return list(csv.DictReader(fh))

    stats_cache, counter_cache = {}, {}

    def stats_of(run):
        if run not in stats_cache:
            stats_cache[run] = {r["Name"]: r for r in rows(f"{run}/t_kernel_stats.csv")}
        return stats_cache[run]

    def counters_of(run):
        if run not in counter_cache:
            agg = collections.defaultdict(lambda: collections.defaultdict(list))
            for r in rows(f"{run}/c_counter_collection.csv"):
                agg[r["Kernel_Name"]][r["Counter_Name"]].append(float(r["Counter_Value"]))
            counter_cache[run] = agg
        return counter_cache[run]

    copy_kib = 262144.0                                    # the 256 MiB device copy of bench_copy, each way

    def copy_scale(run, counter):
        vals = counters_of(run).get("__amd_rocclr_copyBuffer", {}).get(counter)
        if not vals:
            raise SystemExit(f"{run}: no {counter} value for the device copy")
        return copy_kib / max(vals), max(vals)

    def cmd(key):
        return "`cd /tmp && export TMPDIR=/tmp && " + PROFILE_RUNS[key].replace("DIR", "$GRAFT_REPO_ROOT/gpurun_out").replace(
            "bench.py", "$GRAFT_REPO_ROOT/bench.py") + "`"

    def short(name):
        return name.replace("(anonymous namespace)::", "")

    trace_cache = {}

    def dispatch_stats(run, name, grid):
        """Calls / average / min / max (ns) over the dispatches of `name` with `grid` threads."""
        if run not in trace_cache:
            trace_cache[run] = rows(f"{run}/t_kernel_trace.csv")
        ns = [float(r["End_Timestamp"]) - float(r["Start_Timestamp"]) for r in trace_cache[run]
              if r["Kernel_Name"] == name and int(r["Grid_Size_X"]) == grid]
        if not ns:
            return None
        return {"Calls": str(len(ns)), "AverageNs": sum(ns) / len(ns), "MinNs": min(ns), "MaxNs": max(ns)}

    def counters_by_grid(run, grid):
        agg = collections.defaultdict(lambda: collections.defaultdict(list))
        for r in rows(f"{run}/c_counter_collection.csv"):
            if int(r["Grid_Size"]) == grid:
                agg[r["Kernel_Name"]][r["Counter_Name"]].append(float(r["Counter_Value"]))
        return agg

    traffic, missing = {}, []
    for entry in PROFILE_WORKLOADS:
        fname, trace_run, pmc_runs, sq_run, frags, workload = entry[:6]
        grid = entry[6] if len(entry) > 6 else None
        stats = stats_of(trace_run)
        names = [n for n in stats if "cm::" in n and any(f in n for f in frags)]
        if grid is not None:
            stats = {n: dispatch_stats(trace_run, n, grid) for n in names}
            names = [n for n in names if stats[n]]
        if not names:
            missing.append(fname)
            continue
        text = [f"# rocprofv3 summary: {fname}", "", f"Workload: {workload} (one MI355X, synthetic inputs resident in HBM).", "",
                "## Kernel durations (`--kernel-trace --stats`)", "", "Command: " + cmd(trace_run), "",
                "| kernel | calls | avg us | min us | max us |", "|---|---|---|---|---|"]
        for n in names:
            r = stats[n]
            text.append("| `%s` | %s | %.2f | %.2f | %.2f |" % (short(n), r["Calls"], float(r["AverageNs"]) / 1e3,
                                                              float(r["MinNs"]) / 1e3, float(r["MaxNs"]) / 1e3))
        if pmc_runs:
            fetch, write = counters_of(pmc_runs[0]), counters_of(pmc_runs[1])
            if grid is not None:
                fetch, write = counters_by_grid(pmc_runs[0], grid), counters_by_grid(pmc_runs[1], grid)
            (scale_f, copy_f), (scale_w, copy_w) = copy_scale(pmc_runs[0], "FETCH_SIZE"), copy_scale(pmc_runs[1], "WRITE_SIZE")
            text += ["", "## HBM traffic per dispatch (`--pmc FETCH_SIZE`, then `--pmc WRITE_SIZE`, KiB)", "",
                     "Commands: " + cmd(pmc_runs[0]) + " and " + cmd(pmc_runs[1]) + ".", "",
                     "Scale factors from the 256 MiB device copy in the same runs (`__amd_rocclr_copyBuffer`, 262144 KiB each way): "
                     "FETCH_SIZE read %.1f KiB -> x%.3f, WRITE_SIZE read %.1f KiB -> x%.3f." % (copy_f, scale_f, copy_w, scale_w), "",
                     "| kernel | FETCH_SIZE KiB | WRITE_SIZE KiB | scaled read MiB | scaled write MiB |", "|---|---|---|---|---|"]
            total = 0.0
            for n in names:
                fv, wv = fetch.get(n, {}).get("FETCH_SIZE", []), write.get(n, {}).get("WRITE_SIZE", [])
                f = sum(fv) / len(fv) if fv else 0.0
                w = sum(wv) / len(wv) if wv else 0.0
                text.append("| `%s` | %.1f | %.1f | %.1f | %.1f |" % (short(n), f, w, f * scale_f / 1024, w * scale_w / 1024))
                total += (f * scale_f + w * scale_w) * 1024
            if total <= 0:
                missing.append(fname + " (no counter rows)")
            traffic[fname] = {"hbm_bytes_per_launch": int(total), "kernels": names}
        if sq_run and os.path.exists(os.path.join(src, f"{sq_run}/c_counter_collection.csv")):
            sq = {}
            for n, cs in counters_of(sq_run).items():
                if "sparse_mla_latent_kernel" in n:
                    sq = {k: sum(v) / len(v) for k, v in cs.items()}
            text += ["", "## SQ counters of the main kernel (one `--pmc` pass, average per dispatch, summed over its wavefronts)", "",
                     "Command: " + cmd(sq_run), "", "| counter | value |", "|---|---|"]
            for k in sorted(sq):
                text.append("| %s | %.0f |" % (k, sq[k]))
            if sq.get("SQ_WAVE_CYCLES"):
                text += ["", "SQ_VALU_MFMA_BUSY_CYCLES / (4 x SQ_WAVE_CYCLES) = %.3f: the matrix-core busy fraction of the wavefronts' "
                         "lifetime (wave cycles count in units of 4 clocks)." % (sq.get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0) / (4 * sq["SQ_WAVE_CYCLES"]))]
        with open(os.path.join(out_dir, fname + ".md"), "w") as fh:
            fh.write("\n".join(text) + "\n")
    with open(os.path.join(out_dir, "traffic.json"), "w") as fh:
        json.dump({"workloads": traffic}, fh, indent=1)
    if missing:
        print("summarise-profiles: no kernel rows for: " + ", ".join(missing), file=sys.stderr)
        return 5
    print(f"wrote {len(PROFILE_WORKLOADS)} summaries and traffic.json to {out_dir}")
    return 0


DEFAULT_PARTS = "decode,vecmat,topk,prefill"
REL_TOL = 2e-2                                               # max-abs error over the oracle's output scale


def main() -> int:
    global REPLAYS
    ap = argparse.ArgumentParser()
    ap.add_argument("--summarise-profiles", metavar="DIR", default=None,
                    help="no GPU work: turn the rocprofv3 CSVs under DIR (see PROFILE_RUNS) into profiles/*.md and profiles/traffic.json")
    ap.add_argument("--print-profile-commands", action="store_true", help="no GPU work: print PROFILE_RUNS, one command per line")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--replays", type=int, default=7, help="timed replays of the captured steps; rows report the median and the fastest")
    ap.add_argument("--only", type=str, default=DEFAULT_PARTS)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.summarise_profiles:
        return summarise_profiles(args.summarise_profiles)
    if args.print_profile_commands:
        for k, v in PROFILE_RUNS.items():
            print(k + "\t" + v)
        return 0
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU; the path shards without communication "
              "(rows / sequences / queries per GPU), so --gpus N>1 is not run here.", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP kernels have no CPU path.", file=sys.stderr)
        return 3
    REPLAYS = max(1, args.replays)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    from cppmega_mlx_amd import native_status
    native_status()
    parts = set(args.only.split(","))
    cpu = not args.no_cpu_baseline
    failed = []

    line = {
        "metric": "sparse_mla_decode_tflops",
        "value": None,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "replays": REPLAYS,
        "ms_per_step": None,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {},
    }

    def decode_row(res):
        t = res["t"]
        return {"ms_per_step": sig(t["median"] * 1e3), "min_ms_per_step": sig(t["min"] * 1e3),
                "tflops": sig(res["flops"] / t["median"] / 1e12), "frac": sig(res["flops"] / t["median"] / 1e12 / MFMA_BF16_PEAK_TFLOPS)}

    if parts & {"decode", "decode_general", "decode_pow2"}:
        pow2_row = None
        if parts & {"decode", "decode_pow2"}:
            res_pow2, sample = bench_decode(args, device, pow2=True)
            pow2_row = decode_row(res_pow2)
            pow2_row["max_rel_err_vs_oracle_on_sample"] = sig(decode_sample_error(sample, (0,)))
            if pow2_row["max_rel_err_vs_oracle_on_sample"] > REL_TOL:
                failed.append("decode (power-of-two scales)")
            del sample
            torch.cuda.empty_cache()
        if parts & {"decode", "decode_general"}:
            res, sample = bench_decode(args, device, pow2=False)
            t = res["t"]
            tfl = res["flops"] / t["median"] / 1e12
            line["value"] = sig(tfl, 5)
            line["ms_per_step"] = sig(t["median"] * 1e3, 5)
            line["config"] = {"workload": res["workload"], "kernel": res["kernel"], "flops_per_step": res["flops"],
                              "algorithmic_bytes_per_step": res["bytes"], "min_ms_per_step": sig(t["min"] * 1e3),
                              "max_ms_per_step": sig(t["max"] * 1e3), "host_ms_per_step": sig(t["host"] * 1e3),
                              "hbm_gbs": sig(res["bytes"] / t["median"] / 1e9)}
            line["roofline"] = {"bound": "mfma", "achieved": sig(tfl), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                "frac": sig(tfl / MFMA_BF16_PEAK_TFLOPS), "traffic": measured_traffic("sparse_mla_decode")}
            err = decode_sample_error(sample)
            line["config"]["max_rel_err_vs_oracle_on_sample"] = sig(err)
            if err > REL_TOL:
                failed.append("decode")
            if cpu:
                line["cpu_baseline"] = cpu_baseline_decode(sample)
            del sample
            torch.cuda.empty_cache()
        if pow2_row is not None:
            if line["config"]:
                line["config"]["power_of_two_block_scales"] = pow2_row
            else:
                line["decode_pow2"] = pow2_row
    vec = {}
    for M, part in ((1, "vecmat"), (4, "vecmat"), (16, "vecmat"), (32, "vecmat_m32")):
        if part not in parts:
            continue
        res, sample = bench_vecmat(args, device, M)
        res["max_rel_err_vs_oracle_on_sample"] = sig(vecmat_sample_error(sample))
        if res["max_rel_err_vs_oracle_on_sample"] > REL_TOL:
            failed.append(f"vecmat M={M}")
        if cpu and M == 1:
            res["cpu_baseline"] = cpu_baseline_vecmat(sample)
        vec[f"M{M}"] = res
        del sample
        torch.cuda.empty_cache()
    if "vecmat_fp8x" in parts:
        vec["M1_fp8x"] = bench_vecmat_fp8x(args, device)
        torch.cuda.empty_cache()
    if vec:
        line["vecmat"] = vec
    for part, order, key in (("topk", "index", "topk"), ("topk_value", "value", "topk_value_order")):
        if part not in parts:
            continue
        res, sample = bench_topk(args, device, order)
        res["bit_exact_vs_oracle_on_sample"] = topk_sample_exact(sample, order)
        if not res["bit_exact_vs_oracle_on_sample"]:
            failed.append(key)
        if cpu and order == "index":
            res["cpu_baseline"] = cpu_baseline_topk(sample)
        line[key] = res
        del sample
        torch.cuda.empty_cache()
    if "topk_wide" in parts:
        line["topk_decode_shape"] = bench_topk_wide(args, device)
        torch.cuda.empty_cache()
    if parts & {"prefill", "prefill_general", "prefill_pow2"}:
        row = None
        if parts & {"prefill", "prefill_general"}:
            row = bench_prefill(args, device, pow2=False)
            if row["max_rel_err_vs_oracle_on_sample"] > REL_TOL:
                failed.append("prefill")
            torch.cuda.empty_cache()
        if parts & {"prefill", "prefill_pow2"}:
            p2 = bench_prefill(args, device, pow2=True)
            if p2["max_rel_err_vs_oracle_on_sample"] > REL_TOL:
                failed.append("prefill (power-of-two scales)")
            if row is None:
                row = p2
            else:
                row["power_of_two_block_scales"] = {k: p2[k] for k in ("ms_per_step", "min_ms_per_step", "max_rel_err_vs_oracle_on_sample")}
                row["power_of_two_block_scales"]["frac"] = p2["roofline"]["frac"]
            torch.cuda.empty_cache()
        line["prefill"] = row
    if "prefill_rows" in parts:
        line["prefill_row_layouts"] = bench_prefill_rows(args, device)
    if "copy" in parts:
        line["copy"] = bench_copy(args, device)
    if "next" in parts:
        line["next_rows"] = bench_next_rows(args, device)
    line["self_checks"] = "failed: " + ", ".join(failed) if failed else "passed"
    print(json.dumps(line, separators=(",", ":")))
    if failed:
        print("bench.py: parity check failed for " + ", ".join(failed), file=sys.stderr)
        return 4
    return 0


if __name__ == "__main__":
    sys.exit(main())
