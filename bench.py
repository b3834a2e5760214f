#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: each workload of the benchmark definition run through
the C-ABI library on synthetic, HBM-resident inputs, timed with HIP events on the launch stream.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workloads gdn,moe_decode,mla,moe_prefill]
                    [--no-cpu-baseline]

Prints ONE JSON line. The headline (`metric`/`value`/`roofline`/`cpu_baseline`) is workload
configs[1], the batched GDN decode step; the other single-GPU workloads are reported under
`workloads` with the same fields. A "step" is one launch of the operator on one batch.

Algorithmic work per launch (what `roofline.achieved` is computed from):
  gdn          2*B*Hv*dk*dv*4 (state read + write) + q,k,v,g,beta,o        = 1 082 195 968 B
  moe_decode   n_active*(44 040 192 + 10 752) + x + logits + out           (n_active measured)
  mla          B*topk*576*2 gathered bytes                                  =   150 994 944 B
  moe_prefill  T*8*(2*H*2I + 2*I*H) flop                                    = 5.772e12 flop
Inputs that fit the 256 MB last-level cache are rotated over several sets so that repeated steps
do not read from cache what the workload would read from HBM.
"""

import argparse
import json
import os
import sys
import time
from pathlib import Path

REPO = Path(__file__).resolve().parent
if str(REPO) not in sys.path:
    sys.path.insert(0, str(REPO))

HBM_PEAK_GBS = 8000.0
FP8_PEAK_TFLOPS = 5033.0
METRIC = "GB/s & % HBM peak (GDN/MoE/MLA decode); fp8 TFLOP/s % MFMA peak (MoE prefill)"

# HBM bytes per step (summed over the workload's kernels) from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled
# by the same counters read on a plain 512 MiB copy kernel (FETCH_SIZE x 1.99986, WRITE_SIZE x 1,
# both in KiB); the counter summary is profiles/all_workloads_hbm_traffic_pmc.md, whose "HBM bytes" column
# holds each of these figures (a test checks that). None = not measured.
# Stamp: taken from the library as built from the sources of this tree; a change to a kernel's data movement needs
# a new run of the two commands in that file.
MEASURED_TRAFFIC = {'gdn': 1085858000, 'moe_decode': 10002073000, 'mla': 238270000, 'index_scores': 553927000,
                    'index_scores_fp8': 289777000, 'moe_prefill': 22426952000, 'mla_fp8_cache': 187610000,
                    'topk_select': 9216000}
# Matrix-pipe occupancy of the dominant kernels from rocprofv3 --pmc (SQ_VALU_MFMA_BUSY_CYCLES over 1024 SIMDs x
# GRBM_GUI_ACTIVE cycles per XCD, the timed launches of bench.py's own loop; the derived MfmaUtil counter reads
# 33.3 / 33.7 / 23.5 %) and the clock by GRBM_GUI_ACTIVE / 8 / duration in the same run (SQ_BUSY_CU_CYCLES / 256 /
# duration for the short sparse-MLA kernel); the summary is profiles/moe_prefill_mla_matrix_core_counters_pmc.md.
# Measured figures of that run, not of this one.
MEASURED_MFMA = {
    'moe_prefill': dict(mfma_busy=0.343, clock_ghz=1.97, kernel='moe_tiled_gemm_kernel<true> (gate/up)',
                        mfma_busy_down=0.345, clock_ghz_down=1.84),
    'mla': dict(mfma_busy=0.241, clock_ghz=2.05, kernel='sparse_mla_split8_kernel<false>'),
}


SETTLE_SECONDS = 0.05


def timed_launches(torch, launch, steps, warmup):
    """Average device time of one launch in seconds, HIP events on the current (launch) stream.

    Before the `warmup` untimed steps the same launch is repeated for about SETTLE_SECONDS, untimed:
    the first few milliseconds of work after the inputs were generated run at lower clocks (the first
    workload of a process measured 5-6 % low without it).
    """
    launch(0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n = 0
    while time.perf_counter() - t0 < SETTLE_SECONDS:
        launch(n)
        n += 1
        if n % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        launch(warmup + i)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / steps


def cpu_time(fn, min_seconds=3.0, max_iters=5):
    fn()  # warm-up
    t0 = time.perf_counter()
    n = 0
    while n < max_iters and (n == 0 or time.perf_counter() - t0 < min_seconds):
        fn()
        n += 1
    return (time.perf_counter() - t0) / n


def bench_gdn(torch, capi, dev, steps, warmup, cpu_baseline):
    from oracle import gdn
    B, Hv, Hqk = 256, 32, 16
    gen = torch.Generator(device=dev).manual_seed(20251)
    sets = []
    for _ in range(3):  # 3 x 537 MB of state: each step streams a set the cache no longer holds
        q = torch.randn(B, Hqk, 128, device=dev, generator=gen)
        k = torch.randn(B, Hqk, 128, device=dev, generator=gen)
        q = (q / q.norm(dim=-1, keepdim=True)).bfloat16()
        k = (k / k.norm(dim=-1, keepdim=True)).bfloat16()
        v = torch.randn(B, Hv, 128, device=dev, generator=gen).bfloat16()
        g = torch.exp(-0.5 * torch.log1p(torch.exp(torch.randn(B, Hv, device=dev, generator=gen))))
        beta = torch.sigmoid(torch.randn(B, Hv, device=dev, generator=gen))
        state = 0.02 * torch.randn(B, Hv, 128, 128, device=dev, generator=gen)
        o = torch.empty(B, Hv, 128, device=dev)
        sets.append((o, state, q, k, v, g, beta))
    sec = timed_launches(torch, lambda i: capi.gdn_decode_launch(*sets[i % 3]), steps, warmup)
    work = 2 * B * Hv * 128 * 128 * 4 + 2 * B * Hqk * 128 * 2 + B * Hv * 128 * 2 + 2 * B * Hv * 4 + B * Hv * 128 * 4
    res = dict(
        workload="configs[1]: GDN batched decode B=256, Hv=32/Hqk=16 (GQA 2:1), dk=dv=128, bf16 q/k/v, "
                 "fp32 state 537 MB updated in place, seed 20251",
        value=work / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="f32", kernel="gdn_decode_kernel",
        roofline=dict(bound="hbm", achieved=work / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=work / sec / 1e9 / HBM_PEAK_GBS, traffic=MEASURED_TRAFFIC['gdn']),
        algorithmic_bytes=work)
    if cpu_baseline:
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
        cgen = torch.Generator().manual_seed(20251)
        ins = gdn.gdn_make_inputs(B, Hv, Hqk, qkv_dtype=torch.bfloat16, generator=cgen)
        csec = cpu_time(lambda: gdn.gdn_decode_step(*ins))
        res['cpu_baseline'] = dict(value=work / csec / 1e9, unit="GB/s", cores=cores, kind="port",
                                   sample="the full configs[1] step (eager PyTorch oracle, state in place), "
                                          "1 warm-up + up to 5 timed steps")
    return res


def bench_gdn_single(torch, capi, dev, steps, warmup, cpu_baseline):
    """configs[0]: one request, 16 heads, fp32 q/k/v: 2 MB of state, a latency measurement (no target)."""
    from oracle import gdn
    B, Hv, Hqk = 1, 16, 16
    gen = torch.Generator().manual_seed(20250)
    host = gdn.gdn_make_inputs(B, Hv, Hqk, qkv_dtype=torch.float32, generator=gen)
    q, k, v, g, beta, state0 = (t.to(dev) for t in host)
    sets = [(torch.empty(B, Hv, 128, device=dev), state0.clone()) for _ in range(3)]
    sec = timed_launches(torch, lambda i: capi.gdn_decode_launch(*sets[i % 3], q, k, v, g, beta), steps, warmup)
    work = 2 * B * Hv * 128 * 128 * 4 + 3 * B * Hv * 128 * 4 + 2 * B * Hv * 4 + B * Hv * 128 * 4
    res = dict(
        workload="configs[0]: GDN single-request decode B=1, 16 heads, dk=dv=128, fp32, seed 20250 (1 MB of state "
                 "read and written: launch latency, not bandwidth, sets the time)",
        value=work / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="f32", kernel="gdn_decode_kernel",
        roofline=dict(bound="hbm", achieved=work / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=work / sec / 1e9 / HBM_PEAK_GBS, traffic=None),
        algorithmic_bytes=work)
    if cpu_baseline:
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
        csec = cpu_time(lambda: gdn.gdn_decode_step(*host), min_seconds=1.0, max_iters=200)
        res['cpu_baseline'] = dict(value=work / csec / 1e9, unit="GB/s", cores=cores, kind="port",
                                   sample="the full configs[0] step (eager PyTorch oracle, state in place), the case "
                                          "the workload definition names as CPU-runnable")
    return res


def bench_gdn_fused_norm(torch, capi, dev, steps, warmup, cpu_baseline):
    """configs[1] sizes through the launcher that does the pre-step, the recurrence and the gated RMS
    normalisation of the read-out: the gate z is read (bf16) and the output is bf16 instead of fp32."""
    from oracle import gdn
    B, Hv, Hqk = 256, 32, 16
    gen = torch.Generator().manual_seed(20261)
    host = gdn.gdn_make_raw_inputs(B, Hv, Hqk, qkv_dtype=torch.bfloat16, generator=gen)
    hz = (torch.randn(B, Hv, 128, generator=gen) * 2).bfloat16()
    hw = (1.0 + 0.1 * torch.randn(128, generator=gen)).bfloat16()
    q, k, v, a, b, a_log, dt_bias, state0 = (t.to(dev) for t in host)
    z, norm_w = hz.to(dev), hw.to(dev)
    sets = [(torch.empty(B, Hv, 128, dtype=torch.bfloat16, device=dev), state0.clone()) for _ in range(3)]
    sec = timed_launches(
        torch, lambda i: capi.gdn_decode_fused_norm_launch(*sets[i % 3], q, k, v, a, b, a_log, dt_bias, z, norm_w),
        steps, warmup)
    work = 2 * B * Hv * 128 * 128 * 4 + 2 * B * Hqk * 128 * 2 + 3 * B * Hv * 128 * 2 + 2 * B * Hv * 4 + 2 * Hv * 4 + 256
    res = dict(
        workload="configs[1] sizes with the pre-step and the gated RMS normalisation of the read-out fused "
                 "(bf16 gate in, bf16 output), seed 20261",
        value=work / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="f32", kernel="gdn_decode_kernel<fused,norm>",
        roofline=dict(bound="hbm", achieved=work / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=work / sec / 1e9 / HBM_PEAK_GBS, traffic=None),
        algorithmic_bytes=work)
    if cpu_baseline:
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
        csec = cpu_time(lambda: gdn.gdn_decode_fused_norm_step(*host, hz, hw))
        res['cpu_baseline'] = dict(value=work / csec / 1e9, unit="GB/s", cores=cores, kind="port",
                                   sample="the full step (eager PyTorch oracle, state in place)")
    return res


def bench_gdn_fused(torch, capi, dev, steps, warmup, cpu_baseline):
    """configs[1] sizes through the launcher that also does the caller's pre-step (L2 normalisation of
    q and k, decay and write gates): same bytes, the gate inputs a, b take the place of g, beta."""
    from oracle import gdn
    B, Hv, Hqk = 256, 32, 16
    gen = torch.Generator().manual_seed(20256)
    host = gdn.gdn_make_raw_inputs(B, Hv, Hqk, qkv_dtype=torch.bfloat16, generator=gen)
    q, k, v, a, b, a_log, dt_bias, state0 = (t.to(dev) for t in host)
    sets = [(torch.empty(B, Hv, 128, device=dev), state0.clone()) for _ in range(3)]
    sec = timed_launches(
        torch, lambda i: capi.gdn_decode_fused_launch(*sets[i % 3], q, k, v, a, b, a_log, dt_bias), steps, warmup)
    work = 2 * B * Hv * 128 * 128 * 4 + 2 * B * Hqk * 128 * 2 + B * Hv * 128 * 2 + 2 * B * Hv * 4 + B * Hv * 128 * 4 \
        + 2 * Hv * 4
    res = dict(
        workload="configs[1] sizes with the pre-step fused (raw q/k normalised in the kernel, gates from a, b, "
                 "A_log, dt_bias), seed 20256",
        value=work / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="f32", kernel="gdn_decode_kernel<fused>",
        roofline=dict(bound="hbm", achieved=work / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=work / sec / 1e9 / HBM_PEAK_GBS, traffic=None),
        algorithmic_bytes=work)
    if cpu_baseline:
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
        csec = cpu_time(lambda: gdn.gdn_decode_fused_step(*host))
        res['cpu_baseline'] = dict(value=work / csec / 1e9, unit="GB/s", cores=cores, kind="port",
                                   sample="the full step (eager PyTorch oracle, state in place), 1 warm-up + up to "
                                          "5 timed steps")
    return res


def bench_conv1d(torch, capi, dev, steps, warmup, cpu_baseline):
    """The convolution update in front of the configs[1] GDN step: 256 requests, 2*2048 + 4096 channels,
    4 taps, a 4-column state per channel, bf16."""
    from oracle import gdn
    B, key_dim, value_dim, L, K = 256, 2048, 4096, 4, 4
    C = 2 * key_dim + value_dim
    gen = torch.Generator().manual_seed(20257)
    host = gdn.conv_make_inputs(B, key_dim, value_dim, L, K, torch.bfloat16, generator=gen)
    x, state0, weight, bias = (t.to(dev) for t in host)
    # 24 state copies (403 MB): one 17 MB state would be served from the cache
    states = [state0.clone() for _ in range(24)]
    q = torch.empty(B, key_dim, dtype=torch.bfloat16, device=dev)
    k = torch.empty_like(q)
    v = torch.empty(B, value_dim, dtype=torch.bfloat16, device=dev)
    sec = timed_launches(
        torch, lambda i: capi.causal_conv1d_update_launch(q, k, v, states[i % 24], x, weight, bias), steps, warmup)
    work = B * C * (2 * L + 2) * 2 + C * (K + 1) * 2
    res = dict(
        workload="single-token causal convolution update in front of configs[1]: B=256, 8192 channels, 4 taps, "
                 "4-column bf16 state, SiLU, seed 20257",
        value=work / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="f32",
        kernel="causal_conv1d_update_kernel",
        roofline=dict(bound="hbm", achieved=work / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=work / sec / 1e9 / HBM_PEAK_GBS, traffic=None),
        algorithmic_bytes=work)
    if cpu_baseline:
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
        csec = cpu_time(lambda: gdn.causal_conv1d_update(*host))
        res['cpu_baseline'] = dict(value=work / csec / 1e9, unit="GB/s", cores=cores, kind="port",
                                   sample="the full update (eager PyTorch oracle, state in place)")
    return res


def bench_router(torch, capi, dev, steps, warmup, cpu_baseline, prefill):
    """The router in front of configs[2] / configs[4]: logits = x . w^T in fp32, then group-limited routing with a
    selection bias (8 groups, 4 stay, top-8)."""
    from oracle import moe
    T, H, E, k = (8192 if prefill else 64), 7168, 256, 8
    gen = torch.Generator(device=dev).manual_seed(20260)
    x = torch.randn(T, H, device=dev, generator=gen).bfloat16()
    w = torch.randn(E, H, device=dev, generator=gen) * H ** -0.5
    bias = 0.1 * torch.randn(E, device=dev, generator=gen)
    logits = torch.empty(T, E, device=dev)
    ids = torch.empty(T, k, dtype=torch.int32, device=dev)
    wts = torch.empty(T, k, device=dev)
    nbytes = capi.moe_router_logits_workspace_bytes(T, H, E)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev) if nbytes else None

    def launch(i):
        capi.moe_router_logits_launch(logits, x, w, ws)
        capi.moe_route_grouped_launch(ids, wts, logits, bias, 8, 4, True, 2.5)

    sec = timed_launches(torch, launch, steps, warmup)
    # the same chain with the weight prepared once as three bf16 planes (projection on the bf16 matrix cores)
    planes = torch.empty(3, E, H, dtype=torch.bfloat16, device=dev)
    capi.moe_router_split_weight_launch(planes, w)

    def launch_split(i):
        capi.moe_router_logits_split_launch(logits, x, planes, ws)
        capi.moe_route_grouped_launch(ids, wts, logits, bias, 8, 4, True, 2.5)

    sec_split = timed_launches(torch, launch_split, steps, warmup)
    flops = 2 * T * H * E
    nbytes_alg = E * H * 4 + T * H * 2 + T * E * 4 + 2 * T * k * 4
    if prefill:
        res = dict(
            workload="router in front of configs[4]: T=8192 bf16 hidden states x fp32 weight [256, 7168] -> fp32 "
                     "logits, then group-limited biased top-8, seed 20260",
            value=flops / sec / 1e12, unit="TFLOP/s", ms_per_step=sec * 1e3, dtype="f32",
            kernel="moe_router_gemm_kernel",
            roofline=dict(bound="mfma", achieved=flops / sec / 1e12, peak=157.3, unit="TFLOP/s",
                          frac=flops / sec / 1e12 / 157.3, traffic=None),
            algorithmic_flops=flops)
    else:
        res = dict(
            workload="router in front of configs[2]: T=64 bf16 hidden states x fp32 weight [256, 7168] -> fp32 "
                     "logits (K split 16 ways + ordered reduce), then group-limited biased top-8, seed 20260",
            value=nbytes_alg / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="f32",
            kernel="moe_router_gemm_kernel",
            roofline=dict(bound="hbm", achieved=nbytes_alg / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                          frac=nbytes_alg / sec / 1e9 / HBM_PEAK_GBS, traffic=None),
            algorithmic_bytes=nbytes_alg)
    res['with_split_weight'] = dict(ms_per_step=sec_split * 1e3,
                                    kernel="moe_router_gemm_split_tiled_kernel" if prefill else "moe_router_gemm_split_kernel",
                                    note="fp32 weight as three bf16 planes, 3 exact bf16 products per weight")
    if cpu_baseline:
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
        n_tok = min(T, 512)
        hx, hw, hb = x[:n_tok].cpu(), w.cpu(), bias.cpu()
        csec = cpu_time(lambda: moe.route_grouped(moe.router_logits(hx, hw), hb, 8, 8, 4, True, 2.5))
        cval = 2 * n_tok * H * E / csec / 1e12 if prefill else nbytes_alg / csec / 1e9
        res['cpu_baseline'] = dict(value=cval, unit=res['unit'], cores=cores, kind="port",
                                   sample=f"tokens 0..{n_tok - 1}, eager PyTorch oracle (fp32 matmul, grouped top-k)")
    return res


def bench_rmsnorm_quant(torch, capi, dev, steps, warmup, cpu_baseline):
    """The norm in front of configs[4] fused with the layer's quantiser: 8192 rows of 7168 bf16."""
    from oracle import moe
    T, H = 8192, 7168
    gen = torch.Generator(device=dev).manual_seed(20263)
    xs = [torch.randn(T, H, device=dev, generator=gen).bfloat16() for _ in range(3)]     # 3 x 117 MB
    w = (1.0 + 0.1 * torch.randn(H, device=dev, generator=gen)).bfloat16()
    q = torch.empty(T, H, dtype=torch.uint8, device=dev)
    sc = torch.empty(T, H // 128, device=dev)
    y = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    sec = timed_launches(torch, lambda i: capi.moe_rmsnorm_quant_launch(q, sc, y, xs[i % 3], w), steps, warmup)
    work = T * H * (2 + 2 + 1) + T * (H // 128) * 4 + H * 2
    res = dict(
        workload="RMS norm + activation quantiser in front of configs[4]: 8192 x 7168 bf16 in; bf16 normalised rows, "
                 "e4m3 codes and group scales out, seed 20263",
        value=work / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="f32", kernel="moe_rmsnorm_quant_kernel",
        roofline=dict(bound="hbm", achieved=work / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=work / sec / 1e9 / HBM_PEAK_GBS, traffic=None),
        algorithmic_bytes=work)
    if cpu_baseline:
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
        hx, hw = xs[0][:1024].cpu(), w.cpu()
        csec = cpu_time(lambda: moe.quantize_groups(moe.rmsnorm_bf16(hx, hw).float()))
        res['cpu_baseline'] = dict(value=work / 8 / csec / 1e9, unit="GB/s", cores=cores, kind="port",
                                   sample="rows 0..1023 (1/8), eager PyTorch oracle")
    return res


def bench_index_scores(torch, capi, dev, steps, warmup, cpu_baseline):
    """The indexer scores in front of the selection: 64 requests, 64 index heads of 128, 32768 cached index keys
    (bf16) per request."""
    from oracle import mla
    B, Hi, N = 64, 64, 32768
    gen = torch.Generator(device=dev).manual_seed(20262)
    q = torch.randn(B, Hi, 128, device=dev, generator=gen).bfloat16()
    k = torch.randn(B, N, 128, device=dev, generator=gen).bfloat16()     # 537 MB: twice the last-level cache
    w = torch.randn(B, Hi, device=dev, generator=gen) / 8
    scores = torch.empty(B, N, device=dev)
    sec = timed_launches(torch, lambda i: capi.mla_index_scores_launch(scores, q, k, w), steps, warmup)
    work = B * N * 128 * 2 + B * N * 4 + B * Hi * 128 * 2 + B * Hi * 4
    flops = 2 * B * Hi * N * 128
    res = dict(
        workload="indexer scores in front of configs[3]: B=64, 64 index heads x 128, 32768 bf16 index keys per "
                 "request, seed 20262",
        value=work / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="bf16", kernel="mla_index_scores_kernel",
        roofline=dict(bound="hbm", achieved=work / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=work / sec / 1e9 / HBM_PEAK_GBS, traffic=MEASURED_TRAFFIC['index_scores']),
        algorithmic_bytes=work, tflops=flops / sec / 1e12)
    if cpu_baseline:
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
        nb = 4
        hq, hk, hw = q[:nb].cpu(), k[:nb].cpu(), w[:nb].cpu()
        csec = cpu_time(lambda: mla.index_scores(hq, hk, hw))
        res['cpu_baseline'] = dict(value=work / B * nb / csec / 1e9, unit="GB/s", cores=cores, kind="port",
                                   sample="requests 0..3 (1/16 of the batch), eager PyTorch oracle")
    return res


def bench_index_scores_fp8(torch, capi, dev, steps, warmup, cpu_baseline):
    """The indexer scores over e4m3 index keys: the same shape as index_scores, 128 one-byte codes and one fp32
    scale per cached position."""
    from oracle import mla
    B, Hi, N = 64, 64, 32768
    gen = torch.Generator(device=dev).manual_seed(20263)
    q = torch.randn(B, Hi, 128, device=dev, generator=gen).to(torch.float8_e4m3fn).view(torch.uint8)
    # two key caches used in turn: one (277 MB with its scales) is about the size of the last-level cache
    ks = [torch.randn(B, N, 128, device=dev, generator=gen).to(torch.float8_e4m3fn).view(torch.uint8) for _ in range(2)]
    ss = [torch.rand(B, N, device=dev, generator=gen) + 0.5 for _ in range(2)]
    w = torch.randn(B, Hi, device=dev, generator=gen) / 8
    scores = torch.empty(B, N, device=dev)
    sec = timed_launches(torch, lambda i: capi.mla_index_scores_fp8_launch(scores, q, ks[i % 2], ss[i % 2], w),
                         steps, warmup)
    work = B * N * 128 + B * N * 4 + B * N * 4 + B * Hi * 128 + B * Hi * 4
    flops = 2 * B * Hi * N * 128
    res = dict(
        workload="indexer scores over e4m3 index keys: B=64, 64 index heads x 128, 32768 keys per request "
                 "(128 codes + one fp32 scale each), seed 20263",
        value=work / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="e4m3", kernel="mla_index_scores_fp8_kernel",
        roofline=dict(bound="hbm", achieved=work / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=work / sec / 1e9 / HBM_PEAK_GBS, traffic=MEASURED_TRAFFIC.get('index_scores_fp8')),
        algorithmic_bytes=work, tflops=flops / sec / 1e12)
    if cpu_baseline:
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
        nb = 2
        hq, hk, hs, hw = q[:nb].cpu(), ks[0][:nb].cpu(), ss[0][:nb].cpu(), w[:nb].cpu()
        csec = cpu_time(lambda: mla.index_scores_fp8(hq, hk, hs, hw))
        res['cpu_baseline'] = dict(value=work / B * nb / csec / 1e9, unit="GB/s", cores=cores, kind="port",
                                   sample="requests 0..1 (1/32 of the batch), eager PyTorch oracle in float64")
    return res


def bench_topk_select(torch, capi, dev, steps, warmup, cpu_baseline):
    """The selection in front of configs[3]: 2048 of 32768 index scores per request, 64 requests."""
    from oracle import mla
    B, N, k = 64, 32768, 2048
    gen = torch.Generator(device=dev).manual_seed(20259)
    sets = [torch.randn(B, N, device=dev, generator=gen) for _ in range(8)]
    idx = torch.empty(B, k, dtype=torch.int32, device=dev)
    sec = timed_launches(torch, lambda i: capi.topk_select_launch(idx, sets[i % 8]), steps, warmup)
    work = B * N * 4 + B * k * 4
    res = dict(
        workload="top-k selection in front of configs[3]: B=64, 2048 of 32768 fp32 index scores per request, "
                 "seed 20259 (one workgroup per request)",
        value=work / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="u32", kernel="topk_select_kernel",
        roofline=dict(bound="hbm", achieved=work / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=work / sec / 1e9 / HBM_PEAK_GBS, traffic=MEASURED_TRAFFIC['topk_select']),
        algorithmic_bytes=work)
    if cpu_baseline:
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
        host = sets[0].cpu()
        csec = cpu_time(lambda: mla.topk_select(host, k))
        res['cpu_baseline'] = dict(value=work / csec / 1e9, unit="GB/s", cores=cores, kind="port",
                                   sample="the full selection (oracle: stable sort per request)")
    return res


def bench_mla(torch, capi, dev, steps, warmup, cpu_baseline, paged=False):
    from oracle import mla
    B, H, N, topk = 64, 128, 32768, 2048
    gen = torch.Generator(device=dev).manual_seed(20253)
    q = torch.randn(B, H, 576, device=dev, generator=gen).bfloat16()
    kv = torch.randn(B, N, 576, device=dev, generator=gen).bfloat16()
    # 4 index sets: the 151 MB gathered by one step would otherwise be served from the cache
    idxs = [torch.stack([torch.randperm(N, device=dev, generator=gen)[:topk] for _ in range(B)]).int()
            for _ in range(4)]
    out = torch.empty(B, H, 512, device=dev, dtype=torch.bfloat16)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, topk), dtype=torch.uint8, device=dev)
    if paged:
        # the same bytes seen as one pool of 64-row pages; every request's block table maps its 512
        # logical pages to random pages of the pool
        page = 64
        pool = kv.view(B * N // page, page, 576)
        table = torch.randperm(B * N // page, device=dev, generator=gen).int().view(B, N // page)
        launch = lambda i: capi.sparse_mla_decode_paged_launch(out, q, pool, table, idxs[i % 4], ws)
    else:
        launch = lambda i: capi.sparse_mla_decode_launch(out, q, kv, idxs[i % 4], ws)
    sec = timed_launches(torch, launch, steps, warmup)
    work = B * topk * 576 * 2
    flops = 2 * B * H * topk * (576 + 512)
    res = dict(
        workload="configs[3]: sparse-MLA decode B=64, 128 heads, 576-dim latent rows, top-k 2048 of 32768, "
                 "bf16, seed 20253 (split kernel + merge per step)" +
                 ("; cache held as one pool of 64-row pages behind a block table" if paged else ""),
        value=work / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="bf16", kernel="sparse_mla_split8_kernel",
        roofline=dict(bound="hbm", achieved=work / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=work / sec / 1e9 / HBM_PEAK_GBS, traffic=None if paged else MEASURED_TRAFFIC['mla'],
                      **({} if paged else MEASURED_MFMA['mla'])),
        algorithmic_bytes=work, tflops=flops / sec / 1e12)
    if cpu_baseline and not paged:
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
        nb = 8
        cq, ckv, cidx = q[:nb].cpu(), kv[:nb].cpu(), idxs[0][:nb].cpu()
        csec = cpu_time(lambda: mla.sparse_mla_decode(cq, ckv, cidx))
        res['cpu_baseline'] = dict(value=nb * topk * 576 * 2 / csec / 1e9, unit="GB/s", cores=cores, kind="port",
                                   sample="requests 0..7 of configs[3] (1/8 of the batch), eager PyTorch oracle")
    return res


def bench_mla_fp8_cache(torch, capi, dev, steps, warmup, cpu_baseline):
    """configs[3] over the e4m3 storage form of the latent cache (656-byte rows): the split kernel gathers the
    656-byte rows and dequantises each tile in LDS; config 5000 times the two-step form beside it (gather +
    dequantise of the selected rows into the workspace, then the bf16 decode kernels on that block)."""
    B, H, N, topk = 64, 128, 32768, 2048
    gen = torch.Generator(device=dev).manual_seed(20253)
    q = torch.randn(B, H, 576, device=dev, generator=gen).bfloat16()
    cache = torch.empty(B, N, 656, dtype=torch.uint8, device=dev)
    for b0 in range(0, B, 8):
        capi.mla_latent_quant_launch(cache[b0:b0 + 8], torch.randn(8, N, 576, device=dev, generator=gen).bfloat16())
    idxs = [torch.stack([torch.randperm(N, device=dev, generator=gen)[:topk] for _ in range(B)]).int()
            for _ in range(4)]
    out = torch.empty(B, H, 512, device=dev, dtype=torch.bfloat16)
    ws = torch.empty(capi.sparse_mla_fp8_workspace_bytes(B, H, topk), dtype=torch.uint8, device=dev)
    sec = timed_launches(torch, lambda i: capi.sparse_mla_decode_fp8_launch(out, q, cache, idxs[i % 4], ws), steps, warmup)
    two_step = timed_launches(
        torch, lambda i: capi.sparse_mla_decode_fp8_launch(out, q, cache, idxs[i % 4], ws, config=5000), steps, warmup)
    work = B * topk * 656
    return dict(
        workload="configs[3] over an e4m3 latent cache: B=64, 128 heads, top-k 2048 of 32768 rows of 656 bytes (512 "
                 "codes, 4 scales, 64 bf16 rope values), seed 20253 (split kernel that dequantises its tiles in LDS, "
                 "merge per step)",
        value=work / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, ms_per_step_two_step_form=two_step * 1e3,
        dtype="bf16", kernel="sparse_mla_split8_kernel",
        roofline=dict(bound="hbm", achieved=work / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                      frac=work / sec / 1e9 / HBM_PEAK_GBS, traffic=MEASURED_TRAFFIC['mla_fp8_cache']),
        algorithmic_bytes=work)


def make_moe(torch, dev, tokens, biased):
    """The workload's tensors. The weight buffers hold one more expert behind the 256 routed ones (the shared
    expert of the `with_shared_expert` timings, seed 20258); the routed experts are views of the first 256."""
    H, I, E = 7168, 2048, 256
    gen = torch.Generator(device=dev).manual_seed(20252 if not biased else 20254)
    w13_all = torch.empty(E + 1, 2 * I, H, dtype=torch.float8_e4m3fn, device=dev)
    w2_all = torch.empty(E + 1, H, I, dtype=torch.float8_e4m3fn, device=dev)
    for e in range(E):
        w13_all[e] = (torch.randn(2 * I, H, device=dev, generator=gen) * (448 / H ** 0.5)).to(torch.float8_e4m3fn)
        w2_all[e] = (torch.randn(H, I, device=dev, generator=gen) * (448 / I ** 0.5)).to(torch.float8_e4m3fn)
    w13_s = (0.5 + torch.rand(E, 2 * I // 128, H // 128, device=dev, generator=gen)) / 448
    w2_s = (0.5 + torch.rand(E, H // 128, I // 128, device=dev, generator=gen)) / 448
    x = torch.randn(tokens, H, device=dev, generator=gen).bfloat16()
    logits = torch.randn(tokens, E, device=dev, generator=gen)
    if biased:
        logits[:, torch.randperm(E, device=dev, generator=gen)[:16]] += 2.0
    gen = torch.Generator(device=dev).manual_seed(20258)
    w13_all[E] = (torch.randn(2 * I, H, device=dev, generator=gen) * (448 / H ** 0.5)).to(torch.float8_e4m3fn)
    w2_all[E] = (torch.randn(H, I, device=dev, generator=gen) * (448 / I ** 0.5)).to(torch.float8_e4m3fn)
    w13_s_all = torch.cat([w13_s, ((0.5 + torch.rand(1, 2 * I // 128, H // 128, device=dev, generator=gen)) / 448)])
    w2_s_all = torch.cat([w2_s, ((0.5 + torch.rand(1, H // 128, I // 128, device=dev, generator=gen)) / 448)])
    stacked = (w13_all, w13_s_all, w2_all, w2_s_all)
    return (x, logits, w13_all[:E], w13_s, w2_all[:E], w2_s), stacked


def moe_cpu_baseline(torch, tensors, n_tokens):
    from oracle import moe
    cores = len(os.sched_getaffinity(0))
    torch.set_num_threads(cores)
    x, logits, w13_q, w13_s, w2_q, w2_s = tensors
    ids, _ = moe.route(logits[:n_tokens].cpu(), 8)
    used = torch.unique(ids).tolist()
    remap = {e: i for i, e in enumerate(used)}
    sub = torch.full((n_tokens, len(used)), -30.0)
    for t in range(n_tokens):
        for e in ids[t].tolist():
            sub[t, remap[e]] = logits[t, e].item()
    sel = torch.tensor(used, device=x.device)
    host = [t.cpu() for t in (x[:n_tokens], )] + [sub] + [t[sel].cpu() for t in (w13_q, w13_s, w2_q, w2_s)]
    csec = cpu_time(lambda: moe.moe_forward(*host, top_k=8), min_seconds=2.0, max_iters=2)
    return csec, len(used), cores


def bench_moe(torch, capi, dev, steps, warmup, cpu_baseline, prefill, plain=False):
    T = 8192 if prefill else 64
    H, I, E, k = 7168, 2048, 256, 8
    tensors, stacked = make_moe(torch, dev, T, prefill)
    x, logits, w13_q, w13_s, w2_q, w2_s = tensors
    ws = torch.empty(capi.moe_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=dev)
    out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    sec = timed_launches(torch, lambda i: capi.moe_fp8_launch(out, x, logits, w13_q, w13_s, w2_q, w2_s, ws),
                         steps, warmup)
    off = capi.moe_workspace_views(ws, T, H, I, E, k)['expert_offsets'].cpu()
    n_active = int(((off[1:] - off[:-1]) > 0).sum())
    flops = T * k * (2 * H * 2 * I + 2 * I * H)
    wbytes = n_active * (3 * I * H + (3 * I * H // (128 * 128)) * 4) + T * H * 2 + T * E * 4 + T * H * 2
    if prefill:
        res = dict(
            workload="configs[4]: FP8 MoE prefill T=8192, hidden 7168, 256 experts x inter 2048, top-8, +2 logit "
                     "bias on 16 experts, e4m3 with 128x128 block scales, seed 20254 (whole layer per step)",
            value=flops / sec / 1e12, unit="TFLOP/s", ms_per_step=sec * 1e3, dtype="f8e4m3",
            kernel="moe_tiled_gemm_kernel",
            roofline=dict(bound="mfma", achieved=flops / sec / 1e12, peak=FP8_PEAK_TFLOPS, unit="TFLOP/s",
                          frac=flops / sec / 1e12 / FP8_PEAK_TFLOPS, traffic=MEASURED_TRAFFIC['moe_prefill'],
                          **MEASURED_MFMA['moe_prefill']),
            algorithmic_flops=flops, active_experts=n_active)
    else:
        res = dict(
            workload="configs[2]: FP8 MoE decode T=64, hidden 7168, 256 experts x inter 2048, top-8, e4m3 with "
                     "128x128 block scales, seed 20252 (whole layer per step)",
            value=wbytes / sec / 1e9, unit="GB/s", ms_per_step=sec * 1e3, dtype="f8e4m3",
            kernel="moe_stream_gemm_lds_kernel",
            roofline=dict(bound="hbm", achieved=wbytes / sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                          frac=wbytes / sec / 1e9 / HBM_PEAK_GBS, traffic=MEASURED_TRAFFIC['moe_decode']),
            algorithmic_bytes=wbytes, active_experts=n_active, tflops=flops / sec / 1e12)
    if plain:  # (the workload's own kernels only: what a profiler run wants)
        return res
    # the same layer with a shared expert (one more block-scaled MLP of inter 2048 on every token): as launches
    # of its own, and stored behind the routed experts so that it runs inside their launches
    sw13_q, sw13_s, sw2_q, sw2_s = (t[E] for t in stacked)
    del ws
    ws2 = torch.empty(capi.moe_shared_workspace_bytes(T, H, I, I, E, k), dtype=torch.uint8, device=dev)
    sec2 = timed_launches(
        torch, lambda i: capi.moe_fp8_shared_launch(out, x, logits, w13_q, w13_s, w2_q, w2_s, sw13_q, sw13_s,
                                                    sw2_q, sw2_s, ws2), steps, warmup)
    del ws2
    ws2 = torch.empty(capi.moe_workspace_bytes(T, H, I, E + 1, k + 1), dtype=torch.uint8, device=dev)
    sec2f = timed_launches(torch, lambda i: capi.moe_fp8_fused_shared_launch(out, x, logits, *stacked, ws2),
                           steps, warmup)
    flops2 = flops + T * (2 * H * 2 * I + 2 * I * H)
    wbytes2 = wbytes + 3 * I * H + (3 * I * H // (128 * 128)) * 4
    res['with_shared_expert'] = dict(
        ms_per_step=sec2f * 1e3, unit=res['unit'],
        value=flops2 / sec2f / 1e12 if prefill else wbytes2 / sec2f / 1e9,
        ms_per_step_separate_launches=sec2 * 1e3,
        note="the layer above plus one shared expert of inter 2048, seed 20258: moe_fp8_fused_shared_launcher "
             "(stored as expert 256, inside the routed experts' launches); ms_per_step_separate_launches is "
             "moe_fp8_shared_launcher (its own launches)")
    del ws2
    # the same layer with power-of-two (UE8M0) block scales: the weight scales rounded up to powers of two,
    # activations quantised with power-of-two scales, the tiled GEMMs scaled by the MFMA itself
    p13_s = torch.exp2(torch.ceil(torch.log2(w13_s)))
    p2_s = torch.exp2(torch.ceil(torch.log2(w2_s)))
    ws3 = torch.empty(capi.moe_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=dev)
    sec3 = timed_launches(
        torch, lambda i: capi.moe_fp8_launch(out, x, logits, w13_q, p13_s, w2_q, p2_s, ws3, config=32), steps, warmup)
    res['with_ue8m0_scales'] = dict(
        ms_per_step=sec3 * 1e3, unit=res['unit'], value=flops / sec3 / 1e12 if prefill else wbytes / sec3 / 1e9,
        note="moe_fp8_launcher with config 32: the same workload with every block scale a power of two")
    # how the intermediate is requantised. Decode: the gate/up GEMM runs on the bf16 matrix core (codes agree with
    # an fp32 evaluation), config 512 puts it on the e4m3 one. Prefill: e4m3 matrix core with the codes of the large
    # elements repaired in the epilogue; config 256 runs gate/up on the bf16 matrix core instead (every code
    # exact), config 512 leaves the e4m3 matrix core's codes as they come.
    for key, other in ((('gate_up_on_bf16_matrix_core', 256), ('e4m3_matrix_core_without_repair', 512)) if prefill
                       else (('gate_up_on_e4m3_matrix_core', 512),)):
        sec4 = timed_launches(
            torch, lambda i: capi.moe_fp8_launch(out, x, logits, w13_q, w13_s, w2_q, w2_s, ws3, config=other),
            max(2, steps // 2), 1)
        res[key] = dict(
            ms_per_step=sec4 * 1e3, unit=res['unit'], value=flops / sec4 / 1e12 if prefill else wbytes / sec4 / 1e9,
            note=f"moe_fp8_launcher with config {other}")
    del ws3
    if cpu_baseline:
        n_tok = 4
        csec, n_used, cores = moe_cpu_baseline(torch, tensors, n_tok)
        if prefill:
            cval = n_tok * k * (2 * H * 2 * I + 2 * I * H) / csec / 1e12
        else:
            cval = (n_used * (3 * I * H + (3 * I * H // (128 * 128)) * 4)) / csec / 1e9
        res['cpu_baseline'] = dict(
            value=cval, unit=res['unit'], cores=cores, kind="port",
            sample=f"tokens 0..{n_tok - 1} of the workload and the {n_used} experts they route to, eager "
                   "PyTorch oracle (dequantise to fp32, dense matmul)")
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--workloads', default='gdn,gdn_single,gdn_fused,gdn_fused_norm,conv1d,moe_decode,router_decode,index_scores,index_scores_fp8,topk_select,mla,mla_paged,mla_fp8_cache,moe_prefill,router_prefill,rmsnorm_quant')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--plain', action='store_true',
                    help='MoE workloads: time the workload itself only, not its variants (shared expert, UE8M0 '
                         'scales, requantisation forms), so that a profiler run sees one set of kernels')
    ap.add_argument('--calibrate-copy', action='store_true',
                    help='also run 3 plain device copies of 536 870 912 bytes (a kernel of known traffic, '
                         'for scaling the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)')
    ap.add_argument('--calibrate-mfma', action=argparse.BooleanOptionalAction, default=True,
                    help='measure what the matrix cores sustain on random operands, alone and beside an HBM stream '
                         '(about a second): reported as roofline.sustained_peak')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py: this build measures one GPU only (no collectives, no sharding); run with --gpus 1')

    import torch
    import __graft_entry__
    __graft_entry__.load_package()
    from cuda_agent_amd import capi
    capi.library()  # raises if the HIP library is not built: there is no fallback path
    if not torch.cuda.is_available():
        sys.exit('bench.py: no GPU visible')
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    cpu = not args.no_cpu_baseline
    if args.calibrate_copy:
        src = torch.ones(536870912 // 4, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    wanted = [w.strip() for w in args.workloads.split(',') if w.strip()]
    results = {}
    for name in wanted:
        if name == 'gdn':
            results[name] = bench_gdn(torch, capi, dev, args.steps, args.warmup, cpu)
        elif name == 'gdn_fused':
            results[name] = bench_gdn_fused(torch, capi, dev, args.steps, args.warmup, cpu)
        elif name == 'gdn_single':
            results[name] = bench_gdn_single(torch, capi, dev, args.steps, args.warmup, cpu)
        elif name == 'gdn_fused_norm':
            results[name] = bench_gdn_fused_norm(torch, capi, dev, args.steps, args.warmup, cpu)
        elif name == 'conv1d':
            results[name] = bench_conv1d(torch, capi, dev, args.steps, args.warmup, cpu)
        elif name in ('router_decode', 'router_prefill'):
            results[name] = bench_router(torch, capi, dev, args.steps, args.warmup, cpu, name == 'router_prefill')
        elif name == 'rmsnorm_quant':
            results[name] = bench_rmsnorm_quant(torch, capi, dev, args.steps, args.warmup, cpu)
        elif name == 'index_scores_fp8':
            results[name] = bench_index_scores_fp8(torch, capi, dev, args.steps, args.warmup, cpu)
        elif name == 'index_scores':
            results[name] = bench_index_scores(torch, capi, dev, args.steps, args.warmup, cpu)
        elif name == 'topk_select':
            results[name] = bench_topk_select(torch, capi, dev, args.steps, args.warmup, cpu)
        elif name == 'mla':
            results[name] = bench_mla(torch, capi, dev, args.steps, args.warmup, cpu)
        elif name == 'mla_fp8_cache':
            results[name] = bench_mla_fp8_cache(torch, capi, dev, args.steps, args.warmup, cpu)
        elif name == 'mla_paged':
            results[name] = bench_mla(torch, capi, dev, args.steps, args.warmup, cpu, paged=True)
        elif name == 'moe_decode':
            results[name] = bench_moe(torch, capi, dev, args.steps, args.warmup, cpu, prefill=False, plain=args.plain)
        elif name == 'moe_prefill':
            results[name] = bench_moe(torch, capi, dev, args.steps, max(1, args.warmup // 2), cpu,
                                      prefill=True, plain=args.plain)
        else:
            sys.exit(f'bench.py: unknown workload {name}')
        results[name].setdefault('steps_timed', args.steps)
        torch.cuda.empty_cache()

    head_name = 'gdn' if 'gdn' in results else wanted[0]
    head = results[head_name]
    line = {
        "metric": METRIC, "value": head['value'], "unit": head['unit'], "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": head['ms_per_step'], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": head['dtype'], "data": "synthetic",
        "config": {"workload": head['workload'],
                   "settle": f"{SETTLE_SECONDS} s of untimed launches before the warm-up steps of every workload"},
        "roofline": head['roofline'],
    }
    # the four workloads the targets are stated on, inside the headline's roofline object
    line["roofline"] = dict(head['roofline'], per_workload={
        k: dict(ms_per_step=results[k]['ms_per_step'], frac=results[k]['roofline']['frac'],
                achieved=results[k]['roofline']['achieved'], unit=results[k]['roofline']['unit'],
                steps_timed=results[k]['steps_timed'])
        for k in ('gdn', 'moe_decode', 'mla', 'moe_prefill') if k in results})
    if args.calibrate_mfma:
        # measured ceilings next to the data-sheet peaks: a stream of MFMAs on random operands, alone and with half
        # of every CU's wavefronts streaming 2 GiB from HBM meanwhile (csrc/calibrate.hip)
        alone, _, _ = capi.calibrate_mfma(0.25, 0, False)
        beside, tbs, _ = capi.calibrate_mfma(0.25, 2 << 30, False)
        alone_bf16, _, _ = capi.calibrate_mfma(0.25, 0, True)
        sustained = dict(e4m3_mfma_alone_pflops=alone, e4m3_mfma_beside_hbm_stream_pflops=beside,
                         hbm_stream_beside_e4m3_mfma_tbs=tbs, bf16_mfma_alone_pflops=alone_bf16)
        # the clock the matrix pipes run at against the share of the chip that is busy: the same loop (which keeps
        # every SIMD's pipe full: 8192 flops per CU and cycle) on 32, 128 and all 256 CUs
        sustained['e4m3_mfma_clock_ghz_by_busy_cus'] = {
            str(n): capi.calibrate_mfma(0.15, 0, False, n)[0] * 1e6 / (n * 8192) for n in (32, 128, 256)}
        sustained['note'] = ("calibrate_mfma_launcher: 256 workgroups, 4 wavefronts of each issuing MFMAs on random "
                             "operands (v_mfma_f32_32x32x64_f8f6f4 / v_mfma_f32_32x32x16_bf16), 4 streaming 16-byte loads; "
                             "rates over the MFMA loops' own wall-clock ticks, mean of the second half of 0.25 s of launches")
        line["roofline"]["sustained_peak"] = sustained
    if 'cpu_baseline' in head:
        line["cpu_baseline"] = head['cpu_baseline']
    shown = ('workload', 'value', 'unit', 'ms_per_step', 'dtype', 'roofline', 'cpu_baseline')
    details = {k: v for k, v in head.items() if k not in shown}
    if details:
        line["details"] = details
    line["workloads"] = {k: v for k, v in results.items() if k != head_name}
    print(json.dumps(line))


if __name__ == '__main__':
    main()
