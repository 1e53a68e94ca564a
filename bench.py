#!/usr/bin/env python3
"""Benchmark of the xKV compressed-KV decode path on one MI355X.

Default workload (configuration 3 of the five target shapes): fused RoPE-aware xKV decode, Llama-3.1-8B attention shape,
batch 16, 32 q / 8 kv heads, head_dim 128, context 32768, rank 512, bf16; one token basis A shared by
K and V and by the 4 layers of a group, per-layer B_l / B_v,l.  A "step" is ONE layer's decode step
(stage 1 + merge) cycling through the 4 layers of the group.

Prints one JSON line: the metric (us per layer decode step), the roofline of the dominant kernel
(stage 1, MFMA-bound) measured live with HIP events, the uncompressed bf16 flash-decode comparator of
the same shape, and the CPU oracle timed on a bounded sample of the same workload.
Other workloads (--config c2|c4|c4v|c5) print the same line for their own shape and bound.
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0
PEAK_BF16_TFLOPS = 2500.0
# HBM bytes of one stage-1 launch at the default c3 shape, from two rocprofv3 --pmc runs of this file
# (FETCH_SIZE, WRITE_SIZE; each scaled by what the counter reads for --calib-copy's 512 MiB copies).
# A counter cannot be read from inside the timed process, so the figure is recorded here.
C3_STAGE1_HBM_BYTES = 535406 * 1024
C5_RING_HBM_BYTES = 602885 * 1024     # same method, latent_ring_kernel at the default c5 shape


def _events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def time_loop(fn, steps, warmup):
    """Exactly `steps` timed calls bracketed by synchronize; returns total ms."""
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3


def time_kernel(fn, steps, warmup):
    """Average duration (ms) of one launch, HIP events recorded on the stream the kernel runs on."""
    for i in range(warmup):
        fn(i)
    st, en = _events(steps), _events(steps)
    torch.cuda.synchronize()
    for i in range(steps):
        st[i].record()
        fn(i)
        en[i].record()
    torch.cuda.synchronize()
    ts = sorted(s.elapsed_time(e) for s, e in zip(st, en))
    return sum(ts) / len(ts), ts[len(ts) // 2]


def randn_dev(shape, std, dev, dtype=torch.bfloat16, gen=None):
    return (torch.randn(shape, device=dev, dtype=torch.float32, generator=gen) * std).to(dtype)


# ------------------------------------------------------------------------------------------------
def bench_c3(args, dev):
    import kernel_collections_amd.flash_recontruction as fr
    from kernel_collections_amd import ops
    from kernel_collections_amd.flash_decoding import gqa
    B, Hq, Hkv, d, L, r, theta, layers = 16, 32, 8, 128, args.ctx, 512, 5e5, 4
    gen = torch.Generator(device=dev).manual_seed(0)
    A = randn_dev((B, L, r), 1.0, dev, gen=gen)
    kB = [randn_dev((r, Hkv * d), r ** -0.5, dev, gen=gen).view(r, Hkv, d).permute(1, 0, 2).unsqueeze(0).expand(B, Hkv, r, d)
          for _ in range(layers)]
    vB = [randn_dev((r, Hkv * d), r ** -0.5, dev, gen=gen).view(r, Hkv, d).permute(1, 0, 2).unsqueeze(0).expand(B, Hkv, r, d)
          for _ in range(layers)]
    q = [randn_dev((B, Hq, d), 1.0, dev, gen=gen) for _ in range(layers)]  # stands for the already-rotated query
    o = torch.empty((B, Hq, d), dtype=torch.bfloat16, device=dev)
    S = args.splits or ops.occupancy_splits(B, Hkv, L, tile=32, waves=1)
    ns = ops.uniform_splits(B, S, dev)
    scale = d ** -0.5

    def step(i):
        l = i % layers
        fr.gqa_xKV_rope(q[l], A, kB[l], A, vB[l], o, ns, S, scale, theta)

    total_ms = time_loop(step, args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps

    # dominant kernel alone: stage 1
    partial, lse = ops.workspaces(B, Hq, S, r, dev)
    inv = ops.rope_inv_freq(d, theta, dev)

    def stage1(i):
        l = i % layers
        ops.recon_stage1(q[l], A, kB[l], A, partial, lse, None, ns, None, B, Hq, Hkv, L, S, scale, True, inv, 0, None)

    k_avg_ms, k_med_ms = time_kernel(stage1, args.steps, args.warmup)
    flops = B * L * (2 * r * Hkv * d + 2 * Hq * d + 2 * Hq * r)
    achieved = flops / (k_avg_ms * 1e-3) / 1e12
    algo_bytes = B * L * r * 2 + 2 * r * Hkv * d * 2

    # comparator: uncompressed bf16 flash decoding of the same shape
    comp_us = None
    if not args.no_comparator:
        K = randn_dev((B, L, Hkv, d), 1.0, dev, gen=gen)
        V = randn_dev((B, L, Hkv, d), 1.0, dev, gen=gen)
        Sc = ops.occupancy_splits(B, Hkv, L)
        nsc = ops.uniform_splits(B, Sc, dev)
        comp_ms = time_loop(lambda i: gqa.decode_attention_fwd(q[i % layers], K, V, o, nsc, Sc, scale), args.steps, args.warmup)
        comp_us = comp_ms * 1e3 / args.steps
        del K, V

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline_c3(Hq, Hkv, d, L, r, theta, B)

    return {
        "metric": "us_per_layer_decode_step", "value": round(us, 2), "unit": "us",
        "higher_is_better": False,
        "ms_per_step": total_ms / args.steps,
        "tokens_per_s": B / (us * 1e-6), "kv_tokens_scanned_per_s": B * L / (us * 1e-6),
        "config": {"workload": "c3 fused RoPE xKV decode: batch 16, 32q/8kv heads, d128, ctx %d, rank 512, "
                               "A shared by K/V and by a 4-layer group, per layer" % L, "kv_splits": S},
        "roofline": {"bound": "mfma", "kernel": "recon_fast_kernel", "achieved": round(achieved, 1),
                     "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                     "traffic": C3_STAGE1_HBM_BYTES if (L == 32768 and not args.splits) else None,
                     "kernel_avg_us": round(k_avg_ms * 1e3, 2), "kernel_median_us": round(k_med_ms * 1e3, 2),
                     "algorithmic_flop": flops, "hbm_side_GBps": round(algo_bytes / (k_avg_ms * 1e-3) / 1e9, 1)},
        "uncompressed_flash_decode_us": None if comp_us is None else round(comp_us, 2),
        "cpu_baseline": cpu,
    }


def cpu_baseline_c3(Hq, Hkv, d, L, r, theta, B):
    """The CPU oracle (eager fp32 restatement of the reference semantics) on ONE of the B sequences,
    repeated for >= ~10 s; value scaled to the whole batch (sequences are independent)."""
    import oracle
    torch.manual_seed(0)
    nthreads = torch.get_num_threads()
    A = torch.randn(1, L, r)
    kB, vB = torch.randn(1, Hkv, r, d) * r ** -0.5, torch.randn(1, Hkv, r, d) * r ** -0.5
    q = torch.randn(1, Hq, 1, d)
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta)
    oracle.gqa_factorized_rope(q, A, kB, A, vB, cos, sin)
    n, t0 = 0, time.perf_counter()
    while True:
        oracle.gqa_factorized_rope(q, A, kB, A, vB, cos, sin)
        n += 1
        el = time.perf_counter() - t0
        if el > 10.0 or n >= 50:
            break
    per_seq_us = el / n * 1e6
    return {"value": round(per_seq_us * B, 1), "unit": "us", "cores": nthreads, "kind": "port",
            "sample": "1 of %d sequences (ctx %d) x %d repeats, eager fp32 oracle.gqa_factorized_rope; "
                      "value = per-sequence time x %d" % (B, L, n, B)}


# ------------------------------------------------------------------------------------------------
def bench_c2(args, dev):
    import kernel_collections_amd.flash_recontruction as fr
    from kernel_collections_amd import ops
    B, Hq, Hkv, d, L, r = 8, 32, 8, 128, 16384, 512
    gen = torch.Generator(device=dev).manual_seed(0)
    # rotate through several A buffers (> 256 MiB in total) so the scan cannot be served from cache
    nbuf = 4
    As = [randn_dev((B, L, r), 1.0, dev, gen=gen) for _ in range(nbuf)]
    Bm = randn_dev((r, Hkv * d), r ** -0.5, dev, gen=gen).view(r, Hkv, d).permute(1, 0, 2).unsqueeze(0).expand(B, Hkv, r, d)
    q = randn_dev((B, Hq, 1, d), 1.0, dev, gen=gen)
    scale = d ** -0.5
    total_ms = time_loop(lambda i: fr.qAB_no_pe_v1(q, As[i % nbuf], Bm, sm_scale=scale, out_dtype=torch.float32),
                         args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    q3 = q.reshape(B, Hq, d)
    hi, lo = ops.absorb_q(q3, Bm)
    out = torch.empty((B, Hq, 1, L), dtype=torch.float32, device=dev)
    S = args.splits or ops.latent_splits(B, 1, L, r)
    ns = ops.uniform_splits(B, S, dev)

    def scan(i):
        A = As[i % nbuf]
        ops.latent_stage1(hi, lo, None, (A, A.stride(0), A.stride(1), 0, r), None, None, None, None, out, ns, None,
                          B, Hq, 1, L, S, scale)

    k_avg_ms, k_med_ms = time_kernel(scan, args.steps, args.warmup)
    algo_bytes = B * L * r * 2 + B * Hq * L * 4 + r * Hkv * d * 2 + B * Hq * d * 2
    gbs = algo_bytes / (k_avg_ms * 1e-3) / 1e9
    return {
        "metric": "us_per_qAB_no_pe_call", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps,
        "config": {"workload": "c2 qAB_no_pe scores: batch 8, 32q/8kv, d128, L16384, rank 512, bf16 in / fp32 out", "kv_splits": S},
        "roofline": {"bound": "hbm", "kernel": "latent_ring_kernel(scores)", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None,
                     "kernel_avg_us": round(k_avg_ms * 1e3, 2), "kernel_median_us": round(k_med_ms * 1e3, 2),
                     "algorithmic_bytes": algo_bytes},
        "cpu_baseline": None,
    }


def bench_c5(args, dev):
    from kernel_collections_amd import ops
    from kernel_collections_amd.flash_decoding import mla2
    B, H, L, c, e = 64, 16, 8192, 512, 64
    gen = torch.Generator(device=dev).manual_seed(0)
    ckv, kpe = randn_dev((B, L, 1, c), 1.0, dev, gen=gen), randn_dev((B, L, 1, e), 1.0, dev, gen=gen)
    qn, qr = randn_dev((B, H, c), 0.3, dev, gen=gen), randn_dev((B, H, e), 1.0, dev, gen=gen)
    scale = 1 / math.sqrt(192)
    total_ms = time_loop(lambda i: mla2.mla_decode_attention_fwd(qn, qr, ckv, kpe, scale), args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    S = args.splits or ops.latent_splits(B, 1, L, 512)
    ns = ops.uniform_splits(B, S, dev)
    partial, lse = ops.workspaces(B, H, S, c, dev)
    k_avg_ms, k_med_ms = time_kernel(lambda i: mla2.decoding_stage1(qn, qr, ckv, kpe, partial, lse, ns, S, scale),
                                     args.steps, args.warmup)
    algo_bytes = B * L * (c + e) * 2
    gbs = algo_bytes / (k_avg_ms * 1e-3) / 1e9
    flops = B * L * H * (c + e + c) * 2
    return {
        "metric": "us_per_mla_decode_step", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps,
        "config": {"workload": "c5 MLA absorbed decode: batch 64, 16 heads, latent 512 + rope 64, ctx 8192, bf16", "kv_splits": S},
        "roofline": {"bound": "hbm", "kernel": "latent_ring_kernel", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None if args.splits else C5_RING_HBM_BYTES,
                     "kernel_avg_us": round(k_avg_ms * 1e3, 2), "kernel_median_us": round(k_med_ms * 1e3, 2),
                     "algorithmic_bytes": algo_bytes, "mfma_TFLOPs": round(flops / (k_avg_ms * 1e-3) / 1e12, 1)},
        "cpu_baseline": None,
    }


def bench_c4(args, dev, vfact):
    from kernel_collections_amd import ops
    from kernel_collections_amd.flash_decoding import gqa
    B, Hq, Hkv, d, rv, split = 32, 32, 8, 128, 512, 4096
    g = torch.Generator().manual_seed(0)
    u = torch.rand(B, generator=g)
    lens = torch.floor(torch.exp(math.log(1024) + u * (math.log(131072) - math.log(1024)))).to(torch.int64).tolist()
    Lmax = max(lens)
    gen = torch.Generator(device=dev).manual_seed(0)
    K = randn_dev((B, Lmax, Hkv, d), 1.0, dev, gen=gen)
    q = randn_dev((B, Hq, d), 1.0, dev, gen=gen)
    o = torch.empty_like(q)
    if vfact:
        split = args.splits or split  # the wrapper cuts long splits itself (one workgroup serves all 32 heads of a split)
    elif args.splits:
        split = args.splits
    ns_l = [-(-n // split) for n in lens]
    S = max(ns_l)
    ns = torch.tensor(ns_l, dtype=torch.int32, device=dev)
    kl = torch.tensor(lens, dtype=torch.int32, device=dev)
    scale = d ** -0.5
    if vfact:
        vA = randn_dev((B, Lmax, rv), 1.0, dev, gen=gen)
        vB = randn_dev((B, Hkv, rv, d), rv ** -0.5, dev, gen=gen)
        fn = lambda i: gqa.decode_attention_fwd_v_factorized(q, K, vA, vB, o, ns, S, scale, kv_lens=kl)
        per_tok = 2048 + 1024
    else:
        V = randn_dev((B, Lmax, Hkv, d), 1.0, dev, gen=gen)
        fn = lambda i: gqa.decode_attention_fwd(q, K, V, o, ns, S, scale, kv_lens=kl)
        per_tok = 4096
    total_ms = time_loop(fn, args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    algo_bytes = sum(lens) * per_tok
    gbs = algo_bytes / (us * 1e-6) / 1e9
    return {
        "metric": "us_per_ragged_decode_step", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps,
        "config": {"workload": "c4 ragged split-K GQA%s: batch 32, lens log-uniform [1024,131072], split %d"
                               % (" V-factorised r512" if vfact else "", split), "sum_len": sum(lens), "max_len": Lmax,
                   "kv_splits_max": S},
        "roofline": {"bound": "hbm", "kernel": "latent_ring_kernel" if vfact else "latent_stage1_kernel",
                     "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None,
                     "note": "whole call (stage 1 + merge) over algorithmic bytes", "algorithmic_bytes": algo_bytes},
        "cpu_baseline": None,
    }


def bench_pdsep(args, dev):
    """Prefix + tail decode at the shape of the reference's own script (test_mla_decoding_new.py:66-73): batch 1,
    32 heads on one kv head, head_dim 512, prefix 262144 tokens factorised at rank 512, 128 decoded tokens, fp16."""
    from kernel_collections_amd.flash_decoding import deepseek_mla
    B, H, hd, Lp, Ld, r = 1, 32, 512, 262144, 128, 512
    dt = torch.float16
    gen = torch.Generator(device=dev).manual_seed(0)
    q = randn_dev((B, H, hd), 1.0, dev, dt, gen)
    kA, vA = randn_dev((B, Lp, r), 1.0, dev, dt, gen), randn_dev((B, Lp, r), 1.0, dev, dt, gen)
    kB, vB = randn_dev((B, 1, r, hd), r ** -0.5, dev, dt, gen), randn_dev((B, 1, r, hd), r ** -0.5, dev, dt, gen)
    Kd, Vd = randn_dev((B, Ld, 1, hd), 1.0, dev, dt, gen), randn_dev((B, Ld, 1, hd), 1.0, dev, dt, gen)
    scale = hd ** -0.5
    fn = lambda i: deepseek_mla.mla_decode_attention_fwd_pd_sep_xKV(q, kA, kB, vA, vB, Kd, Vd, scale)
    total_ms = time_loop(fn, args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    algo_bytes = B * Lp * 2 * r * 2 + B * Ld * 2 * hd * 2 + 2 * r * hd * 2
    gbs = algo_bytes / (us * 1e-6) / 1e9
    return {
        "metric": "us_per_prefix_tail_decode_step", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps,
        "config": {"workload": "prefix + tail decode: batch 1, 32 heads / 1 kv head, head_dim 512, prefix 262144 at rank 512 "
                               "(k_A, v_A), tail 128 plain, fp16"},
        "roofline": {"bound": "hbm", "kernel": "latent_ring_kernel", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None,
                     "note": "whole call (absorb, 2 x stage 1, 2 x merge) over algorithmic bytes", "algorithmic_bytes": algo_bytes},
        "cpu_baseline": None,
    }


def bench_qabrope(args, dev):
    """RoPE-aware key reconstruction scores at the shape of the reference's own sweep (test_qAB_rope.py:85-125):
    batch 1, 32 q / 8 kv heads, head_dim 128, rank 192, fp16, kv_len = --ctx (the sweep runs 16K .. 128K)."""
    import kernel_collections_amd.flash_recontruction as fr
    B, Hq, Hkv, d, r, L, theta = 1, 32, 8, 128, args.rank, args.ctx, 1e7
    dt = torch.float16 if args.dtype == "fp16" else torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(0)
    q = randn_dev((B, Hq, 1, d), 0.2, dev, dt, gen)
    A = randn_dev((B, L, r), 0.2, dev, dt, gen)
    Bk = randn_dev((B, Hkv, r, d), 0.2, dev, dt, gen)
    total_ms = time_loop(lambda i: fr.qAB_rope_v1(q, A, Bk, theta), args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    flops = B * L * (2 * r * Hkv * d + 2 * Hq * d)
    tf = flops / (us * 1e-6) / 1e12
    return {
        "metric": "us_per_qAB_rope_call", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps,
        "config": {"workload": "qAB with RoPE, scores only: batch 1, 32q/8kv, d128, rank %d, kv_len %d, %s" % (r, L, args.dtype)},
        "roofline": {"bound": "mfma", "kernel": "recon_stage1_kernel(scores)", "achieved": round(tf, 1), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tf / PEAK_BF16_TFLOPS, 4), "traffic": None,
                     "note": "whole call over algorithmic FLOP", "algorithmic_flop": flops,
                     "hbm_side_GBps": round((B * L * r * 2 + B * Hq * L * 2) / (us * 1e-6) / 1e9, 1)},
        "cpu_baseline": None,
    }


def bench_ropedecode(args, dev):
    """Fused xKV decode with RoPE and SEPARATE key / value bases at the default shape of the reference's variant table
    (test_attention_profiling.py:511-517): batch 1, 32 q / 8 kv heads, head_dim 128, kv_len 131072, K rank 384, V rank 512."""
    import kernel_collections_amd.flash_recontruction as fr
    from kernel_collections_amd import ops
    B, Hq, Hkv, d, L, rk, rv, theta = 1, 32, 8, 128, 131072, args.rank if args.rank != 192 else 384, 512, 5e5
    gen = torch.Generator(device=dev).manual_seed(0)
    q = randn_dev((B, Hq, d), 1.0, dev, torch.bfloat16, gen)
    kA, vA = randn_dev((B, L, rk), 1.0, dev, torch.bfloat16, gen), randn_dev((B, L, rv), 1.0, dev, torch.bfloat16, gen)
    kB = randn_dev((B, Hkv, rk, d), rk ** -0.5, dev, torch.bfloat16, gen)
    vB = randn_dev((B, Hkv, rv, d), rv ** -0.5, dev, torch.bfloat16, gen)
    o = torch.empty_like(q)
    S = args.splits or ops.occupancy_splits(B, Hkv, L, tile=32, waves=1)
    ns = ops.uniform_splits(B, S, dev)
    total_ms = time_loop(lambda i: fr.gqa_xKV_rope(q, kA, kB, vA, vB, o, ns, S, d ** -0.5, theta), args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    flops = B * L * (2 * rk * Hkv * d + 2 * Hq * d + 2 * Hq * rv)
    tf = flops / (us * 1e-6) / 1e12
    return {
        "metric": "us_per_layer_decode_step", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps,
        "config": {"workload": "fused RoPE xKV decode, separate bases: batch 1, 32q/8kv, d128, kv_len %d, K rank %d, V rank %d, bf16"
                               % (L, rk, rv), "kv_splits": S},
        "roofline": {"bound": "mfma", "kernel": "recon_duo_kernel", "achieved": round(tf, 1), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tf / PEAK_BF16_TFLOPS, 4), "traffic": None,
                     "note": "whole call (pack, stage 1, merge) over algorithmic FLOP", "algorithmic_flop": flops,
                     "hbm_side_GBps": round(B * L * (rk + rv) * 2 / (us * 1e-6) / 1e9, 1)},
        "cpu_baseline": None,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--config", default="c3", choices=["c2", "c3", "c4", "c4v", "c5", "pdsep", "qabrope", "ropedecode"])
    ap.add_argument("--ctx", type=int, default=32768)
    ap.add_argument("--splits", type=int, default=0)
    ap.add_argument("--rank", type=int, default=192, help="rank of the qabrope workload (ropedecode: K rank, default 384)")
    ap.add_argument("--dtype", default="fp16", choices=["fp16", "bf16"], help="operand type of the qabrope workload")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-comparator", action="store_true")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run 3 plain device copies of 512 MiB (a kernel of known traffic, for scaling rocprof's "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    from kernel_collections_amd import _lib
    _lib.lib()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.calib_copy:
        src = torch.empty(512 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.config == "c3":
        res = bench_c3(args, dev)
    elif args.config == "c2":
        res = bench_c2(args, dev)
    elif args.config == "c5":
        res = bench_c5(args, dev)
    elif args.config == "pdsep":
        res = bench_pdsep(args, dev)
    elif args.config == "qabrope":
        res = bench_qabrope(args, dev)
    elif args.config == "ropedecode":
        res = bench_ropedecode(args, dev)
    else:
        res = bench_c4(args, dev, args.config == "c4v")
    line = {"metric": res.pop("metric"), "value": res.pop("value"), "unit": res.pop("unit"), "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": res.pop("ms_per_step"),
            "higher_is_better": res.pop("higher_is_better"), "scaling": "weak", "vs_baseline": None,
            "dtype": "fp16" if (args.config == "pdsep" or (args.config == "qabrope" and args.dtype == "fp16")) else "bf16", "data": "synthetic"}
    line.update(res)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
