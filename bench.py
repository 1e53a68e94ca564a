#!/usr/bin/env python3
"""Benchmark of the xKV compressed-KV decode path on one MI355X.

Default workload (configuration 3 of the five target shapes): fused RoPE-aware xKV decode, Llama-3.1-8B attention shape,
batch 16, 32 q / 8 kv heads, head_dim 128, context 32768, rank 512, bf16; one token basis A shared by
K and V and by the 4 layers of a group, per-layer B_l / B_v,l.  A "step" is ONE layer's decode step
(stage 1 + merge) cycling through the 4 layers of the group.

Prints one JSON line: the metric (us per layer decode step, wall clock over exactly --steps steps after --warmup
untimed ones), per-step quantiles from HIP events, the roofline of the dominant kernel measured live with HIP events,
the uncompressed bf16 flash-decode comparator of the same shape, the same workload with a value basis of its own, and the
CPU oracle timed on a bounded sample of the same workload.  Every configuration first checks what it is about to time
against the CPU oracle on a slice (outside the timed region) and refuses to print a number for a wrong result.
Other workloads: --config c1|c2|c4|c4v|c5|pdsep|qabrope|ropedecode|ceilings.
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

# published peaks of the MI355X, the denominators of roofline.frac
PEAK_HBM_GBS = 8000.0
PEAK_BF16_TFLOPS = 2500.0
# roofline.traffic: HBM bytes of one launch of a workload's dominant kernel, from two rocprofv3 --pmc runs of this file
# (FETCH_SIZE, WRITE_SIZE; each scaled by what the counter reads for --calib-copy's 512 MiB copies).  A counter cannot be read
# from inside the timed process, so the figures are kept in profiles/hbm_traffic_table.txt, one line per workload:
#   <workload> <bytes> <kernel source file>:<first 16 hex digits of its sha256> ...
# A figure is reported only while every source file it names still has the recorded hash: after a kernel change the line
# reads null until the counters have been collected again (`bench.py --traffic-line <workload> <bytes>` prints a fresh line).
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic_table.txt")
CSRC = os.path.join(ROOT, "kernel_collections_amd", "csrc")
TRAFFIC_SOURCES = {
    "c3": ["recon_spec_impl.h", "recon_fast_impl.h", "recon_stage1.hip"],
    "c2": ["latent_ring.hip", "latent_ring.h"], "c5": ["latent_ring.hip", "latent_ring.h"], "c4": ["latent_ring.hip", "latent_ring.h"],
}


def _source_hash(name):
    import hashlib
    return hashlib.sha256(open(os.path.join(CSRC, name), "rb").read()).hexdigest()[:16]


def traffic_line(workload, nbytes):
    return " ".join([workload, str(int(nbytes))] + ["%s:%s" % (f, _source_hash(f)) for f in TRAFFIC_SOURCES[workload]])


def recorded_traffic(workload):
    try:
        rows = [l.split() for l in open(TRAFFIC_TABLE) if l.strip() and not l.startswith("#")]
    except OSError:
        return None
    for row in rows:
        if row[0] == workload:
            ok = all(_source_hash(f) == h for f, h in (x.split(":") for x in row[2:]))
            return int(row[1]) if ok else None
    return None


OUT_ATOL, SCORE_RTOL = 2e-2, 1e-2     # the parity bars (attention output max-abs, scores max|delta| / max|ref|)


def _events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def _quantiles(ts):
    ts = sorted(ts)
    pick = lambda f: ts[min(len(ts) - 1, int(f * len(ts)))]
    return {"median": round(pick(0.5) * 1e3, 2), "p20": round(pick(0.2) * 1e3, 2), "p80": round(pick(0.8) * 1e3, 2)}


SETTLE_S = 1.5


def _settle(fn):
    """Untimed calls of the workload about to be measured, for SETTLE_S seconds: a device that has idled (while the CPU
    oracle ran, say) or has just run a different kernel needs tens of milliseconds of this load before it runs it at the
    clock it sustains; until then every kernel is 4-10 % slower.  The --warmup steps still follow."""
    t_end = time.perf_counter() + SETTLE_S
    i = 0
    while time.perf_counter() < t_end:
        for _ in range(20):
            fn(i)
            i += 1
        torch.cuda.synchronize()


def time_loop(fn, steps, warmup, settle=True):
    """Settling calls, `warmup` untimed calls, then exactly `steps` timed calls bracketed by synchronize.  Returns (total
    wall-clock ms, per-step quantiles in us from HIP events recorded between the steps on the launch stream)."""
    if settle:
        _settle(fn)
    for i in range(warmup):
        fn(i)
    ev = _events(steps + 1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        ev[i].record()
        fn(i)
    ev[steps].record()
    torch.cuda.synchronize()
    total = (time.perf_counter() - t0) * 1e3
    return total, _quantiles([ev[i].elapsed_time(ev[i + 1]) for i in range(steps)])


def time_kernel(fn, steps, warmup, settle=True):
    """Average and median duration (ms) of one launch, HIP events recorded on the stream the kernel runs on."""
    if settle:
        _settle(fn)
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
    out = torch.empty(shape, dtype=dtype, device=dev)
    flat = out.view(-1)
    for i in range(0, flat.numel(), 1 << 28):
        n = min(1 << 28, flat.numel() - i)
        flat[i:i + n] = (torch.randn(n, device=dev, dtype=torch.float32, generator=gen) * std).to(dtype)
    return out


def require_close(got, ref, what, scores=False):
    """Parity gate of a bench configuration: the 16-bit result against the fp32 oracle on the same 16-bit inputs."""
    got, ref = got.float().cpu(), ref.float().cpu()
    if not torch.isfinite(got).all():
        sys.exit(f"bench.py: {what}: non-finite output - no number is reported for a wrong result")
    err = (got - ref).abs().max().item()
    if scores:
        err /= max(ref.abs().max().item(), 1e-30)
    bar = SCORE_RTOL if scores else OUT_ATOL
    if err > bar:
        sys.exit(f"bench.py: {what}: error {err:.3e} against the oracle exceeds {bar} - no number is reported for a wrong result")
    return round(err, 6)


def cpu_time(fn, budget_s=10.0, max_n=50, warm=1):
    for _ in range(warm):
        fn()
    ts = []
    t0 = time.perf_counter()
    while True:
        t1 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t1)
        if time.perf_counter() - t0 > budget_s or len(ts) >= max_n:
            break
    ts.sort()
    return ts[len(ts) // 2], len(ts)


def device_info(dev):
    p = torch.cuda.get_device_properties(dev)
    info = {"name": p.name, "compute_units": int(p.multi_processor_count)}
    mhz = getattr(p, "clock_rate", 0) / 1e3
    if mhz:
        info["max_engine_clock_mhz"] = round(mhz)
        # 4096 dense bf16 FLOP per clock and CU (4 SIMDs x one v_mfma_f32_32x32x16 = 32768 FLOP per 32 clocks)
        info["derived_bf16_peak_tflops"] = round(p.multi_processor_count * mhz * 1e6 * 4096 / 1e12, 1)
    mem_mhz, bus = getattr(p, "memory_clock_rate", 0) / 1e3, getattr(p, "memory_bus_width", 0)
    if mem_mhz and bus:
        info["memory_clock_mhz"], info["memory_bus_bits"] = round(mem_mhz), int(bus)
        info["derived_hbm_peak_gbs"] = round(mem_mhz * 1e6 * 2 * bus / 8 / 1e9, 1)   # double data rate
    info["hbm_gib"] = round(p.total_memory / 2 ** 30, 1)
    if not mhz:
        info["clock_note"] = "this torch build exposes no clock attribute; see roofline.sustained_mfma_clock_mhz (c3) and sysfs"
    info["sysfs"] = sysfs_gpu_state()
    return info


def sysfs_gpu_state():
    """Clock and power figures the driver exposes through sysfs, read best-effort (an ordinary user may read them on most
    installations): the engine clock level in force and the power cap / draw.  None where the files are absent."""
    import glob
    out = {}
    for card in sorted(glob.glob("/sys/class/drm/card[0-9]*/device")):
        try:
            lines = open(os.path.join(card, "pp_dpm_sclk")).read().split("\n")
        except OSError:
            continue
        cur = [l for l in lines if l.strip().endswith("*")]
        out["sclk_levels"] = [l.strip() for l in lines if l.strip()][:4]
        if cur:
            out["sclk_in_force"] = cur[0].strip()
        for name, key in (("power1_cap", "power_cap_w"), ("power1_average", "power_draw_w"), ("power1_input", "power_draw_w")):
            for f in glob.glob(os.path.join(card, "hwmon", "hwmon*", name)):
                try:
                    out[key] = round(int(open(f).read().strip()) / 1e6, 1)
                except (OSError, ValueError):
                    pass
        break
    return out or None


def sustained_mfma(dev, seconds=0.05):
    """What this box sustains right now with nothing but v_mfma_f32_32x32x16_bf16 on every SIMD (two waves each): the kernel
    of `--config ceilings`, run for about `seconds` after the same settling as the workload.  Also the clock that rate
    implies (4096 dense bf16 FLOP per clock and CU), which is the clock the power manager grants under matrix load."""
    from kernel_collections_amd import _lib, ops
    lib = _lib.lib()
    cus = ops.num_cus(dev)
    st = _lib.stream_ptr(torch.empty(1, device=dev))
    out = torch.empty(cus * 2 * 256, dtype=torch.float32, device=dev)
    iters, wgs = 2000, cus * 2
    fn = lambda i: _lib.check(lib.xkv_ceiling_mfma(_lib.ptr(out), wgs, iters, _lib.XKV_BF16, st), "xkv_ceiling_mfma")
    flop = wgs * 4 * iters * 32 * 32768
    _settle(fn)
    n = max(3, int(seconds / (flop / 1.8e15)))
    avg_ms, _ = time_kernel(fn, n, 2, settle=False)
    tf = flop / (avg_ms * 1e-3) / 1e12
    return round(tf, 1), round(tf * 1e12 / (cus * 4096) / 1e6)


# ------------------------------------------------------------------------------------------------
def bench_c3(args, dev):
    import oracle
    import kernel_collections_amd.flash_recontruction as fr
    from kernel_collections_amd import ops
    from kernel_collections_amd.flash_decoding import gqa
    from kernel_collections_amd.flash_recontruction.rope.sin_cos import rotary_apply
    B, Hq, Hkv, d, L, r, theta, layers = 16, 32, 8, 128, args.ctx, 512, 5e5, 4
    gen = torch.Generator(device=dev).manual_seed(0)
    A = randn_dev((B, L, r), 1.0, dev, gen=gen)
    kB = [randn_dev((r, Hkv * d), r ** -0.5, dev, gen=gen).view(r, Hkv, d).permute(1, 0, 2).unsqueeze(0).expand(B, Hkv, r, d)
          for _ in range(layers)]
    vB = [randn_dev((r, Hkv * d), r ** -0.5, dev, gen=gen).view(r, Hkv, d).permute(1, 0, 2).unsqueeze(0).expand(B, Hkv, r, d)
          for _ in range(layers)]
    # the decode queries, rotated to position L on the device (what a caller does before these entry points)
    q = [rotary_apply(randn_dev((B, Hq, d), 1.0, dev, gen=gen), L, theta) for _ in range(layers)]
    o = torch.empty((B, Hq, d), dtype=torch.bfloat16, device=dev)
    S = args.splits or ops.occupancy_splits(B, Hkv, L, tile=32, waves=1)
    ns = ops.uniform_splits(B, S, dev)
    scale = d ** -0.5

    def step(i):
        l = i % layers
        fr.gqa_xKV_rope(q[l], A, kB[l], A, vB[l], o, ns, S, scale, theta)

    # parity gate: sequence 0 of layer 0 against the oracle
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta)
    ref0 = oracle.gqa_factorized_rope(q[0][:1].float().cpu().unsqueeze(2), A[:1].float().cpu(), kB[0][:1].float().cpu(),
                                      A[:1].float().cpu(), vB[0][:1].float().cpu(), cos, sin, sm_scale=scale)[:, :, 0]
    step(0)
    parity = {"shared_basis": require_close(o[:1], ref0, "c3, sequence 0")}

    # dominant kernel alone: stage 1
    partial, lse = ops.workspaces(B, Hq, S, r, dev)
    inv = ops.rope_inv_freq(d, theta, dev)

    def stage1(i):
        l = i % layers
        ops.recon_stage1(q[l], A, kB[l], A, partial, lse, None, ns, None, B, Hq, Hkv, L, S, scale, True, inv, 0, None)

    first_ms = None
    if args.headline_first:   # diagnosis: the same loop as the first GPU work of the process
        first_ms, _ = time_loop(step, args.steps, args.warmup, settle=False)
    # headline: exactly --steps layer steps after the settling and --warmup steps of the same workload
    total_ms, step_q = time_loop(step, args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    k_avg_ms, k_med_ms = time_kernel(stage1, max(args.steps, 50), max(args.warmup, 10))
    flops = B * L * (2 * r * Hkv * d + 2 * Hq * d + 2 * Hq * r)
    achieved = flops / (k_avg_ms * 1e-3) / 1e12
    algo_bytes = B * L * r * 2 + 2 * r * Hkv * d * 2
    # the same box's MFMA ceiling, measured next to the kernel: tells a slower box from a slower kernel
    sus_tf, sus_mhz = sustained_mfma(dev)

    # the same workload with a value basis of its own (A_v distinct from A)
    distinct = None
    if not args.no_comparator:
        Av = randn_dev((B, L, r), 1.0, dev, gen=gen)
        o2 = torch.empty_like(o)
        fr.gqa_xKV_rope(q[0], A, kB[0], Av, vB[0], o2, ns, S, scale, theta)
        ref_d = oracle.gqa_factorized_rope(q[0][:1].float().cpu().unsqueeze(2), A[:1].float().cpu(), kB[0][:1].float().cpu(),
                                           Av[:1].float().cpu(), vB[0][:1].float().cpu(), cos, sin, sm_scale=scale)[:, :, 0]
        parity["distinct_value_basis"] = require_close(o2[:1], ref_d, "c3 with its own value basis, sequence 0")
        d_ms, d_q = time_loop(lambda i: fr.gqa_xKV_rope(q[i % layers], A, kB[i % layers], Av, vB[i % layers], o2, ns, S, scale, theta),
                              args.steps, args.warmup)
        distinct = {"us": round(d_ms * 1e3 / args.steps, 2), "step_us": d_q, "kernel": "recon_spec_kernel (scores) + latent_ring_kernel (given scores), two passes",
                    "hbm_bytes": 2 * B * L * r * 2}
        del Av

    # comparator: uncompressed bf16 flash decoding of the same shape
    comp = None
    if not args.no_comparator:
        K = randn_dev((B, L, Hkv, d), 1.0, dev, gen=gen)
        V = randn_dev((B, L, Hkv, d), 1.0, dev, gen=gen)
        Sc = ops.occupancy_splits(B, Hkv, L)
        nsc = ops.uniform_splits(B, Sc, dev)
        gqa.decode_attention_fwd(q[0], K, V, o, nsc, Sc, scale)
        parity["comparator"] = require_close(o[:1], oracle.gqa_plain(q[0][:1].float().cpu(), K[:1].float().cpu(), V[:1].float().cpu(), scale),
                                             "uncompressed comparator, sequence 0")
        comp_ms, comp_q = time_loop(lambda i: gqa.decode_attention_fwd(q[i % layers], K, V, o, nsc, Sc, scale), args.steps, args.warmup)
        comp = {"us": round(comp_ms * 1e3 / args.steps, 2), "step_us": comp_q}
        del K, V

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline_c3(Hq, Hkv, d, L, r, theta, B)

    res = {
        "metric": "us_per_layer_decode_step", "value": round(us, 2), "unit": "us",
        "higher_is_better": False,
        "ms_per_step": total_ms / args.steps, "step_us": step_q,
        "tokens_per_s": B / (us * 1e-6), "kv_tokens_scanned_per_s": B * L / (us * 1e-6),
        "config": {"workload": "c3 fused RoPE xKV decode: batch 16, 32q/8kv heads, d128, ctx %d, rank 512, "
                               "A shared by K/V and by a 4-layer group, per layer" % L, "kv_splits": S},
        "roofline": {"bound": "mfma", "kernel": "recon_spec_kernel", "achieved": round(achieved, 1),
                     "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                     "traffic": recorded_traffic("c3") if (L == 32768 and not args.splits) else None,
                     "kernel_avg_us": round(k_avg_ms * 1e3, 2), "kernel_median_us": round(k_med_ms * 1e3, 2),
                     "algorithmic_flop": flops, "hbm_side_GBps": round(algo_bytes / (k_avg_ms * 1e-3) / 1e9, 1),
                     "sustained_mfma_tflops": sus_tf, "frac_of_sustained": round(achieved / sus_tf, 4),
                     "sustained_mfma_clock_mhz": sus_mhz},
        "uncompressed_flash_decode_us": None if comp is None else comp["us"],
        "uncompressed_flash_decode_step_us": None if comp is None else comp["step_us"],
        "distinct_value_basis": distinct,
        "parity_vs_oracle": parity,
        "cpu_baseline": cpu,
    }
    if first_ms is not None:
        res["same_loop_as_first_gpu_work_us"] = round(first_ms * 1e3 / args.steps, 2)
    return res


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
    med, n = cpu_time(lambda: oracle.gqa_factorized_rope(q, A, kB, A, vB, cos, sin))
    return {"value": round(med * 1e6 * B, 1), "unit": "us", "cores": nthreads, "kind": "port",
            "sample": "1 of %d sequences (ctx %d) x %d repeats (median), eager fp32 oracle.gqa_factorized_rope; "
                      "value = per-sequence time x %d" % (B, L, n, B)}


# ------------------------------------------------------------------------------------------------
def bench_c1(args, dev):
    """Target configuration 1, the reference's own CPU-runnable case: eager fp32 factorised decode with RoPE at batch 1,
    32 q / 8 kv heads, d 128, 4096 tokens, rank 256 (K and V bases distinct), theta 5e5, query at position 4096.  The CPU
    oracle at full size is the figure the configuration names; the HIP path on the same inputs (rounded to bf16) beside it."""
    import oracle
    import kernel_collections_amd.flash_recontruction as fr
    from kernel_collections_amd import ops
    torch.manual_seed(0)
    b, Hq, Hkv, d, L, r, theta = 1, 32, 8, 128, 4096, 256, 5e5
    q = torch.randn(b, Hq, 1, d)
    A, Av = torch.randn(b, L, r), torch.randn(b, L, r)
    kB, vB = torch.randn(b, Hkv, r, d) / 16, torch.randn(b, Hkv, r, d) / 16
    cq, sq = oracle.rope_cos_sin(torch.tensor([L]), d, theta)
    q_pe = oracle.apply_rope(q, cq[0], sq[0])
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta)
    nthreads = torch.get_num_threads()
    run = lambda: oracle.gqa_factorized_rope(q_pe, A, kB, Av, vB, cos, sin)
    for _ in range(3):
        run()
    ts = []
    for _ in range(max(20, args.steps)):
        t0 = time.perf_counter()
        run()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    cpu_med = ts[len(ts) // 2]
    bf = torch.bfloat16
    q16, A16, Av16, kB16, vB16 = (t.to(bf).to(dev) for t in (q_pe[:, :, 0], A, Av, kB, vB))
    ref = oracle.gqa_factorized_rope(q16.float().cpu().unsqueeze(2), A16.float().cpu(), kB16.float().cpu(), Av16.float().cpu(),
                                     vB16.float().cpu(), cos, sin)[:, :, 0]
    o = torch.empty(b, Hq, d, dtype=bf, device=dev)
    S = args.splits or 8
    ns = ops.uniform_splits(b, S, dev)
    step = lambda i: fr.gqa_xKV_rope(q16, A16, kB16, Av16, vB16, o, ns, S, d ** -0.5, theta)
    step(0)
    parity = require_close(o, ref, "c1")
    total_ms, step_q = time_loop(step, args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    flops = b * L * (2 * r * Hkv * d + 2 * Hq * d + 2 * Hq * r)
    tf = flops / (us * 1e-6) / 1e12
    return {
        "metric": "us_per_layer_decode_step", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps, "step_us": step_q,
        "config": {"workload": "c1 factorised decode with RoPE: batch 1, 32q/8kv, d128, 4096 tokens, K rank 256 / V rank 256 "
                               "(HIP path in bf16 on the CPU case's inputs)", "kv_splits": S},
        "roofline": {"bound": "mfma", "kernel": "recon_duo_kernel", "achieved": round(tf, 2), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tf / PEAK_BF16_TFLOPS, 5), "traffic": None,
                     "note": "whole call over algorithmic FLOP; at 4096 tokens the call is launch- and latency-bound",
                     "algorithmic_flop": flops},
        "parity_vs_oracle": parity,
        "cpu_baseline": {"value": round(cpu_med * 1e6, 1), "unit": "us", "cores": nthreads, "kind": "port",
                         "p20": round(ts[len(ts) // 5] * 1e6, 1), "p80": round(ts[len(ts) * 4 // 5] * 1e6, 1),
                         "sample": "the whole configuration (fp32, full size), median of %d runs after 3 warm-ups, "
                                   "eager oracle.gqa_factorized_rope" % len(ts)},
    }


# ------------------------------------------------------------------------------------------------
def bench_c2(args, dev):
    import oracle
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
    call = lambda i: fr.qAB_no_pe_v1(q, As[i % nbuf], Bm, sm_scale=scale, out_dtype=torch.float32)
    ref0 = oracle.qab_nope(q[:1].float().cpu(), As[0][:1].float().cpu(), Bm[:1].float().cpu()) * scale
    parity = require_close(call(0)[:1], ref0, "c2, sequence 0", scores=True)
    q3 = q.reshape(B, Hq, d)
    hi, lo = ops.absorb_q(q3, Bm)
    out = torch.empty((B, Hq, 1, L), dtype=torch.float32, device=dev)
    S = args.splits or ops.latent_splits(B, 1, L, r)
    ns = ops.uniform_splits(B, S, dev)

    def scan(i):
        A = As[i % nbuf]
        ops.latent_stage1(hi, lo, None, (A, A.stride(0), A.stride(1), 0, r), None, None, None, None, out, ns, None,
                          B, Hq, 1, L, S, scale)

    k_avg_ms, k_med_ms = time_kernel(scan, max(args.steps, 50), max(args.warmup, 10))
    warm_avg_ms, _ = time_kernel(lambda i: (scan(0)), max(args.steps, 50), max(args.warmup, 10))   # one buffer: may sit in cache
    total_ms, step_q = time_loop(call, args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    algo_bytes = B * L * r * 2 + B * Hq * L * 4 + r * Hkv * d * 2 + B * Hq * d * 2
    gbs = algo_bytes / (k_avg_ms * 1e-3) / 1e9
    cpu = None
    if not args.no_cpu:
        qc, Ac, Bc = torch.randn(B, Hq, 1, d), torch.randn(B, L, r), (torch.randn(1, Hkv, r, d) * r ** -0.5).expand(B, Hkv, r, d)
        med, n = cpu_time(lambda: oracle.qab_nope(qc, Ac, Bc) * scale, budget_s=12.0, max_n=20)
        cpu = {"value": round(med * 1e6, 1), "unit": "us", "cores": torch.get_num_threads(), "kind": "port",
               "sample": "the whole configuration (fp32, full size), median of %d runs, eager oracle.qab_nope "
                         "(reconstructs K, as the reference's eager form does)" % n}
    return {
        "metric": "us_per_qAB_no_pe_call", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps, "step_us": step_q,
        "config": {"workload": "c2 qAB_no_pe scores: batch 8, 32q/8kv, d128, L16384, rank 512, bf16 in / fp32 out", "kv_splits": S,
                   "buffers_rotated": nbuf},
        "roofline": {"bound": "hbm", "kernel": "latent_ring_kernel(scores)", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None if args.splits else recorded_traffic("c2"),
                     "kernel_avg_us": round(k_avg_ms * 1e3, 2), "kernel_median_us": round(k_med_ms * 1e3, 2),
                     "kernel_avg_us_one_buffer": round(warm_avg_ms * 1e3, 2), "algorithmic_bytes": algo_bytes},
        "parity_vs_oracle": parity,
        "cpu_baseline": cpu,
    }


def bench_c5(args, dev):
    import oracle
    from kernel_collections_amd import ops
    from kernel_collections_amd.flash_decoding import mla2
    B, H, L, c, e = 64, 16, 8192, 512, 64
    gen = torch.Generator(device=dev).manual_seed(0)
    nbuf = 2   # 2 x 576 MiB of latent + rope keys: more than the 256 MiB last-level cache
    ckvs = [randn_dev((B, L, 1, c), 1.0, dev, gen=gen) for _ in range(nbuf)]
    kpes = [randn_dev((B, L, 1, e), 1.0, dev, gen=gen) for _ in range(nbuf)]
    qn, qr = randn_dev((B, H, c), 0.3, dev, gen=gen), randn_dev((B, H, e), 1.0, dev, gen=gen)
    scale = 1 / math.sqrt(192)
    call = lambda i: mla2.mla_decode_attention_fwd(qn, qr, ckvs[i % nbuf], kpes[i % nbuf], scale)
    parity = require_close(call(0)[:1], oracle.mla_ref(qn[:1].float().cpu(), qr[:1].float().cpu(), ckvs[0][:1].float().cpu(),
                                                       kpes[0][:1].float().cpu(), scale), "c5, sequence 0")
    S = args.splits or ops.latent_splits(B, 1, L, 512)
    ns = ops.uniform_splits(B, S, dev)
    partial, lse = ops.workspaces(B, H, S, c, dev)
    k_avg_ms, k_med_ms = time_kernel(lambda i: mla2.decoding_stage1(qn, qr, ckvs[i % nbuf], kpes[i % nbuf], partial, lse, ns, S, scale),
                                     max(args.steps, 50), max(args.warmup, 10))
    total_ms, step_q = time_loop(call, args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    algo_bytes = B * L * (c + e) * 2
    gbs = algo_bytes / (k_avg_ms * 1e-3) / 1e9
    flops = B * L * H * (c + e + c) * 2
    cpu = None
    if not args.no_cpu:
        qnc, qrc = torch.randn(B, H, c) * 0.3, torch.randn(B, H, e)
        cc, kc = torch.randn(B, L, 1, c), torch.randn(B, L, 1, e)
        med, n = cpu_time(lambda: oracle.mla_ref(qnc, qrc, cc, kc, scale), budget_s=12.0, max_n=20)
        cpu = {"value": round(med * 1e6, 1), "unit": "us", "cores": torch.get_num_threads(), "kind": "port",
               "sample": "the whole configuration (fp32, full size), median of %d runs, eager oracle.mla_ref" % n}
    return {
        "metric": "us_per_mla_decode_step", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps, "step_us": step_q,
        "config": {"workload": "c5 MLA absorbed decode: batch 64, 16 heads, latent 512 + rope 64, ctx 8192, bf16", "kv_splits": S,
                   "buffers_rotated": nbuf},
        "roofline": {"bound": "hbm", "kernel": "latent_ring_kernel", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None if args.splits else recorded_traffic("c5"),
                     "kernel_avg_us": round(k_avg_ms * 1e3, 2), "kernel_median_us": round(k_med_ms * 1e3, 2),
                     "algorithmic_bytes": algo_bytes, "mfma_TFLOPs": round(flops / (k_avg_ms * 1e-3) / 1e12, 1)},
        "parity_vs_oracle": parity,
        "cpu_baseline": cpu,
    }


def c4_lengths(B=32):
    g = torch.Generator().manual_seed(0)
    u = torch.rand(B, generator=g)
    return torch.floor(torch.exp(math.log(1024) + u * (math.log(131072) - math.log(1024)))).to(torch.int64).tolist()


def bench_c4(args, dev, vfact):
    import oracle
    from kernel_collections_amd import ops
    from kernel_collections_amd.flash_decoding import gqa
    B, Hq, Hkv, d, rv, split = 32, 32, 8, 128, 512, args.splits or 4096
    lens = c4_lengths(B)
    Lmax = max(lens)
    gen = torch.Generator(device=dev).manual_seed(0)
    K = randn_dev((B, Lmax, Hkv, d), 1.0, dev, gen=gen)
    q = randn_dev((B, Hq, d), 1.0, dev, gen=gen)
    o = torch.empty_like(q)
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
        ref_of = lambda i, n: oracle.gqa_v_only(q[i:i + 1].float().cpu().unsqueeze(2), K[i:i + 1, :n].float().cpu().transpose(1, 2),
                                                vA[i:i + 1, :n].float().cpu(), vB[i:i + 1].float().cpu(), sm_scale=scale)[:, :, 0]
    else:
        V = randn_dev((B, Lmax, Hkv, d), 1.0, dev, gen=gen)
        fn = lambda i: gqa.decode_attention_fwd(q, K, V, o, ns, S, scale, kv_lens=kl)
        per_tok = 4096
        ref_of = lambda i, n: oracle.gqa_plain(q[i:i + 1].float().cpu(), K[i:i + 1, :n].float().cpu(), V[i:i + 1, :n].float().cpu(), scale)
    order = sorted(range(B), key=lambda i: lens[i])
    fn(0)
    parity = {"sequence_%d_len_%d" % (i, lens[i]): require_close(o[i:i + 1], ref_of(i, lens[i]), "c4, sequence %d" % i)
              for i in (order[0], order[B // 2], order[-1])}
    total_ms, step_q = time_loop(fn, args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    # the same call with the caller's splits taken as they are (split_cap_tokens = 0: the kernels add no splits)
    saved = gqa.MAX_SPLIT_TOKENS, gqa.MAX_SPLIT_TOKENS_WIDE
    gqa.MAX_SPLIT_TOKENS = gqa.MAX_SPLIT_TOKENS_WIDE = 0
    try:
        asis_ms, _ = time_loop(fn, args.steps, args.warmup)
    finally:
        gqa.MAX_SPLIT_TOKENS, gqa.MAX_SPLIT_TOKENS_WIDE = saved
    algo_bytes = sum(lens) * per_tok
    gbs = algo_bytes / (us * 1e-6) / 1e9
    # the split length the wrappers planned on the device for this batch (read back here, outside every timed region)
    plan_S = ops.capped_splits(Lmax, S, gqa.MAX_SPLIT_TOKENS_WIDE)
    limit = int(ops.plan_splits(kl, ns, plan_S, gqa.MAX_SPLIT_TOKENS_WIDE, ops.num_cus())[0].item())
    cpu = None
    if not args.no_cpu:
        # an eighth of every length (fp32): the scan is linear in the number of tokens, value = time x 8
        l8 = [max(1, n // 8) for n in lens]
        L8 = max(l8)
        qc, Kc = torch.randn(B, Hq, d), torch.randn(B, L8, Hkv, d)
        if vfact:
            vAc, vBc = torch.randn(B, L8, rv), torch.randn(B, Hkv, rv, d) * rv ** -0.5
            run = lambda: oracle.ragged_apply(
                lambda q_, K_, vA_, vB_: oracle.gqa_v_only(q_.unsqueeze(2), K_.transpose(1, 2), vA_, vB_, sm_scale=scale)[:, :, 0],
                l8, (qc, Kc, vAc, vBc), (None, 1, 1, None))
        else:
            Vc = torch.randn(B, L8, Hkv, d)
            run = lambda: oracle.ragged_apply(oracle.gqa_plain, l8, (qc, Kc, Vc), (None, 1, 1), sm_scale=scale)
        med, n = cpu_time(run, budget_s=12.0, max_n=20)
        cpu = {"value": round(med * 1e6 * 8, 1), "unit": "us", "cores": torch.get_num_threads(), "kind": "port",
               "sample": "all 32 sequences at an eighth of their lengths (fp32), median of %d runs, eager oracle via ragged_apply; "
                         "value = time x 8 (the scan is linear in tokens)" % n}
    return {
        "metric": "us_per_ragged_decode_step", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps, "step_us": step_q,
        "config": {"workload": "c4 ragged split-K GQA%s: batch 32, lens log-uniform [1024,131072], %d-token splits at the call"
                               % (" V-factorised r512" if vfact else "", split), "sum_len": sum(lens), "max_len": Lmax,
                   "kv_splits_max_at_the_call": S,
                   "split_length_planned_on_the_device_tokens": limit,
                   "kv_splits_max_in_the_kernel": max(max(s_, -(-n // limit)) for n, s_ in zip(lens, ns_l)),
                   "workgroups_with_work": sum(max(s_, -(-n // limit)) for n, s_ in zip(lens, ns_l)),
                   "compute_units": ops.num_cus()},
        "roofline": {"bound": "hbm", "kernel": "latent_ring_kernel",
                     "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4),
                     "traffic": recorded_traffic("c4") if (not vfact and split == 4096) else None,
                     "note": "whole call (stage 1 + merge) over algorithmic bytes", "algorithmic_bytes": algo_bytes},
        "caller_splits_as_they_are_us": round(asis_ms * 1e3 / args.steps, 2),
        "parity_vs_oracle": parity,
        "cpu_baseline": cpu,
    }


def bench_pdsep(args, dev):
    """Prefix + tail decode at the shape of the reference's own script (test_mla_decoding_new.py:66-73): batch 1,
    32 heads on one kv head, head_dim 512, prefix 262144 tokens factorised at rank 512, 128 decoded tokens, fp16."""
    import oracle
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
    Kp = oracle.reconstruct(kA.float().cpu(), kB.float().cpu()).transpose(1, 2)
    Vp = oracle.reconstruct(vA.float().cpu(), vB.float().cpu()).transpose(1, 2)
    ref = oracle.gqa_plain(q.float().cpu(), torch.cat([Kp, Kd.float().cpu()], 1), torch.cat([Vp, Vd.float().cpu()], 1), scale)
    parity = require_close(fn(0), ref, "prefix + tail")
    del Kp, Vp
    total_ms, step_q = time_loop(fn, args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    algo_bytes = B * Lp * 2 * r * 2 + B * Ld * 2 * hd * 2 + 2 * r * hd * 2
    gbs = algo_bytes / (us * 1e-6) / 1e9
    return {
        "metric": "us_per_prefix_tail_decode_step", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps, "step_us": step_q,
        "config": {"workload": "prefix + tail decode: batch 1, 32 heads / 1 kv head, head_dim 512, prefix 262144 at rank 512 "
                               "(k_A, v_A), tail 128 plain, fp16"},
        "roofline": {"bound": "hbm", "kernel": "latent_ring_kernel", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None,
                     "note": "whole call (absorb, 2 x stage 1, 2 x merge) over algorithmic bytes", "algorithmic_bytes": algo_bytes},
        "parity_vs_oracle": parity,
        "cpu_baseline": None,
    }


def bench_qabrope(args, dev):
    """RoPE-aware key reconstruction scores at the shape of the reference's own sweep (test_qAB_rope.py:85-125):
    batch 1, 32 q / 8 kv heads, head_dim 128, rank 192, fp16, kv_len = --ctx (the sweep runs 16K .. 128K)."""
    import oracle
    import kernel_collections_amd.flash_recontruction as fr
    B, Hq, Hkv, d, r, L, theta = 1, 32, 8, 128, args.rank, args.ctx, 1e7
    dt = torch.float16 if args.dtype == "fp16" else torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(0)
    q = randn_dev((B, Hq, 1, d), 0.2, dev, dt, gen)
    A = randn_dev((B, L, r), 0.2, dev, dt, gen)
    Bk = randn_dev((B, Hkv, r, d), 0.2, dev, dt, gen)
    n = min(L, 8192)
    cos, sin = oracle.rope_cos_sin(torch.arange(n), d, theta)
    ref = oracle.qab_rope(q.float().cpu(), A[:, :n].float().cpu(), Bk.float().cpu(), cos, sin)
    parity = require_close(fr.qAB_rope_v1(q, A, Bk, theta)[..., :n], ref, "qAB with RoPE, first %d tokens" % n, scores=True)
    total_ms, step_q = time_loop(lambda i: fr.qAB_rope_v1(q, A, Bk, theta), args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    flops = B * L * (2 * r * Hkv * d + 2 * Hq * d)
    tf = flops / (us * 1e-6) / 1e12
    return {
        "metric": "us_per_qAB_rope_call", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps, "step_us": step_q,
        "config": {"workload": "qAB with RoPE, scores only: batch 1, 32q/8kv, d128, rank %d, kv_len %d, %s" % (r, L, args.dtype)},
        "roofline": {"bound": "mfma", "kernel": "recon_stage1_kernel(scores)", "achieved": round(tf, 1), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tf / PEAK_BF16_TFLOPS, 4), "traffic": None,
                     "note": "whole call over algorithmic FLOP", "algorithmic_flop": flops,
                     "hbm_side_GBps": round((B * L * r * 2 + B * Hq * L * 2) / (us * 1e-6) / 1e9, 1)},
        "parity_vs_oracle": parity,
        "cpu_baseline": None,
    }


def bench_ropedecode(args, dev):
    """Fused xKV decode with RoPE and SEPARATE key / value bases at the default shape of the reference's variant table
    (test_attention_profiling.py:511-517): batch 1, 32 q / 8 kv heads, head_dim 128, kv_len 131072, K rank 384, V rank 512."""
    import oracle
    import kernel_collections_amd.flash_recontruction as fr
    from kernel_collections_amd import ops
    from kernel_collections_amd.flash_decoding import gqa
    B, Hq, Hkv, d, L, rk, rv, theta = 1, 32, 8, 128, 131072, args.rank if args.rank != 192 else 384, 512, 5e5
    gen = torch.Generator(device=dev).manual_seed(0)
    q = randn_dev((B, Hq, d), 1.0, dev, torch.bfloat16, gen)
    kA, vA = randn_dev((B, L, rk), 1.0, dev, torch.bfloat16, gen), randn_dev((B, L, rv), 1.0, dev, torch.bfloat16, gen)
    kB = randn_dev((B, Hkv, rk, d), rk ** -0.5, dev, torch.bfloat16, gen)
    vB = randn_dev((B, Hkv, rv, d), rv ** -0.5, dev, torch.bfloat16, gen)
    o = torch.empty_like(q)
    S = args.splits or ops.occupancy_splits(B, Hkv, L, tile=32, waves=1)
    ns = ops.uniform_splits(B, S, dev)
    fn = lambda i: fr.gqa_xKV_rope(q, kA, kB, vA, vB, o, ns, S, d ** -0.5, theta)
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta)
    ref = oracle.gqa_factorized_rope(q.float().cpu().unsqueeze(2), kA.float().cpu(), kB.float().cpu(), vA.float().cpu(),
                                     vB.float().cpu(), cos, sin, sm_scale=d ** -0.5)[:, :, 0]
    fn(0)
    parity = require_close(o, ref, "fused RoPE decode, separate bases")
    total_ms, step_q = time_loop(fn, args.steps, args.warmup)
    us = total_ms * 1e3 / args.steps
    K, V = randn_dev((B, L, Hkv, d), 1.0, dev, gen=gen), randn_dev((B, L, Hkv, d), 1.0, dev, gen=gen)
    Sc = ops.occupancy_splits(B, Hkv, L)
    nsc = ops.uniform_splits(B, Sc, dev)
    comp_ms, _ = time_loop(lambda i: gqa.decode_attention_fwd(q, K, V, o, nsc, Sc, d ** -0.5), args.steps, args.warmup)
    flops = B * L * (2 * rk * Hkv * d + 2 * Hq * d + 2 * Hq * rv)
    tf = flops / (us * 1e-6) / 1e12
    return {
        "metric": "us_per_layer_decode_step", "value": round(us, 2), "unit": "us", "higher_is_better": False,
        "ms_per_step": total_ms / args.steps, "step_us": step_q,
        "config": {"workload": "fused RoPE xKV decode, separate bases: batch 1, 32q/8kv, d128, kv_len %d, K rank %d, V rank %d, bf16"
                               % (L, rk, rv), "kv_splits": S},
        "roofline": {"bound": "mfma", "kernel": "recon_spec_kernel (scores) + latent_ring_kernel (given scores), two passes", "achieved": round(tf, 1), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tf / PEAK_BF16_TFLOPS, 4), "traffic": None,
                     "note": "whole call (pack, stage 1, merge) over algorithmic FLOP", "algorithmic_flop": flops,
                     "hbm_side_GBps": round(B * L * (rk + rv) * 2 / (us * 1e-6) / 1e9, 1)},
        "uncompressed_flash_decode_us": round(comp_ms * 1e3 / args.steps, 2),
        "parity_vs_oracle": parity,
        "cpu_baseline": None,
    }


def bench_ceilings(args, dev):
    """What the device sustains with nothing but the bounding instruction: v_mfma_f32_32x32x16_bf16 on register operands
    on every wave, and a plain HBM read stream (into registers, and directly into LDS)."""
    from ctypes import c_int64
    from kernel_collections_amd import _lib, ops
    lib = _lib.lib()
    cus = ops.num_cus(dev)
    st = _lib.stream_ptr(torch.empty(1, device=dev))
    out = torch.empty(cus * 8 * 256, dtype=torch.float32, device=dev)
    res = {}
    iters = 4000
    for wpc in (1, 2):          # workgroups per CU: 4 or 8 waves per CU, i.e. 1 or 2 per SIMD
        wgs = cus * wpc
        fn = lambda i: _lib.check(lib.xkv_ceiling_mfma(_lib.ptr(out), wgs, iters, _lib.XKV_BF16, st), "xkv_ceiling_mfma")
        avg_ms, _ = time_kernel(fn, 20, 5)
        res["mfma_32x32x16_bf16_%d_waves_per_simd_tflops" % wpc] = round(wgs * 4 * iters * 32 * 32768 / (avg_ms * 1e-3) / 1e12, 1)
    nbytes = 2 << 30
    bufs = [torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(i + 1) for i in range(2)]   # 2 x 2 GiB: no cache reuse
    for name, to_lds, depth, wpc in (("registers_2wg", 0, 1, 2), ("registers_4wg", 0, 1, 4), ("registers_8wg", 0, 1, 8),
                                     ("lds_depth4_1wg", 1, 4, 1), ("lds_depth2_2wg", 1, 2, 2), ("lds_depth3_1wg", 1, 3, 1),
                                     ("registers_then_lds_depth2_1wg", 2, 2, 1), ("registers_then_lds_depth4_1wg", 2, 4, 1),
                                     ("registers_then_lds_depth6_1wg", 2, 6, 1), ("registers_then_lds_depth4_2wg", 2, 4, 2)):
        wgs = cus * wpc
        got = wgs * 4 * 8192 * (nbytes // (wgs * 4 * 8192))
        if to_lds == 2:
            got = wgs * 4 * 8192 * (nbytes // (wgs * 4 * 8192) // depth * depth)
        fn = lambda i: _lib.check(lib.xkv_ceiling_stream(_lib.ptr(bufs[i % 2]), c_int64(nbytes), wgs, to_lds, depth, _lib.ptr(out), st),
                                  "xkv_ceiling_stream")
        avg_ms, _ = time_kernel(fn, 20, 5)
        if to_lds == 2:   # the kernel counts the 16-byte packets it handed on: every byte it is credited with was read
            torch.cuda.synchronize()
            seen = int(out[:wgs * 256].double().sum().item())
            if seen * 16 != got:
                sys.exit("bench.py: ceilings: the stream kernel handed on %d bytes, expected %d" % (seen * 16, got))
        res["hbm_stream_to_%s_gbs" % name] = round(got / (avg_ms * 1e-3) / 1e9, 1)
    best_mfma = max(v for k, v in res.items() if k.startswith("mfma"))
    best_hbm = max(v for k, v in res.items() if k.startswith("hbm"))
    return {
        "metric": "sustained_ceilings", "value": best_mfma, "unit": "TFLOP/s", "higher_is_better": True, "ms_per_step": 0.0,
        "config": {"workload": "ceilings: pure v_mfma_f32_32x32x16_bf16 loop on every wave; plain 2 GiB HBM read stream"},
        "roofline": {"bound": "mfma", "kernel": "ceiling_mfma_kernel", "achieved": best_mfma, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(best_mfma / PEAK_BF16_TFLOPS, 4), "traffic": None},
        "hbm_stream": {"achieved": best_hbm, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(best_hbm / PEAK_HBM_GBS, 4)},
        "ceilings": res,
        "cpu_baseline": None,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--config", default="c3", choices=["c1", "c2", "c3", "c4", "c4v", "c5", "pdsep", "qabrope", "ropedecode", "ceilings"])
    ap.add_argument("--ctx", type=int, default=32768)
    ap.add_argument("--splits", type=int, default=0, help="kv splits (c4 / c4v: tokens per split at the call, default 4096)")
    ap.add_argument("--rank", type=int, default=192, help="rank of the qabrope workload (ropedecode: K rank, default 384)")
    ap.add_argument("--dtype", default="fp16", choices=["fp16", "bf16"], help="operand type of the qabrope workload")
    ap.add_argument("--settle", type=float, default=1.5,
                    help="seconds of untimed calls of a workload before each of its measurements (the device reaches the clock "
                         "it sustains under that load); reported as settle_s")
    ap.add_argument("--traffic-line", nargs=2, metavar=("WORKLOAD", "BYTES"),
                    help="print the line of profiles/hbm_traffic_table.txt for a workload's measured HBM bytes and exit")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-comparator", action="store_true")
    ap.add_argument("--headline-first", action="store_true",
                    help="c3: also time the step loop as the first GPU work of the process (a device that has not reached its "
                         "sustained clock), reported as same_loop_as_first_gpu_work_us")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run 3 plain device copies of 512 MiB (a kernel of known traffic, for scaling rocprof's "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.traffic_line:
        print(traffic_line(args.traffic_line[0], int(float(args.traffic_line[1]))))
        return
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    from kernel_collections_amd import _lib
    _lib.lib()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    global SETTLE_S
    SETTLE_S = max(0.0, args.settle)
    if args.calib_copy:
        src = torch.empty(512 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    fns = {"c1": bench_c1, "c2": bench_c2, "c3": bench_c3, "c5": bench_c5, "pdsep": bench_pdsep, "qabrope": bench_qabrope,
           "ropedecode": bench_ropedecode, "ceilings": bench_ceilings,
           "c4": lambda a, d_: bench_c4(a, d_, False), "c4v": lambda a, d_: bench_c4(a, d_, True)}
    res = fns[args.config](args, dev)
    line = {"metric": res.pop("metric"), "value": res.pop("value"), "unit": res.pop("unit"), "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": res.pop("ms_per_step"),
            "higher_is_better": res.pop("higher_is_better"), "scaling": "weak", "vs_baseline": None,
            "dtype": "fp16" if (args.config == "pdsep" or (args.config == "qabrope" and args.dtype == "fp16")) else "bf16", "data": "synthetic"}
    line.update(res)
    line["settle_s"] = args.settle
    line["device"] = device_info(dev)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
