"""Variant table for one decode step, in the spirit of the reference's test_attention_profiling.py:213-474:
every attention variant of the path on the same synthetic shape, its time, its speed-up over eager attention and over
the uncompressed flash decode, and its distance from the eager result.

    python -m kernel_collections_amd.profiling --kv_len 131072 --k_rank 384 --v_rank 512 [--batch 1] [--dtype bf16]

Same flags as the reference script (:511-517: --num_heads --num_kv_heads --head_dim --kv_len --k_rank --v_rank).
--profile runs one pass over the variants under torch.profiler, one ``record_function`` range per variant, prints the
per-kernel table and exports the chrome trace (``--trace_path``, default ./xkv_profile_trace.json), as the reference's
profiling pass does (:118-211).
--sweep is the key-reconstruction sweep of the reference's test_qAB_rope.py:85-167 / test_fused_key_reconstruction.py:94-100:
kv_len 2^14 .. 2^17 at batch 1, rank --k_rank (192 there), fp16 by default; per kv_len the plain q.K^T of torch and the
four qAB-with-RoPE entry points (v2 on a precomputed sin/cos table), each as median / 20 % / 80 % quantile over --repeat
timed calls after --warmup (the reference: 100 after 25).
The eager and SDPA rows are torch on the same device (comparators, as in the reference); every other row runs the
HIP kernels of this package."""
from __future__ import annotations

import argparse
import math

import torch

import kernel_collections_amd.flash_recontruction as fr
from kernel_collections_amd import ops
from kernel_collections_amd.flash_decoding import gqa


def _time(fn, warmup=5, repeat=20):
    for _ in range(warmup):
        fn()
    st, en = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    st.record()
    for _ in range(repeat):
        fn()
    en.record()
    torch.cuda.synchronize()
    return st.elapsed_time(en) / repeat


def _quantiles(fn, warmup=25, repeat=100):
    """(median, 20 %, 80 %) in ms over `repeat` calls timed one by one with HIP events (what triton.testing.do_bench
    returns for quantiles=[0.5, 0.2, 0.8], test_qAB_rope.py:136-163)."""
    for _ in range(warmup):
        fn()
    st = [torch.cuda.Event(enable_timing=True) for _ in range(repeat)]
    en = [torch.cuda.Event(enable_timing=True) for _ in range(repeat)]
    torch.cuda.synchronize()
    for i in range(repeat):
        st[i].record()
        fn()
        en[i].record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in zip(st, en))
    pick = lambda f: ts[min(repeat - 1, int(f * repeat))]
    return pick(0.5), pick(0.2), pick(0.8)


def sweep(args):
    """kv_len sweep of the RoPE key-reconstruction scores; returns [(kv_len, {operation: (median, p20, p80)})]."""
    from kernel_collections_amd.flash_recontruction.rope.sin_cos import rotary_sin_cos
    dev = torch.device("cuda:0")
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float16
    hq, hkv, d, r, theta = args.num_heads, args.num_kv_heads, args.head_dim, args.k_rank, 1e7
    g = torch.Generator(device=dev).manual_seed(0)
    rnd = lambda shape: torch.randn(shape, device=dev, dtype=torch.float32, generator=g).to(dtype)
    rows = []
    for e in range(args.sweep_min, args.sweep_max + 1):
        L = 2 ** e
        q, K = rnd((1, hq, 1, d)), rnd((1, hkv, L, d))
        Ak, Bk = rnd((1, L, r)), rnd((1, hkv, r, d))
        sin, cos = rotary_sin_cos(L, theta, 0, dtype=dtype, device=dev)
        sin_cos = torch.cat((sin, cos), dim=-1)
        qg = q.reshape(1, hkv, hq // hkv, d)
        ops_ = {
            "qK (torch)": lambda: torch.matmul(qg, K.transpose(-1, -2)),
            "qAB_v1": lambda: fr.qAB_rope_v1(q, Ak, Bk, theta),
            "qAB_v2 (table)": lambda: fr.qAB_rope_v2(q, Ak, Bk, sin_cos),
            "qAB_v3": lambda: fr.qAB_rope_v3(q, Ak, Bk, theta),
            "qAB_v4": lambda: fr.qAB_rope_v4(q, Ak, Bk, theta),
        }
        rows.append((L, {name: _quantiles(fn, args.warmup, args.repeat) for name, fn in ops_.items()}))
    names = list(rows[0][1])
    print("\n=== qK vs qAB with RoPE: batch 1, %d q / %d kv heads, head_dim %d, rank %d, %s; ms as median [20 %% .. 80 %%] ==="
          % (hq, hkv, d, r, args.dtype))
    print("%10s " % "kv_len" + " ".join("%26s" % n for n in names))
    for L, res in rows:
        print("%10d " % L + " ".join("%10.4f [%6.4f..%6.4f]" % res[n] for n in names))
    return rows


def eager_attention(q, K, V, scale):
    """Plain GQA decode in torch (attention.py:7-60 of the reference): q [b,Hq,d], K/V [b,L,Hkv,d]."""
    b, hq, d = q.shape
    hkv = K.shape[2]
    s = torch.einsum("bkgd,blkd->bkgl", q.reshape(b, hkv, hq // hkv, d), K) * scale
    p = torch.softmax(s, dim=-1, dtype=torch.float32).to(q.dtype)
    return torch.einsum("bkgl,blkd->bkgd", p, V).reshape(b, hq, V.shape[-1])


def sdpa_attention(q, K, V, scale):
    b, hq, d = q.shape
    hkv = K.shape[2]
    Kh = K.permute(0, 2, 1, 3).repeat_interleave(hq // hkv, dim=1)
    Vh = V.permute(0, 2, 1, 3).repeat_interleave(hq // hkv, dim=1)
    return torch.nn.functional.scaled_dot_product_attention(q.unsqueeze(2), Kh, Vh, scale=scale).squeeze(2)


def build_variants(batch, hq, hkv, d, L, rk, rv, dtype, dev, theta=5e5):
    g = torch.Generator(device=dev).manual_seed(0)
    rnd = lambda shape, std: (torch.randn(shape, device=dev, dtype=torch.float32, generator=g) * std).to(dtype)
    q = rnd((batch, hq, d), 1.0)
    kA, vA = rnd((batch, L, rk), 1.0), rnd((batch, L, rv), 1.0)
    kB, vB = rnd((batch, hkv, rk, d), rk ** -0.5), rnd((batch, hkv, rv, d), rv ** -0.5)
    # the uncompressed cache the factorised one stands for (so that every row answers the same question)
    K = torch.einsum("blr,bhrd->blhd", kA.float(), kB.float()).to(dtype)
    V = torch.einsum("blr,bhrd->blhd", vA.float(), vB.float()).to(dtype)
    scale = 1.0 / math.sqrt(d)
    S = ops.occupancy_splits(batch, hkv, L)
    ns = ops.uniform_splits(batch, S, dev)
    S1 = ops.latent_splits(batch, 1, L, rk, absorbed=True)
    ns1 = ops.uniform_splits(batch, S1, dev)
    Sr = ops.occupancy_splits(batch, hkv, L, tile=32, waves=1)
    Sv = ops.occupancy_splits(batch, 1, L, tile=32, waves=1)   # V-only factorised: one workgroup serves every head of a split
    nsv = ops.uniform_splits(batch, Sv, dev)
    nsr = ops.uniform_splits(batch, Sr, dev)
    o = torch.empty_like(q)
    variants = [
        ("Standard attention (torch eager)", lambda: eager_attention(q, K, V, scale), "plain"),
        ("SDPA (torch)", lambda: sdpa_attention(q, K, V, scale), "plain"),
        ("Flash decode (uncompressed K, V)", lambda: gqa.decode_attention_fwd(q, K, V, o, ns, S, scale), "plain"),
        ("Factorised V only", lambda: gqa.decode_attention_fwd_v_factorized(q, K, vA, vB, o, nsv, Sv, scale), "plain"),
        ("Fused xKV, K only", lambda: fr.gqa_xKV_no_pe_k_only(q, kA, kB, V, o, ns1, S1, scale), "plain"),
        ("Fused xKV", lambda: fr.gqa_xKV_no_pe(q, kA, kB, vA, vB, o, ns1, S1, scale), "plain"),
        ("Fused xKV v2", lambda: fr.gqa_xKV_no_pe_v2(q, kA, kB, vA, vB, ns1, S1, scale), "plain"),
        ("Fused xKV with RoPE", lambda: fr.gqa_xKV_rope(q, kA, kB, vA, vB, o, nsr, Sr, scale, theta), "rope"),
    ]
    return variants


def run(args):
    dev = torch.device("cuda:0")
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float16
    variants = build_variants(args.batch, args.num_heads, args.num_kv_heads, args.head_dim, args.kv_len, args.k_rank,
                              args.v_rank, dtype, dev)
    if args.profile:
        from torch.profiler import ProfilerActivity, profile, record_function
        for _, fn, _ in variants:   # first calls (module load, allocator growth) stay out of the trace
            fn()
        torch.cuda.synchronize()
        with profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA]) as prof:
            for name, fn, _ in variants:
                with record_function(name):
                    fn()
                torch.cuda.synchronize()
        print(prof.key_averages().table(sort_by="cuda_time_total", row_limit=20))
        prof.export_chrome_trace(args.trace_path)
        print("chrome trace written to %s" % args.trace_path)
        return []
    ref = variants[0][1]().float()
    rows = []
    for name, fn, kind in variants:
        out = fn()
        err = (out.float() - ref).abs().max().item() if kind == "plain" else float("nan")
        rows.append((name, _time(fn, args.warmup, args.repeat), err))
    t_std = rows[0][1]
    t_flash = rows[2][1]
    print("\n=== Benchmark results: batch %d, %d q / %d kv heads, head_dim %d, kv_len %d, K rank %d, V rank %d, %s ==="
          % (args.batch, args.num_heads, args.num_kv_heads, args.head_dim, args.kv_len, args.k_rank, args.v_rank, args.dtype))
    print("%-36s %10s %12s %12s %14s" % ("variant", "ms", "vs standard", "vs flash", "max |diff|"))
    for name, t, err in rows:
        print("%-36s %10.4f %11.2fx %11.2fx %14s" % (name, t, t_std / t, t_flash / t, "-" if math.isnan(err) else "%.3e" % err))
    total = args.num_kv_heads * args.head_dim
    print("\n=== Rank information ===")
    print("Per-layer K rank: %d (compression %.2fx)   V rank: %d (compression %.2fx)" %
          (args.k_rank, total / args.k_rank, args.v_rank, total / args.v_rank))
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description="Benchmark the attention variants of the xKV decode path")
    ap.add_argument("--num_heads", type=int, default=32)
    ap.add_argument("--num_kv_heads", type=int, default=8)
    ap.add_argument("--head_dim", type=int, default=128)
    ap.add_argument("--kv_len", type=int, default=128 * 1024)
    ap.add_argument("--k_rank", type=int, default=384)
    ap.add_argument("--v_rank", type=int, default=512)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp16"])
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--repeat", type=int, default=20)
    ap.add_argument("--profile", action="store_true", help="one profiled pass over the variants; writes a chrome trace")
    ap.add_argument("--trace_path", default="xkv_profile_trace.json")
    ap.add_argument("--sweep", action="store_true", help="kv_len sweep of the qAB-with-RoPE entry points (rank = --k_rank)")
    ap.add_argument("--sweep_min", type=int, default=14, help="log2 of the first kv_len of the sweep")
    ap.add_argument("--sweep_max", type=int, default=17, help="log2 of the last kv_len of the sweep")
    args = ap.parse_args(argv)
    return sweep(args) if args.sweep else run(args)


if __name__ == "__main__":
    main()
