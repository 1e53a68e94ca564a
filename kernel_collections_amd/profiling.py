"""Variant table for one decode step, in the spirit of the reference's test_attention_profiling.py:213-474:
every attention variant of the path on the same synthetic shape, its time, its speed-up over eager attention and over
the uncompressed flash decode, and its distance from the eager result.

    python -m kernel_collections_amd.profiling --kv_len 131072 --k_rank 384 --v_rank 512 [--batch 1] [--dtype bf16]

Same flags as the reference script (:511-517: --num_heads --num_kv_heads --head_dim --kv_len --k_rank --v_rank);
--profile prints the per-kernel table of torch.profiler for one pass over the variants instead of writing a trace.
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
        from torch.profiler import ProfilerActivity, profile
        with profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA]) as prof:
            for _, fn, _ in variants:
                fn()
            torch.cuda.synchronize()
        print(prof.key_averages().table(sort_by="cuda_time_total", row_limit=20))
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
    ap.add_argument("--profile", action="store_true")
    return run(ap.parse_args(argv))


if __name__ == "__main__":
    main()
