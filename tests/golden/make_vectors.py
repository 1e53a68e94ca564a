"""Writes tests/golden/xkv_vectors.npz: small seeded inputs and the CPU oracle's outputs for every operation on the path.

The reference project ships no golden vectors for this path (its tests draw unseeded CUDA randoms), and its kernels
need Triton on a GPU, so these vectors come from the oracle (oracle/xkv_oracle.py, itself pinned by tests/test_oracle.py).
They freeze the oracle: a later change to it that moves any output fails tests/test_golden.py, and the GPU parity
suite checks the HIP path against the same file.  Run from the repository root:  python tests/golden/make_vectors.py
"""
import math
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402


def gen(shape, std, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(torch.bfloat16).float()   # exactly representable in bf16


def build():
    b, hq, hkv, d, L, r, theta = 2, 8, 2, 128, 96, 64, 5e5
    q = gen((b, hq, 1, d), 0.5, 1)
    A, Av = gen((b, L, r), 1.0, 2), gen((b, L, r), 1.0, 3)
    kB, vB = gen((b, hkv, r, d), r ** -0.5, 4), gen((b, hkv, r, d), r ** -0.5, 5)
    K, V = gen((b, L, hkv, d), 1.0, 6), gen((b, L, hkv, d), 1.0, 7)
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta)
    scale = 1.0 / math.sqrt(d)
    out = {
        "q": q, "A": A, "Av": Av, "kB": kB, "vB": vB, "K": K, "V": V, "theta": torch.tensor(theta), "scale": torch.tensor(scale),
        "qab_nope": oracle.qab_nope(q, A, kB),
        "qab_rope": oracle.qab_rope(q, A, kB, cos, sin),
        "gqa_xkv": oracle.gqa_xkv(q[:, :, 0], A, kB, Av, vB, sm_scale=scale),
        "gqa_factorized_rope": oracle.gqa_factorized_rope(q, A, kB, Av, vB, cos, sin)[:, :, 0],
        "gqa_plain": oracle.gqa_plain(q[:, :, 0], K, V, scale),
        "gqa_v_only": oracle.gqa_v_only(q, K.transpose(1, 2), Av, vB, sm_scale=scale)[:, :, 0],
        "sin_cos_table": oracle.sin_cos_table(L, d, theta),
    }
    # MLA: 16 heads over a 512 + 64 latent
    H, c, e, Lm = 16, 512, 64, 80
    qn, qr = gen((1, H, c), 1 / 3, 8), gen((1, H, e), 1 / 3, 9)
    ckv, kpe = gen((1, Lm, 1, c), 1 / 3, 10), gen((1, Lm, 1, e), 1 / 3, 11)
    out.update({"mla_qn": qn, "mla_qr": qr, "mla_ckv": ckv, "mla_kpe": kpe, "mla_scale": torch.tensor(1.0 / math.sqrt(c + e)),
                "mla_ref": oracle.mla_ref(qn, qr, ckv, kpe, 1.0 / math.sqrt(c + e))})
    # split arithmetic
    cases = [(1000, 4, 4), (100, 8, 8), (4096, 3, 5), (33, 2, 2), (64, 1, 3), (131072, 32, 32)]
    out["split_cases"] = torch.tensor(cases)
    out["split_bounds"] = torch.tensor([[oracle.split_bounds(L_, n, i) for i in range(32)] for (L_, n, _) in cases])
    return {k: v.numpy() for k, v in out.items()}


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "xkv_vectors.npz")
    np.savez_compressed(path, **build())
    print("wrote", path, os.path.getsize(path), "bytes")
