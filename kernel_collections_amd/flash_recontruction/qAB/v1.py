"""Fused key reconstruction WITH RoPE: ``q_pe @ RoPE(Ak @ Bk)^T``.

Call surface of the reference's flash_recontruction/qAB/v1.py:90-148 (``qAB``; v3.py:84 / v4.py:85 /
ref.py:88 share it) and v2.py:132-187 (``qAB_precomp``).  The key tile is rebuilt on MFMA with
``Bk[kv_head]`` stationary in registers, rotated in registers (rotate-half pairs are lane-local)
and dotted with the already-rotated query; K never reaches HBM.  Keys sit at absolute positions
``pos_offset .. pos_offset + kv_len - 1``; angles are ``float(pos) * theta**(-2j/128)`` as in the
eager closed form (rope/rope_ref.py:3-9), not the fast-math variant of the Triton helper.
"""
from __future__ import annotations

from typing import Optional

import torch

from kernel_collections_amd import ops


def _check(q, Ak, Bk):
    assert q.dim() == 4, f"Expected q to be 4D, got {q.dim()}D"
    assert Ak.dim() == 3, f"Expected Ak to be 3D, got {Ak.dim()}D"
    assert Bk.dim() == 4, f"Expected Bk to be 4D, got {Bk.dim()}D"
    bsz, num_heads, q_len, head_dim = q.shape
    bsz_a, kv_len, rank = Ak.shape
    bsz_b, num_kv_heads, rank_b, head_dim_b = Bk.shape
    assert bsz == bsz_a == bsz_b, "Batch size mismatch"
    assert rank == rank_b, "Rank mismatch"
    assert head_dim == head_dim_b, "Head dimension mismatch"
    assert q_len == 1, "Only supporting q_len=1 for now"
    assert num_heads % num_kv_heads == 0, "num_heads must be divisible by num_kv_heads"
    assert head_dim == 128, "the RoPE reconstruction kernels are built for head_dim 128"
    assert num_heads // num_kv_heads <= 16, "at most 16 query heads per kv head"
    assert rank % 32 == 0 and rank <= 512, "rank must be a multiple of 32, at most 512"
    ops.check_16bit(q, Ak, Bk)
    return bsz, num_heads, num_kv_heads, head_dim, kv_len, rank


def _scores(q, Ak, Bk, inv_freq, sin_cos, pos_offset, sm_scale, out_dtype):
    bsz, num_heads, num_kv_heads, head_dim, kv_len, rank = _check(q, Ak, Bk)
    out_dtype = out_dtype or q.dtype
    assert out_dtype in (q.dtype, torch.float32)
    q3 = ops._q3(q.reshape(bsz, num_heads, head_dim))
    Ak = ops.as_rows(Ak)
    Bk = Bk if Bk.stride(-1) == 1 else Bk.contiguous()
    out = torch.empty((bsz, num_heads, 1, kv_len), dtype=out_dtype, device=q.device)
    # ranks 384 / 512 run the wave-specialised MFMA kernel, one workgroup per CU; rank 256 the 4-wave kernel, whose scores-only
    # form fits a CU twice (252 registers, 78 KB of LDS); below, the register-staged scores kernel keeps 2-3
    n_splits = ops.occupancy_splits(bsz, num_kv_heads, kv_len, tile=32, waves=1 if rank > 256 else (2 if rank > 128 else 3))
    splits = ops.uniform_splits(bsz, n_splits, q.device)
    ops.recon_stage1(q3, Ak, Bk, None, None, None, out, splits, None, bsz, num_heads, num_kv_heads, kv_len,
                     n_splits, 1.0 if sm_scale is None else float(sm_scale), True, inv_freq, int(pos_offset), sin_cos)
    return out


def qAB(q: torch.Tensor, Ak: torch.Tensor, Bk: torch.Tensor, theta: float = 10000000.0, *,
        sm_scale: Optional[float] = None, out_dtype: Optional[torch.dtype] = None,
        pos_offset: int = 0) -> torch.Tensor:
    """q (already rotated) ``(bsz, num_heads, 1, 128)``, Ak ``(bsz, kv_len, rank)``,
    Bk ``(bsz, num_kv_heads, rank, 128)`` -> ``(bsz, num_heads, 1, kv_len)``; no scale unless given."""
    inv = ops.rope_inv_freq(q.shape[-1], theta, q.device)
    return _scores(q, Ak, Bk, inv, None, pos_offset, sm_scale, out_dtype)


def qAB_precomp(q: torch.Tensor, Ak: torch.Tensor, Bk: torch.Tensor, sin_cos: torch.Tensor, *,
                sm_scale: Optional[float] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Same contract with a precomputed table ``sin_cos [kv_len, head_dim]``,
    ``[:, :64] = sin`` and ``[:, 64:] = cos`` (reference qAB/v2.py:138-139)."""
    kv_len, head_dim_sc = sin_cos.shape
    assert head_dim_sc == q.shape[-1], "sin_cos.head_dim mismatch"
    assert kv_len == Ak.shape[1], "sin_cos must have one row per key"
    if sin_cos.dtype != q.dtype or sin_cos.stride(-1) != 1:
        sin_cos = sin_cos.to(q.dtype).contiguous()
    return _scores(q, Ak, Bk, None, sin_cos, 0, sm_scale, out_dtype)
