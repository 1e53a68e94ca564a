"""Fused key reconstruction without positional encoding: scores ``q @ (Ak @ Bk)^T``.

Same call surface as the reference's flash_recontruction/qAB_no_pe/v1.py:78-135 (``qAB``) and
v2.py:72-130 (``qAB_v3``).  The HIP path never reconstructs K: the query is absorbed into
``Bk`` (``q~ = q @ Bk^T``, the eager form attention.py:312-318) and the scores become a
bandwidth-bound scan ``q~ @ Ak^T`` that reads ``Ak`` once for all query heads.
"""
from __future__ import annotations

from typing import Optional

import torch

from kernel_collections_amd import ops


def qAB(q: torch.Tensor, Ak: torch.Tensor, Bk: torch.Tensor, *,
        sm_scale: Optional[float] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """q ``(bsz, num_heads, 1, head_dim)``, Ak ``(bsz, kv_len, rank)``,
    Bk ``(bsz, num_kv_heads, rank, head_dim)`` -> ``(bsz, num_heads, 1, kv_len)``.

    ``sm_scale`` (default: none, like the reference) multiplies the scores; ``out_dtype``
    (default ``q.dtype``) may be ``torch.float32``."""
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
    assert rank % 32 == 0, "rank must be a multiple of 32"
    ops.check_16bit(q, Ak, Bk)
    out_dtype = out_dtype or q.dtype
    assert out_dtype in (q.dtype, torch.float32)

    q3 = ops._q3(q.reshape(bsz, num_heads, head_dim))
    Ak = ops.as_rows(Ak)
    qt_hi, qt_lo = ops.absorb_q(q3, Bk, want_lo=True)
    out = torch.empty((bsz, num_heads, 1, kv_len), dtype=out_dtype, device=q.device)
    groups = ops.head_groups(num_heads)
    n_splits = ops.latent_splits(bsz, groups, kv_len, rank, absorbed=True)
    splits = ops.uniform_splits(bsz, n_splits, q.device)
    ops.latent_stage1(qt_hi, qt_lo, None, (Ak, Ak.stride(0), Ak.stride(1), 0, rank), None, None,
                      None, None, out, splits, None, bsz, num_heads, groups, kv_len, n_splits,
                      1.0 if sm_scale is None else float(sm_scale))
    return out


qAB_v3 = qAB
