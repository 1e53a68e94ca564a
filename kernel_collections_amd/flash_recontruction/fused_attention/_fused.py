"""Shared host logic of the fused xKV decode wrappers (no-PE, K-only, RoPE)."""
from __future__ import annotations

from typing import Optional

import torch

from kernel_collections_amd import ops


def _common(q, k_A, k_B, num_kv_splits, max_kv_splits):
    assert q.dim() == 3, "q must be [batch, num_q_heads, head_dim]"
    batch, num_q_heads, head_dim = q.shape
    num_kv_heads = k_B.shape[1]
    assert k_A.shape[0] == batch and k_B.shape[0] == batch, "Batch size mismatch"
    assert k_A.shape[-1] == k_B.shape[2], "Rank mismatch between k_A and k_B"
    assert k_B.shape[-1] == head_dim, "Head dimension mismatch"
    assert num_q_heads % num_kv_heads == 0
    kv_group_num = num_q_heads // num_kv_heads
    assert kv_group_num >= 1
    assert k_A.shape[-1] % 32 == 0, "rank must be a multiple of 32"
    splits = ops.as_int32_dev(num_kv_splits, batch, q.device)
    return batch, num_q_heads, num_kv_heads, head_dim, int(max_kv_splits), splits


def _lens(kv_lens, batch, device):
    return None if kv_lens is None else ops.as_int32_dev(kv_lens, batch, device)


def decode_nope(q, k_A, k_B, v_A, v_B, o, num_kv_splits, max_kv_splits, sm_scale, kv_lens=None):
    """K and V factorised, no positional encoding: absorb q into k_B, scan k_A / v_A once for
    all heads, merge in rank space, then multiply by v_B."""
    assert v_A.shape[1] == k_A.shape[1]
    assert v_B.shape[1] == k_B.shape[1]
    batch, hq, hkv, d, S, splits = _common(q, k_A, k_B, num_kv_splits, max_kv_splits)
    ops.check_16bit(q, k_A, k_B, v_A, v_B)
    rank_v = v_A.shape[-1]
    assert rank_v == v_B.shape[2], "Rank mismatch between v_A and v_B"
    assert rank_v % 64 == 0 and rank_v <= 512, "v rank must be a multiple of 64, at most 512"
    kv_len = k_A.shape[1]
    lens = _lens(kv_lens, batch, q.device)
    q3 = ops._q3(q)
    k_A, v_A = ops.as_rows(k_A), ops.as_rows(v_A)
    qt_hi, qt_lo = ops.absorb_q(q3, k_B, want_lo=True)
    partial, lse = ops.workspaces(batch, hq, S, rank_v, q.device)
    groups = ops.head_groups(hq)
    ops.latent_stage1(qt_hi, qt_lo, None, (k_A, k_A.stride(0), k_A.stride(1), 0, k_A.shape[-1]), None,
                      (v_A, v_A.stride(0), v_A.stride(1), 0, rank_v), partial, lse, None, splits, lens,
                      batch, hq, groups, kv_len, S, float(sm_scale))
    return ops.merge_stage2(partial, lse, o, v_B, splits, lens, batch, hq, hkv, kv_len, S)


def decode_k_only(q, k_A, k_B, v_buffer, o, num_kv_splits, max_kv_splits, sm_scale, kv_lens=None):
    """K factorised (absorbed), V plain ``[batch, kv_len, num_kv_heads, head_dim]``."""
    batch, hq, hkv, d, S, splits = _common(q, k_A, k_B, num_kv_splits, max_kv_splits)
    ops.check_16bit(q, k_A, k_B, v_buffer)
    assert v_buffer.shape[1] == k_A.shape[1] and v_buffer.shape[2] == hkv
    dv = v_buffer.shape[-1]
    assert dv % 64 == 0 and dv <= 512
    kv_len = k_A.shape[1]
    lens = _lens(kv_lens, batch, q.device)
    q3 = ops._q3(q)
    k_A, v_buffer = ops.as_rows(k_A), ops.as_rows(v_buffer)
    qt_hi, qt_lo = ops.absorb_q(q3, k_B, want_lo=True)
    partial, lse = ops.workspaces(batch, hq, S, dv, q.device)
    ops.latent_stage1(qt_hi, qt_lo, None, (k_A, k_A.stride(0), k_A.stride(1), 0, k_A.shape[-1]), None,
                      (v_buffer, v_buffer.stride(0), v_buffer.stride(1), v_buffer.stride(2), dv),
                      partial, lse, None, splits, lens, batch, hq, hkv, kv_len, S, float(sm_scale))
    return ops.merge_stage2(partial, lse, o, None, splits, lens, batch, hq, hq, kv_len, S)


# key ranks at which fused RoPE decode with a value basis of its own runs as two passes (scores, then softmax + P.v_A)
# A value basis of its own runs as two passes (scores, then softmax + P.v_A) at these key ranks once the call scans at
# least TWO_PASS_MIN_TOKENS tokens (batch x kv_len); below, the extra launches cost more than the second row stream of
# the fused 8-wave kernel (measured crossover: 32768 tokens at every rank).
TWO_PASS_KEY_RANKS = (512, 384, 256)
TWO_PASS_MIN_TOKENS = 49152


def decode_rope(q_pe, k_A, k_B, v_A, v_B, o, num_kv_splits, max_kv_splits, sm_scale, theta, sin_cos,
                pos_offset=0, kv_lens=None):
    """K = RoPE(k_A @ k_B) rebuilt and rotated in registers, V factorised."""
    assert v_A.shape[1] == k_A.shape[1]
    assert v_B.shape[1] == k_B.shape[1]
    batch, hq, hkv, d, S, splits = _common(q_pe, k_A, k_B, num_kv_splits, max_kv_splits)
    ops.check_16bit(q_pe, k_A, k_B, v_A, v_B)
    assert d == 128, "the RoPE reconstruction kernels are built for head_dim 128"
    assert hq // hkv <= 16 and k_A.shape[-1] <= 512
    rank_v = v_A.shape[-1]
    assert rank_v == v_B.shape[2], "Rank mismatch between v_A and v_B"
    assert rank_v % 64 == 0 and rank_v <= 512
    kv_len = k_A.shape[1]
    lens = _lens(kv_lens, batch, q_pe.device)
    q3 = ops._q3(q_pe)
    k_A, v_A = ops.as_rows(k_A), ops.as_rows(v_A)
    k_B = k_B if k_B.stride(-1) == 1 else k_B.contiguous()
    inv = None
    if sin_cos is None:
        inv = ops.rope_inv_freq(d, theta, q_pe.device)
    else:
        assert sin_cos.shape == (kv_len, d), "sin_cos must be [kv_len, head_dim]"
        if sin_cos.dtype != q_pe.dtype or sin_cos.stride(-1) != 1:
            sin_cos = sin_cos.to(q_pe.dtype).contiguous()
    same_basis = (v_A.data_ptr() == k_A.data_ptr() and v_A.shape == k_A.shape and v_A.stride() == k_A.stride())
    if (not same_basis and k_A.shape[-1] in TWO_PASS_KEY_RANKS and batch * kv_len >= TWO_PASS_MIN_TOKENS
            and sin_cos is None and hq // hkv <= 8 and hq <= 32
            and rank_v in (256, 384, 512) and kv_len % 4 == 0 and ops.USE_RECON_WORKSPACE):
        # A value basis of its own: two passes.  The scores-only form of the reconstruction kernel runs at the rate of the
        # shared-basis fused kernel (one row stream, no P.A); softmax and P.v_A then stream v_A once for all heads at HBM
        # rate.  Fused into one kernel, the second row stream costs more than the 2 x 4 bytes per score this moves.
        scores = torch.empty((batch, hq, kv_len), dtype=torch.float32, device=q_pe.device)
        # the scores do not depend on how pass 1 cuts the range: one round of workgroups per CU, two at key rank 256, whose
        # scores-only kernel is small enough for two workgroups to share a CU
        S1 = ops.occupancy_splits(batch, hkv, kv_len, tile=32, waves=2 if k_A.shape[-1] == 256 else 1)
        ops.recon_stage1(q3, k_A, k_B, None, None, None, scores, ops.uniform_splits(batch, S1, q_pe.device), lens, batch, hq,
                         hkv, kv_len, S1, float(sm_scale), True, inv, int(pos_offset), None)
        S2 = ops.latent_splits(batch, 1, kv_len, rank_v, absorbed=True)
        splits2 = ops.uniform_splits(batch, S2, q_pe.device)
        partial, lse = ops.workspaces(batch, hq, S2, rank_v, q_pe.device)
        ops.softmax_pv_stage1(scores, v_A, partial, lse, splits2, lens, batch, hq, kv_len, S2, q_pe.dtype)
        return ops.merge_stage2(partial, lse, o, v_B, splits2, lens, batch, hq, hkv, kv_len, S2)
    partial, lse = ops.workspaces(batch, hq, S, rank_v, q_pe.device)
    ops.recon_stage1(q3, k_A, k_B, v_A, partial, lse, None, splits, lens, batch, hq, hkv, kv_len, S,
                     float(sm_scale), True, inv, int(pos_offset), sin_cos)
    return ops.merge_stage2(partial, lse, o, v_B, splits, lens, batch, hq, hkv, kv_len, S)
