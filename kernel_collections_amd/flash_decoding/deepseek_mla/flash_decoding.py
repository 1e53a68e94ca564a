"""Decode over a long prefix plus a short buffer of recently decoded tokens
(reference flash_decoding/deepseek_mla/flash_decoding.py).

``mla_decode_attention_fwd``            :6-62    one buffer
``mla_decode_attention_fwd_pd_sep``     :66-155  prefix + tail, both plain
``mla_decode_attention_fwd_pd_sep_xKV`` :159-255 prefix factorised (``K = k_A k_B``, ``V = v_A v_B``), tail plain

Differences from the reference, none of which changes the result beyond fp32 rounding: the number of prefix splits
comes from occupancy instead of a fixed 128 (:86, :186); prefix and tail stage 1 write into ONE workspace (the tail at a
split offset) instead of two that are concatenated afterwards (:137-138, :238-239); in the factorised form the prefix
partials are merged in rank space first and up-projected once per head (the reference multiplies all 128 split rows by
``v_B`` in fp16, :218), and that merged row enters the final merge as a single split with its own log-sum-exp."""
from __future__ import annotations

import torch

from kernel_collections_amd import ops
from kernel_collections_amd.flash_decoding.mla import stage1_operands


def _all_live(n_splits: int, batch: int, device):
    """(kv_len, num_kv_splits) under which every one of `n_splits` workspace rows counts as live in the merge."""
    return 32 * n_splits, ops.uniform_splits(batch, n_splits, device)


def _stage1_into(q, k_buffer, v_buffer, partial, lse, first_split, n_splits, sm_scale, logit_cap):
    """Stage 1 of one buffer into rows first_split .. first_split + n_splits - 1 of a shared workspace."""
    batch, num_q_heads, _ = q.shape
    kv_len = k_buffer.shape[1]
    qn, qr, C, R, V, groups, dn, dv = stage1_operands(q, k_buffer, v_buffer)
    splits = ops.uniform_splits(batch, n_splits, q.device)
    ops.latent_stage1(qn, None, qr, C, R, V, partial[:, :, first_split:], lse[:, :, first_split:], None, splits, None,
                      batch, num_q_heads, groups, kv_len, partial.shape[2], float(sm_scale), float(logit_cap))


def _tail_splits(decode_kv_len: int, want: int) -> int:
    return ops.settled_splits(decode_kv_len, want)           # every split of the shared workspace must be live


def mla_decode_attention_fwd(q, k_buffer, v_buffer, sm_scale=1.0, logit_cap=0.0):
    batch, num_q_heads, _ = q.shape
    kv_len, dv = k_buffer.shape[1], v_buffer.shape[-1]
    groups = stage1_operands(q, k_buffer, v_buffer)[5]
    S = ops.latent_splits(batch, groups, kv_len, k_buffer.shape[-1])
    partial, lse = ops.workspaces(batch, num_q_heads, S, dv, q.device)
    _stage1_into(q, k_buffer, v_buffer, partial, lse, 0, S, sm_scale, logit_cap)
    o = torch.empty((batch, num_q_heads, dv), dtype=q.dtype, device=q.device)
    ops.merge_stage2(partial, lse, o, None, ops.uniform_splits(batch, S, q.device), None, batch, num_q_heads, num_q_heads,
                     kv_len, S)
    return o


def mla_decode_attention_fwd_pd_sep(q, k_buffer, v_buffer, k_buffer_decoded, v_buffer_decoded, sm_scale=1.0, logit_cap=0.0):
    batch, num_q_heads, _ = q.shape
    prefill_kv_len, decode_kv_len = k_buffer.shape[1], k_buffer_decoded.shape[1]
    dv = v_buffer.shape[-1]
    assert v_buffer_decoded.shape[-1] == dv
    groups = stage1_operands(q, k_buffer, v_buffer)[5]
    S1 = ops.settled_splits(prefill_kv_len, ops.latent_splits(batch, groups, prefill_kv_len, k_buffer.shape[-1]))
    S2 = _tail_splits(decode_kv_len, 2)                      # the reference uses 2 (:89)
    partial, lse = ops.workspaces(batch, num_q_heads, S1 + S2, dv, q.device)
    _stage1_into(q, k_buffer, v_buffer, partial, lse, 0, S1, sm_scale, logit_cap)
    _stage1_into(q, k_buffer_decoded, v_buffer_decoded, partial, lse, S1, S2, sm_scale, logit_cap)
    o = torch.empty((batch, num_q_heads, dv), dtype=q.dtype, device=q.device)
    live_len, live_splits = _all_live(S1 + S2, batch, q.device)
    ops.merge_stage2(partial, lse, o, None, live_splits, None, batch, num_q_heads, num_q_heads, live_len, S1 + S2)
    return o


def mla_decode_attention_fwd_pd_sep_xKV(q, k_A_buffer, k_B_buffer, v_A_buffer, v_B_buffer, k_buffer_decoded,
                                        v_buffer_decoded, sm_scale=1.0, logit_cap=0.0):
    batch, num_q_heads, head_dim = q.shape
    _, prefill_kv_len, rank = k_A_buffer.shape
    num_kv_heads = k_B_buffer.shape[1]
    decode_kv_len = k_buffer_decoded.shape[1]
    v_dim = v_buffer_decoded.shape[-1]
    assert num_kv_heads == 1, "Only one KV head is supported for now"     # reference :176
    assert v_B_buffer.shape[-1] == v_dim and v_A_buffer.shape[-1] == v_B_buffer.shape[2]
    ops.check_16bit(q, k_A_buffer, k_B_buffer, v_A_buffer, v_B_buffer)
    rank_v = v_A_buffer.shape[-1]
    q3 = ops._q3(q)
    k_A, v_A = ops.as_rows(k_A_buffer), ops.as_rows(v_A_buffer)
    groups = ops.head_groups(num_q_heads)

    # prefix: q absorbed into k_B (the reference's torch.matmul at :178), scan over k_A / v_A, partials in rank space
    qt_hi, qt_lo = ops.absorb_q(q3, k_B_buffer, want_lo=True)
    S1 = ops.latent_splits(batch, groups, prefill_kv_len, rank, absorbed=True)
    splits1 = ops.uniform_splits(batch, S1, q.device)
    part1, lse1 = ops.workspaces(batch, num_q_heads, S1, rank_v, q.device)
    shared = v_A.data_ptr() == k_A.data_ptr() and v_A.stride() == k_A.stride() and rank_v == rank
    Cop = (k_A, k_A.stride(0), k_A.stride(1), 0, rank)
    Vop = Cop if shared else (v_A, v_A.stride(0), v_A.stride(1), 0, rank_v)
    ops.latent_stage1(qt_hi, qt_lo, None, Cop, None, Vop, part1, lse1, None, splits1, None, batch, num_q_heads, groups,
                      prefill_kv_len, S1, float(sm_scale), float(logit_cap))

    # final workspace: row 0 = the merged, up-projected prefix with its log-sum-exp; rows 1.. = the tail's splits
    S2 = _tail_splits(decode_kv_len, 4)                      # the reference uses 4 (:189)
    partial, lse = ops.workspaces(batch, num_q_heads, 1 + S2, v_dim, q.device)
    ops.merge_stage2(part1, lse1, partial[:, :, 0], v_B_buffer, splits1, None, batch, num_q_heads, num_kv_heads,
                     prefill_kv_len, S1, lse_out=lse[:, :, 0])
    _stage1_into(q, k_buffer_decoded, v_buffer_decoded, partial, lse, 1, S2, sm_scale, logit_cap)
    o = torch.empty((batch, num_q_heads, v_dim), dtype=q.dtype, device=q.device)
    live_len, live_splits = _all_live(1 + S2, batch, q.device)
    ops.merge_stage2(partial, lse, o, None, live_splits, None, batch, num_q_heads, num_q_heads, live_len, 1 + S2)
    return o
