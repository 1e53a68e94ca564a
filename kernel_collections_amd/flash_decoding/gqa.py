"""Split-K flash decoding for grouped-query attention on plain K/V buffers.

Call surface of the reference's flash_decoding/gqa.py:339-434 (``decode_attention_fwd``), plus
  * ``kv_lens``: optional int32 ``[batch]`` of per-sequence lengths (ragged batch; the reference has
    one length, ``k_buffer.shape[1]``, for the whole batch - gqa.py:60,194);
  * ``decode_attention_fwd_v_factorized``: K plain, ``V = v_A @ v_B`` (the eager semantics of
    ``group_query_attention_factorized_v_only``, reference attention.py:202-274) as a split-K kernel
    that accumulates ``P @ v_A`` in rank space and multiplies by ``v_B`` after the merge.
Split ranges follow gqa.py:95-99 exactly; ``sm_scale`` multiplies the scores (gqa.py:122).  The caller's split counts are a
lower bound: a sequence is cut into more splits when that is what fills the device (split-K is exact under the merge), by a
fixed cap in the per-head form and by a per-call plan computed on the device in the all-heads forms.
"""
from __future__ import annotations

import torch

from kernel_collections_amd import ops


# Longest split, in tokens, that stage 1 scans as one workgroup (0: the caller's splits as they are).  The kernels raise a
# sequence's split count to ceil(len / this) when the caller asked for fewer (`split_cap_tokens` of the C entry points):
# split-K is exact under the merge, so the caller's count is a lower bound on the parallelism, not part of the result, and a
# ragged batch scanned in 4096-token splits would otherwise leave most CUs idle behind its longest sequences.
MAX_SPLIT_TOKENS = 1024
# The all-heads ("wide") forms run one workgroup per CU and per (sequence, split), hkv times fewer workgroups than the
# per-head form.  There the split length is planned per call: the shortest that still cuts the batch into at most one split
# per CU, so that every CU gets one job and the jobs are as equal as the lengths allow - never below this floor, which is
# also what sizes the workspaces (0: the caller's splits as they are).
MAX_SPLIT_TOKENS_WIDE = 1024


def _plan_wide(lens, splits, S, batch, kv_len):
    """(cap that sizes the workspaces, their split dimension, split plan on the device or None) of an all-heads call."""
    floor = MAX_SPLIT_TOKENS_WIDE
    if not floor:
        return 0, S, None
    jobs = ops.num_cus()
    if lens is None:      # one length: plain host arithmetic
        per_seq = max(1, jobs // batch)
        cap = max(floor, -(-(-(-kv_len // per_seq)) // 32) * 32)
        return cap, ops.capped_splits(kv_len, S, cap), None
    S = ops.capped_splits(kv_len, S, floor)
    return floor, S, ops.plan_splits(lens, splits, S, floor, jobs)


def _prep(q, k_buffer, num_kv_splits, max_kv_splits, kv_lens):
    assert q.dim() == 3 and k_buffer.dim() == 4
    batch, num_q_heads, head_dim = q.shape
    num_kv_heads = k_buffer.shape[2]
    assert k_buffer.shape[0] == batch and k_buffer.shape[-1] == head_dim
    kv_group_num = num_q_heads // num_kv_heads
    assert kv_group_num >= 1 and num_q_heads % num_kv_heads == 0
    assert kv_group_num <= 32, "at most 32 query heads per kv head"
    assert head_dim % 32 == 0, "head_dim must be a multiple of 32"
    splits = ops.as_int32_dev(num_kv_splits, batch, q.device)
    lens = None if kv_lens is None else ops.as_int32_dev(kv_lens, batch, q.device)
    return batch, num_q_heads, num_kv_heads, head_dim, int(max_kv_splits), splits, lens


def decode_attention_fwd(q, k_buffer, v_buffer, o, num_kv_splits, max_kv_splits, sm_scale=1.0, *, kv_lens=None):
    """q ``[batch, Hq, d]``; k_buffer / v_buffer ``[batch, kv_len, Hkv, d]``; o ``[batch, Hq, d]`` (filled,
    returned); num_kv_splits int32 ``[batch]`` on the device; max_kv_splits int."""
    batch, hq, hkv, d, S, splits, lens = _prep(q, k_buffer, num_kv_splits, max_kv_splits, kv_lens)
    ops.check_16bit(q, k_buffer, v_buffer)
    assert k_buffer.shape[-1] == v_buffer.shape[-1], "head dim of K and V must be the same"
    dv = v_buffer.shape[-1]
    assert dv % 64 == 0 and dv <= 512
    kv_len = k_buffer.shape[1]
    q3 = ops._q3(q)
    k_buffer, v_buffer = ops.as_rows(k_buffer), ops.as_rows(v_buffer)
    # 8 kv heads of 128 side by side in a token row: stage 1 serves every head of a split from one workgroup (whole 2 KiB
    # rows through its LDS ring), so there are hkv times fewer workgroups and a split may be twice as long
    wide = (hkv * d == 1024 and d == 128 and hq <= 32 and k_buffer.stride(2) == d and v_buffer.stride(2) == d
            and k_buffer.stride(1) >= 1024 and v_buffer.stride(1) >= 1024)
    if wide:
        cap, S, plan = _plan_wide(lens, splits, S, batch, kv_len)
    else:   # room in the workspaces for the splits the kernels may add (host arithmetic only)
        cap, S, plan = MAX_SPLIT_TOKENS, ops.capped_splits(kv_len, S, MAX_SPLIT_TOKENS), None
    partial, lse = ops.workspaces(batch, hq, S, dv, q.device)
    ops.latent_stage1(q3, None, None,
                      (k_buffer, k_buffer.stride(0), k_buffer.stride(1), k_buffer.stride(2), d), None,
                      (v_buffer, v_buffer.stride(0), v_buffer.stride(1), v_buffer.stride(2), dv),
                      partial, lse, None, splits, lens, batch, hq, hkv, kv_len, S, float(sm_scale), split_cap=cap,
                      split_plan=plan)
    return ops.merge_stage2(partial, lse, o, None, splits, lens, batch, hq, hq, kv_len, S, split_cap=cap, split_plan=plan)


def decode_attention_fwd_v_factorized(q, k_buffer, v_A_buffer, v_B_buffer, o, num_kv_splits, max_kv_splits,
                                      sm_scale=1.0, *, kv_lens=None):
    """K plain ``[batch, kv_len, Hkv, d]``; v_A ``[batch, kv_len, rv]``; v_B ``[batch, Hkv, rv, d]``."""
    batch, hq, hkv, d, S, splits, lens = _prep(q, k_buffer, num_kv_splits, max_kv_splits, kv_lens)
    ops.check_16bit(q, k_buffer, v_A_buffer, v_B_buffer)
    rv = v_A_buffer.shape[-1]
    assert v_A_buffer.shape[1] == k_buffer.shape[1] and v_B_buffer.shape[1] == hkv and v_B_buffer.shape[2] == rv
    assert rv % 64 == 0 and rv <= 512
    kv_len = k_buffer.shape[1]
    q3 = ops._q3(q)
    k_buffer, v_A_buffer = ops.as_rows(k_buffer), ops.as_rows(v_A_buffer)
    # 8 kv heads of 128 side by side in a token row: stage 1 serves every head of a split from one workgroup, and the value
    # basis (shared by the heads) is read once per token instead of once per kv head
    wide8 = hkv * d == 1024 and d == 128 and rv in (256, 384, 512) and hq <= 32 and k_buffer.stride(2) == d
    # 512-wide token rows (4 x 128, 2 x 256 ...): the same form, with the block-diagonal query built here
    wide4 = hkv * d == 512 and rv == 512 and hq <= 32 and k_buffer.stride(2) == d
    cap, S, plan = _plan_wide(lens, splits, S, batch, kv_len) if (wide8 or wide4) else (0, S, None)
    partial, lse = ops.workspaces(batch, hq, S, rv, q.device)
    if wide4:
        ops.latent_stage1(ops.blockdiag_q(q3, hkv), None, None,
                          (k_buffer, k_buffer.stride(0), k_buffer.stride(1), 0, hkv * d), None,
                          (v_A_buffer, v_A_buffer.stride(0), v_A_buffer.stride(1), 0, rv),
                          partial, lse, None, splits, lens, batch, hq, 1, kv_len, S, float(sm_scale), split_cap=cap,
                          split_plan=plan)
    else:
        ops.latent_stage1(q3, None, None,
                          (k_buffer, k_buffer.stride(0), k_buffer.stride(1), k_buffer.stride(2), d), None,
                          (v_A_buffer, v_A_buffer.stride(0), v_A_buffer.stride(1), 0, rv),
                          partial, lse, None, splits, lens, batch, hq, hkv, kv_len, S, float(sm_scale), split_cap=cap,
                          split_plan=plan)
    return ops.merge_stage2(partial, lse, o, v_B_buffer, splits, lens, batch, hq, hkv, kv_len, S, split_cap=cap,
                            split_plan=plan)
