"""MLA-style decode on concatenated key buffers (reference flash_decoding/mla.py:388-471).

``decode_attention_fwd(q, k_buffer, v_buffer, o, sm_scale=1.0, logit_cap=0.0)`` writes ``o`` in place and
returns ``None`` like the reference.  A 576-wide key is split 512 (latent) + 64 (RoPE part) and a
288-wide one 256 + 32 (mla.py:227-235); ``logit_cap > 0`` applies ``cap * tanh(x / cap)`` (mla.py:157-158).
When ``v_buffer`` is a view of the key's latent part the latent tile is loaded once for both products.
The number of KV splits is chosen from occupancy instead of the reference's fixed 128 (mla.py:405-406);
the merged result is independent of it up to fp32 rounding.  The log-sum-exp workspace is indexed
``[batch, head, split]`` (the reference derives that index by an integer division that is only exact
when key and value widths are equal)."""
from __future__ import annotations

import torch

from kernel_collections_amd import ops


def _split_dims(dk: int):
    if dk == 576:
        return 512, 64
    if dk == 288:
        return 256, 32
    return dk, 0


def stage1_operands(q, k_buffer, v_buffer):
    """Shape checks and operand descriptors shared by every entry built on this kernel:
    returns ``(qn, qr, C, R, V, groups, dn, dv)``."""
    batch, num_q_heads, head_dim = q.shape
    _, kv_len, num_kv_heads, dk = k_buffer.shape
    assert dk == head_dim
    kv_group_num = num_q_heads // num_kv_heads
    assert kv_group_num >= 1 and num_q_heads % num_kv_heads == 0
    ops.check_16bit(q, k_buffer, v_buffer)
    dn, dr = _split_dims(dk)
    dv = v_buffer.shape[-1]
    assert dn % 32 == 0 and dv % 64 == 0 and dv <= 512
    k_buffer, v_buffer = ops.as_rows(k_buffer), ops.as_rows(v_buffer)
    qn = ops._q3(q[..., :dn])
    qr = ops._q3(q[..., dn:]) if dr else None
    # query heads of one kv head must fit 32 rows; more heads -> several groups over the same rows
    per_kv_groups = ops.head_groups(kv_group_num)
    assert per_kv_groups == 1 or num_kv_heads == 1, "more than 32 query heads per kv head needs num_kv_heads == 1"
    groups = num_kv_heads * per_kv_groups
    sh = k_buffer.stride(2) if per_kv_groups == 1 else 0
    svh = v_buffer.stride(2) if per_kv_groups == 1 else 0
    C = (k_buffer, k_buffer.stride(0), k_buffer.stride(1), sh, dn)
    R = (k_buffer[..., dn:], k_buffer.stride(0), k_buffer.stride(1), sh, dr) if dr else None
    V = (v_buffer, v_buffer.stride(0), v_buffer.stride(1), svh, dv)
    return qn, qr, C, R, V, groups, dn, dv


def decode_attention_fwd(q, k_buffer, v_buffer, o, sm_scale=1.0, logit_cap=0.0):
    batch, num_q_heads, _ = q.shape
    kv_len = k_buffer.shape[1]
    qn, qr, C, R, V, groups, dn, dv = stage1_operands(q, k_buffer, v_buffer)
    S = ops.latent_splits(batch, groups, kv_len, dn)
    splits = ops.uniform_splits(batch, S, q.device)
    partial, lse = ops.workspaces(batch, num_q_heads, S, dv, q.device)
    ops.latent_stage1(qn, None, qr, C, R, V, partial, lse, None, splits, None, batch, num_q_heads, groups,
                      kv_len, S, float(sm_scale), float(logit_cap))
    ops.merge_stage2(partial, lse, o, None, splits, None, batch, num_q_heads, num_q_heads, kv_len, S)
    return None


def decode_attention_reference(q, k_buffer, v_buffer, o, sm_scale):
    """Eager form with the reference's name (mla.py:442-471).  The reference divides the scores by
    ``sm_scale`` there while its kernel multiplies (they agree only at 1.0); this one multiplies, like
    the kernel, and returns the result (the reference's version rebinds ``o`` and returns nothing)."""
    batch, hq, d = q.shape
    hkv = k_buffer.shape[2]
    s = torch.einsum("bkgd,blkd->bkgl", q.reshape(batch, hkv, hq // hkv, d), k_buffer) * sm_scale
    p = torch.softmax(s, dim=-1, dtype=torch.float32).to(s.dtype)
    return torch.einsum("bkgl,blkd->bkgd", p, v_buffer).reshape(batch, hq, v_buffer.shape[-1])
