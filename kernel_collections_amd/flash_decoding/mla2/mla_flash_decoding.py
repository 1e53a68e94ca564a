"""Absorbed MLA decode (reference flash_decoding/mla2/mla_flash_decoding.py:6-130).

``mla_decode_attention_fwd`` returns the latent-space output ``[batch, H, lora_rank]``;
``mla_decode_attention_xKV`` takes a latent that is itself factorised (``c_kv = kv_A @ kv_B``), absorbs
``q_nope`` into ``kv_B`` and un-absorbs the output.  The split count is chosen from occupancy instead of the
reference's fixed 128 (:20-21); workspaces are ``torch.empty`` (dead splits are never read)."""
from __future__ import annotations

import torch

from kernel_collections_amd import ops
from .stage1 import decoding_stage1
from .stage2 import decoding_stage2


def _run(q_nope, q_rope, kv_nope, k_rope, sm_scale, q_nope_lo=None, up_proj=None):
    batch, num_q_heads, width = q_nope.shape
    kv_len = kv_nope.shape[1]
    groups = ops.head_groups(num_q_heads)
    S = ops.latent_splits(batch, groups, kv_len, width)
    splits = ops.uniform_splits(batch, S, q_nope.device)
    attn_logits, attn_lse = ops.workspaces(batch, num_q_heads, S, width, q_nope.device)
    decoding_stage1(q_nope, q_rope, kv_nope, k_rope, attn_logits, attn_lse, splits, S, sm_scale, q_nope_lo=q_nope_lo)
    if up_proj is None:
        o = torch.empty_like(q_nope)
        decoding_stage2(attn_logits, attn_lse, o, kv_seq_len=kv_len, num_kv_splits=splits, max_kv_splits=S)
        return o
    o = torch.empty((batch, num_q_heads, up_proj.shape[-1]), dtype=q_nope.dtype, device=q_nope.device)
    return ops.merge_stage2(attn_logits, attn_lse, o, up_proj, splits, None, batch, num_q_heads, 1, kv_len, S)


def mla_decode_attention_fwd(q_nope, q_rope, kv_nope, k_rope, sm_scale=1.0):
    """q_nope ``[batch, H, lora]``, q_rope ``[batch, H, rope]``, kv_nope ``[batch, kv_len, 1, lora]``,
    k_rope ``[batch, kv_len, 1, rope]`` -> ``[batch, H, lora]``."""
    assert kv_nope.shape[2] == 1
    return _run(q_nope, q_rope, kv_nope, k_rope, sm_scale)


def mla_decode_attention_xKV(q_nope, q_rope, kv_A_nope, kv_B_nope, k_rope, sm_scale=1.0):
    """kv_A_nope ``[batch, kv_len, 1, rank]``, kv_B_nope ``[batch, 1, rank, lora]``.  The absorb
    ``q_nope @ kv_B^T`` (reference :81-82) runs in ``xkv_absorb_q`` and is kept as a high + low 16-bit pair, so the scan over
    ``kv_A`` sees the query at ~16 mantissa bits; the un-absorb ``o @ kv_B`` (:128) is the up-projection of the merge
    kernel, applied to the fp32 merged latent."""
    assert kv_A_nope.shape[2] == 1
    assert kv_B_nope.shape[1] == 1
    assert kv_B_nope.shape[-1] <= 512 and kv_B_nope.shape[-1] % 8 == 0, "lora rank: a multiple of 8, at most 512"
    q_hi, q_lo = ops.absorb_q(ops._q3(q_nope), kv_B_nope, want_lo=True)
    return _run(q_hi, q_rope, kv_A_nope, k_rope, sm_scale, q_nope_lo=q_lo, up_proj=kv_B_nope)
