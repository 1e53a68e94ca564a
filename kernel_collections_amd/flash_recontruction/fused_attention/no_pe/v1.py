"""Fused xKV decode without positional encoding, K and V both factorised.

Call surface of the reference's flash_recontruction/fused_attention/no_pe/v1.py:365-473
(``decode_attention_fwd`` -> exported as ``gqa_xKV_no_pe``): fills and returns ``o``.
HIP path: ``xkv_absorb_q`` -> ``xkv_latent_stage1`` (one scan of k_A / v_A for all query heads,
online softmax per split, partials in v-rank space) -> ``xkv_merge_stage2`` with the ``@ v_B``
up-projection fused behind the merge.  The reference multiplies every split partial by v_B before
merging (v1.py:458-460); the merge is linear, so multiplying once afterwards gives the same result.
"""
from .._fused import decode_nope


def decode_attention_fwd(q, k_A_buffer, k_B_buffer, v_A_buffer, v_B_buffer, o, num_kv_splits, max_kv_splits,
                         sm_scale=1.0, *, kv_lens=None):
    """q ``[batch, Hq, d]``; k_A ``[batch, kv_len, rk]``; k_B ``[batch, Hkv, rk, d]``; v_A ``[batch, kv_len, rv]``;
    v_B ``[batch, Hkv, rv, d]``; o ``[batch, Hq, d]``; num_kv_splits int32 ``[batch]`` (device)."""
    return decode_nope(q, k_A_buffer, k_B_buffer, v_A_buffer, v_B_buffer, o, num_kv_splits, max_kv_splits,
                       sm_scale, kv_lens)
