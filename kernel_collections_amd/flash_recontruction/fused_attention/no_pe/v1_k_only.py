"""``gqa_xKV_no_pe_k_only`` (reference flash_recontruction/fused_attention/no_pe/v1_k_only.py,
``decode_attention_fwd``): K factorised, V a plain ``[batch, kv_len, Hkv, d]`` buffer; fills and returns ``o``."""
from .._fused import decode_k_only


def decode_attention_fwd(q, k_A_buffer, k_B_buffer, v_buffer, o, num_kv_splits, max_kv_splits, sm_scale=1.0, *,
                         kv_lens=None):
    return decode_k_only(q, k_A_buffer, k_B_buffer, v_buffer, o, num_kv_splits, max_kv_splits, sm_scale, kv_lens)
