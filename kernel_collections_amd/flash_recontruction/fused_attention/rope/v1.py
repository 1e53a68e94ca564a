"""Fused xKV decode WITH RoPE - the composition the reference does not have as one kernel:
key reconstruction + rotation (flash_recontruction/qAB/v1.py:54-86) inside the split-K stage 1 of
fused_attention/no_pe/v1.py:40-190, then the rank-space merge and ``@ v_B``.

``q_pe`` is the already-rotated query; keys sit at absolute positions ``pos_offset + l``.
Either ``theta`` (angles ``float(pos) * theta**(-2j/128)``) or a ``sin_cos [kv_len, 128]`` table
(``[:, :64] = sin``, ``[:, 64:] = cos``) selects the rotation."""
from .._fused import decode_rope


def decode_attention_fwd(q_pe, k_A_buffer, k_B_buffer, v_A_buffer, v_B_buffer, o, num_kv_splits, max_kv_splits,
                         sm_scale=1.0, theta=10000000.0, sin_cos=None, *, pos_offset=0, kv_lens=None):
    return decode_rope(q_pe, k_A_buffer, k_B_buffer, v_A_buffer, v_B_buffer, o, num_kv_splits, max_kv_splits,
                       sm_scale, theta, sin_cos, pos_offset, kv_lens)
