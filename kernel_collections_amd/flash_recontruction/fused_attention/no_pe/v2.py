"""``gqa_xKV_no_pe_v2`` (reference flash_recontruction/fused_attention/no_pe/v2.py:364-473): like v1 but
takes no ``o`` and returns a new tensor; merge in rank space first, ``@ v_B`` once afterwards."""
import torch

from .._fused import decode_nope


def decode_attention_fwd(q, k_A_buffer, k_B_buffer, v_A_buffer, v_B_buffer, num_kv_splits, max_kv_splits,
                         sm_scale=1.0, *, kv_lens=None):
    o = torch.empty((q.shape[0], q.shape[1], v_B_buffer.shape[-1]), dtype=q.dtype, device=q.device)
    return decode_nope(q, k_A_buffer, k_B_buffer, v_A_buffer, v_B_buffer, o, num_kv_splits, max_kv_splits,
                       sm_scale, kv_lens)
