"""``decoding_stage2`` of the reference's flash_decoding/deepseek_mla/stage2.py: log-sum-exp merge of the split partials.
Same argument list as the reference (``q`` and ``v_dim`` are accepted and unused: the width is the workspace's)."""
from kernel_collections_amd import ops


def decoding_stage2(attn_logits, attn_lse, q, o, v_dim, kv_seq_len, num_kv_splits, max_kv_splits):
    batch, head_num = attn_logits.shape[0], attn_logits.shape[1]
    assert attn_logits.is_contiguous() and attn_lse.is_contiguous() and attn_logits.shape[2] == int(max_kv_splits)
    splits = ops.as_int32_dev(num_kv_splits, batch, attn_logits.device)
    ops.merge_stage2(attn_logits, attn_lse, o, None, splits, None, batch, head_num, head_num, int(kv_seq_len),
                     int(max_kv_splits))
