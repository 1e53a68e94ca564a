"""``decoding_stage2`` of the reference's flash_decoding/mla2/stage2.py:102-136: LSE merge of the split partials."""
from kernel_collections_amd import ops


def decoding_stage2(attn_logits, attn_lse, o, kv_seq_len, num_kv_splits, max_kv_splits):
    batch, head_num = attn_logits.shape[0], attn_logits.shape[1]
    splits = ops.as_int32_dev(num_kv_splits, batch, attn_logits.device)
    ops.merge_stage2(attn_logits, attn_lse, o, None, splits, None, batch, head_num, head_num, int(kv_seq_len),
                     int(max_kv_splits))
