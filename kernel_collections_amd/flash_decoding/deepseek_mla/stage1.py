"""``decoding_stage1`` of the reference's flash_decoding/deepseek_mla/stage1.py:214-287: split-K stage 1 into caller-owned
workspaces.  ``attn_out`` / ``attn_lse`` may be views that start at a split offset of a larger workspace (their
split stride is what counts), which is how prefix and tail partials end up side by side without a concatenation."""
from kernel_collections_amd import ops
from kernel_collections_amd.flash_decoding.mla import stage1_operands


def decoding_stage1(q, k_buffer, v_buffer, attn_out, attn_lse, num_kv_splits, max_kv_splits, sm_scale, logit_cap=0.0):
    batch, num_q_heads, _ = q.shape
    kv_len = k_buffer.shape[1]
    qn, qr, C, R, V, groups, dn, dv = stage1_operands(q, k_buffer, v_buffer)
    assert attn_out.shape[-1] == dv and attn_out.stride(-1) == 1 and attn_out.stride(2) == dv
    assert attn_out.stride(1) == attn_lse.stride(1) * dv and attn_out.stride(0) == attn_lse.stride(0) * dv
    stride_splits = attn_lse.stride(1)          # splits per (sequence, head) row of the underlying workspace
    assert stride_splits >= int(max_kv_splits) and attn_lse.stride(0) == stride_splits * num_q_heads
    splits = ops.as_int32_dev(num_kv_splits, batch, q.device)
    ops.latent_stage1(qn, None, qr, C, R, V, attn_out, attn_lse, None, splits, None, batch, num_q_heads, groups,
                      kv_len, stride_splits, float(sm_scale), float(logit_cap))
