"""``decoding_stage1`` of the reference's flash_decoding/mla2/stage1.py:181-249: split-K stage 1 of absorbed MLA.
``qk = q_nope . kv_nope + q_rope . k_rope`` on MFMA, online softmax, ``acc += p . kv_nope`` with the latent
tile loaded once (the reference reuses it through ``tl.trans``, stage1.py:150)."""
from kernel_collections_amd import ops


def decoding_stage1(q_nope, q_rope, kv_nope, k_rope, attn_out, attn_lse, num_kv_splits, max_kv_splits, sm_scale, *,
                    q_nope_lo=None):
    """``q_nope_lo`` (keyword-only, not in the reference): residual of an absorbed query kept as a high + low 16-bit pair
    (``ops.absorb_q``); its dot with the latent is added to the scores."""
    batch, head_num, dmodel = q_nope.shape
    assert kv_nope.dim() == 4 and k_rope.dim() == 4
    n_kv = kv_nope.shape[2]
    assert head_num % n_kv == 0
    ops.check_16bit(q_nope, q_rope, kv_nope, k_rope)
    assert dmodel % 64 == 0 and dmodel <= 512, "latent width must be a multiple of 64, at most 512"
    assert q_rope.shape[-1] % 32 == 0 and q_rope.shape[-1] <= 128
    kv_len = kv_nope.shape[1]
    kv_nope, k_rope = ops.as_rows(kv_nope), ops.as_rows(k_rope)
    per_kv_groups = ops.head_groups(head_num // n_kv)
    assert per_kv_groups == 1 or n_kv == 1
    groups = n_kv * per_kv_groups
    sh_c = kv_nope.stride(2) if per_kv_groups == 1 else 0
    sh_r = k_rope.stride(2) if per_kv_groups == 1 else 0
    splits = ops.as_int32_dev(num_kv_splits, batch, q_nope.device)
    C = (kv_nope, kv_nope.stride(0), kv_nope.stride(1), sh_c, dmodel)
    R = (k_rope, k_rope.stride(0), k_rope.stride(1), sh_r, k_rope.shape[-1])
    ops.latent_stage1(ops._q3(q_nope), None if q_nope_lo is None else ops._q3(q_nope_lo), ops._q3(q_rope), C, R, C, attn_out, attn_lse, None, splits, None,
                      batch, head_num, groups, kv_len, int(max_kv_splits), float(sm_scale))
