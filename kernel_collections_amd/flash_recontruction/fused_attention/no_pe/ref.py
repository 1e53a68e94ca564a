"""Eager PyTorch forms with the reference's surface (flash_recontruction/fused_attention/no_pe/ref.py:4-161):
3-D query, no softmax scale, fp32 softmax cast back to the query dtype before the value product.
Plain torch ops on the tensors' device; no kernel in this package calls them."""
import torch


def _probs(query, key_A, key_B):
    bsz, hq, d = query.shape
    hkv = key_B.shape[1]
    assert key_A.shape[-1] == key_B.shape[2], "Rank mismatch between key_A and key_B"
    assert hq % hkv == 0, "num_heads must be divisible by num_kv_heads"
    absorbed = torch.einsum("bkgd,bkrd->bkgr", query.reshape(bsz, hkv, hq // hkv, d), key_B).reshape(bsz, hq, -1)
    logits = torch.einsum("bhr,blr->bhl", absorbed, key_A)
    return torch.softmax(logits, dim=-1, dtype=torch.float32).to(query.dtype)


def group_query_attention_xKV(query, key_A, key_B, value_A, value_B, attn_mask=None, dropout_p=0.0):
    assert attn_mask is None and dropout_p == 0.0, "decode path: no mask, no dropout"
    assert value_A.shape[-1] == value_B.shape[2], "Rank mismatch between value_A and value_B"
    bsz, hq, d = query.shape
    hkv = key_B.shape[1]
    p = _probs(query, key_A, key_B)
    latent = torch.einsum("bhl,blr->bhr", p, value_A).reshape(bsz, hkv, hq // hkv, -1)
    return torch.einsum("bkgr,bkrd->bkgd", latent, value_B).reshape(bsz, hq, value_B.shape[-1])


def group_query_attention_xKV_k_only(query, key_A, key_B, value, attn_mask=None, dropout_p=0.0):
    assert attn_mask is None and dropout_p == 0.0, "decode path: no mask, no dropout"
    bsz, hq, d = query.shape
    hkv = key_B.shape[1]
    p = _probs(query, key_A, key_B).reshape(bsz, hkv, hq // hkv, -1)
    return torch.einsum("bkgl,blkd->bkgd", p, value).reshape(bsz, hq, value.shape[-1])
