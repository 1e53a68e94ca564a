"""Eager form of absorbed MLA decode with the reference's name (flash_decoding/mla2/ref.py:3-33).
The reference divides by ``sm_scale`` here while its kernel multiplies (stage1.py:136); this one multiplies."""
import torch


def mla_decode_attention_fwd_ref(q_nope, q_rope, kv_nope, k_rope, sm_scale=1.0):
    assert kv_nope.shape[2] == 1
    latent, rope_keys = kv_nope[:, :, 0, :], k_rope[:, :, 0, :]
    logits = torch.einsum("bhc,blc->bhl", q_nope, latent) + torch.einsum("bhe,ble->bhl", q_rope, rope_keys)
    p = torch.softmax(logits * sm_scale, dim=-1, dtype=torch.float32).to(logits.dtype)
    return torch.einsum("bhl,blc->bhc", p, latent)
