"""Eager PyTorch form of ``q @ (Ak @ Bk)^T`` with the reference's ``qAB_ref`` surface
(flash_recontruction/qAB_no_pe/ref.py:4-25).  Plain torch ops on whatever device the tensors
live on; no kernel in this package calls it."""
import torch


def qAB_ref(q: torch.Tensor, Ak: torch.Tensor, Bk: torch.Tensor) -> torch.Tensor:
    bsz, num_heads, q_len, head_dim = q.shape
    assert bsz == Ak.shape[0] == Bk.shape[0], "Batch size mismatch"
    num_kv_heads = Bk.shape[1]
    group = num_heads // num_kv_heads
    keys = torch.einsum("blr,bhrd->bhld", Ak, Bk)
    out = torch.einsum("bhgd,bhld->bhgl", q.reshape(bsz, num_kv_heads, group * q_len, head_dim), keys)
    return out.reshape(bsz, num_heads, q_len, Ak.shape[1])
