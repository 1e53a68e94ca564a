"""Eager RoPE helpers with the reference's names (flash_recontruction/rope/rope_ref.py:3-20):
``LlamaRotaryEmbedding`` returns ``(cos, sin)`` of shape ``[end, dim]`` with the halves duplicated,
``rotate_half`` / ``apply_rotary_pos_emb_pytorch`` use the rotate-half pairing (j, j + dim/2)."""
import torch


def LlamaRotaryEmbedding(dim: int, end: int, theta: float = 10000.0):
    inv_freq = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.int64).float() / dim))
    angles = torch.outer(torch.arange(end, dtype=torch.int64).to(inv_freq.dtype), inv_freq)
    angles = torch.cat((angles, angles), dim=-1)
    return angles.cos(), angles.sin()


def rotate_half(x):
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rotary_pos_emb_pytorch(x, cos, sin, unsqueeze_dim=0):
    cos = cos.unsqueeze(unsqueeze_dim).to(x.device)
    sin = sin.unsqueeze(unsqueeze_dim).to(x.device)
    return x * cos + rotate_half(x) * sin
