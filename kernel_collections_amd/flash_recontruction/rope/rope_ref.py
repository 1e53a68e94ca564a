"""Eager RoPE helpers under the reference's names (flash_recontruction/rope/rope_ref.py:3-20).

``LlamaRotaryEmbedding(dim, end, theta)`` -> ``(cos, sin)``, each ``[end, dim]`` fp32 with the ``dim/2``
pair angles repeated twice along the last axis; ``rotate_half`` / ``apply_rotary_pos_emb_pytorch`` use the
rotate-half pairing (feature j with feature j + dim/2).  These run in torch on whatever device the
arguments live on; the HIP table generator is ``rotary_sin_cos`` in ``sin_cos.py``."""
import torch


def _pair_angles(dim: int, end: int, theta: float) -> torch.Tensor:
    """angle[l, j] = l * theta^(-2j/dim), evaluated in fp32 (position and frequency both fp32)."""
    exponent = torch.arange(0, dim, 2, dtype=torch.float32) / dim
    inv_freq = torch.pow(torch.tensor(theta, dtype=torch.float32), exponent).reciprocal()
    return torch.arange(end, dtype=torch.float32)[:, None] * inv_freq[None, :]


def LlamaRotaryEmbedding(dim: int, end: int, theta: float = 10000.0):
    a = _pair_angles(dim, end, theta)
    return a.cos().repeat(1, 2), a.sin().repeat(1, 2)


def rotate_half(x):
    lo, hi = x.chunk(2, dim=-1)
    return torch.cat((hi.neg(), lo), dim=-1)


def apply_rotary_pos_emb_pytorch(x, cos, sin, unsqueeze_dim=0):
    c, s = (t.unsqueeze(unsqueeze_dim).to(x.device) for t in (cos, sin))
    return x * c + rotate_half(x) * s
