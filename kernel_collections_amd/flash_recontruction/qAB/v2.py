"""``qAB_precomp`` (reference flash_recontruction/qAB/v2.py:132-187): RoPE scores from a
precomputed ``[kv_len, head_dim]`` sin|cos table.  Implemented beside ``qAB`` in v1."""
from .v1 import qAB_precomp  # noqa: F401
