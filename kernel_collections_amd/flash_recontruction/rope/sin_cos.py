"""RoPE sin/cos tables on the device (reference flash_recontruction/rope/sin_cos.py:72-99).

``rotary_sin_cos`` keeps the reference signature and its return order ``(sin, cos)``, each
``[seqlen, 64]``.  The HIP kernel evaluates ``float(starting_idx + l) * theta**(-2j/128)`` in fp32 and
takes a fully range-reduced sincos, i.e. it matches the eager closed form to fp32 rounding rather
than the ~1e-3 of the reference's fast-math helper."""
from __future__ import annotations

import torch

from kernel_collections_amd import ops


def rotary_sin_cos(seqlen: int, theta: float = 10_000.0, starting_idx: int = 0, *,
                   block_size: int = 16, dtype: torch.dtype = torch.float32,
                   device="cuda", stream=None):
    """``block_size`` is accepted for signature compatibility (the launch shape is fixed);
    ``stream``, if given, is made current for the launch."""
    assert block_size > 0
    if stream is not None:
        with torch.cuda.stream(stream):
            return ops.rope_table(seqlen, theta, starting_idx, dtype, device)
    return ops.rope_table(seqlen, theta, starting_idx, dtype, device)


def rotary_apply(x, positions, theta: float = 10_000.0, *, out=None):
    """Rotate ``x`` to absolute ``positions`` on the device - what a caller of the ``q_pe`` entry points otherwise does
    in eager torch (reference rope_ref.py:17-20 on the tables of rope_ref.py:3-9).  ``x`` is ``[batch, heads, dim]`` (one
    position per sequence: the decode query) or ``[batch, rows, heads, dim]`` (row r at ``positions[b] + r``: a tail of new
    keys); ``positions`` an int or an integer tensor ``[batch]``.  Returns a new tensor (or ``out``; ``out=x`` rotates in
    place)."""
    return ops.rope_apply(x, positions, theta, out)
