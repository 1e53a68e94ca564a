"""Eager CPU restatement of the reference semantics for the xKV decode path.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  Every function cites the
reference lines (relative to the reference repository root) whose arithmetic it
follows.  All functions are dtype-agnostic: run them in float32 for the parity
bar, in float64 to measure the oracle's own rounding.

Parity status (what pins each function, none of it by re-typing the formula):
  * ``split_bounds`` / ``live_splits``      - exhaustive tiling properties + C brute force
  * ``rope_cos_sin`` / ``apply_rope``       - identities (pos 0, norm, relative position) + C fp64
  * ``qab_nope`` / ``qab_rope``             - associativity, C brute-force triple loop
  * ``gqa_*`` / ``mla_ref``                 - torch SDPA on reconstructed K/V, C brute force
  * ``splitk_stage1`` / ``merge_stage2``    - S=1 equals direct softmax, split-count invariance
The reference holds no golden vectors for this path (its tests draw unseeded
CUDA randoms), so no function is pinned against a reference fixture.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch

__all__ = [
    "MIN_BLOCK_KV", "split_bounds", "live_splits",
    "rope_inv_freq", "rope_cos_sin", "rotate_half", "apply_rope", "sin_cos_table",
    "qab_nope", "qab_rope", "reconstruct", "reconstruct_rope",
    "softmax_pv", "gqa_plain", "gqa_v_only", "gqa_factorized", "gqa_factorized_rope",
    "gqa_xkv", "gqa_xkv_k_only", "mla_ref", "mla_xkv_ref",
    "splitk_stage1", "merge_stage2", "ragged_apply",
]

MIN_BLOCK_KV = 32  # flash_decoding/gqa.py:38


# --------------------------------------------------------------------------- #
# split arithmetic (integer, bit-exact)                                        #
# --------------------------------------------------------------------------- #
def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


def split_bounds(kv_len: int, num_splits: int, split_id: int) -> Tuple[int, int]:
    """Token range ``[start, end)`` of one KV split.  flash_decoding/gqa.py:95-99
    (stage 1) and :273-281 (stage 2) use the same arithmetic.  A split is live
    iff ``end > start``."""
    per = _cdiv(_cdiv(kv_len, num_splits), MIN_BLOCK_KV) * MIN_BLOCK_KV
    start = per * split_id
    end = min(start + per, kv_len)
    return start, end


def live_splits(kv_len: int, num_splits: int, max_splits: int):
    """``[(split_id, start, end)]`` for every live split among the ``max_splits``
    programs the grid launches (gqa.py:197-201 launches MAX_KV_SPLITS on axis 2;
    :106 / :282 skip the dead ones)."""
    out = []
    for i in range(max_splits):
        s, e = split_bounds(kv_len, num_splits, i)
        if e > s:
            out.append((i, s, e))
    return out


# --------------------------------------------------------------------------- #
# RoPE                                                                         #
# --------------------------------------------------------------------------- #
def rope_inv_freq(dim: int, theta: float) -> torch.Tensor:
    """fp32 ``theta**(-2j/dim)``, j < dim/2.  flash_recontruction/rope/rope_ref.py:4."""
    return 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.int64).float() / dim))


def rope_cos_sin(positions: torch.Tensor, dim: int, theta: float, dtype=torch.float32):
    """``(cos, sin)`` each ``[len(positions), dim]`` with the two halves duplicated.
    Angles are formed in fp32 as ``float(pos) * inv_freq`` exactly like
    rope_ref.py:4-9; pass ``dtype=torch.float64`` to get the same fp32 angles
    evaluated in double."""
    inv = rope_inv_freq(dim, theta)
    ang = torch.outer(positions.to(torch.int64).float(), inv)
    ang = torch.cat((ang, ang), dim=-1).to(dtype)
    return ang.cos(), ang.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """rope_ref.py:11-15."""
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """``x*cos + rotate_half(x)*sin`` (rope_ref.py:17-20); cos/sin broadcast
    against ``x[..., L, dim]``."""
    return x * cos + rotate_half(x) * sin


def sin_cos_table(kv_len: int, dim: int, theta: float, start: int = 0) -> torch.Tensor:
    """The precomputed table the v2 RoPE kernel consumes: ``[kv_len, dim]`` with
    ``[:, :dim/2] = sin`` and ``[:, dim/2:] = cos`` (qAB/v2.py:138-139;
    test_qAB_rope.py:61)."""
    cos, sin = rope_cos_sin(torch.arange(start, start + kv_len), dim, theta)
    return torch.cat((sin[:, : dim // 2], cos[:, : dim // 2]), dim=-1)


# --------------------------------------------------------------------------- #
# scores                                                                       #
# --------------------------------------------------------------------------- #
def reconstruct(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """``K[b,h,l,:] = A[b,l,:] @ B[b,h,:,:]``.  qAB_no_pe/ref.py:18."""
    return torch.matmul(A.unsqueeze(1), B)


def qab_nope(q: torch.Tensor, A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """``q @ (A @ B)^T``: q ``[b,Hq,1,d]`` -> ``[b,Hq,1,L]``, no scale, no mask.
    qAB_no_pe/ref.py:4-25."""
    b, hq, ql, d = q.shape
    hkv = B.shape[1]
    g = hq // hkv
    K = reconstruct(A, B)
    out = torch.matmul(q.reshape(b, hkv, g * ql, d), K.transpose(-1, -2))
    return out.reshape(b, hq, ql, A.shape[1])


def reconstruct_rope(A, B, cos, sin) -> torch.Tensor:
    """``RoPE(A @ B)`` with cos/sin ``[L, d]`` at the keys' absolute positions.
    test_qAB_rope.py:34-36 (rotation applied to K only)."""
    return apply_rope(reconstruct(A, B), cos, sin)


def qab_rope(q_pe: torch.Tensor, A, B, cos, sin) -> torch.Tensor:
    """Scores of an already-rotated query against rotated reconstructed keys;
    the rotated K is cast to the query dtype before the dot.  test_qAB_rope.py:19-43."""
    b, hq, ql, d = q_pe.shape
    hkv = B.shape[1]
    g = hq // hkv
    K = reconstruct_rope(A, B, cos.to(A.dtype), sin.to(A.dtype)).to(q_pe.dtype)
    out = torch.matmul(q_pe.reshape(b, hkv, g * ql, d), K.transpose(-1, -2))
    return out.reshape(b, hq, ql, A.shape[1])


# --------------------------------------------------------------------------- #
# softmax + PV                                                                 #
# --------------------------------------------------------------------------- #
def softmax_pv(scores: torch.Tensor, q_dtype) -> torch.Tensor:
    """fp32 softmax over the last axis, then cast to the query dtype before the
    PV product.  attention.py:330.  (float64 scores keep float64, so the oracle can be
    run in double to measure its own rounding.)"""
    sdt = torch.float64 if scores.dtype == torch.float64 else torch.float32
    return torch.softmax(scores, dim=-1, dtype=sdt).to(q_dtype)


def gqa_plain(q, K, V, sm_scale: float) -> torch.Tensor:
    """Plain GQA decode.  q ``[b,Hq,d]``, K/V ``[b,L,Hkv,d]`` -> ``[b,Hq,d]``.
    flash_decoding/mla.py:442-471 and test_triton_gqa.py:4-23, except that the
    scale MULTIPLIES (the kernels multiply, gqa.py:122; the reference's eager
    helpers divide and only agree at sm_scale=1)."""
    b, hq, d = q.shape
    hkv = K.shape[2]
    g = hq // hkv
    Kt = K.transpose(1, 2)
    Vt = V.transpose(1, 2)
    s = torch.matmul(q.reshape(b, hkv, g, d), Kt.transpose(-1, -2)) * sm_scale
    p = softmax_pv(s, q.dtype)
    return torch.matmul(p, Vt).reshape(b, hq, V.shape[-1])


def gqa_v_only(q, K, vA, vB, sm_scale: Optional[float] = None) -> torch.Tensor:
    """K plain, V = vA @ vB evaluated as (P @ vA) @ vB.  q ``[b,Hq,1,d]``,
    K ``[b,Hkv,L,d]``.  attention.py:202-274 (scale 1/sqrt(d) at :241)."""
    b, hq, ql, d = q.shape
    hkv = K.shape[1]
    g = hq // hkv
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    s = torch.matmul(q.reshape(b, hkv, g * ql, d), K.transpose(-1, -2)) * sm_scale
    p = softmax_pv(s, q.dtype)
    t = torch.matmul(p.reshape(b, hq * ql, -1), vA).reshape(b, hkv, g * ql, -1)
    return torch.matmul(t, vB).reshape(b, hq, ql, vB.shape[-1])


def _factorized_out(scores, q_dtype, vA, vB, hkv):
    b, hq, _, L = scores.shape
    g = hq // hkv
    p = softmax_pv(scores, q_dtype)
    t = torch.matmul(p.reshape(b, hq, L), vA).reshape(b, hkv, g, -1)
    return torch.matmul(t, vB).reshape(b, hq, 1, vB.shape[-1])


def gqa_factorized(q, kA, kB, vA, vB, sm_scale: Optional[float] = None) -> torch.Tensor:
    """Both K and V factorised; q absorbed into kB first.  q ``[b,Hq,1,d]``.
    attention.py:276-357 (absorb :314, scan :318, scale :322, softmax :330,
    P@vA :345, @vB :352)."""
    b, hq, ql, d = q.shape
    hkv = kB.shape[1]
    g = hq // hkv
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    lat = torch.matmul(q.reshape(b, hkv, g * ql, d), kB.transpose(-1, -2)).reshape(b, hq * ql, -1)
    s = torch.matmul(lat, kA.transpose(-1, -2)).reshape(b, hq, ql, -1) * sm_scale
    return _factorized_out(s, q.dtype, vA, vB, hkv)


def gqa_factorized_rope(q_pe, kA, kB, vA, vB, cos, sin, sm_scale: Optional[float] = None):
    """The factorised pipeline of attention.py:276-357 with the score step
    replaced by ``q_pe . RoPE(kA @ kB)^T`` (test_qAB_rope.py:19-43).  The shape of
    the pipeline is attention.py:360-431, which however hard-codes theta and drops
    the scale (:393-396); here the scale is applied (default 1/sqrt(d))."""
    d = q_pe.shape[-1]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    s = qab_rope(q_pe, kA, kB, cos, sin) * sm_scale
    return _factorized_out(s, q_pe.dtype, vA, vB, kB.shape[1])


def gqa_xkv(q, kA, kB, vA, vB, sm_scale: float = 1.0) -> torch.Tensor:
    """3-D-query form of the fully factorised decode.  q ``[b,Hq,d]`` -> ``[b,Hq,d]``.
    fused_attention/no_pe/ref.py:4-87 (which leaves the scale out, :52; the
    kernels it is compared with multiply by ``sm_scale``)."""
    return gqa_factorized(q.unsqueeze(2), kA, kB, vA, vB, sm_scale).squeeze(2)


def gqa_xkv_k_only(q, kA, kB, V, sm_scale: float = 1.0) -> torch.Tensor:
    """K factorised, V plain ``[b,L,Hkv,d]``.  fused_attention/no_pe/ref.py:92-161."""
    b, hq, d = q.shape
    hkv = kB.shape[1]
    g = hq // hkv
    lat = torch.matmul(q.reshape(b, hkv, g, d), kB.transpose(-1, -2)).reshape(b, hq, -1)
    s = torch.matmul(lat, kA.transpose(-1, -2)) * sm_scale
    p = softmax_pv(s, q.dtype).reshape(b, hkv, g, -1)
    return torch.matmul(p, V.transpose(1, 2)).reshape(b, hq, V.shape[-1])


def mla_ref(q_nope, q_rope, kv_nope, k_rope, sm_scale: float = 1.0) -> torch.Tensor:
    """Absorbed MLA decode in latent space.  q_nope ``[b,H,c]``, q_rope ``[b,H,e]``,
    kv_nope ``[b,L,1,c]``, k_rope ``[b,L,1,e]`` -> ``[b,H,c]``.
    flash_decoding/mla2/ref.py:3-33 with the scale MULTIPLIED (stage1.py:136
    multiplies; ref.py:28 divides and only agrees at sm_scale=1)."""
    c = kv_nope.squeeze(2)
    r = k_rope.squeeze(2)
    s = torch.matmul(q_nope, c.transpose(-1, -2)) + torch.matmul(q_rope, r.transpose(-1, -2))
    p = softmax_pv(s * sm_scale, q_nope.dtype)
    return torch.matmul(p, c)


def mla_xkv_ref(q_nope, q_rope, kv_A, kv_B, k_rope, sm_scale: float = 1.0) -> torch.Tensor:
    """MLA whose latent is itself factorised, ``c_kv = kv_A @ kv_B``:
    kv_A ``[b,L,1,r]``, kv_B ``[b,1,r,c]``.  Result ``[b,H,c]``.
    flash_decoding/mla2/mla_flash_decoding.py:66-130 (absorb :81-82, un-absorb :128)."""
    c = torch.matmul(kv_A.squeeze(2), kv_B.squeeze(1)).unsqueeze(2)
    return mla_ref(q_nope, q_rope, c, k_rope, sm_scale)


# --------------------------------------------------------------------------- #
# split-K flash decoding: stage 1 partials and stage 2 merge                   #
# --------------------------------------------------------------------------- #
def splitk_stage1(scores: torch.Tensor, values: torch.Tensor,
                  num_kv_splits: Sequence[int], max_kv_splits: int,
                  kv_lens: Optional[Sequence[int]] = None):
    """Per-split normalised partial output and log-sum-exp.

    scores ``[b,H,L]`` (already scaled), values ``[b,H or 1,L,Dv]``.
    Returns ``partial [b,H,S,Dv]``, ``lse [b,H,S]`` and ``live [b,S]`` (bool); dead
    splits are left as NaN so that a consumer that reads one is caught.
    gqa.py:95-172: partial = acc / sum (:159), lse = max + log(sum) (:170)."""
    b, H, L = scores.shape
    Dv = values.shape[-1]
    partial = torch.full((b, H, max_kv_splits, Dv), float("nan"), dtype=scores.dtype)
    lse = torch.full((b, H, max_kv_splits), float("nan"), dtype=scores.dtype)
    live = torch.zeros((b, max_kv_splits), dtype=torch.bool)
    for ib in range(b):
        n = int(kv_lens[ib]) if kv_lens is not None else L
        for i, s, e in live_splits(n, int(num_kv_splits[ib]), max_kv_splits):
            sc = scores[ib, :, s:e]
            m = sc.max(dim=-1, keepdim=True).values
            p = torch.exp(sc - m)
            den = p.sum(dim=-1, keepdim=True)
            v = values[ib, :, s:e, :]
            partial[ib, :, i, :] = torch.matmul(p.unsqueeze(1), v.expand(H, -1, -1)).squeeze(1) / den
            lse[ib, :, i] = (m + torch.log(den)).squeeze(-1)
            live[ib, i] = True
    return partial, lse, live


def merge_stage2(partial: torch.Tensor, lse: torch.Tensor,
                 num_kv_splits: Sequence[int], max_kv_splits: int, kv_len: int,
                 kv_lens: Optional[Sequence[int]] = None) -> torch.Tensor:
    """LSE-weighted merge of the live splits, visited in increasing split id.
    gqa.py:258-299."""
    b, H, S, Dv = partial.shape
    out = torch.zeros((b, H, Dv), dtype=partial.dtype)
    for ib in range(b):
        n = int(kv_lens[ib]) if kv_lens is not None else kv_len
        g_lse = torch.full((H, 1), -float("inf"), dtype=partial.dtype)
        g_sum = torch.zeros((H, 1), dtype=partial.dtype)
        acc = torch.zeros((H, Dv), dtype=partial.dtype)
        for i, _, _ in live_splits(n, int(num_kv_splits[ib]), max_kv_splits):
            inc = lse[ib, :, i].unsqueeze(-1)
            new = torch.maximum(inc, g_lse)
            old_scale = torch.exp(g_lse - new)
            w = torch.exp(inc - new)
            acc = acc * old_scale + w * partial[ib, :, i, :]
            g_sum = g_sum * old_scale + w
            g_lse = new
        out[ib] = acc / g_sum
    return out


def ragged_apply(fn, kv_lens: Sequence[int], batched: Sequence[torch.Tensor],
                 seq_axes: Sequence[Optional[int]], **kw) -> torch.Tensor:
    """Ragged semantics by definition: sequence ``i`` of a ragged batch equals the
    same call on its own first ``kv_lens[i]`` tokens with batch size 1.
    ``seq_axes[j]`` is the token axis of ``batched[j]`` (None: no token axis)."""
    outs = []
    for i, n in enumerate(kv_lens):
        args = []
        for t, ax in zip(batched, seq_axes):
            ti = t[i:i + 1]
            if ax is not None:
                ti = ti.narrow(ax, 0, int(n))
            args.append(ti)
        outs.append(fn(*args, **kw))
    return torch.cat(outs, dim=0)
