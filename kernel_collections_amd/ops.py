"""Thin host layer over the C ABI: marshals torch tensors into the `xkv_*` entry points.

Everything here launches HIP kernels on the current stream and returns without synchronising.
Workspaces are `torch.empty` tensors owned by the caller's allocator; the C side allocates nothing.
"""
from __future__ import annotations

from ctypes import c_float, c_int, c_int64, c_void_p
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import check, dtype_code, kv_operand, ptr, q_operand, stream_ptr

_16BIT = (torch.float16, torch.bfloat16)
_num_cu_cache = {}


def num_cus(device=None) -> int:
    """Compute units of the device, read from its properties (256 on an MI355X)."""
    if not torch.cuda.is_available():
        return 256   # planning a split count off the device (CPU-side tests): the MI355X figure
    idx = torch.cuda.current_device() if device is None else torch.device(device).index
    if idx is None:
        idx = torch.cuda.current_device()
    n = _num_cu_cache.get(idx)
    if n is None:
        n = _num_cu_cache[idx] = int(torch.cuda.get_device_properties(idx).multi_processor_count)
    return n

USE_RECON_WORKSPACE = True  # False: never hand xkv_recon_stage1 a workspace (it then takes its generic kernel)


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


# ------------------------------------------------------------------------------------------------
# small cached device constants (no per-call host->device traffic on the hot path)
# ------------------------------------------------------------------------------------------------
_inv_freq_cache = {}
_splits_cache = {}


def rope_inv_freq(dim: int, theta: float, device) -> torch.Tensor:
    """fp32 `theta**(-2j/dim)` evaluated exactly as the reference's eager RoPE does on the host
    (flash_recontruction/rope/rope_ref.py:4), cached per (dim, theta, device)."""
    key = (int(dim), float(theta), str(device))
    t = _inv_freq_cache.get(key)
    if t is None:
        inv = 1.0 / (float(theta) ** (torch.arange(0, dim, 2, dtype=torch.int64).float() / dim))
        t = inv.to(device=device, dtype=torch.float32).contiguous()
        _inv_freq_cache[key] = t
    return t


def uniform_splits(batch: int, n: int, device) -> torch.Tensor:
    """int32 `[batch]` tensor filled with `n` (what the reference builds with torch.ones(...)*128,
    flash_decoding/mla2/mla_flash_decoding.py:20), cached."""
    key = (int(batch), int(n), str(device))
    t = _splits_cache.get(key)
    if t is None:
        t = torch.full((batch,), int(n), dtype=torch.int32, device=device)
        _splits_cache[key] = t
    return t


def occupancy_splits(batch: int, groups: int, kv_len: int, tile: int = 64, waves: int = 2) -> int:
    """Number of KV splits that gives about `waves` workgroups per CU without making a split
    shorter than 4 tiles."""
    want = _cdiv(waves * num_cus(), max(1, batch * groups))
    cap = max(1, kv_len // (4 * tile))
    return max(1, min(want, cap))


def settled_splits(kv_len: int, n: int) -> int:
    """Largest split count <= n under which EVERY split is live: with `per = cdiv(cdiv(kv_len, n), 32) * 32` tokens per
    split only the first cdiv(kv_len, per) splits hold tokens (flash_decoding/gqa.py:95-99 of the reference)."""
    n = max(1, int(n))
    while True:
        per = _cdiv(_cdiv(kv_len, n), 32) * 32
        live = max(1, _cdiv(kv_len, per))
        if live == n:
            return n
        n = live


def latent_splits(batch: int, groups: int, kv_len: int, width: int, absorbed: bool = False) -> int:
    """Split count for the dot-product stage 1.  512-wide rows - and 256- / 384-wide ones scanned with an absorbed
    query (hi + lo parts, no RoPE features) - run the LDS-ring kernel (one workgroup per CU, 32-token tiles);
    everything else the register-staged one (two workgroups per CU, 64-token tiles)."""
    if width == 512 or (absorbed and width in (256, 384)):
        return occupancy_splits(batch, groups, kv_len, tile=32, waves=1)
    return occupancy_splits(batch, groups, kv_len)


def _row_ok(t: torch.Tensor) -> bool:
    """Unit stride on the feature axis, every other stride a multiple of 8 elements, 16-byte base."""
    if t.stride(-1) != 1 or t.data_ptr() % 16:
        return False
    return all(s % 8 == 0 for s in t.stride()[:-1])


def as_rows(t: torch.Tensor) -> torch.Tensor:
    return t if _row_ok(t) else t.contiguous()


def _q3(q: torch.Tensor) -> torch.Tensor:
    q = q.contiguous()
    assert q.data_ptr() % 16 == 0
    return q


# ------------------------------------------------------------------------------------------------
# entry-point wrappers
# ------------------------------------------------------------------------------------------------
def rope_table(seqlen: int, theta: float, start: int, dtype, device, half_dim: int = 64):
    sin = torch.empty((seqlen, half_dim), dtype=dtype, device=device)
    cos = torch.empty_like(sin)
    inv = rope_inv_freq(2 * half_dim, theta, sin.device)
    check(_lib.lib().xkv_rope_table(ptr(sin), ptr(cos), ptr(inv), c_int64(seqlen), c_int64(start), half_dim,
                                    dtype_code(dtype), stream_ptr(sin)), "xkv_rope_table")
    return sin, cos


def rope_apply(x: torch.Tensor, positions, theta: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotate-half RoPE on the device.  x ``[batch, heads, dim]`` (one row per sequence, e.g. the decode query) or
    ``[batch, rows, heads, dim]`` (row r of sequence b sits at ``positions[b] + r``); ``positions`` an int or an integer
    tensor ``[batch]`` (kept on the device: no host synchronisation).  fp32 angles ``float(pos) * inv_freq`` as in the
    reference's eager form (flash_recontruction/rope/rope_ref.py:3-20); x may be float32, float16 or bfloat16."""
    _lib.require_gpu(x)
    assert x.dim() in (3, 4) and x.stride(-1) == 1 and x.shape[-1] % 2 == 0
    x4 = x.unsqueeze(1) if x.dim() == 3 else x
    if out is None:
        out = torch.empty_like(x)
    assert out.shape == x.shape and out.dtype == x.dtype and out.stride(-1) == 1 and out.device == x.device
    o4 = out.unsqueeze(1) if out.dim() == 3 else out
    b, rows, heads, dim = x4.shape
    pos_t, pos0 = None, 0
    if torch.is_tensor(positions):
        assert positions.numel() == b
        pos_t = positions.to(device=x.device, dtype=torch.int64).contiguous()
    else:
        pos0 = int(positions)
    inv = rope_inv_freq(dim, theta, x.device)
    check(_lib.lib().xkv_rope_apply(ptr(x4), ptr(o4), ptr(inv), ptr(pos_t), c_int64(pos0), b, rows, heads, dim,
                                    c_int64(x4.stride(0)), c_int64(x4.stride(1)), c_int64(x4.stride(2)),
                                    c_int64(o4.stride(0)), c_int64(o4.stride(1)), c_int64(o4.stride(2)),
                                    dtype_code(x.dtype), stream_ptr(x)), "xkv_rope_apply")
    return out


def absorb_q(q3: torch.Tensor, Bk: torch.Tensor, want_lo: bool = True) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """q3 `[b,Hq,d]`, Bk `[b,Hkv,r,d]` (any batch/head/rank strides) -> q~ hi (and lo) `[b,Hq,r]`."""
    b, hq, d = q3.shape
    _, hkv, r, _ = Bk.shape
    if hkv == 1 and hq > 32:   # the kernel serves at most 32 query heads per kv head: one shared matrix seen as several heads
        hkv = head_groups(hq)
        Bk = Bk.expand(-1, hkv, -1, -1)
    Bk = as_rows(Bk)
    hi = torch.empty((b, hq, r), dtype=q3.dtype, device=q3.device)
    lo = torch.empty_like(hi) if want_lo else None
    check(_lib.lib().xkv_absorb_q(ptr(q3), ptr(Bk), ptr(hi), ptr(lo), b, hq, hkv, d, r,
                                  c_int64(Bk.stride(0)), c_int64(Bk.stride(1)), c_int64(Bk.stride(2)),
                                  dtype_code(q3.dtype), stream_ptr(q3)), "xkv_absorb_q")
    return hi, lo


def blockdiag_q(q3: torch.Tensor, hkv: int) -> torch.Tensor:
    """``[batch, hq, d]`` -> ``[batch, hq, hkv * d]`` with head h's row non-zero only in the slot of its kv head."""
    batch, hq, d = q3.shape
    out = torch.empty((batch, hq, hkv * d), dtype=q3.dtype, device=q3.device)
    check(_lib.lib().xkv_blockdiag_q(ptr(q3), ptr(out), batch, hq, hkv, d, dtype_code(q3.dtype), stream_ptr(q3)),
          "xkv_blockdiag_q")
    return out


def latent_stage1(qn, qn_lo, qr, C, R, V, partial, lse, scores, num_kv_splits, kv_lens,
                  batch, hq, groups, kv_len, max_splits, sm_scale, logit_cap=0.0, split_cap=0, split_plan=None):
    """C / R / V are `(tensor, stride_b, stride_l, stride_h, dim)` tuples or None.  `split_cap` > 0: no split longer than that
    many tokens (the kernels then scan sequence b with ``max(num_kv_splits[b], ceil(len_b / split_cap))`` splits; `max_splits`,
    the split dimension of the workspaces, must cover ``ceil(kv_len / split_cap)``).  `split_plan`: the int32 device
    array `plan_splits` returned; the cap in force is then the larger of the two and stage 1 takes its jobs from the list."""
    def op(x):
        return kv_operand(None) if x is None else kv_operand(*x)
    sd = dtype_code(scores.dtype) if scores is not None else 0
    check(_lib.lib().xkv_latent_stage1(
        q_operand(qn), ptr(qn_lo), q_operand(qr), op(C), op(R), op(V), ptr(partial), ptr(lse), ptr(scores), sd,
        ptr(num_kv_splits), ptr(kv_lens), batch, hq, groups, kv_len, max_splits, int(split_cap), ptr(split_plan),
        c_float(sm_scale), c_float(logit_cap), dtype_code(qn.dtype), stream_ptr(qn)), "xkv_latent_stage1")


def softmax_pv_stage1(scores, V, partial, lse, num_kv_splits, kv_lens, batch, hq, kv_len, max_splits, dtype,
                      split_cap=0, split_plan=None):
    """Stage 1 over given scores (fp32 ``[batch, hq, kv_len]``, already scaled): online softmax and ``P @ V`` per split, with V
    ``[batch, kv_len, dv]`` one row per token for every head.  `dtype`: the 16-bit type of V (and of the rounded weights)."""
    v = V.reshape(V.shape[0], V.shape[1], V.shape[-1]) if V.dim() == 4 else V
    check(_lib.lib().xkv_softmax_pv_stage1(
        ptr(scores), kv_operand(v, v.stride(0), v.stride(1), 0, v.shape[-1]), ptr(partial), ptr(lse), ptr(num_kv_splits),
        ptr(kv_lens), batch, hq, kv_len, max_splits, int(split_cap), ptr(split_plan), dtype_code(dtype), stream_ptr(scores)),
        "xkv_softmax_pv_stage1")


def recon_stage1(q3, kA, kB, vA, partial, lse, scores, num_kv_splits, kv_lens, batch, hq, hkv, kv_len, max_splits,
                 sm_scale, rope, inv_freq, pos_offset, sin_cos):
    a_op = kv_operand(kA, kA.stride(0), kA.stride(1), 0, kA.shape[-1])
    ws, ws_bytes = None, 0
    if USE_RECON_WORKSPACE:
        ws_bytes = _lib.lib().xkv_recon_workspace_bytes(batch, hkv, kA.shape[-1], c_int64(kB.stride(0)))
        if ws_bytes:
            ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=q3.device)
    v_op = kv_operand(None) if vA is None else kv_operand(vA, vA.stride(0), vA.stride(1), 0, vA.shape[-1])
    sd = dtype_code(scores.dtype) if scores is not None else 0
    check(_lib.lib().xkv_recon_stage1(
        ptr(q3), a_op, ptr(kB), c_int64(kB.stride(0)), c_int64(kB.stride(1)), c_int64(kB.stride(2)), v_op,
        ptr(partial), ptr(lse), ptr(scores), sd, ptr(num_kv_splits), ptr(kv_lens), batch, hq, hkv, kv_len, max_splits,
        c_float(sm_scale), int(rope), ptr(inv_freq), c_int64(pos_offset), ptr(sin_cos),
        c_int64(sin_cos.stride(0) if sin_cos is not None else 0), ptr(ws), c_int64(ws_bytes),
        dtype_code(q3.dtype), stream_ptr(q3)),
        "xkv_recon_stage1")


def merge_stage2(partial, lse, out, vB, num_kv_splits, kv_lens, batch, hq, hkv, kv_len, max_splits, lse_out=None, split_cap=0,
                 split_plan=None):
    """out `[b,Hq,*]` (strides honoured on the first two axes).  `lse_out` `[b,Hq]` (any strides, fp32): log-sum-exp
    of the merged range.  Up-projections wider than 512 columns run as column blocks of 512."""
    dv = partial.shape[-1]
    assert out.stride(-1) == 1
    sl = (0, 0) if lse_out is None else (lse_out.stride(0), lse_out.stride(1))

    def call(o, w, d_out, sv, vdt, lo):
        check(_lib.lib().xkv_merge_stage2(
            ptr(partial), ptr(lse), ptr(o), ptr(w), c_int64(sv[0]), c_int64(sv[1]), c_int64(sv[2]), d_out, vdt,
            ptr(num_kv_splits), ptr(kv_lens), batch, hq, hkv, kv_len, max_splits, int(split_cap), ptr(split_plan), dv,
            c_int64(o.stride(0)), c_int64(o.stride(1)), dtype_code(o.dtype), ptr(lo), c_int64(sl[0]), c_int64(sl[1]),
            stream_ptr(partial)), "xkv_merge_stage2")

    if vB is None:
        call(out, None, dv, (0, 0, 0), _lib.XKV_BF16, lse_out)
        return out
    if hkv == 1 and hq > 32:   # at most 32 query heads per kv head in the up-projecting merge: the shared matrix as several heads
        hkv = head_groups(hq)
        vB = vB.expand(-1, hkv, -1, -1)
    vB = as_rows(vB)
    sv, vdt = (vB.stride(0), vB.stride(1), vB.stride(2)), dtype_code(vB.dtype)
    for c0 in range(0, vB.shape[-1], 512):
        c1 = min(c0 + 512, vB.shape[-1])
        call(out[..., c0:c1], vB[..., c0:c1], c1 - c0, sv, vdt, lse_out if c0 == 0 else None)
    return out


def plan_splits(kv_lens: torch.Tensor, num_kv_splits: torch.Tensor, max_splits: int, floor_tokens: int, target_jobs: int):
    """The int32 device array `xkv_plan_splits` fills: [0] the smallest multiple of 32, not below `floor_tokens`, that cuts the
    sequences of the batch into at most `target_jobs` splits; [1] the number of live (sequence, split) pairs; then the pairs.
    Pass it as `split_plan` (with `split_cap=floor_tokens` and the same `max_splits`) to stage 1 and the merge."""
    batch = kv_lens.numel()
    plan = torch.empty(2 + 2 * batch * int(max_splits), dtype=torch.int32, device=kv_lens.device)
    check(_lib.lib().xkv_plan_splits(ptr(kv_lens), ptr(num_kv_splits), batch, int(max_splits), int(floor_tokens),
                                     int(target_jobs), ptr(plan), stream_ptr(kv_lens)), "xkv_plan_splits")
    return plan


def capped_splits(kv_len: int, max_kv_splits: int, cap_tokens: int) -> int:
    """Split dimension of the workspaces when no split may be longer than `cap_tokens` tokens (0: no cap)."""
    return max(int(max_kv_splits), _cdiv(kv_len, cap_tokens)) if cap_tokens else int(max_kv_splits)


def workspaces(batch: int, hq: int, max_splits: int, dv: int, device):
    partial = torch.empty((batch, hq, max_splits, dv), dtype=torch.float32, device=device)
    lse = torch.empty((batch, hq, max_splits), dtype=torch.float32, device=device)
    return partial, lse


def head_groups(hq: int, limit: int = 32) -> int:
    """Smallest number of equal head groups with at most `limit` heads each."""
    g = _cdiv(hq, limit)
    while hq % g:
        g += 1
    return g


def check_16bit(*ts):
    dt = ts[0].dtype
    assert dt in _16BIT, f"xkv HIP kernels take float16 or bfloat16 operands, got {dt}"
    for t in ts:
        if t is not None:
            assert t.dtype == dt, f"operand dtypes differ: {t.dtype} vs {dt}"
            _lib.require_gpu(t)


def as_int32_dev(x, batch: int, device) -> torch.Tensor:
    if torch.is_tensor(x):
        assert x.numel() == batch
        if x.dtype != torch.int32 or x.device != device:
            x = x.to(device=device, dtype=torch.int32)
        return x.contiguous()
    return uniform_splits(batch, int(x), device)
