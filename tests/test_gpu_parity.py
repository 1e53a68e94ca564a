"""GPU parity tests: HIP kernels (through the C ABI) vs the CPU oracle on identical seeded inputs.

Inputs are drawn on the CPU in fp32, rounded to the 16-bit operand type, and BOTH sides see those
rounded values: the oracle runs in fp32 on them (the "fp32 eager reference"), the kernels in 16-bit
with fp32 accumulation.  Bars: attention output max-abs <= 2e-2 (and, tighter, <= 2e-2 of the largest
reference magnitude); pre-softmax scores max|delta|/max|ref| <= 1e-2; split handling bit-exact.
"""
import math

import pytest
import torch

import oracle
from util import OUT_ATOL, check_out, check_scores, f32, gen, max_abs, rel_max, rope_q

pytestmark = pytest.mark.gpu

import kernel_collections_amd.flash_recontruction as fr  # noqa: E402
from kernel_collections_amd import ops  # noqa: E402
from kernel_collections_amd.flash_decoding import deepseek_mla, gqa, mla, mla2  # noqa: E402
from kernel_collections_amd.flash_recontruction.rope.sin_cos import rotary_sin_cos  # noqa: E402

BF, FP = torch.bfloat16, torch.float16


def dev_(dev, *ts):
    return [None if t is None else t.to(dev) for t in ts]


def splits_t(vals, dev):
    return torch.tensor(vals, dtype=torch.int32, device=dev)


# ------------------------------------------------------------------------------------ RoPE table
@pytest.mark.parametrize("theta,start", [(1e4, 0), (5e5, 4096), (1e7, 131072 - 100)])
def test_rope_table(dev, theta, start):
    sin, cos = rotary_sin_cos(300, theta, start, device=dev)
    ocos, osin = oracle.rope_cos_sin(torch.arange(start, start + 300), 128, theta)
    assert sin.shape == (300, 64) and sin.dtype == torch.float32
    # same fp32 angle on both sides; what is left is sincos rounding (the reference's own test holds 1e-3)
    assert max_abs(sin, osin[:, :64]) < 2e-6 and max_abs(cos, ocos[:, :64]) < 2e-6


@pytest.mark.parametrize("dtype", [torch.float32, BF, FP])
def test_rope_apply(dev, dtype):
    """Device-side rotation of a decode query (one position per sequence) and of a tail of new keys (consecutive
    positions) against the oracle's eager rotate-half form on fp32 angles, at positions 0, 4096 and 131071."""
    from kernel_collections_amd.flash_recontruction.rope.sin_cos import rotary_apply
    theta, d = 5e5, 128
    pos = [0, 4096, 131071]
    q = gen((3, 32, d), dtype=dtype, seed=1)
    cos, sin = oracle.rope_cos_sin(torch.tensor(pos), d, theta)
    ref = oracle.apply_rope(q.float(), cos[:, None, :], sin[:, None, :])
    tol = 2e-6 if dtype == torch.float32 else (2.0 ** -8 if dtype == BF else 2.0 ** -11)   # one rounding of the output type
    out = rotary_apply(q.to(dev), torch.tensor(pos, device=dev), theta)
    assert out.dtype == dtype and out.shape == q.shape
    assert rel_max(out, ref) <= tol
    assert max_abs(rotary_apply(q[1:2].to(dev), 4096, theta), ref[1:2]) <= tol * ref.abs().max().item()   # integer position
    # a tail of 70 keys per sequence, starting at 131071 - 69 / 0 / 4096, written in place into a strided view
    L, hkv = 70, 8
    K = gen((3, L, hkv, d + 8), dtype=dtype, seed=2)
    starts = [131071 - (L - 1), 0, 4096]
    refs = []
    for i, s0 in enumerate(starts):
        c, s_ = oracle.rope_cos_sin(torch.arange(s0, s0 + L), d, theta)
        refs.append(oracle.apply_rope(K[i, :, :, :d].float(), c[:, None, :], s_[:, None, :]))
    Kd = K.to(dev)
    view = Kd[..., :d]
    assert rotary_apply(view, torch.tensor(starts, device=dev), theta, out=view) is view
    assert rel_max(Kd[..., :d], torch.stack(refs)) <= tol
    assert torch.equal(Kd[..., d:].cpu(), K[..., d:]), "the padding columns of the strided view are untouched"


# ------------------------------------------------------------------------------------ qAB, no PE
@pytest.mark.parametrize("dtype", [BF, FP])
@pytest.mark.parametrize("b,hq,hkv,L,r", [(2, 32, 8, 1000, 512), (1, 8, 8, 77, 192), (3, 16, 2, 4133, 256),
                                          (1, 64, 8, 300, 384), (2, 4, 1, 64, 64),
                                          (1, 32, 8, 5, 512), (2, 16, 2, 33, 512)])   # shorter than one tile / one token over
def test_qab_nope(dev, dtype, b, hq, hkv, L, r):
    d = 128
    q, A, B = gen((b, hq, 1, d), dtype=dtype, seed=1), gen((b, L, r), dtype=dtype, seed=2), \
        gen((b, hkv, r, d), std=r ** -0.5, dtype=dtype, seed=3)
    ref = oracle.qab_nope(*f32(q, A, B))
    qd, Ad, Bd = dev_(dev, q, A, B)
    out = fr.qAB_no_pe_v1(qd, Ad, Bd)
    assert out.shape == (b, hq, 1, L) and out.dtype == dtype
    check_scores(out, ref, "qAB_no_pe_v1")
    out32 = fr.qAB_no_pe_v2(qd, Ad, Bd, sm_scale=1 / math.sqrt(d), out_dtype=torch.float32)
    assert out32.dtype == torch.float32
    er = check_scores(out32, ref / math.sqrt(d), "qAB_no_pe_v2 fp32")
    assert er < 2e-3, f"hi/lo absorbed query should hold ~1e-3, got {er}"


def test_qab_nope_shared_factor_stride0_and_row_strides(dev):
    b, hq, hkv, L, r, d = 3, 32, 8, 500, 512, 128
    q, A = gen((b, hq, 1, d), seed=1), gen((b, L, r + 64), seed=2)
    Bm = gen((r, hkv * d), std=r ** -0.5, seed=3)                 # one 512 x 1024 matrix for the whole batch
    Bv = Bm.view(r, hkv, d).permute(1, 0, 2).unsqueeze(0).expand(b, hkv, r, d)
    Av = A[:, :, :r]                                              # row stride r + 64, unit feature stride
    ref = oracle.qab_nope(*f32(q, Av, Bv))
    Bd = Bm.to(dev).view(r, hkv, d).permute(1, 0, 2).unsqueeze(0).expand(b, hkv, r, d)
    Ad = A.to(dev)[:, :, :r]
    assert Bd.stride(0) == 0 and Ad.stride(1) == r + 64
    check_scores(fr.qAB_no_pe_v1(q.to(dev), Ad, Bd), ref)


# ------------------------------------------------------------------------------------ qAB with RoPE
@pytest.mark.parametrize("dtype", [BF, FP])
@pytest.mark.parametrize("b,hq,hkv,L,r,theta", [(2, 32, 8, 1000, 512, 5e5), (1, 8, 2, 77, 256, 1e7),
                                                (1, 16, 1, 2085, 384, 1e4), (2, 4, 4, 40, 192, 1e7),
                                                (2, 8, 2, 300, 384, 5e5),    # wave-specialised kernel at rank 384, scores mode
                                                (1, 16, 2, 1500, 256, 1e7),   # ... at rank 256, 8 heads per kv head
                                                (1, 48, 8, 700, 512, 5e5), (2, 15, 3, 333, 384, 1e4)])  # 6 and 5 heads per kv head
def test_qab_rope(dev, dtype, b, hq, hkv, L, r, theta):
    d = 128
    q, A, B = gen((b, hq, 1, d), std=0.5, dtype=dtype, seed=1), gen((b, L, r), dtype=dtype, seed=2), \
        gen((b, hkv, r, d), std=r ** -0.5, dtype=dtype, seed=3)
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta)
    ref = oracle.qab_rope(*f32(q, A, B), cos, sin)
    qd, Ad, Bd = dev_(dev, q, A, B)
    for fn in (fr.qAB_rope_v1, fr.qAB_rope_v3, fr.qAB_rope_v4):
        out = fn(qd, Ad, Bd, theta)
        assert out.shape == (b, hq, 1, L) and out.dtype == dtype
        check_scores(out, ref, fn.__name__)
    table = oracle.sin_cos_table(L, d, theta).to(dtype)
    tcos = torch.cat((table[:, 64:], table[:, 64:]), -1).float()
    tsin = torch.cat((table[:, :64], table[:, :64]), -1).float()
    ref2 = oracle.qab_rope(*f32(q, A, B), tcos, tsin)            # the table as the kernel sees it (16-bit)
    check_scores(fr.qAB_rope_v2(qd, Ad, Bd, table.to(dev)), ref2, "qAB_rope_v2")


def test_qab_rope_long_positions(dev):
    # keys at absolute positions ~128K: angle addition in the kernel vs fp32 angles in the oracle
    b, hq, hkv, L, r, theta, off = 1, 8, 2, 3000, 256, 5e5, 131072 - 3000
    q, A, B = gen((b, hq, 1, 128), std=0.5, seed=1), gen((b, L, r), seed=2), gen((b, hkv, r, 128), std=r ** -0.5, seed=3)
    cos, sin = oracle.rope_cos_sin(torch.arange(off, off + L), 128, theta)
    ref = oracle.qab_rope(*f32(q, A, B), cos, sin)
    out = fr.qAB_rope_v1(*dev_(dev, q, A, B), theta, pos_offset=off, out_dtype=torch.float32)
    check_scores(out, ref)


# ------------------------------------------------------------------------------------ fused xKV decode, no PE
@pytest.mark.parametrize("dtype", [BF, FP])
@pytest.mark.parametrize("b,hq,hkv,L,rk,rv,S", [(2, 32, 8, 3000, 256, 384, 8), (1, 32, 8, 700, 512, 512, 3),
                                                (3, 8, 8, 129, 192, 64, 2), (1, 16, 4, 4096, 384, 256, 16),
                                                (2, 32, 8, 40, 512, 512, 2), (1, 8, 2, 3, 512, 512, 4),   # fewer live splits than asked
                                                (2, 16, 8, 1000, 384, 256, 4), (1, 8, 8, 777, 512, 256, 3),
                                                (1, 128, 8, 600, 512, 512, 2)])   # 16 heads per kv head: the merge's head groups
def test_fused_nope(dev, dtype, b, hq, hkv, L, rk, rv, S):
    d = 128
    q = gen((b, hq, d), std=1 / 3, dtype=dtype, seed=1)
    kA, kB = gen((b, L, rk), dtype=dtype, seed=2), gen((b, hkv, rk, d), std=rk ** -0.5, dtype=dtype, seed=3)
    vA, vB = gen((b, L, rv), dtype=dtype, seed=4), gen((b, hkv, rv, d), std=rv ** -0.5, dtype=dtype, seed=5)
    V = gen((b, L, hkv, d), dtype=dtype, seed=6)
    scale = 0.7
    ref = oracle.gqa_xkv(*f32(q, kA, kB, vA, vB), sm_scale=scale)
    ref_k = oracle.gqa_xkv_k_only(*f32(q, kA, kB, V), sm_scale=scale)
    qd, kAd, kBd, vAd, vBd, Vd = dev_(dev, q, kA, kB, vA, vB, V)
    ns = splits_t([S] * b, dev)
    o = torch.zeros_like(qd)
    ret = fr.gqa_xKV_no_pe(qd, kAd, kBd, vAd, vBd, o, ns, S, scale)
    assert ret is o
    check_out(o, ref, "gqa_xKV_no_pe")
    o2 = fr.gqa_xKV_no_pe_v2(qd, kAd, kBd, vAd, vBd, ns, S, scale)
    assert o2.shape == o.shape and o2.dtype == dtype
    check_out(o2, ref, "gqa_xKV_no_pe_v2")
    o3 = torch.zeros_like(qd)
    check_out(fr.gqa_xKV_no_pe_k_only(qd, kAd, kBd, Vd, o3, ns, S, scale), ref_k, "k_only")


def test_fused_nope_shared_basis_tile_reuse(dev):
    # k_A is v_A (one basis for K and V): the kernel loads each tile once
    b, hq, hkv, L, r, S = 2, 32, 8, 2500, 512, 5
    q = gen((b, hq, 128), seed=1)
    A, kB, vB = gen((b, L, r), seed=2), gen((b, hkv, r, 128), std=r ** -0.5, seed=3), gen((b, hkv, r, 128), std=r ** -0.5, seed=4)
    ref = oracle.gqa_xkv(*f32(q, A, kB, A, vB), sm_scale=128 ** -0.5)
    qd, Ad, kBd, vBd = dev_(dev, q, A, kB, vB)
    o = fr.gqa_xKV_no_pe_v2(qd, Ad, kBd, Ad, vBd, splits_t([S] * b, dev), S, 128 ** -0.5)
    check_out(o, ref)


# ------------------------------------------------------------------------------------ fused xKV decode with RoPE
@pytest.mark.parametrize("dtype", [BF, FP])
@pytest.mark.parametrize("b,hq,hkv,L,rk,rv,S,shared", [(2, 32, 8, 3000, 512, 512, 4, True),
                                                       (1, 32, 8, 1500, 256, 384, 3, False),
                                                       (2, 8, 2, 200, 192, 192, 2, True),
                                                       (1, 16, 1, 4096, 384, 128, 8, False)])
def test_fused_rope(dev, dtype, b, hq, hkv, L, rk, rv, S, shared):
    d, theta = 128, 5e5
    q = rope_q(gen((b, hq, d), dtype=dtype, seed=1), L, theta).to(dtype)
    kA, kB = gen((b, L, rk), dtype=dtype, seed=2), gen((b, hkv, rk, d), std=rk ** -0.5, dtype=dtype, seed=3)
    vA = kA if shared else gen((b, L, rv), dtype=dtype, seed=4)
    vB = gen((b, hkv, vA.shape[-1], d), std=vA.shape[-1] ** -0.5, dtype=dtype, seed=5)
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta)
    scale = d ** -0.5
    ref = oracle.gqa_factorized_rope(*f32(q.unsqueeze(2), kA, kB, vA, vB), cos, sin, sm_scale=scale)[:, :, 0]
    qd, kAd, kBd, vBd = dev_(dev, q, kA, kB, vB)
    vAd = kAd if shared else vA.to(dev)
    o = torch.zeros_like(qd)
    ret = fr.gqa_xKV_rope(qd, kAd, kBd, vAd, vBd, o, splits_t([S] * b, dev), S, scale, theta)
    assert ret is o
    check_out(o, ref, "gqa_xKV_rope")
    table = oracle.sin_cos_table(L, d, theta).to(dtype)
    tcos = torch.cat((table[:, 64:], table[:, 64:]), -1).float()
    tsin = torch.cat((table[:, :64], table[:, :64]), -1).float()
    ref_t = oracle.gqa_factorized_rope(*f32(q.unsqueeze(2), kA, kB, vA, vB), tcos, tsin, sm_scale=scale)[:, :, 0]
    o2 = torch.zeros_like(qd)
    fr.gqa_xKV_rope(qd, kAd, kBd, vAd, vBd, o2, splits_t([S] * b, dev), S, scale, sin_cos=table.to(dev))
    check_out(o2, ref_t, "gqa_xKV_rope table")


@pytest.mark.parametrize("dtype", [BF, FP])
@pytest.mark.parametrize("b,hq,hkv,rk,rv,shared,lens,S,off", [
    (2, 32, 8, 512, 512, False, [1000, 333], 4, 0),        # every shape the 8-wave kernels are built for (fused form)
    (1, 16, 2, 384, 512, False, [2100], 3, 4096),          # 8 query heads per kv head
    (2, 8, 8, 384, 384, False, [17, 64], 2, 0),            # shorter than a tile / exactly two tiles; one head per kv head
    (3, 32, 8, 256, 256, False, [700, 5, 2048], 5, 100000),
    (1, 24, 8, 256, 512, False, [1500], 7, 0),             # the last splits are dead
    (2, 32, 8, 384, 384, True, [900, 1200], 4, 0),
    (2, 16, 4, 256, 256, True, [33, 4000], 6, 131072 - 4000),
    (1, 16, 2, 384, 384, True, [1500], 3, 0),              # the wave-specialised kernel at ranks 384 / 256: 8 heads per kv head ...
    (2, 8, 8, 256, 256, True, [100, 257], 2, 50000),       # ... and one
    (1, 48, 8, 512, 512, True, [1100], 3, 0),              # 6 query heads per kv head: head slots 6 and 7 of the 8 are empty
    (2, 40, 8, 384, 256, False, [70, 1300], 2, 7),         # 5 per kv head
    (1, 21, 3, 256, 256, True, [999], 4, 0),               # 7 per kv head, 3 kv heads
    (2, 32, 8, 512, 512, True, [1, 32], 2, 0),             # one token; exactly one tile (the second split is dead)
    (2, 32, 8, 512, 512, True, [192, 193], 1, 31),         # exactly the six tiles of one unrolled block, and one token more
    (2, 16, 4, 384, 384, False, [1, 191], 3, 0)])
@pytest.mark.parametrize("form", ["fused", "two_pass", "as_shipped"])
def test_fused_rope_wide_kernels(dev, dtype, b, hq, hkv, rk, rv, shared, lens, S, off, form, monkeypatch):
    # a value basis of its own runs either fused (one kernel, two row streams) or as two passes (scores, then softmax + P.v_A);
    # as shipped the choice follows the key rank and the number of tokens scanned: here both forms are forced in turn
    from kernel_collections_amd.flash_recontruction.fused_attention import _fused
    if form == "fused":
        monkeypatch.setattr(_fused, "TWO_PASS_KEY_RANKS", ())
    elif form == "two_pass":
        monkeypatch.setattr(_fused, "TWO_PASS_KEY_RANKS", (512, 384, 256))
        monkeypatch.setattr(_fused, "TWO_PASS_MIN_TOKENS", 0)
    d, theta = 128, 5e5
    L = max(lens)
    q = gen((b, hq, d), std=0.4, dtype=dtype, seed=21)
    kA, kB = gen((b, L, rk), dtype=dtype, seed=22), gen((b, hkv, rk, d), std=rk ** -0.5, dtype=dtype, seed=23)
    vA = kA if shared else gen((b, L, rv), dtype=dtype, seed=24)
    vB = gen((b, hkv, vA.shape[-1], d), std=vA.shape[-1] ** -0.5, dtype=dtype, seed=25)
    scale = d ** -0.5
    qd, kAd, kBd, vBd = dev_(dev, q, kA, kB, vB)
    vAd = kAd if shared else vA.to(dev)
    o = torch.zeros_like(qd)
    fr.gqa_xKV_rope(qd, kAd, kBd, vAd, vBd, o, splits_t([S] * b, dev), S, scale, theta, pos_offset=off,
                    kv_lens=torch.tensor(lens, dtype=torch.int32, device=dev))
    for i, n in enumerate(lens):   # every sequence against the oracle on its own length
        cos, sin = oracle.rope_cos_sin(torch.arange(off, off + n), d, theta)
        ref = oracle.gqa_factorized_rope(*f32(q[i:i + 1].unsqueeze(2), kA[i:i + 1, :n], kB[i:i + 1], vA[i:i + 1, :n], vB[i:i + 1]),
                                         cos, sin, sm_scale=scale)[:, :, 0]
        check_out(o[i:i + 1], ref, "gqa_xKV_rope wide, sequence %d" % i)


def test_config1_shape_factorized_rope(dev):
    """Target configuration 1 (batch 1, 32/8 heads, d 128, L 4096, rank 256, theta 5e5, query at 4096)."""
    torch.manual_seed(0)
    b, hq, hkv, d, L, r, theta = 1, 32, 8, 128, 4096, 256, 5e5
    q = torch.randn(b, hq, 1, d)
    A, Av = torch.randn(b, L, r), torch.randn(b, L, r)
    B, Bv = torch.randn(b, hkv, r, d) / 16, torch.randn(b, hkv, r, d) / 16
    q_pe = rope_q(q[:, :, 0], L, theta)
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta)
    q16, A16, Av16, B16, Bv16 = [t.to(BF) for t in (q_pe, A, Av, B, Bv)]
    ref = oracle.gqa_factorized_rope(*f32(q16.unsqueeze(2), A16, B16, Av16, Bv16), cos, sin)[:, :, 0]
    o = torch.empty(b, hq, d, dtype=BF, device=dev)
    S = 8
    fr.gqa_xKV_rope(*dev_(dev, q16, A16, B16, Av16, Bv16), o, splits_t([S], dev), S, d ** -0.5, theta)
    check_out(o, ref, "config 1")


# ------------------------------------------------------------------------------------ plain flash decoding
@pytest.mark.parametrize("dtype", [BF, FP])
@pytest.mark.parametrize("b,hq,hkv,L,S", [(2, 32, 8, 3000, 8), (1, 8, 8, 100, 4), (3, 16, 2, 4099, 5), (1, 64, 2, 640, 2)])
def test_gqa_plain(dev, dtype, b, hq, hkv, L, S):
    d = 128
    q, K, V = gen((b, hq, d), dtype=dtype, seed=1), gen((b, L, hkv, d), dtype=dtype, seed=2), gen((b, L, hkv, d), dtype=dtype, seed=3)
    scale = d ** -0.5
    ref = oracle.gqa_plain(*f32(q, K, V), scale)
    qd, Kd, Vd = dev_(dev, q, K, V)
    o = torch.zeros_like(qd)
    assert gqa.decode_attention_fwd(qd, Kd, Vd, o, splits_t([S] * b, dev), S, scale) is o
    check_out(o, ref, "gqa plain")


def _ragged_lens(b, lo, hi, seed):
    g = torch.Generator().manual_seed(seed)
    u = torch.rand(b, generator=g)
    return torch.floor(torch.exp(math.log(lo) + u * (math.log(hi) - math.log(lo)))).to(torch.int64).tolist()


def test_gqa_ragged_plain_and_v_factorized(dev):
    """Config-4 semantics at reduced size: per-sequence lengths, fixed-size splits, dead splits skipped."""
    b, hq, hkv, d, rv, split = 6, 32, 8, 128, 512, 256
    lens = _ragged_lens(b, 64, 4096, seed=0)
    lens[0], lens[1] = 4096, 33
    Lmax = max(lens)
    q, K, V = gen((b, hq, d), seed=1), gen((b, Lmax, hkv, d), seed=2), gen((b, Lmax, hkv, d), seed=3)
    vA, vB = gen((b, Lmax, rv), seed=4), gen((b, hkv, rv, d), std=rv ** -0.5, seed=5)
    ns = [-(-n // split) for n in lens]
    S = max(ns)
    scale = d ** -0.5
    ref = oracle.ragged_apply(oracle.gqa_plain, lens, f32(q, K, V), (None, 1, 1), sm_scale=scale)
    ref_v = oracle.ragged_apply(
        lambda q_, K_, vA_, vB_: oracle.gqa_v_only(q_.unsqueeze(2), K_.transpose(1, 2), vA_, vB_, sm_scale=scale)[:, :, 0],
        lens, f32(q, K, vA, vB), (None, 1, 1, None))
    qd, Kd, Vd, vAd, vBd = dev_(dev, q, K, V, vA, vB)
    kl, nst = splits_t(lens, dev), splits_t(ns, dev)
    # poison everything past each sequence's end: the kernels must never read it
    for i, n in enumerate(lens):
        Kd[i, n:] = float("nan"); Vd[i, n:] = float("nan"); vAd[i, n:] = float("nan")
    o = torch.zeros_like(qd)
    gqa.decode_attention_fwd(qd, Kd, Vd, o, nst, S, scale, kv_lens=kl)
    check_out(o, ref, "ragged plain")
    o2 = torch.zeros_like(qd)
    gqa.decode_attention_fwd_v_factorized(qd, Kd, vAd, vBd, o2, nst, S, scale, kv_lens=kl)
    check_out(o2, ref_v, "ragged V-factorised")


@pytest.mark.parametrize("dtype", [BF, FP])
@pytest.mark.parametrize("b,hq,hkv,L,rv,S", [(2, 32, 8, 1500, 512, 4),    # all heads from one workgroup (block-diagonal query)
                                             (1, 16, 4, 333, 512, 2),     # same, 512-wide key rows
                                             (2, 8, 2, 700, 256, 3)])     # one workgroup per kv head
def test_gqa_v_factorized(dev, dtype, b, hq, hkv, L, rv, S):
    d = 128
    q, K = gen((b, hq, d), dtype=dtype, seed=1), gen((b, L, hkv, d), dtype=dtype, seed=2)
    vA, vB = gen((b, L, rv), dtype=dtype, seed=3), gen((b, hkv, rv, d), std=rv ** -0.5, dtype=dtype, seed=4)
    scale = d ** -0.5
    ref = oracle.gqa_v_only(*f32(q.unsqueeze(2), K.transpose(1, 2), vA, vB), sm_scale=scale)[:, :, 0]
    qd, Kd, vAd, vBd = dev_(dev, q, K, vA, vB)
    o = torch.zeros_like(qd)
    gqa.decode_attention_fwd_v_factorized(qd, Kd, vAd, vBd, o, splits_t([S] * b, dev), S, scale)
    check_out(o, ref, "V-factorised")


def test_blockdiag_q_is_exact(dev):
    b, hq, hkv, d = 3, 32, 8, 128
    q = gen((b, hq, d), dtype=BF, seed=7).to(dev)
    out = ops.blockdiag_q(q, hkv).view(b, hq, hkv, d)
    ref = torch.zeros_like(out)
    for h in range(hq):
        ref[:, h, h // (hq // hkv)] = q[:, h]
    assert torch.equal(out, ref)


# ------------------------------------------------------------------------------------ MLA
@pytest.mark.parametrize("dtype", [BF, FP])
@pytest.mark.parametrize("L", [2100, 17])
def test_mla2(dev, dtype, L):
    b, H, c, e = 3, 16, 512, 64
    qn, qr = gen((b, H, c), std=1 / 3, dtype=dtype, seed=1), gen((b, H, e), std=1 / 3, dtype=dtype, seed=2)
    ckv, kpe = gen((b, L, 1, c), std=1 / 3, dtype=dtype, seed=3), gen((b, L, 1, e), std=1 / 3, dtype=dtype, seed=4)
    scale = 1 / math.sqrt(192)
    ref = oracle.mla_ref(*f32(qn, qr, ckv, kpe), scale)
    out = mla2.mla_decode_attention_fwd(*dev_(dev, qn, qr, ckv, kpe), scale)
    assert out.shape == (b, H, c) and out.dtype == dtype
    check_out(out, ref, "mla2")
    # latent itself factorised
    r = 256
    kvA, kvB = gen((b, L, 1, r), std=1 / 3, dtype=dtype, seed=5), gen((b, 1, r, c), std=r ** -0.5, dtype=dtype, seed=6)
    ref_x = oracle.mla_xkv_ref(*f32(qn, qr, kvA, kvB, kpe), scale)
    out_x = mla2.mla_decode_attention_xKV(*dev_(dev, qn, qr, kvA, kvB, kpe), scale)
    check_out(out_x, ref_x, "mla2 xKV")


def test_mla_many_heads(dev):
    b, H, L, c, e = 1, 128, 700, 512, 64
    qn, qr, ckv, kpe = gen((b, H, c), std=1 / 3, seed=1), gen((b, H, e), std=1 / 3, seed=2), \
        gen((b, L, 1, c), std=1 / 3, seed=3), gen((b, L, 1, e), std=1 / 3, seed=4)
    ref = oracle.mla_ref(*f32(qn, qr, ckv, kpe), 0.1)
    check_out(mla2.mla_decode_attention_fwd(*dev_(dev, qn, qr, ckv, kpe), 0.1), ref)


@pytest.mark.parametrize("b,H", [(2, 128), (1, 64), (1, 48)])
def test_mla2_xkv_many_heads(dev, b, H):
    """More than 32 heads share the one factor matrix: the absorb and the up-projecting merge see it as head groups of <= 32."""
    L, c, e, r = 600, 512, 64, 256
    qn, qr, kpe = gen((b, H, c), std=1 / 3, seed=1), gen((b, H, e), std=1 / 3, seed=2), gen((b, L, 1, e), std=1 / 3, seed=4)
    kvA, kvB = gen((b, L, 1, r), std=1 / 3, seed=5), gen((b, 1, r, c), std=r ** -0.5, seed=6)
    ref = oracle.mla_xkv_ref(*f32(qn, qr, kvA, kvB, kpe), 0.1)
    out = mla2.mla_decode_attention_xKV(*dev_(dev, qn, qr, kvA, kvB, kpe), 0.1)
    assert out.shape == (b, H, c)
    check_out(out, ref, "mla2 xKV, %d heads" % H)


@pytest.mark.parametrize("dk,dv,hkv", [(384, 384, 1), (576, 512, 1), (288, 256, 2), (128, 128, 4)])
def test_mla_py_concat_layout(dev, dk, dv, hkv):
    b, H, L = 2, 16, 1100
    q, K = gen((b, H, dk), std=1 / 3, seed=1), gen((b, L, hkv, dk), std=1 / 3, seed=2)
    Kd = K.to(dev)
    if dk == dv:
        V, Vd = gen((b, L, hkv, dv), std=1 / 3, seed=3), None
        Vd = V.to(dev)
    else:
        V, Vd = K[..., :dv], Kd[..., :dv]                         # value = latent part of the key buffer (a view)
    ref = oracle.gqa_plain(*f32(q, K, V), 0.2)
    o = torch.zeros(b, H, dv, dtype=q.dtype, device=dev)
    assert mla.decode_attention_fwd(q.to(dev), Kd, Vd, o, 0.2) is None
    check_out(o, ref, f"mla.py {dk}/{dv}")
    # logit cap
    s = torch.einsum("bkgd,blkd->bkgl", q.float().reshape(b, hkv, H // hkv, dk), K.float()) * 0.2
    p = torch.softmax(30.0 * torch.tanh(s / 30.0), -1)
    ref_c = torch.einsum("bkgl,blkd->bkgd", p, V.float()).reshape(b, H, dv)
    o2 = torch.zeros_like(o)
    mla.decode_attention_fwd(q.to(dev), Kd, Vd, o2, 0.2, 30.0)
    check_out(o2, ref_c, "mla.py logit cap")


# ------------------------------------------------------------------------------------ prefix + tail decode
@pytest.mark.parametrize("dtype", [BF, FP])
@pytest.mark.parametrize("b,H,hd,Lp,Ld,r", [(2, 32, 512, 1500, 100, 512),   # the reference test's shape, shortened
                                            (1, 16, 576, 700, 33, 512),     # 512 + 64 RoPE features, tail shorter than 2 blocks
                                            (3, 8, 128, 300, 1, 256)])      # one decoded token
def test_prefix_tail_decode(dev, dtype, b, H, hd, Lp, Ld, r):
    """flash_decoding/deepseek_mla: attention over [prefix | tail] computed as two stage-1 passes and one merge equals
    plain attention over the concatenation; in the factorised form the prefix is K = k_A k_B, V = v_A v_B."""
    scale = hd ** -0.5
    q = gen((b, H, hd), dtype=dtype, seed=1)
    kA, vA = gen((b, Lp, r), dtype=dtype, seed=2), gen((b, Lp, r), dtype=dtype, seed=3)
    kB, vB = gen((b, 1, r, hd), std=r ** -0.5, dtype=dtype, seed=4), gen((b, 1, r, hd), std=r ** -0.5, dtype=dtype, seed=5)
    Kd, Vd = gen((b, Ld, 1, hd), dtype=dtype, seed=6), gen((b, Ld, 1, hd), dtype=dtype, seed=7)
    # the plain-buffer entry points see the prefix rounded to the operand type; the factorised one reconstructs it in fp32
    Kp32 = oracle.reconstruct(*f32(kA, kB)).transpose(1, 2)
    Vp32 = oracle.reconstruct(*f32(vA, vB)).transpose(1, 2)
    Kp, Vp = Kp32.to(dtype), Vp32.to(dtype)
    qd, kAd, vAd, kBd, vBd, Kdd, Vdd, Kpd, Vpd = dev_(dev, q, kA, vA, kB, vB, Kd, Vd, Kp, Vp)
    if hd != 576:
        ref_plain = oracle.gqa_plain(q.float(), torch.cat([Kp.float(), Kd.float()], 1),
                                     torch.cat([Vp.float(), Vd.float()], 1), scale)
        ref_xkv = oracle.gqa_plain(q.float(), torch.cat([Kp32, Kd.float()], 1), torch.cat([Vp32, Vd.float()], 1), scale)
        o_one = deepseek_mla.mla_decode_attention_fwd(qd, torch.cat([Kpd, Kdd], 1), torch.cat([Vpd, Vdd], 1), scale)
        check_out(o_one, ref_plain, "one buffer")
        o_sep = deepseek_mla.mla_decode_attention_fwd_pd_sep(qd, Kpd, Vpd, Kdd, Vdd, scale)
        check_out(o_sep, ref_plain, "prefix + tail, plain")
        assert max_abs(o_sep, o_one) < 4e-3, "splitting the buffer in two must not change the result beyond rounding"
        if hd <= 256 or hd == 512:
            o_x = deepseek_mla.mla_decode_attention_fwd_pd_sep_xKV(qd, kAd, kBd, vAd, vBd, Kdd, Vdd, scale)
            check_out(o_x, ref_xkv, "prefix factorised + tail plain")
    else:
        # MLA layout: a 576-wide key buffer whose first 512 features are also the values
        o_sep = deepseek_mla.mla_decode_attention_fwd_pd_sep(qd, Kpd, Kpd[..., :512], Kdd, Kdd[..., :512], scale)
        Kall = torch.cat([Kp.float(), Kd.float()], 1)
        check_out(o_sep, oracle.gqa_plain(q.float(), Kall, Kall[..., :512], scale), "prefix + tail, MLA layout")


# ------------------------------------------------------------------------------------ committed vectors
def test_committed_golden_vectors(dev):
    """The HIP path on the committed inputs (tests/golden/xkv_vectors.npz; all values exactly representable in bf16)
    against the committed oracle outputs."""
    import os
    import numpy as np
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "xkv_vectors.npz"), allow_pickle=False)
    g = {k: torch.from_numpy(z[k]) for k in z.files}
    h = lambda k: g[k].to(BF).to(dev)
    q, A, Av, kB, vB, K, V = (h(k) for k in ("q", "A", "Av", "kB", "vB", "K", "V"))
    theta, scale = float(g["theta"]), float(g["scale"])
    b, hq = q.shape[0], q.shape[1]
    S = 2
    ns = splits_t([S] * b, dev)
    check_scores(fr.qAB_no_pe_v1(q, A, kB, out_dtype=torch.float32), g["qab_nope"], "qab_nope")
    check_scores(fr.qAB_rope_v1(q, A, kB, theta, out_dtype=torch.float32), g["qab_rope"], "qab_rope")
    q3 = q[:, :, 0].contiguous()
    check_out(fr.gqa_xKV_no_pe_v2(q3, A, kB, Av, vB, ns, S, scale), g["gqa_xkv"], "gqa_xkv")
    o = torch.empty_like(q3)
    fr.gqa_xKV_rope(q3, A, kB, Av, vB, o, ns, S, scale, theta)
    check_out(o, g["gqa_factorized_rope"], "gqa_factorized_rope")
    o = torch.empty_like(q3)
    gqa.decode_attention_fwd(q3, K, V, o, ns, S, scale)
    check_out(o, g["gqa_plain"], "gqa_plain")
    o = torch.empty_like(q3)
    gqa.decode_attention_fwd_v_factorized(q3, K, Av, vB, o, ns, S, scale)
    check_out(o, g["gqa_v_only"], "gqa_v_only")
    sin, cos = rotary_sin_cos(A.shape[1], theta, 0, device=dev)
    assert max_abs(torch.cat((sin, cos), -1), g["sin_cos_table"]) < 2e-6
    out = mla2.mla_decode_attention_fwd(h("mla_qn"), h("mla_qr"), h("mla_ckv"), h("mla_kpe"), float(g["mla_scale"]))
    check_out(out, g["mla_ref"], "mla_ref")


# ------------------------------------------------------------------------------------ split handling, bit-exact
@pytest.mark.parametrize("L,ns,S", [(1000, 4, 4), (100, 8, 8), (4096, 3, 5), (33, 2, 2), (64, 1, 3)])
def test_split_index_handling_is_exact(dev, L, ns, S):
    """Which (batch, split) slots get written is decided by integer arithmetic that must equal the
    reference's: poison the workspaces with NaN, run stage 1, and compare the written/untouched pattern
    with oracle.live_splits; then compare the written partials and lse with the oracle's split-K values."""
    b, hq, hkv, d = 2, 8, 2, 128
    q, K, V = gen((b, hq, d), seed=1), gen((b, L, hkv, d), seed=2), gen((b, L, hkv, d), seed=3)
    lens = [L, max(1, L // 3)]
    qd, Kd, Vd = dev_(dev, q, K, V)
    partial = torch.full((b, hq, S, d), float("nan"), device=dev)
    lse = torch.full((b, hq, S), float("nan"), device=dev)
    ops.latent_stage1(qd, None, None, (Kd, Kd.stride(0), Kd.stride(1), Kd.stride(2), d), None,
                      (Vd, Vd.stride(0), Vd.stride(1), Vd.stride(2), d), partial, lse, None,
                      splits_t([ns, ns], dev), splits_t(lens, dev), b, hq, hkv, L, S, 0.1)
    g = hq // hkv
    scores = torch.einsum("bkgd,blkd->bkgl", q.float().reshape(b, hkv, g, d), K.float()).reshape(b, hq, L) * 0.1
    vals = V.float().permute(0, 2, 1, 3).repeat_interleave(g, dim=1)
    op, ol, live = oracle.splitk_stage1(scores, vals, [ns, ns], S, kv_lens=lens)
    written = ~torch.isnan(lse.cpu())
    assert torch.equal(written, live.unsqueeze(1).expand(b, hq, S)), "live/dead split pattern differs"
    assert torch.equal(~torch.isnan(partial.cpu()).any(-1), written)
    m = written
    assert (lse.cpu()[m] - ol[m]).abs().max() < 2e-3
    assert (partial.cpu()[m] - op[m]).abs().max() < OUT_ATOL
    out = torch.empty(b, hq, d, device=dev)
    ops.merge_stage2(partial, lse, out, None, splits_t([ns, ns], dev), splits_t(lens, dev), b, hq, hq, L, S)
    ref = oracle.merge_stage2(partial.cpu(), lse.cpu(), [ns, ns], S, L, kv_lens=lens)
    assert max_abs(out, ref) < 1e-5, "stage 2 merges exactly the live splits"


def test_split_count_invariance_and_v1_v2_order(dev):
    b, hq, hkv, L, r = 1, 32, 8, 5000, 256
    q = gen((b, hq, 128), std=0.5, seed=1)
    kA, kB, vA, vB = gen((b, L, r), seed=2), gen((b, hkv, r, 128), std=r ** -0.5, seed=3), gen((b, L, r), seed=4), \
        gen((b, hkv, r, 128), std=r ** -0.5, seed=5)
    args = dev_(dev, q, kA, kB, vA, vB)
    outs = [fr.gqa_xKV_no_pe_v2(*args, splits_t([S], dev), S, 0.1).float() for S in (1, 2, 7, 32)]
    for o in outs[1:]:
        assert max_abs(o, outs[0]) < 4e-3, "result must not depend on the number of splits beyond rounding"


# ------------------------------------------------------------------------------------ full-size properties
def test_full_size_config3_properties(dev):
    """Target configuration 3 shape (batch 16, L 32768, rank 512) is too big for the CPU oracle as a whole:
    check one sequence against the oracle, and the rest through size-independent properties -
    batch permutation equivariance and linearity in v_B."""
    b, hq, hkv, d, L, r, theta = 16, 32, 8, 128, 32768, 512, 5e5
    g = torch.Generator(device="cpu").manual_seed(0)
    A1 = gen((1, L, r), g=g)
    q = rope_q(gen((b, hq, d), g=g), L, theta).to(BF)
    kB, vB = gen((1, hkv, r, d), std=r ** -0.5, g=g), gen((1, hkv, r, d), std=r ** -0.5, g=g)
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta)
    ref0 = oracle.gqa_factorized_rope(*f32(q[:1].unsqueeze(2), A1, kB, A1, vB), cos, sin)[0, :, 0]
    # device batch: sequence 0 = A1, the others = deterministic row rolls of it (cheap to build on device)
    A1d = A1.to(dev)
    Ad = torch.cat([torch.roll(A1d, shifts=17 * i, dims=2) for i in range(b)], dim=0).contiguous()
    qd, kBd, vBd = q.to(dev), kB.to(dev).expand(b, hkv, r, d), vB.to(dev).expand(b, hkv, r, d)
    S = 4
    ns = splits_t([S] * b, dev)
    o = torch.empty(b, hq, d, dtype=BF, device=dev)
    fr.gqa_xKV_rope(qd, Ad, kBd, Ad, vBd, o, ns, S, d ** -0.5, theta)
    check_out(o[0], ref0, "config 3, sequence 0")
    perm = torch.arange(b - 1, -1, -1, device=dev)
    o_p = torch.empty_like(o)
    Ap = Ad[perm].contiguous()   # passed as k_A and v_A: one tensor, so the shared-basis kernel runs as above
    fr.gqa_xKV_rope(qd[perm], Ap, kBd, Ap, vBd, o_p, ns, S, d ** -0.5, theta)
    assert torch.equal(o_p, o[perm]), "sequences are independent: permuting the batch permutes the output bit for bit"
    o2 = torch.empty_like(o)
    fr.gqa_xKV_rope(qd, Ad, kBd, Ad, (vBd * 2).contiguous(), o2, ns, S, d ** -0.5, theta)
    assert rel_max(o2.float(), o.float() * 2) < 1e-2, "output is linear in v_B"
