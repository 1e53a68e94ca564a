"""CPU tests that PIN the oracle: every check is an identity, invariant, library routine or an
independent brute-force implementation (oracle/xkv_oracle.c), never the oracle's own formula retyped."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import cbrute

torch.manual_seed(0)


def rnd(*shape, std=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float64) * std


# ----------------------------------------------------------------------------- split arithmetic
def test_split_bounds_tile_the_sequence_exhaustive():
    for L in list(range(1, 700)) + [1023, 1024, 1025, 4095, 4096, 4097, 131071, 131072, 262144]:
        for ns in list(range(1, 40)) + [64, 128]:
            live = oracle.live_splits(L, ns, ns + 3)
            per = None
            pos = 0
            for k, (i, s, e) in enumerate(live):
                assert i == k, "live splits are a prefix of the split ids"
                assert s == pos and e > s
                if k + 1 < len(live):
                    per = per or (e - s)
                    assert e - s == per and per % 32 == 0
                pos = e
            assert pos == L, "live splits cover [0, L) exactly"
            assert len(live) <= ns


def test_split_bounds_match_c_bruteforce():
    for L in (1, 31, 32, 33, 1000, 4096, 5000, 131072):
        for ns in (1, 2, 3, 7, 32, 128):
            for i in range(ns + 2):
                assert oracle.split_bounds(L, ns, i) == cbrute.split_bounds(L, ns, i)


def test_split_known_values():
    # ceil(ceil(4096/3)/32)*32 = 1376
    assert oracle.split_bounds(4096, 3, 0) == (0, 1376)
    assert oracle.split_bounds(4096, 3, 2) == (2752, 4096)
    # a request for more splits than 32-token blocks leaves the tail splits dead
    assert [x[0] for x in oracle.live_splits(100, 8, 8)] == [0, 1, 2, 3]
    assert oracle.live_splits(100, 8, 8)[-1] == (3, 96, 100)


# ----------------------------------------------------------------------------- RoPE
def test_rope_position_zero_is_identity_and_norm_is_preserved():
    x = rnd(5, 128).float()
    cos, sin = oracle.rope_cos_sin(torch.tensor([0, 1, 17, 4096, 131071]), 128, 5e5)
    y = oracle.apply_rope(x, cos, sin)
    assert torch.equal(y[0], x[0])
    pair_norm = lambda t: t[:, :64] ** 2 + t[:, 64:] ** 2
    assert torch.allclose(pair_norm(y), pair_norm(x), rtol=1e-5, atol=1e-6)


def test_rope_inner_product_depends_on_relative_position_only():
    q, k = rnd(1, 128, seed=1), rnd(1, 128, seed=2)
    def dot(m, n):
        cm, sm = oracle.rope_cos_sin(torch.tensor([m]), 128, 1e4, dtype=torch.float64)
        cn, sn = oracle.rope_cos_sin(torch.tensor([n]), 128, 1e4, dtype=torch.float64)
        return (oracle.apply_rope(q, cm, sm) * oracle.apply_rope(k, cn, sn)).sum().item()
    # small positions so the fp32 angle rounding (the oracle forms angles in fp32) stays ~1e-6
    assert abs(dot(7, 3) - dot(14, 10)) < 1e-4
    assert abs(dot(7, 3) - dot(3, 7)) > 1e-3  # and it is not symmetric: sign of the rotation matters


def test_rope_closed_form_matches_c_double():
    dim, theta = 128, 5e5
    pos = torch.tensor([0, 1, 5, 100, 4095, 32768])
    cos, sin = oracle.rope_cos_sin(pos, dim, theta)
    assert cos.shape == (6, 128) and torch.equal(cos[:, :64], cos[:, 64:])
    for a, p in enumerate(pos.tolist()):
        for j in (0, 1, 7, 31, 63):
            c, s = cbrute.rope_cs(p, j, dim, theta)
            # fp32 angle: |delta angle| <= ulp(angle) ~ angle * 2^-23 (+ inv_freq rounding, same order)
            tol = 4 * max(p * theta ** (-2 * j / dim), 1.0) * 2.0 ** -23 + 1e-6
            assert abs(cos[a, j].item() - c) < tol and abs(sin[a, j].item() - s) < tol


def test_sin_cos_table_layout():
    t = oracle.sin_cos_table(9, 128, 1e7, start=3)
    cos, sin = oracle.rope_cos_sin(torch.arange(3, 12), 128, 1e7)
    assert torch.equal(t[:, :64], sin[:, :64]) and torch.equal(t[:, 64:], cos[:, :64])


# ----------------------------------------------------------------------------- scores
@pytest.mark.parametrize("hq,hkv", [(8, 2), (4, 4), (6, 1)])
def test_qab_nope_bruteforce_and_associativity(hq, hkv):
    b, d, L, r = 2, 16, 37, 12
    q, A, B = rnd(b, hq, 1, d, seed=1), rnd(b, L, r, seed=2), rnd(b, hkv, r, d, seed=3)
    got = oracle.qab_nope(q, A, B)
    ref = cbrute.qab(q[:, :, 0].numpy(), A.numpy(), B.numpy())
    assert np.allclose(got[:, :, 0].numpy(), ref, rtol=1e-10, atol=1e-10)
    # q (A B)^T == (q B^T) A^T
    g = hq // hkv
    absorbed = torch.einsum("bkgd,bkrd->bkgr", q.reshape(b, hkv, g, d), B).reshape(b, hq, r)
    assert torch.allclose(torch.einsum("bhr,blr->bhl", absorbed, A), got[:, :, 0], rtol=1e-10, atol=1e-10)


def test_qab_rope_matches_bruteforce():
    b, hq, hkv, d, L, r, theta = 1, 4, 2, 128, 40, 8, 1e4
    q, A, B = rnd(b, hq, 1, d, seed=4), rnd(b, L, r, seed=5), rnd(b, hkv, r, d, seed=6, std=0.3)
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta, dtype=torch.float64)
    got = oracle.qab_rope(q, A, B, cos, sin)[:, :, 0].numpy()
    ref = cbrute.qab(q[:, :, 0].numpy(), A.numpy(), B.numpy(), rope=True, theta=theta)
    # positions < 40: fp32 angle rounding <= 40 * 2^-23 per pair
    assert np.allclose(got, ref, rtol=0, atol=1e-4 * np.abs(ref).max())
    # rotating K by R(l) equals rotating q by R(-l): un-rotate q per key and use plain K
    K = oracle.reconstruct(A, B)
    g = hq // hkv
    for l in (0, 13, 39):
        q_back = oracle.apply_rope(q[:, :, 0], cos[l], -sin[l])
        s = torch.einsum("bkgd,bkd->bkg", q_back.reshape(b, hkv, g, d), K[:, :, l]).reshape(b, hq)
        assert np.allclose(s.numpy(), got[:, :, l], atol=1e-9)


# ----------------------------------------------------------------------------- full decode
def _sdpa(q4, K, V, scale):
    return F.scaled_dot_product_attention(q4, K, V, scale=scale, enable_gqa=True)


def test_gqa_factorized_vs_sdpa_and_bruteforce():
    b, hq, hkv, d, L, rk, rv = 2, 8, 2, 16, 50, 6, 10
    q = rnd(b, hq, 1, d, seed=1)
    kA, kB = rnd(b, L, rk, seed=2), rnd(b, hkv, rk, d, seed=3, std=0.5)
    vA, vB = rnd(b, L, rv, seed=4), rnd(b, hkv, rv, d, seed=5, std=0.5)
    got = oracle.gqa_factorized(q, kA, kB, vA, vB)            # default scale 1/sqrt(d)
    K, V = oracle.reconstruct(kA, kB), oracle.reconstruct(vA, vB)
    assert torch.allclose(got, _sdpa(q, K, V, 1 / math.sqrt(d)), rtol=1e-9, atol=1e-9)
    ref = cbrute.decode_factorized(q[:, :, 0], kA, kB, vA, vB, 1 / math.sqrt(d))
    assert np.allclose(got[:, :, 0].numpy(), ref, rtol=1e-9, atol=1e-9)
    # 3-D query form, explicit scale
    got3 = oracle.gqa_xkv(q[:, :, 0], kA, kB, vA, vB, sm_scale=0.37)
    assert np.allclose(got3.numpy(), cbrute.decode_factorized(q[:, :, 0], kA, kB, vA, vB, 0.37), atol=1e-9)


def test_gqa_factorized_rope_vs_bruteforce():
    b, hq, hkv, d, L, rk, rv, theta = 1, 4, 2, 128, 33, 8, 12, 5e5
    q = rnd(b, hq, 1, d, seed=1, std=0.5)
    kA, kB = rnd(b, L, rk, seed=2), rnd(b, hkv, rk, d, seed=3, std=0.3)
    vA, vB = rnd(b, L, rv, seed=4), rnd(b, hkv, rv, d, seed=5, std=0.3)
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta, dtype=torch.float64)
    got = oracle.gqa_factorized_rope(q, kA, kB, vA, vB, cos, sin)[:, :, 0].numpy()
    ref = cbrute.decode_factorized(q[:, :, 0], kA, kB, vA, vB, 1 / math.sqrt(d), rope=True, theta=theta)
    assert np.allclose(got, ref, rtol=0, atol=1e-4 * np.abs(ref).max())


def test_plain_vonly_konly_mla_consistency():
    b, hq, hkv, d, L, r = 2, 8, 4, 16, 45, 6
    q = rnd(b, hq, d, seed=1)
    K, V = rnd(b, L, hkv, d, seed=2), rnd(b, L, hkv, d, seed=3)
    got = oracle.gqa_plain(q, K, V, 0.3)
    assert np.allclose(got.numpy(), cbrute.decode_plain(q, K, V, 0.3), atol=1e-10)
    assert torch.allclose(got, _sdpa(q.unsqueeze(2), K.transpose(1, 2), V.transpose(1, 2), 0.3)[:, :, 0], atol=1e-10)
    # V-only factorised == plain with V reconstructed
    vA, vB = rnd(b, L, r, seed=4), rnd(b, hkv, r, d, seed=5)
    Vrec = oracle.reconstruct(vA, vB).transpose(1, 2)          # [b, L, hkv, d]
    a = oracle.gqa_v_only(q.unsqueeze(2), K.transpose(1, 2), vA, vB, sm_scale=0.3)[:, :, 0]
    assert torch.allclose(a, oracle.gqa_plain(q, K, Vrec, 0.3), atol=1e-10)
    # K-only factorised == plain with K reconstructed
    kA, kB = rnd(b, L, r, seed=6), rnd(b, hkv, r, d, seed=7)
    Krec = oracle.reconstruct(kA, kB).transpose(1, 2)
    assert torch.allclose(oracle.gqa_xkv_k_only(q, kA, kB, V, 0.3), oracle.gqa_plain(q, Krec, V, 0.3), atol=1e-10)
    # MLA == plain GQA with one kv head, K = cat(c, pe), V = c
    H, c, e = 6, 12, 4
    qn, qr, ckv, kpe = rnd(b, H, c, seed=8), rnd(b, H, e, seed=9), rnd(b, L, 1, c, seed=10), rnd(b, L, 1, e, seed=11)
    m = oracle.mla_ref(qn, qr, ckv, kpe, 0.21)
    assert torch.allclose(m, oracle.gqa_plain(torch.cat((qn, qr), -1), torch.cat((ckv, kpe), -1), ckv, 0.21), atol=1e-10)
    assert np.allclose(m.numpy(), cbrute.mla(qn, qr, ckv, kpe, 0.21), atol=1e-10)
    # xKV-MLA: factorised latent
    kvA, kvB = rnd(b, L, 1, 5, seed=12), rnd(b, 1, 5, c, seed=13)
    full = torch.matmul(kvA.squeeze(2), kvB.squeeze(1)).unsqueeze(2)
    assert torch.allclose(oracle.mla_xkv_ref(qn, qr, kvA, kvB, kpe, 0.21), oracle.mla_ref(qn, qr, full, kpe, 0.21), atol=1e-10)


def test_softmax_cast_order():
    """Probabilities are formed in fp32 and rounded to the query dtype BEFORE the value product (attention.py:330).  The two
    orders give different results in bf16, and the oracle equals the rounded-first one bit for bit."""
    b, hq, hkv, d, L = 1, 4, 2, 16, 64
    q, K, V = (rnd(b, hq, d, seed=1).to(torch.bfloat16), rnd(b, L, hkv, d, seed=2).to(torch.bfloat16),
               rnd(b, L, hkv, d, seed=3).to(torch.bfloat16))
    out = oracle.gqa_plain(q, K, V, 0.7)
    assert out.dtype == torch.bfloat16
    assert oracle.softmax_pv(torch.zeros(1, 4), torch.bfloat16).dtype == torch.bfloat16
    g = hq // hkv
    s = torch.matmul(q.reshape(b, hkv, g, d), K.transpose(1, 2).transpose(-1, -2)) * 0.7
    p32 = torch.softmax(s, dim=-1, dtype=torch.float32)
    rounded_first = torch.matmul(p32.to(torch.bfloat16), V.transpose(1, 2)).reshape(b, hq, d)
    rounded_last = torch.matmul(p32, V.transpose(1, 2).float()).to(torch.bfloat16).reshape(b, hq, d)
    assert torch.equal(out, rounded_first)
    assert not torch.equal(rounded_first, rounded_last), "the cast order must be observable for this test to pin anything"


# ----------------------------------------------------------------------------- split-K + merge
def test_splitk_merge_equals_direct_softmax_for_any_split_count():
    b, H, L, Dv = 2, 3, 300, 7
    scores, vals = rnd(b, H, L, seed=1, std=3.0), rnd(b, 1, L, Dv, seed=2)
    direct = torch.einsum("bhl,bld->bhd", torch.softmax(scores, -1), vals[:, 0])
    for ns, mx in ((1, 1), (2, 4), (7, 8), (16, 16), (10, 32)):
        part, lse, live = oracle.splitk_stage1(scores, vals, [ns] * b, mx)
        assert live.sum().item() == b * len(oracle.live_splits(L, ns, mx))
        assert torch.isnan(part[~live.unsqueeze(1).expand(b, H, mx)]).all(), "dead splits stay untouched"
        out = oracle.merge_stage2(part, lse, [ns] * b, mx, L)
        assert torch.allclose(out, direct, rtol=1e-10, atol=1e-12)
    # S = 1: lse is the log-sum-exp, partial is the softmax average itself
    part, lse, _ = oracle.splitk_stage1(scores, vals, [1] * b, 1)
    assert torch.allclose(lse[:, :, 0], torch.logsumexp(scores, -1)) and torch.allclose(part[:, :, 0], direct)


def test_ragged_batch_is_per_sequence_slices():
    b, H, L, Dv = 3, 2, 200, 5
    lens = [200, 37, 129]
    scores, vals = rnd(b, H, L, seed=3), rnd(b, 1, L, Dv, seed=4)
    part, lse, live = oracle.splitk_stage1(scores, vals, [4, 2, 3], 4, kv_lens=lens)
    out = oracle.merge_stage2(part, lse, [4, 2, 3], 4, L, kv_lens=lens)
    for i, n in enumerate(lens):
        ref = torch.einsum("hl,ld->hd", torch.softmax(scores[i, :, :n], -1), vals[i, 0, :n])
        assert torch.allclose(out[i], ref, atol=1e-12)
    K, V, q = rnd(b, L, 2, 8, seed=5), rnd(b, L, 2, 8, seed=6), rnd(b, 4, 8, seed=7)
    rag = oracle.ragged_apply(oracle.gqa_plain, lens, (q, K, V), (None, 1, 1), sm_scale=0.5)
    assert torch.allclose(rag[1], oracle.gqa_plain(q[1:2], K[1:2, :37], V[1:2, :37], 0.5)[0])
