"""Randomised parity sweep: shapes drawn from a seeded generator over the envelope of each entry point (ranks, head
groupings, ragged lengths, split counts, both operand types), HIP path against the CPU oracle.  Sizes are kept small
enough for the oracle to finish in seconds; the draw is fixed by the seed, so a failure names its case."""
import math
import random

import pytest
import torch

import oracle
from util import check_out, check_scores, f32, gen

pytestmark = pytest.mark.gpu

import kernel_collections_amd.flash_recontruction as fr  # noqa: E402
from kernel_collections_amd.flash_decoding import gqa, mla2  # noqa: E402

BF, FP = torch.bfloat16, torch.float16


def _cases(n, seed):
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        hkv = rng.choice([1, 2, 4, 8])
        g = rng.choice([1, 2, 4, 7, 8])
        out.append(dict(b=rng.choice([1, 2, 3]), hq=hkv * g, hkv=hkv, L=rng.choice([1, 31, 32, 33, 100, 257, 1000, 2049]),
                        rk=rng.choice([64, 128, 192, 256, 384, 512]), rv=rng.choice([64, 128, 256, 512]),
                        S=rng.choice([1, 2, 3, 5, 8]), dtype=rng.choice([BF, FP]), theta=rng.choice([1e4, 5e5, 1e7]),
                        shared=rng.random() < 0.4, off=rng.choice([0, 0, 4096, 100000])))
    return out


def splits_t(vals, dev):
    return torch.tensor(vals, dtype=torch.int32, device=dev)


@pytest.mark.parametrize("c", _cases(24, seed=1), ids=lambda c: "b%d-h%d/%d-L%d-rk%d-rv%d-S%d%s" % (
    c["b"], c["hq"], c["hkv"], c["L"], c["rk"], c["rv"], c["S"], "-sh" if c["shared"] else ""))
def test_random_factorised_paths(dev, c):
    b, hq, hkv, L, rk, S, dt, theta, d = c["b"], c["hq"], c["hkv"], c["L"], c["rk"], c["S"], c["dtype"], c["theta"], 128
    rv = rk if c["shared"] else c["rv"]
    q = gen((b, hq, d), std=0.4, dtype=dt, seed=11)
    kA, kB = gen((b, L, rk), dtype=dt, seed=12), gen((b, hkv, rk, d), std=rk ** -0.5, dtype=dt, seed=13)
    vA = kA if c["shared"] else gen((b, L, rv), dtype=dt, seed=14)
    vB = gen((b, hkv, rv, d), std=rv ** -0.5, dtype=dt, seed=15)
    scale = 1 / math.sqrt(d)
    qd, kAd, kBd, vBd = (t.to(dev) for t in (q, kA, kB, vB))
    vAd = kAd if c["shared"] else vA.to(dev)
    ns = splits_t([S] * b, dev)
    # scores, with and without RoPE
    check_scores(fr.qAB_no_pe_v1(qd.unsqueeze(2), kAd, kBd, out_dtype=torch.float32), oracle.qab_nope(*f32(q.unsqueeze(2), kA, kB)), "qab_nope")
    cos, sin = oracle.rope_cos_sin(torch.arange(c["off"], c["off"] + L), d, theta)
    check_scores(fr.qAB_rope_v1(qd.unsqueeze(2), kAd, kBd, theta, pos_offset=c["off"], out_dtype=torch.float32),
                 oracle.qab_rope(*f32(q.unsqueeze(2), kA, kB), cos, sin), "qab_rope")
    # fused decode, with and without RoPE
    check_out(fr.gqa_xKV_no_pe_v2(qd, kAd, kBd, vAd, vBd, ns, S, scale), oracle.gqa_xkv(*f32(q, kA, kB, vA, vB), sm_scale=scale), "xkv no pe")
    o = torch.empty_like(qd)
    fr.gqa_xKV_rope(qd, kAd, kBd, vAd, vBd, o, ns, S, scale, theta, pos_offset=c["off"])
    ref = oracle.gqa_factorized_rope(*f32(q.unsqueeze(2), kA, kB, vA, vB), cos, sin, sm_scale=scale)[:, :, 0]
    check_out(o, ref, "xkv rope")


@pytest.mark.parametrize("c", _cases(12, seed=2), ids=lambda c: "b%d-h%d/%d-L%d-rv%d-S%d" % (c["b"], c["hq"], c["hkv"], c["L"], c["rv"], c["S"]))
def test_random_plain_and_v_factorised_ragged(dev, c):
    b, hq, hkv, L, rv, dt, d = c["b"], c["hq"], c["hkv"], c["L"], c["rv"], c["dtype"], 128
    rng = random.Random(c["L"] * 7 + c["b"])
    lens = [rng.randint(1, L) for _ in range(b)]
    lens[0] = L
    split = rng.choice([32, 64, 256])
    ns = [-(-n // split) for n in lens]
    S = max(ns)
    scale = 1 / math.sqrt(d)
    q, K, V = gen((b, hq, d), dtype=dt, seed=21), gen((b, L, hkv, d), dtype=dt, seed=22), gen((b, L, hkv, d), dtype=dt, seed=23)
    vA, vB = gen((b, L, rv), dtype=dt, seed=24), gen((b, hkv, rv, d), std=rv ** -0.5, dtype=dt, seed=25)
    ref = oracle.ragged_apply(oracle.gqa_plain, lens, f32(q, K, V), (None, 1, 1), sm_scale=scale)
    ref_v = oracle.ragged_apply(
        lambda q_, K_, vA_, vB_: oracle.gqa_v_only(q_.unsqueeze(2), K_.transpose(1, 2), vA_, vB_, sm_scale=scale)[:, :, 0],
        lens, f32(q, K, vA, vB), (None, 1, 1, None))
    qd, Kd, Vd, vAd, vBd = (t.to(dev) for t in (q, K, V, vA, vB))
    kl, nst = splits_t(lens, dev), splits_t(ns, dev)
    o = torch.zeros_like(qd)
    gqa.decode_attention_fwd(qd, Kd, Vd, o, nst, S, scale, kv_lens=kl)
    check_out(o, ref, "ragged plain")
    o2 = torch.zeros_like(qd)
    gqa.decode_attention_fwd_v_factorized(qd, Kd, vAd, vBd, o2, nst, S, scale, kv_lens=kl)
    check_out(o2, ref_v, "ragged V-factorised")


@pytest.mark.parametrize("H,L,dtype", [(1, 5, BF), (16, 300, FP), (48, 1025, BF), (128, 64, FP)])
def test_random_mla(dev, H, L, dtype):
    b, c, e = 2, 512, 64
    qn, qr = gen((b, H, c), std=1 / 3, dtype=dtype, seed=31), gen((b, H, e), std=1 / 3, dtype=dtype, seed=32)
    ckv, kpe = gen((b, L, 1, c), std=1 / 3, dtype=dtype, seed=33), gen((b, L, 1, e), std=1 / 3, dtype=dtype, seed=34)
    scale = 1 / math.sqrt(192)
    out = mla2.mla_decode_attention_fwd(*(t.to(dev) for t in (qn, qr, ckv, kpe)), scale)
    check_out(out, oracle.mla_ref(*f32(qn, qr, ckv, kpe), scale), "mla")


def test_profiling_cli_runs_and_agrees(dev, capsys):
    """The variant table of kernel_collections_amd.profiling at a small shape: every non-RoPE row answers the same question
    as eager attention."""
    from kernel_collections_amd import profiling
    rows = profiling.main(["--kv_len", "2048", "--k_rank", "256", "--v_rank", "512", "--batch", "2", "--warmup", "1", "--repeat", "2"])
    assert len(rows) == 8 and "Fused xKV v2" in capsys.readouterr().out
    for name, t, err in rows:
        assert t > 0 and (math.isnan(err) or err < 3e-2), (name, err)


def test_profiling_cli_sweep_and_trace(dev, capsys, tmp_path):
    """--sweep prints median / 20 % / 80 % per kv_len and entry point; --profile leaves a chrome trace with one range per variant."""
    import json
    from kernel_collections_amd import profiling
    rows = profiling.main(["--sweep", "--sweep_min", "10", "--sweep_max", "11", "--k_rank", "192", "--dtype", "fp16", "--warmup", "1",
                           "--repeat", "5"])
    assert [L for L, _ in rows] == [1024, 2048]
    for _, res in rows:
        assert set(res) == {"qK (torch)", "qAB_v1", "qAB_v2 (table)", "qAB_v3", "qAB_v4"}
        for med, p20, p80 in res.values():
            assert 0 < p20 <= med <= p80
    assert "kv_len" in capsys.readouterr().out
    trace = tmp_path / "trace.json"
    profiling.main(["--kv_len", "1024", "--k_rank", "256", "--v_rank", "512", "--profile", "--trace_path", str(trace)])
    events = json.loads(trace.read_text())["traceEvents"]
    names = {e.get("name", "") for e in events}
    assert "Fused xKV with RoPE" in names and any("recon" in n or "latent" in n for n in names), "variant ranges and HIP kernels in the trace"
