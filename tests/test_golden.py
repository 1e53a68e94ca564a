"""The committed vectors (tests/golden/xkv_vectors.npz, written by tests/golden/make_vectors.py from the CPU oracle) against
the oracle as it is now, and against the independent C brute force where that covers the operation.  The reference
project has no vectors of its own for this path."""
import os
import sys

import numpy as np
import torch

import oracle
from oracle import cbrute

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))


def load():
    z = np.load(os.path.join(HERE, "golden", "xkv_vectors.npz"), allow_pickle=False)
    return {k: torch.from_numpy(z[k]) for k in z.files}


def test_oracle_reproduces_the_committed_vectors():
    import make_vectors
    now, then = make_vectors.build(), load()
    assert set(now) == set(then)
    for k in then:
        a, b = torch.from_numpy(now[k]).double(), then[k].double()
        assert a.shape == b.shape, k
        assert (a - b).abs().max().item() <= 2e-6 * max(1.0, b.abs().max().item()), k   # thread-count dependent fp32 summation order


def test_vectors_agree_with_the_c_bruteforce():
    """Independent double-precision loops (oracle/xkv_oracle.c) on the committed inputs.  qab_rope is left out: the
    oracle rounds the rotated key to the query type there (test_oracle.py pins that step)."""
    g = load()
    n = lambda t: t.double().numpy()
    q3, scale, theta = g["q"][:, :, 0], float(g["scale"]), float(g["theta"])
    assert np.abs(cbrute.qab(n(q3), n(g["A"]), n(g["kB"])) - n(g["qab_nope"][:, :, 0])).max() < 1e-4
    ref = cbrute.decode_factorized(n(q3), n(g["A"]), n(g["kB"]), n(g["Av"]), n(g["vB"]), scale)
    assert np.abs(ref - n(g["gqa_xkv"])).max() < 1e-4
    ref = cbrute.decode_factorized(n(q3), n(g["A"]), n(g["kB"]), n(g["Av"]), n(g["vB"]), scale, rope=True, theta=theta)
    assert np.abs(ref - n(g["gqa_factorized_rope"])).max() < 1e-4
    assert np.abs(cbrute.decode_plain(n(q3), n(g["K"]), n(g["V"]), scale) - n(g["gqa_plain"])).max() < 1e-4
    ref = cbrute.mla(n(g["mla_qn"]), n(g["mla_qr"]), n(g["mla_ckv"]), n(g["mla_kpe"]), float(g["mla_scale"]))
    assert np.abs(ref - n(g["mla_ref"])).max() < 1e-4


def test_split_vectors_are_the_integer_arithmetic():
    g = load()
    for (L, n, _), row in zip(g["split_cases"].tolist(), g["split_bounds"].tolist()):
        per = -(-(-(-L // n)) // 32) * 32
        for i, (s, e) in enumerate(row):
            assert s == per * i and e == min(per * (i + 1), L)
