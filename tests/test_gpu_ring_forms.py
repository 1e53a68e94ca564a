"""Every instantiation of the wide-row (LDS ring) stage 1, called through xkv_latent_stage1 + xkv_merge_stage2 on inputs
long enough that each loader wave's register queue wraps several times (6 tiles and more per split), against a plain fp32
computation of the same attention.

The loader waves of that kernel fetch rows with loads the compiler does not track; a register copy the compiler might
insert between such a load and the LDS store that consumes it would hand on stale values from the third or fourth tile of
a split onwards, in that instantiation only.  The shapes below reach every (mode, key width, value width, head blocks,
low-order query part, operand type) combination the dispatcher holds, so such a copy cannot hide behind a shape no other
test happens to run.
"""
import itertools

import pytest
import torch

from util import OUT_ATOL, SCORE_RTOL, max_abs, rel_max

pytestmark = pytest.mark.gpu

from kernel_collections_amd import ops  # noqa: E402

BF, FP = torch.bfloat16, torch.float16


def draw(shape, std, dtype, dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    return (torch.randn(shape, device=dev, dtype=torch.float32, generator=g) * std).to(dtype)


def run_form(dev, dtype, *, hq, dn, lo, rope, mode, dv, lens, S, heads_in_row=0):
    """mode: 'scores' | 'shared' (values = the key rows) | 'row' (a second row stream of dv) | 'heads' (plain per-kv-head
    values [L, 8, 128]).  heads_in_row = 8: keys are 8 plain kv heads of 128 side by side (dn is then 128 per head)."""
    b, L = len(lens), max(lens)
    scale = 0.5
    kv_heads = 8 if (mode == "heads" or heads_in_row) else 1
    hpk = hq // kv_heads
    if heads_in_row:
        K = draw((b, L, 8, 128), 1.0, dtype, dev, 1)
        q = draw((b, hq, 128), 128 ** -0.5, dtype, dev, 2)
        C = (K, K.stride(0), K.stride(1), K.stride(2), 128)
        qf = q.float()
        s = torch.einsum("bhd,blhd->bhl", qf, K.float().repeat_interleave(hpk, dim=2))
        groups, q_lo = 8, None
    else:
        Cm = draw((b, L, dn), 1.0, dtype, dev, 1)
        q = draw((b, hq, dn), dn ** -0.5, dtype, dev, 2)
        q_lo = draw((b, hq, dn), dn ** -0.5 * 2 ** -8, dtype, dev, 3) if lo else None
        C = (Cm, Cm.stride(0), Cm.stride(1), 0, dn)
        qf = q.float() + (q_lo.float() if lo else 0)
        s = torch.einsum("bhd,bld->bhl", qf, Cm.float())
        groups = 8 if mode == "heads" else 1
    R = qr = None
    if rope:
        Rm = draw((b, L, 64), 1.0, dtype, dev, 4)
        qr = draw((b, hq, 64), 0.1, dtype, dev, 5)
        R = (Rm, Rm.stride(0), Rm.stride(1), 0, 64)
        s = s + torch.einsum("bhd,bld->bhl", qr.float(), Rm.float())
    s = s * scale
    splits = torch.full((b,), S, dtype=torch.int32, device=dev)
    kl = torch.tensor(lens, dtype=torch.int32, device=dev)
    what = f"{mode} hq{hq} dn{dn} lo{int(lo)} rope{int(rope)} dv{dv} rows{heads_in_row} {dtype}"
    if mode == "scores":
        out = torch.full((b, hq, 1, L), float("nan"), dtype=torch.float32, device=dev)
        ops.latent_stage1(q, q_lo, qr, C, R, None, None, None, out, splits, kl, b, hq, groups, L, S, scale)
        for i, n in enumerate(lens):
            er = rel_max(out[i, :, 0, :n].cpu(), s[i, :, :n].cpu())
            assert er <= SCORE_RTOL, f"{what}: sequence {i}: scores rel err {er:.3e}"
        return
    if mode == "shared":
        V, vals = C, Cm.float().unsqueeze(2).expand(b, L, hq, dn)
    elif mode == "row":
        Vm = draw((b, L, dv), 1.0, dtype, dev, 6)
        V, vals = (Vm, Vm.stride(0), Vm.stride(1), 0, dv), Vm.float().unsqueeze(2).expand(b, L, hq, dv)
    else:
        Vm = draw((b, L, 8, 128), 1.0, dtype, dev, 6)
        V, vals = (Vm, Vm.stride(0), Vm.stride(1), Vm.stride(2), 128), Vm.float().repeat_interleave(hpk, dim=2)
    dvo = vals.shape[-1]
    partial, lse = ops.workspaces(b, hq, S, dvo, dev)
    ops.latent_stage1(q, q_lo, qr, C, R, V, partial, lse, None, splits, kl, b, hq, groups, L, S, scale)
    o = torch.empty((b, hq, dvo), dtype=dtype, device=dev)
    ops.merge_stage2(partial, lse, o, None, splits, kl, b, hq, hq, L, S)
    for i, n in enumerate(lens):
        p = torch.softmax(s[i, :, :n], dim=-1).to(dtype).float()      # probabilities rounded to the operand type before P.V
        ref = torch.einsum("hl,lhd->hd", p, vals[i, :n])
        err = max_abs(o[i].float().cpu(), ref.cpu())
        assert err <= OUT_ATOL, f"{what}: sequence {i}: max abs err {err:.3e}"


# two sequences, one of them not a multiple of the tile; 2 splits -> 8 .. 10 tiles of 32 tokens (16 .. 20 of 16) per split
LENS, SPLITS = [640, 517], 2


@pytest.mark.parametrize("dtype", [BF, FP], ids=["bf16", "fp16"])
@pytest.mark.parametrize("hq", [8, 32], ids=["one_head_block", "two_head_blocks"])
def test_single_stream_forms(dev, dtype, hq):
    for dn, lo in ((512, True), (512, False), (384, True), (256, True)):
        run_form(dev, dtype, hq=hq, dn=dn, lo=lo, rope=False, mode="scores", dv=0, lens=LENS, S=SPLITS)
        run_form(dev, dtype, hq=hq, dn=dn, lo=lo, rope=False, mode="shared", dv=dn, lens=LENS, S=SPLITS)
    run_form(dev, dtype, hq=hq, dn=512, lo=False, rope=True, mode="shared", dv=512, lens=LENS, S=SPLITS)


@pytest.mark.parametrize("dtype", [BF, FP], ids=["bf16", "fp16"])
@pytest.mark.parametrize("hq", [8, 32], ids=["one_head_block", "two_head_blocks"])
def test_two_stream_forms(dev, dtype, hq):
    for dn, dv in itertools.product((512, 384, 256), (512, 384, 256)):      # absorbed query, keys and values factorised
        run_form(dev, dtype, hq=hq, dn=dn, lo=True, rope=False, mode="row", dv=dv, lens=LENS, S=SPLITS)
    run_form(dev, dtype, hq=hq, dn=512, lo=False, rope=False, mode="row", dv=512, lens=LENS, S=SPLITS)   # plain 512 / 512
    for dv in (512, 384, 256):                                              # 8 plain kv heads in a row, values factorised
        run_form(dev, dtype, hq=hq, dn=128, lo=False, rope=False, mode="row", dv=dv, lens=LENS, S=SPLITS, heads_in_row=8)


@pytest.mark.parametrize("dtype", [BF, FP], ids=["bf16", "fp16"])
@pytest.mark.parametrize("hq", [16, 32], ids=["one_head_block", "two_head_blocks"])
def test_per_head_value_forms(dev, dtype, hq):
    for dn in (512, 384, 256):                                              # absorbed keys, plain per-head values
        run_form(dev, dtype, hq=hq, dn=dn, lo=True, rope=False, mode="heads", dv=128, lens=LENS, S=SPLITS)
    run_form(dev, dtype, hq=hq, dn=128, lo=False, rope=False, mode="heads", dv=128, lens=LENS, S=SPLITS, heads_in_row=8)   # plain GQA


@pytest.mark.parametrize("dtype", [BF, FP], ids=["bf16", "fp16"])
@pytest.mark.parametrize("hq", [8, 32], ids=["one_head_block", "two_head_blocks"])
def test_softmax_pv_over_given_scores(dev, dtype, hq):
    """xkv_softmax_pv_stage1 + merge against torch: scores are an input (peaked: sigma 6), values one row per token."""
    lens, S = [644, 516, 32], 3
    b, L = len(lens), 644
    for dv in (512, 384, 256):
        scores = draw((b, hq, L), 6.0, torch.float32, dev, 11)
        V = draw((b, L, dv), 1.0, dtype, dev, 12)
        splits = torch.full((b,), S, dtype=torch.int32, device=dev)
        kl = torch.tensor(lens, dtype=torch.int32, device=dev)
        partial, lse = ops.workspaces(b, hq, S, dv, dev)
        ops.softmax_pv_stage1(scores, V, partial, lse, splits, kl, b, hq, L, S, dtype)
        o = torch.empty((b, hq, dv), dtype=dtype, device=dev)
        ops.merge_stage2(partial, lse, o, None, splits, kl, b, hq, hq, L, S)
        for i, n in enumerate(lens):
            p = torch.softmax(scores[i, :, :n], dim=-1).to(dtype).float()
            ref = p @ V[i, :n].float()
            err = max_abs(o[i].float().cpu(), ref.cpu())
            assert err <= OUT_ATOL, f"given scores hq{hq} dv{dv} {dtype}: sequence {i}: max abs err {err:.3e}"
