"""Helpers shared by the parity tests: seeded CPU inputs (so oracle and kernels see identical bits),
error measures and the tolerances of the parity contract."""
import torch

# parity contract
OUT_ATOL = 2e-2      # attention output, max abs error of the 16-bit kernel vs the fp32 eager oracle
SCORE_RTOL = 1e-2    # pre-softmax scores, max |delta| / max |ref|
# tighter bound this repo holds itself to: output error relative to the largest reference magnitude
OUT_RTOL = 2e-2


def gen(shape, std=1.0, dtype=torch.bfloat16, seed=None, g=None):
    if g is None:
        g = torch.Generator().manual_seed(0 if seed is None else seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)


def f32(*ts):
    return [None if t is None else t.float() for t in ts]


def max_abs(a, b):
    return (a.float().cpu() - b.float().cpu()).abs().max().item()


def rel_max(a, b):
    b = b.float().cpu()
    return (a.float().cpu() - b).abs().max().item() / max(b.abs().max().item(), 1e-30)


def check_out(got, ref, what=""):
    ea, er = max_abs(got, ref), rel_max(got, ref)
    assert ea <= OUT_ATOL, f"{what}: max abs err {ea:.3e} > {OUT_ATOL}"
    assert er <= OUT_RTOL, f"{what}: rel err {er:.3e} > {OUT_RTOL}"
    return ea, er


def check_scores(got, ref, what=""):
    er = rel_max(got, ref)
    assert er <= SCORE_RTOL, f"{what}: scores rel err {er:.3e} > {SCORE_RTOL}"
    return er


def rope_q(q, pos, theta):
    """Rotate a query [b, H, d] (fp32 math) to absolute position `pos` - what a caller does before
    handing q_pe to the kernels."""
    from oracle import apply_rope, rope_cos_sin
    cos, sin = rope_cos_sin(torch.tensor([pos]), q.shape[-1], theta)
    return apply_rope(q.float(), cos[0], sin[0])
