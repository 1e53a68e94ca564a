"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports exactly the symbols
include/xkv_hip.h declares (no compute call is made), argument validation answers before any launch,
and the Python mirrors expose the reference's names and signatures."""
import ctypes
import inspect
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "xkv_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xkv_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from kernel_collections_amd import _lib
    names = _declared()
    assert set(names) == set(_lib.EXPORTS), (names, _lib.EXPORTS)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} not exported"
    assert _lib.lib().xkv_abi_version() == _lib.ABI_VERSION
    assert _lib.lib().xkv_error_string(0) == b"ok"
    assert b"envelope" in _lib.lib().xkv_error_string(-2)


def test_argument_errors_are_reported_before_any_launch():
    from kernel_collections_amd import _lib
    L = _lib.lib()
    null = ctypes.c_void_p(0)
    assert L.xkv_rope_table(null, null, null, 4, 0, 64, _lib.XKV_F32, null) == -1
    assert L.xkv_absorb_q(null, null, null, null, 1, 4, 2, 128, 64, 0, 0, 0, _lib.XKV_BF16, null) == -1
    q = _lib.QOperand(ctypes.c_void_p(16), 100)
    kv = _lib.KVOperand(ctypes.c_void_p(16), 0, 100, 0, 100)
    none = _lib.KVOperand(null, 0, 0, 0, 0)
    ns = ctypes.c_void_p(16)
    # feature width 100 is outside the envelope (multiple of 32 required)
    rc = L.xkv_latent_stage1(q, null, _lib.QOperand(null, 0), kv, none, kv, ctypes.c_void_p(16), ctypes.c_void_p(16),
                             null, 0, ns, null, 1, 4, 1, 8, 1, 0, null, 1.0, 0.0, _lib.XKV_BF16, null)
    assert rc == -2
    with pytest.raises(RuntimeError, match="envelope"):
        _lib.check(rc, "xkv_latent_stage1")
    # the static-scratch variant refuses a shape whose packed factors exceed its array (8 x 1 MiB here), before any HIP call
    big = _lib.KVOperand(ctypes.c_void_p(16), 512 * 64, 512, 0, 512)
    rc = L.xkv_recon_stage1_static(ctypes.c_void_p(16), big, ctypes.c_void_p(16), 8 * 512 * 128, 512 * 128, 128, big,
                                   ctypes.c_void_p(16), ctypes.c_void_p(16), null, 0, ns, null, 8, 32, 8, 64, 1, 1.0, 1,
                                   ctypes.c_void_p(16), 0, null, 0, _lib.XKV_BF16, null)
    assert rc == _lib.XKV_ESCRATCH and b"static device array" in L.xkv_error_string(rc)
    # the merge keeps one head's merged row and split weights in the LDS: a split count that cannot fit beside the kernel's
    # static buffers is refused before any launch (512 + 14000 floats = 58 KB of the 64 KiB a workgroup may have)
    rc = L.xkv_merge_stage2(ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16), null, 0, 0, 0, 0, _lib.XKV_BF16,
                            ns, null, 1, 8, 1, 14000 * 32, 14000, 0, null, 512, 8 * 512, 512, _lib.XKV_F32, null, 0, 0, null)
    assert rc == -2


def test_python_surface_matches_reference_names_and_argument_order():
    import kernel_collections_amd.flash_recontruction as fr
    from kernel_collections_amd.flash_decoding import gqa, mla, mla2
    for n in ("qAB_no_pe_v1", "qAB_no_pe_v2", "qAB_no_pe_ref", "qAB_rope_v1", "qAB_rope_v2", "qAB_rope_v3",
              "qAB_rope_v4", "gqa_xKV_no_pe_ref", "gqa_xKV_no_pe_k_only_ref", "gqa_xKV_no_pe_k_only",
              "gqa_xKV_no_pe", "gqa_xKV_no_pe_v2"):
        assert n in fr.__all__ and callable(getattr(fr, n))
    pos = lambda f: [p.name for p in inspect.signature(f).parameters.values()
                     if p.kind == p.POSITIONAL_OR_KEYWORD]
    assert pos(fr.qAB_no_pe_v1) == ["q", "Ak", "Bk"]
    assert pos(fr.qAB_rope_v1) == ["q", "Ak", "Bk", "theta"]
    assert inspect.signature(fr.qAB_rope_v1).parameters["theta"].default == 10000000.0
    assert pos(fr.qAB_rope_v2) == ["q", "Ak", "Bk", "sin_cos"]
    assert pos(fr.gqa_xKV_no_pe) == ["q", "k_A_buffer", "k_B_buffer", "v_A_buffer", "v_B_buffer", "o",
                                     "num_kv_splits", "max_kv_splits", "sm_scale"]
    assert pos(fr.gqa_xKV_no_pe_v2) == ["q", "k_A_buffer", "k_B_buffer", "v_A_buffer", "v_B_buffer",
                                        "num_kv_splits", "max_kv_splits", "sm_scale"]
    assert pos(fr.gqa_xKV_no_pe_k_only) == ["q", "k_A_buffer", "k_B_buffer", "v_buffer", "o", "num_kv_splits",
                                            "max_kv_splits", "sm_scale"]
    assert pos(gqa.decode_attention_fwd) == ["q", "k_buffer", "v_buffer", "o", "num_kv_splits", "max_kv_splits",
                                             "sm_scale"]
    assert pos(mla.decode_attention_fwd) == ["q", "k_buffer", "v_buffer", "o", "sm_scale", "logit_cap"]
    assert pos(mla2.mla_decode_attention_fwd) == ["q_nope", "q_rope", "kv_nope", "k_rope", "sm_scale"]
    assert pos(mla2.mla_decode_attention_xKV) == ["q_nope", "q_rope", "kv_A_nope", "kv_B_nope", "k_rope", "sm_scale"]
    from kernel_collections_amd.flash_recontruction.rope.sin_cos import rotary_sin_cos
    assert pos(rotary_sin_cos) == ["seqlen", "theta", "starting_idx"]


def test_reference_asserts_are_kept():
    import kernel_collections_amd.flash_recontruction as fr
    q = torch.zeros(1, 4, 2, 128, dtype=torch.bfloat16)
    A = torch.zeros(1, 8, 64, dtype=torch.bfloat16)
    B = torch.zeros(1, 2, 64, 128, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="q_len=1"):
        fr.qAB_no_pe_v1(q, A, B)
    with pytest.raises(AssertionError, match="Rank mismatch"):
        fr.qAB_rope_v1(q[:, :, :1], A, torch.zeros(1, 2, 32, 128, dtype=torch.bfloat16))
    with pytest.raises(AssertionError, match="4D"):
        fr.qAB_no_pe_v1(q[0], A, B)
    # CPU tensors are refused, never silently computed elsewhere
    with pytest.raises(AssertionError, match="no CPU path"):
        fr.qAB_no_pe_v1(q[:, :, :1], A, B)


def test_eager_surface_functions_agree_with_the_oracle():
    import oracle
    import kernel_collections_amd.flash_recontruction as fr
    from kernel_collections_amd.flash_decoding import mla, mla2
    from kernel_collections_amd.flash_recontruction.rope import rope_ref
    g = torch.Generator().manual_seed(1)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    q, A, B, vA, vB = r(2, 8, 1, 16), r(2, 30, 6), r(2, 2, 6, 16), r(2, 30, 10), r(2, 2, 10, 16)
    assert torch.allclose(fr.qAB_no_pe_ref(q, A, B), oracle.qab_nope(q, A, B))
    assert torch.allclose(fr.gqa_xKV_no_pe_ref(q[:, :, 0], A, B, vA, vB).float(),
                          oracle.gqa_xkv(q[:, :, 0], A, B, vA, vB).float(), atol=1e-5)
    V = r(2, 30, 2, 16)
    assert torch.allclose(fr.gqa_xKV_no_pe_k_only_ref(q[:, :, 0], A, B, V).float(),
                          oracle.gqa_xkv_k_only(q[:, :, 0], A, B, V).float(), atol=1e-5)
    K = r(2, 30, 2, 16)
    assert torch.allclose(mla.decode_attention_reference(q[:, :, 0], K, V, None, 0.4).float(),
                          oracle.gqa_plain(q[:, :, 0], K, V, 0.4).float(), atol=1e-5)
    qn, qr, c, pe = r(2, 4, 12), r(2, 4, 4), r(2, 30, 1, 12), r(2, 30, 1, 4)
    assert torch.allclose(mla2.mla_decode_attention_fwd_ref(qn, qr, c, pe, 0.3).float(),
                          oracle.mla_ref(qn, qr, c, pe, 0.3).float(), atol=1e-5)
    cos, sin = rope_ref.LlamaRotaryEmbedding(128, 50, 5e5)
    ocos, osin = oracle.rope_cos_sin(torch.arange(50), 128, 5e5)
    assert torch.equal(cos, ocos) and torch.equal(sin, osin)
    x = r(50, 128).float()
    assert torch.equal(rope_ref.apply_rotary_pos_emb_pytorch(x, cos, sin)[0], oracle.apply_rope(x, ocos, osin))


def test_settled_splits_leaves_no_dead_split():
    """A workspace shared by two stage-1 passes is merged as 'all rows live': the host must never ask for more splits
    than the split arithmetic fills."""
    import oracle
    from kernel_collections_amd import ops
    for L in list(range(1, 400)) + [1500, 4096, 4097, 131072]:
        for n in (1, 2, 3, 4, 7, 11, 16, 64, 128):
            s = ops.settled_splits(L, n)
            assert 1 <= s <= n
            live = oracle.live_splits(L, s, s)
            assert len(live) == s and live[0][1] == 0 and live[-1][2] == L, (L, n, s)


def test_split_cap_needs_room_in_the_workspace():
    """With split_cap_tokens > 0 a sequence may be scanned with ceil(kv_len / cap) splits: stage 1 and the merge refuse
    (before any launch) a workspace whose split dimension is smaller, and accept one that covers it."""
    from kernel_collections_amd import _lib, ops
    L = _lib.lib()
    null, p16 = ctypes.c_void_p(0), ctypes.c_void_p(16)
    q = _lib.QOperand(p16, 128)
    kv = _lib.KVOperand(p16, 8192 * 128, 128, 0, 128)
    none = _lib.KVOperand(null, 0, 0, 0, 0)
    args = lambda max_splits, cap: (q, null, _lib.QOperand(null, 0), kv, none, kv, p16, p16, null, 0, p16, null,
                                    1, 4, 1, 8192, max_splits, cap, null, 1.0, 0.0, _lib.XKV_BF16, null)
    assert L.xkv_latent_stage1(*args(7, 1024)) == -1          # 8192 tokens at 1024 per split need 8 rows
    assert L.xkv_latent_stage1(*args(2, -5)) == -1
    assert L.xkv_merge_stage2(p16, p16, p16, null, 0, 0, 0, 128, 0, p16, null, 1, 4, 1, 8192, 7, 1024, null, 128, 512, 128,
                              _lib.XKV_BF16, null, 0, 0, null) == -1
    # a split plan's cap only raises the host's value, which is what bounds the workspaces: it needs one
    dev_cap = lambda max_splits, cap: args(max_splits, cap)[:18] + (p16,) + args(max_splits, cap)[19:]
    assert L.xkv_latent_stage1(*dev_cap(8, 0)) == -1
    assert L.xkv_plan_splits(null, p16, 4, 8, 1024, 256, p16, null) == -1 and L.xkv_plan_splits(p16, p16, 4, 8, 0, 256, p16, null) == -1
    assert ops.capped_splits(8192, 2, 1024) == 8 and ops.capped_splits(8192, 16, 1024) == 16 and ops.capped_splits(8192, 2, 0) == 2
    assert ops.capped_splits(104212, 26, 1024) == 102


REFERENCE_IMPORTS = """
from flash_recontruction import qAB_no_pe_v1, qAB_no_pe_v2, qAB_no_pe_ref, qAB_rope_v1, qAB_rope_v2, qAB_rope_v3, qAB_rope_v4
from flash_recontruction import gqa_xKV_no_pe_ref, gqa_xKV_no_pe_k_only_ref, gqa_xKV_no_pe_k_only, gqa_xKV_no_pe, gqa_xKV_no_pe_v2
from flash_recontruction.rope.sin_cos import rotary_sin_cos
from flash_recontruction.rope.rope_ref import LlamaRotaryEmbedding, rotate_half, apply_rotary_pos_emb_pytorch
from flash_decoding.gqa import decode_attention_fwd
from flash_decoding.mla import decode_attention_fwd, decode_attention_reference
from flash_decoding.mla2 import mla_decode_attention_fwd, mla_decode_attention_fwd_ref, mla_decode_attention_xKV
from flash_decoding.deepseek_mla import mla_decode_attention_fwd, mla_decode_attention_fwd_pd_sep, mla_decode_attention_fwd_pd_sep_xKV
"""


def _doc_python_blocks():
    """Every fenced python block of the markdown notes at the repository root."""
    out = []
    for name in sorted(os.listdir(ROOT)):
        if name.endswith(".md"):
            text = open(os.path.join(ROOT, name)).read()
            out += [(name, m.group(1)) for m in re.finditer(r"```python\n(.*?)```", text, flags=re.S)]
    return out


def test_install_aliases_binds_the_reference_module_names():
    """After install_aliases() code written against the reference imports unchanged: every name the reference's scripts
    import (test_gqa_xKV.py:1-10, test_qAB_rope.py:1-8, test_triton_gqa.py:1, test_triton_mla.py:1,
    test_mla_decoding_new.py:1, test_mla_decoding_new2.py:3, test_cos_sin.py:1-3), and the import block the notes print."""
    import sys
    import kernel_collections_amd
    saved = {k: sys.modules.get(k) for k in ("flash_recontruction", "flash_decoding")}
    try:
        kernel_collections_amd.install_aliases()
        exec(REFERENCE_IMPORTS, {})
        blocks = [code for _, code in _doc_python_blocks() if "install_aliases()" in code]
        assert blocks, "the notes show the import route"
        for code in blocks:
            exec(code, {})
        import flash_recontruction
        assert flash_recontruction is sys.modules["kernel_collections_amd.flash_recontruction"]
    finally:
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v


def _load_route_b_stub(monkeypatch):
    import importlib.util
    from kernel_collections_amd import _lib
    monkeypatch.setenv("XKV_HIP_LIB", _lib.LIB_PATH)
    spec = importlib.util.spec_from_file_location("route_b_stub", os.path.join(ROOT, "tests", "route_b_stub.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)      # loads the library, declares the prototype, checks the ABI version
    return mod


def test_ctypes_stub_of_the_notes_loads_and_is_the_printed_one(monkeypatch):
    mod = _load_route_b_stub(monkeypatch)
    assert callable(mod.qAB)
    printed = [code for _, code in _doc_python_blocks() if "xkv_recon_stage1.argtypes" in code]
    assert len(printed) == 1
    body = open(os.path.join(ROOT, "tests", "route_b_stub.py")).read()
    assert body.endswith(printed[0]), "tests/route_b_stub.py must stay word for word what the notes print"
    from kernel_collections_amd import _lib
    assert mod._xkv.xkv_recon_stage1.argtypes[1]._fields_ == _lib.KVOperand._fields_


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_ctypes_stub_of_the_notes_computes_qab_rope(monkeypatch, dtype):
    """The stub binds nothing but ctypes and torch; its qAB must give the reference's RoPE scores."""
    import oracle
    mod = _load_route_b_stub(monkeypatch)
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(5)
    b, hq, hkv, L, r, d, theta = 2, 32, 8, 700, 512, 128, 1e7
    q = (torch.randn(b, hq, 1, d, generator=g) * 0.5).to(dtype)
    A = torch.randn(b, L, r, generator=g).to(dtype)
    B = (torch.randn(b, hkv, r, d, generator=g) * r ** -0.5).to(dtype)
    cos, sin = oracle.rope_cos_sin(torch.arange(L), d, theta)
    ref = oracle.qab_rope(q.float(), A.float(), B.float(), cos, sin)
    out = mod.qAB(q.to(dev), A.to(dev), B.to(dev), theta)
    torch.cuda.synchronize()
    assert out.shape == (b, hq, 1, L) and out.dtype == dtype
    err = (out.float().cpu() - ref).abs().max().item() / ref.abs().max().item()
    assert err <= 1e-2, err
