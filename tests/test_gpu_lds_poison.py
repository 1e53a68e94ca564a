"""Parity with the LDS poisoned: the LDS is not cleared between kernels, so a stage-1 kernel that reads a ring slot before its
tile has landed there (a wrong wait count, a barrier too few, a register handed on before its load has returned) can still
pass a parity test when the previous launch left the same rows in the same place.  Here every stage-1 launch is preceded, on
the same stream, by `xkv_poison_lds`, which leaves a NaN pattern in all 160 KiB of every CU: stale reads then show up as NaNs in
the output.  The cases are the parity tests of test_gpu_parity.py themselves, one or two per kernel family that tracks its own
loads (latent_ring, recon_spec, recon_fast, recon_duo) plus the generic kernels, called again under the poisoning binding.
"""
import pytest
import torch

import test_gpu_parity as tp
from kernel_collections_amd import _lib

pytestmark = pytest.mark.gpu

BF, FP = torch.bfloat16, torch.float16
PATTERN = 0x7FFF7FFF      # a NaN as fp16 (twice), as bf16 (twice) and as fp32
STAGE1 = ("xkv_latent_stage1", "xkv_recon_stage1", "xkv_recon_stage1_static", "xkv_softmax_pv_stage1")


class _Poisoning:
    """The loaded library with a poison launch in front of every stage-1 entry point."""

    def __init__(self, real):
        self._real, self.poisoned = real, 0

    def __getattr__(self, name):
        fn = getattr(self._real, name)
        if name not in STAGE1:
            return fn

        def call(*args):
            rc = self._real.xkv_poison_lds(PATTERN, None, torch.cuda.current_stream().cuda_stream)
            assert rc == 0, rc
            self.poisoned += 1
            return fn(*args)
        return call


@pytest.fixture
def poisoned(monkeypatch):
    proxy = _Poisoning(_lib.lib())
    monkeypatch.setattr(_lib, "lib", lambda: proxy)
    yield proxy
    assert proxy.poisoned > 0, "the case launched no stage-1 kernel through the binding"


def test_poison_is_still_there_for_the_next_kernel(dev):
    """The premise: what one kernel leaves in the LDS is what the next one finds."""
    lib = _lib.lib()
    st = torch.cuda.current_stream().cuda_stream
    seen = torch.zeros(2, dtype=torch.int32, device=dev)
    assert lib.xkv_poison_lds(PATTERN, None, st) == 0
    assert lib.xkv_poison_lds(PATTERN, seen.data_ptr(), st) == 0
    hit, looked = seen.tolist()
    assert looked > 0 and looked % (160 * 1024 // 4) == 0
    assert hit >= 0.9 * looked, f"only {hit} of {looked} LDS words still hold the pattern"
    # and another pattern is not found there
    seen.zero_()
    assert lib.xkv_poison_lds(0x12345678, seen.data_ptr(), st) == 0
    assert seen[0].item() == 0


@pytest.mark.parametrize("dtype", [BF, FP])
def test_ring_kernel_scores_and_decode(dev, dtype, poisoned):
    tp.test_qab_nope(dev, dtype, 2, 32, 8, 1000, 512)          # absorbed scores, 512-wide rows
    tp.test_qab_nope(dev, dtype, 1, 32, 8, 5, 512)             # shorter than one tile
    tp.test_fused_nope(dev, dtype, 1, 32, 8, 700, 512, 512, 3)  # shared basis: values = the latent rows
    tp.test_fused_nope(dev, dtype, 2, 32, 8, 3000, 256, 384, 8)  # a second row stream for the values
    tp.test_gqa_plain(dev, dtype, 2, 32, 8, 3000, 8)           # 8 kv heads as one 1024-wide row
    tp.test_mla2(dev, dtype, 2100)                             # 512 + 64 RoPE features


@pytest.mark.parametrize("dtype", [BF, FP])
def test_reconstruction_kernels(dev, dtype, poisoned):
    tp.test_qab_rope(dev, dtype, 2, 32, 8, 1000, 512, 5e5)     # recon_spec, scores mode, rank 512
    tp.test_qab_rope(dev, dtype, 2, 8, 2, 300, 384, 5e5)       # ... rank 384
    tp.test_qab_rope(dev, dtype, 1, 8, 2, 77, 256, 1e7)        # recon_fast (4 waves), rank 256
    tp.test_qab_rope(dev, dtype, 2, 4, 4, 40, 192, 1e7)        # generic kernel, rank 192
    tp.test_fused_rope(dev, dtype, 2, 32, 8, 3000, 512, 512, 4, True)    # recon_spec fused, shared basis
    tp.test_fused_rope(dev, dtype, 1, 32, 8, 1500, 256, 384, 3, False)   # a value basis of its own


@pytest.mark.parametrize("form", ["fused", "two_pass"])
def test_two_basis_forms(dev, form, poisoned, monkeypatch):
    # recon_duo (one kernel, two row streams) and scores pass + softmax / P.V over given scores, ragged lengths, short tiles
    tp.test_fused_rope_wide_kernels(dev, BF, 2, 32, 8, 512, 512, False, [1000, 333], 4, 0, form, monkeypatch)
    tp.test_fused_rope_wide_kernels(dev, FP, 2, 8, 8, 384, 384, False, [17, 64], 2, 0, form, monkeypatch)
    tp.test_fused_rope_wide_kernels(dev, BF, 3, 32, 8, 256, 256, False, [700, 5, 2048], 5, 100000, form, monkeypatch)


def test_config1_shape(dev, poisoned):
    tp.test_config1_shape_factorized_rope(dev)
