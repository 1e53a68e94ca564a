"""ctypes binding of ``libxkv_hip.so`` - the only bridge between the Python call surface and
the HIP kernels.  There is no fallback: if the library is missing or a call fails, it raises."""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("XKV_HIP_LIB", os.path.join(_HERE, "libxkv_hip.so"))  # override: another build of the same ABI

XKV_F16, XKV_BF16, XKV_F32 = 0, 1, 2
ABI_VERSION = 6

EXPORTS = (
    "xkv_abi_version", "xkv_error_string", "xkv_rope_table", "xkv_absorb_q",
    "xkv_blockdiag_q", "xkv_latent_stage1", "xkv_recon_stage1", "xkv_recon_workspace_bytes", "xkv_merge_stage2",
    "xkv_recon_stage1_static", "xkv_rope_apply", "xkv_ceiling_mfma", "xkv_ceiling_stream", "xkv_plan_splits", "xkv_softmax_pv_stage1",
    "xkv_poison_lds",
)
STATIC_SCRATCH_BYTES = 4 << 20
XKV_ESCRATCH = -5
XKV_ETOOLCHAIN = -6


class KVOperand(Structure):
    _fields_ = [("ptr", c_void_p), ("stride_b", c_int64), ("stride_l", c_int64), ("stride_h", c_int64),
                ("dim", c_int)]


class QOperand(Structure):
    _fields_ = [("ptr", c_void_p), ("dim", c_int)]


_lib = None


def _declare(lib):
    lib.xkv_abi_version.restype = c_int
    lib.xkv_abi_version.argtypes = []
    lib.xkv_error_string.restype = c_char_p
    lib.xkv_error_string.argtypes = [c_int]
    lib.xkv_rope_table.restype = c_int
    lib.xkv_rope_table.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_void_p]
    lib.xkv_rope_apply.restype = c_int
    lib.xkv_rope_apply.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int,
                                   c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p]
    lib.xkv_ceiling_mfma.restype = c_int
    lib.xkv_ceiling_mfma.argtypes = [c_void_p, c_int, c_int, c_int, c_void_p]
    lib.xkv_ceiling_stream.restype = c_int
    lib.xkv_ceiling_stream.argtypes = [c_void_p, c_int64, c_int, c_int, c_int, c_void_p, c_void_p]
    lib.xkv_absorb_q.restype = c_int
    lib.xkv_absorb_q.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                 c_int64, c_int64, c_int64, c_int, c_void_p]
    lib.xkv_blockdiag_q.restype = c_int
    lib.xkv_blockdiag_q.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]
    lib.xkv_latent_stage1.restype = c_int
    lib.xkv_latent_stage1.argtypes = [QOperand, c_void_p, QOperand, KVOperand, KVOperand, KVOperand,
                                      c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                      c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_float, c_float, c_int, c_void_p]
    lib.xkv_recon_stage1.restype = c_int
    lib.xkv_recon_stage1.argtypes = [c_void_p, KVOperand, c_void_p, c_int64, c_int64, c_int64, KVOperand,
                                     c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                     c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_int64,
                                     c_void_p, c_int64, c_void_p, c_int64, c_int, c_void_p]
    lib.xkv_recon_stage1_static.restype = c_int
    lib.xkv_recon_stage1_static.argtypes = lib.xkv_recon_stage1.argtypes[:-4] + [c_int, c_void_p]
    lib.xkv_recon_workspace_bytes.restype = c_int64
    lib.xkv_recon_workspace_bytes.argtypes = [c_int, c_int, c_int, c_int64]
    lib.xkv_merge_stage2.restype = c_int
    lib.xkv_merge_stage2.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int,
                                     c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int,
                                     c_int64, c_int64, c_int, c_void_p, c_int64, c_int64, c_void_p]
    lib.xkv_softmax_pv_stage1.restype = c_int
    lib.xkv_softmax_pv_stage1.argtypes = [c_void_p, KVOperand, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p]
    lib.xkv_poison_lds.restype = c_int
    lib.xkv_poison_lds.argtypes = [ctypes.c_uint32, c_void_p, c_void_p]
    lib.xkv_plan_splits.restype = c_int
    lib.xkv_plan_splits.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p]


def lib():
    """The loaded library; raises RuntimeError if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m kernel_collections_amd.build` "
                "(hipcc, gfx950). There is no non-HIP fallback.")
        l = ctypes.CDLL(LIB_PATH)
        _declare(l)
        v = l.xkv_abi_version()
        if v != ABI_VERSION:
            raise RuntimeError(f"libxkv_hip.so ABI {v} != binding ABI {ABI_VERSION}; rebuild")
        _lib = l
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().xkv_error_string(rc).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {rc})")


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float16:
        return XKV_F16
    if dt == torch.bfloat16:
        return XKV_BF16
    if dt == torch.float32:
        return XKV_F32
    raise AssertionError(f"unsupported dtype {dt}")


def stream_ptr(t: torch.Tensor) -> c_void_p:
    return c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def ptr(t) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def kv_operand(t, stride_b=None, stride_l=None, stride_h=0, dim=None) -> KVOperand:
    if t is None:
        return KVOperand(c_void_p(0), 0, 0, 0, 0)
    return KVOperand(c_void_p(t.data_ptr()), stride_b, stride_l, stride_h, dim)


def q_operand(t) -> QOperand:
    if t is None:
        return QOperand(c_void_p(0), 0)
    return QOperand(c_void_p(t.data_ptr()), t.shape[-1])


def require_gpu(t: torch.Tensor) -> None:
    assert t.is_cuda, "xkv HIP kernels need tensors on a ROCm device (there is no CPU path)"
