"""The ctypes binding a maintainer of the reference would put in flash_recontruction/qAB/v1.py in place of the Triton
launch at :135-145 - nothing but ctypes and torch, no import from this package.  Kept word for word as the integration
notes print it; the tests execute it."""
import ctypes, os, torch
from ctypes import c_void_p, c_int, c_int64, c_float, Structure

_xkv = ctypes.CDLL(os.environ.get("XKV_HIP_LIB", "libxkv_hip.so"))

class KVOperand(Structure):          # xkv_kv_operand
    _fields_ = [("ptr", c_void_p), ("stride_b", c_int64), ("stride_l", c_int64), ("stride_h", c_int64), ("dim", c_int)]

_xkv.xkv_recon_stage1.restype = c_int
_xkv.xkv_recon_stage1.argtypes = [c_void_p, KVOperand, c_void_p, c_int64, c_int64, c_int64, KVOperand,
    c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
    c_float, c_int, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int, c_void_p]
assert _xkv.xkv_abi_version() == 6

def qAB(q, A, B, theta=1e7):                       # same signature as flash_recontruction/qAB/v1.py:90
    bsz, hq, _, d = q.shape; L, r = A.shape[1], A.shape[2]; hkv = B.shape[1]
    out = torch.empty(bsz, hq, 1, L, dtype=q.dtype, device=q.device)
    inv = theta ** (-torch.arange(0, d, 2, device=q.device, dtype=torch.float32) / d)
    ns = torch.ones(bsz, dtype=torch.int32, device=q.device)
    rc = _xkv.xkv_recon_stage1(
        q.contiguous().data_ptr(), KVOperand(A.data_ptr(), A.stride(0), A.stride(1), 0, r),
        B.data_ptr(), B.stride(0), B.stride(1), B.stride(2), KVOperand(None, 0, 0, 0, 0),
        None, None, out.data_ptr(), 1 if q.dtype == torch.bfloat16 else 0, ns.data_ptr(), None,
        bsz, hq, hkv, L, 1, 1.0, 1, inv.data_ptr(), 0, None, 0, None, 0,
        1 if q.dtype == torch.bfloat16 else 0, torch.cuda.current_stream().cuda_stream)
    if rc: raise RuntimeError(f"xkv_recon_stage1 failed with code {rc}")
    return out
