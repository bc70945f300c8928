"""ctypes access to the C ABI (include/sma.h) for the tests: what a foreign-language binding sees."""
import ctypes
import os

import torch  # imported first so that the HIP runtime PyTorch ships is the one in the process

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "sparse-mask-attention_amd", "libsma_hip.so")

SMA_OK = 0
SMA_ERR_NULL_POINTER = -1
SMA_ERR_BAD_SHAPE = -2
SMA_ERR_HEAD_DIM = -3
SMA_ERR_DTYPE = -4
SMA_ERR_SCALE = -5
SMA_ERR_LAUNCH = -6
SMA_ERR_ALIGNMENT = -7
SMA_DTYPE_F16 = 0
SMA_DTYPE_BF16 = 1

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            raise RuntimeError(f"{LIB} is not built; run __graft_entry__.build()")
        lib = ctypes.CDLL(LIB)
        vp, ci, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        lib.sma_version.restype = ci
        lib.sma_version.argtypes = []
        lib.sma_strerror.restype = ctypes.c_char_p
        lib.sma_strerror.argtypes = [ci]
        lib.sma_pack_mask.restype = ci
        lib.sma_pack_mask.argtypes = [vp, vp, ci, ci, ci, vp]
        lib.sma_attn_fwd.restype = ci
        lib.sma_attn_fwd.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, cf, ci, vp]
        lib.sma_attn_bwd.restype = ci
        lib.sma_attn_bwd.argtypes = [vp] * 11 + [ci, ci, ci, ci, cf, ci, vp]
        _lib = lib
    return _lib


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def pack_mask(mask: torch.Tensor) -> torch.Tensor:
    """bool [B,H,N,N] GPU tensor -> int32 [B,H,N,nw] through sma_pack_mask."""
    lib = load()
    B, H, N, _ = mask.shape
    mask = mask.contiguous()
    # poison the output: the kernel must write every word itself
    packed = torch.full((B, H, N, (N + 31) // 32), -1431655766, dtype=torch.int32, device=mask.device)
    st = lib.sma_pack_mask(mask.data_ptr(), packed.data_ptr(), B, H, N, _stream())
    assert st == SMA_OK, lib.sma_strerror(st)
    return packed


def attn_fwd(q, k, v, packed, scale=None, want_lse=False):
    """Fused forward through sma_attn_fwd; returns out (and lse)."""
    lib = load()
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    dt = {torch.float16: SMA_DTYPE_F16, torch.bfloat16: SMA_DTYPE_BF16}[q.dtype]
    out = torch.full_like(q, float("nan"))
    lse = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=q.device) if want_lse else None
    st = lib.sma_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), packed.data_ptr(), out.data_ptr(),
                          lse.data_ptr() if want_lse else None, B, H, N, D, scale, dt, _stream())
    assert st == SMA_OK, lib.sma_strerror(st)
    return (out, lse) if want_lse else out


def attn_bwd(dout, q, k, v, out, lse, packed, scale=None):
    """Backward through sma_attn_bwd; returns (dq, dk, dv, delta).  Outputs are poisoned first."""
    lib = load()
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    dt = {torch.float16: SMA_DTYPE_F16, torch.bfloat16: SMA_DTYPE_BF16}[q.dtype]
    dq, dk, dv = (torch.full_like(q, float("nan")) for _ in range(3))
    delta = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=q.device)
    st = lib.sma_attn_bwd(dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                          lse.data_ptr(), packed.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                          delta.data_ptr(), B, H, N, D, scale, dt, _stream())
    assert st == SMA_OK, lib.sma_strerror(st)
    return dq, dk, dv, delta
