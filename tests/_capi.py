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
SMA_ERR_STRIDE = -8
SMA_ERR_WORKSPACE = -9
SMA_ERR_DEVICE = -10
SMA_STATIC_WS_ROWS = 1 << 20
SMA_DTYPE_F16 = 0
SMA_DTYPE_BF16 = 1

_lib = None
_probe = None


class SmaTensor(ctypes.Structure):
    """struct sma_tensor of include/sma.h."""
    _fields_ = [("data", ctypes.c_void_p), ("stride_b", ctypes.c_int64), ("stride_h", ctypes.c_int64),
                ("stride_n", ctypes.c_int64)]

    @classmethod
    def of(cls, t: torch.Tensor) -> "SmaTensor":
        assert t.dim() == 4 and t.stride(3) == 1
        return cls(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


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
        lib.sma_tile_map_words.restype = ctypes.c_longlong
        lib.sma_tile_map_words.argtypes = [ci]
        lib.sma_tile_map.restype = ci
        lib.sma_tile_map.argtypes = [vp, vp, ci, ci, ci, vp]
        lib.sma_pack_mask_map.restype = ci
        lib.sma_pack_mask_map.argtypes = [vp, vp, vp, ci, ci, ci, vp]
        lib.sma_attn_fwd_map.restype = ci
        lib.sma_attn_fwd_map.argtypes = [vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, cf, ci, vp]
        lib.sma_device_check.restype = ci
        lib.sma_device_check.argtypes = [vp]
        lib.sma_attn_bwd_map.restype = ci
        lib.sma_attn_bwd_map.argtypes = [vp] * 12 + [ci, ci, ci, ci, cf, ci, vp]
        lib.sma_attn_bwd_static_ws.restype = ci
        lib.sma_attn_bwd_static_ws.argtypes = [vp] * 10 + [ci, ci, ci, ci, cf, ci, vp]
        tp, i64 = ctypes.POINTER(SmaTensor), ctypes.c_int64
        lib.sma_attn_fwd_strided.restype = ci
        lib.sma_attn_fwd_strided.argtypes = [tp, tp, tp, vp, i64, i64, tp, vp, ci, ci, ci, ci, cf, ci, vp]
        lib.sma_attn_bwd_strided.restype = ci
        lib.sma_attn_bwd_strided.argtypes = [tp] * 5 + [vp, vp, i64, i64, tp, tp, tp, vp, ci, ci, ci, ci, cf, ci, vp]
        lib.sma_attn_fwd_map_strided.restype = ci
        lib.sma_attn_fwd_map_strided.argtypes = [tp, tp, tp, vp, i64, i64, vp, tp, vp, ci, ci, ci, ci, cf, ci, vp]
        lib.sma_attn_bwd_map_strided.restype = ci
        lib.sma_attn_bwd_map_strided.argtypes = [tp] * 5 + [vp, vp, i64, i64, vp, tp, tp, tp, vp, ci, ci, ci, ci, cf, ci, vp]
        lib.sma_attn_fwd_bool_mask.restype = ci
        lib.sma_attn_fwd_bool_mask.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp, vp, ci, ci, ci, ci, cf, ci, vp]
        lib.sma_attn_fwd_bool_mask_map.restype = ci
        lib.sma_attn_fwd_bool_mask_map.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp, vp, vp, ci, ci, ci, ci, cf, ci, vp]
        lib.sma_attn_fwd_bool_mask_strided.restype = ci
        lib.sma_attn_fwd_bool_mask_strided.argtypes = [tp, tp, tp, vp, i64, i64, tp, vp, vp, vp, ci, ci, ci, ci, cf, ci, vp]
        _lib = lib
    return _lib


def load_probe():
    """libsma_probe.so, the benchmark's MFMA yardstick (benchprobe/mfma_probe.h): not the product."""
    global _probe
    if _probe is None:
        path = os.path.join(os.path.dirname(LIB), "libsma_probe.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is not built; run __graft_entry__.build()")
        lib = ctypes.CDLL(path)
        lib.sma_probe_mfma_stream.restype = ctypes.c_int
        lib.sma_probe_mfma_stream.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        _probe = lib
    return _probe


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


def _new_map(Bm, Hm, N, device):
    """Poisoned tile map tensor [Bm,Hm,T,2,TW] (int32 holding uint32 words)."""
    lib = load()
    QT = (N + 63) // 64
    TW = (QT + 31) // 32
    assert lib.sma_tile_map_words(N) == QT * 2 * TW
    return torch.full((Bm, Hm, QT, 2, TW), -1431655766, dtype=torch.int32, device=device)


def tile_map(packed: torch.Tensor) -> torch.Tensor:
    """int32 [B,H,N,nw] packed words -> tile map through sma_tile_map."""
    lib = load()
    B, H, N, _ = packed.shape
    tm = _new_map(B, H, N, packed.device)
    st = lib.sma_tile_map(packed.data_ptr(), tm.data_ptr(), B, H, N, _stream())
    assert st == SMA_OK, lib.sma_strerror(st)
    return tm


def pack_mask_map(mask: torch.Tensor):
    """bool [B,H,N,N] -> (packed, tile map) through sma_pack_mask_map."""
    lib = load()
    B, H, N, _ = mask.shape
    mask = mask.contiguous()
    packed = torch.full((B, H, N, (N + 31) // 32), -1431655766, dtype=torch.int32, device=mask.device)
    tm = _new_map(B, H, N, mask.device)
    st = lib.sma_pack_mask_map(mask.data_ptr(), packed.data_ptr(), tm.data_ptr(), B, H, N, _stream())
    assert st == SMA_OK, lib.sma_strerror(st)
    return packed, tm


def attn_fwd_map(q, k, v, packed, tm, scale=None, want_lse=False):
    """Fused forward through sma_attn_fwd_map (tile map of the same mask); returns out (and lse)."""
    lib = load()
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    dt = {torch.float16: SMA_DTYPE_F16, torch.bfloat16: SMA_DTYPE_BF16}[q.dtype]
    out = torch.full_like(q, float("nan"))
    lse = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=q.device) if want_lse else None
    st = lib.sma_attn_fwd_map(q.data_ptr(), k.data_ptr(), v.data_ptr(), packed.data_ptr(),
                              tm.data_ptr() if tm is not None else None, out.data_ptr(),
                              lse.data_ptr() if want_lse else None, B, H, N, D, scale, dt, _stream())
    assert st == SMA_OK, lib.sma_strerror(st)
    return (out, lse) if want_lse else out


def attn_fwd_map_strided(q, k, v, packed, tm, out=None, scale=None, want_lse=False):
    """sma_attn_fwd_map_strided: as attn_fwd_strided, with the tile map [Bm,Hm,QT,2,TW] of `packed`."""
    lib = load()
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    dt = {torch.float16: SMA_DTYPE_F16, torch.bfloat16: SMA_DTYPE_BF16}[q.dtype]
    if out is None:
        out = torch.full((B, H, N, D), float("nan"), dtype=q.dtype, device=q.device)
    lse = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=q.device) if want_lse else None
    msb, msh = _mask_strides(packed, B, H)
    tq, tk, tv, to = (SmaTensor.of(t) for t in (q, k, v, out))
    st = lib.sma_attn_fwd_map_strided(tq, tk, tv, packed.data_ptr(), msb, msh, tm.data_ptr(), to,
                                      lse.data_ptr() if want_lse else None, B, H, N, D, scale, dt, _stream())
    assert st == SMA_OK, lib.sma_strerror(st)
    return (out, lse) if want_lse else out


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


def attn_bwd_map(dout, q, k, v, out, lse, packed, tm, scale=None):
    """Backward through sma_attn_bwd_map (tile map of the same mask); returns (dq, dk, dv)."""
    lib = load()
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    dt = {torch.float16: SMA_DTYPE_F16, torch.bfloat16: SMA_DTYPE_BF16}[q.dtype]
    dq, dk, dv = (torch.full_like(q, float("nan")) for _ in range(3))
    delta = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=q.device)
    st = lib.sma_attn_bwd_map(dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                              lse.data_ptr(), packed.data_ptr(), tm.data_ptr() if tm is not None else None,
                              dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), delta.data_ptr(), B, H, N, D, scale, dt,
                              _stream())
    assert st == SMA_OK, lib.sma_strerror(st)
    return dq, dk, dv


def attn_bwd_static_ws(dout, q, k, v, out, lse, packed, scale=None, expect=SMA_OK):
    """Backward through sma_attn_bwd_static_ws (no workspace argument); returns (dq, dk, dv), or the
    status if `expect` is an error code.  Outputs are poisoned first."""
    lib = load()
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    dt = {torch.float16: SMA_DTYPE_F16, torch.bfloat16: SMA_DTYPE_BF16}[q.dtype]
    dq, dk, dv = (torch.full_like(q, float("nan")) for _ in range(3))
    st = lib.sma_attn_bwd_static_ws(dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                    lse.data_ptr(), packed.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                                    dv.data_ptr(), B, H, N, D, scale, dt, _stream())
    if expect != SMA_OK:
        return st
    assert st == SMA_OK, lib.sma_strerror(st)
    return dq, dk, dv


def _mask_strides(packed, B, H):
    """Word strides of a packed mask [Bm,Hm,N,nw] with Bm in {1,B}, Hm in {1,H}; 0 = shared."""
    Bm, Hm, N, nw = packed.shape
    assert Bm in (1, B) and Hm in (1, H) and packed.is_contiguous()
    return (Hm * N * nw if Bm == B and B > 1 else 0), (N * nw if Hm == H and H > 1 else 0)


def attn_fwd_strided(q, k, v, packed, out=None, scale=None, want_lse=False):
    """Forward through sma_attn_fwd_strided: q, k, v (and out, if given) may be any views whose last
    dimension is contiguous; packed may be [1|B, 1|H, N, nw]."""
    lib = load()
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    dt = {torch.float16: SMA_DTYPE_F16, torch.bfloat16: SMA_DTYPE_BF16}[q.dtype]
    if out is None:
        out = torch.full((B, H, N, D), float("nan"), dtype=q.dtype, device=q.device)
    lse = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=q.device) if want_lse else None
    msb, msh = _mask_strides(packed, B, H)
    tq, tk, tv, to = (SmaTensor.of(t) for t in (q, k, v, out))
    st = lib.sma_attn_fwd_strided(tq, tk, tv, packed.data_ptr(), msb, msh, to,
                                  lse.data_ptr() if want_lse else None, B, H, N, D, scale, dt, _stream())
    assert st == SMA_OK, lib.sma_strerror(st)
    return (out, lse) if want_lse else out


def attn_fwd_bool_mask_strided(q, k, v, mask, out=None, scale=None, want_lse=False, want_packed=False, want_map=False,
                               expect=SMA_OK):
    """Forward straight from the boolean mask through sma_attn_fwd_bool_mask_strided: q, k, v (and out,
    if given) may be any views whose last dimension is contiguous.  Returns out (and lse) (and the
    packed words) (and the tile map), or the status if `expect` is an error code."""
    lib = load()
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    dt = {torch.float16: SMA_DTYPE_F16, torch.bfloat16: SMA_DTYPE_BF16}[q.dtype]
    assert mask.dtype == torch.bool and mask.is_contiguous()
    Bm, Hm = mask.shape[:2]
    msb = Hm * N * N if Bm == B and B > 1 else 0
    msh = N * N if Hm == H and H > 1 else 0
    if out is None:
        out = torch.full((B, H, N, D), float("nan"), dtype=q.dtype, device=q.device)
    lse = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=q.device) if want_lse else None
    packed = (torch.full((Bm, Hm, N, (N + 31) // 32), -1431655766, dtype=torch.int32, device=q.device)
              if want_packed else None)
    tm = _new_map(Bm, Hm, N, q.device) if want_map else None
    tq, tk, tv, to = (SmaTensor.of(t) for t in (q, k, v, out))
    st = lib.sma_attn_fwd_bool_mask_strided(tq, tk, tv, mask.data_ptr(), msb, msh, to,
                                            lse.data_ptr() if want_lse else None,
                                            packed.data_ptr() if want_packed else None,
                                            tm.data_ptr() if want_map else None, B, H, N, D, scale, dt, _stream())
    if expect != SMA_OK:
        return st
    assert st == SMA_OK, lib.sma_strerror(st)
    res = (out,) + ((lse,) if want_lse else ()) + ((packed,) if want_packed else ()) + ((tm,) if want_map else ())
    return res if len(res) > 1 else out


def attn_bwd_strided(dout, q, k, v, out, lse, packed, grads=None, scale=None):
    """Backward through sma_attn_bwd_strided; grads = (dq, dk, dv) views to fill, or None for new
    contiguous tensors.  Returns (dq, dk, dv, delta)."""
    lib = load()
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    dt = {torch.float16: SMA_DTYPE_F16, torch.bfloat16: SMA_DTYPE_BF16}[q.dtype]
    if grads is None:
        grads = tuple(torch.full((B, H, N, D), float("nan"), dtype=q.dtype, device=q.device) for _ in range(3))
    dq, dk, dv = grads
    delta = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=q.device)
    msb, msh = _mask_strides(packed, B, H)
    ts = [SmaTensor.of(t) for t in (dout, q, k, v, out, dq, dk, dv)]
    st = lib.sma_attn_bwd_strided(ts[0], ts[1], ts[2], ts[3], ts[4], lse.data_ptr(), packed.data_ptr(), msb, msh,
                                  ts[5], ts[6], ts[7], delta.data_ptr(), B, H, N, D, scale, dt, _stream())
    assert st == SMA_OK, lib.sma_strerror(st)
    return dq, dk, dv, delta


def attn_bwd_map_strided(dout, q, k, v, out, lse, packed, tm, scale=None):
    """Backward through sma_attn_bwd_map_strided (any views, shared masks, tile map of `packed`);
    returns new contiguous (dq, dk, dv)."""
    lib = load()
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    dt = {torch.float16: SMA_DTYPE_F16, torch.bfloat16: SMA_DTYPE_BF16}[q.dtype]
    dq, dk, dv = (torch.full((B, H, N, D), float("nan"), dtype=q.dtype, device=q.device) for _ in range(3))
    delta = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=q.device)
    msb, msh = _mask_strides(packed, B, H)
    ts = [SmaTensor.of(t) for t in (dout, q, k, v, out, dq, dk, dv)]
    st = lib.sma_attn_bwd_map_strided(ts[0], ts[1], ts[2], ts[3], ts[4], lse.data_ptr(), packed.data_ptr(), msb, msh,
                                      tm.data_ptr(), ts[5], ts[6], ts[7], delta.data_ptr(), B, H, N, D, scale, dt,
                                      _stream())
    assert st == SMA_OK, lib.sma_strerror(st)
    return dq, dk, dv


def attn_fwd_bool_mask(q, k, v, mask, scale=None, want_lse=False, expect=SMA_OK, want_packed=False,
                       want_map=False):
    """Forward straight from the boolean mask ([1|B, 1|H, N, N], contiguous) through
    sma_attn_fwd_bool_mask (sma_attn_fwd_bool_mask_map with `want_map`); returns out (and lse) (and
    the packed words it leaves behind) (and the tile map), or the status if `expect` is an error
    code."""
    lib = load()
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    dt = {torch.float16: SMA_DTYPE_F16, torch.bfloat16: SMA_DTYPE_BF16}[q.dtype]
    assert mask.dtype == torch.bool and mask.is_contiguous()
    Bm, Hm = mask.shape[:2]
    msb = Hm * N * N if Bm == B and B > 1 else 0
    msh = N * N if Hm == H and H > 1 else 0
    out = torch.full_like(q, float("nan"))
    lse = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=q.device) if want_lse else None
    packed = (torch.full((Bm, Hm, N, (N + 31) // 32), -1431655766, dtype=torch.int32, device=q.device)
              if want_packed else None)
    if want_map:
        tm = _new_map(Bm, Hm, N, q.device)
        st = lib.sma_attn_fwd_bool_mask_map(q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.data_ptr(), msb, msh,
                                            out.data_ptr(), lse.data_ptr() if want_lse else None,
                                            packed.data_ptr() if want_packed else None, tm.data_ptr(), B, H, N, D,
                                            scale, dt, _stream())
    else:
        st = lib.sma_attn_fwd_bool_mask(q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.data_ptr(), msb, msh,
                                        out.data_ptr(), lse.data_ptr() if want_lse else None,
                                        packed.data_ptr() if want_packed else None, B, H, N, D, scale, dt, _stream())
    if expect != SMA_OK:
        return st
    assert st == SMA_OK, lib.sma_strerror(st)
    res = (out,) + ((lse,) if want_lse else ()) + ((packed,) if want_packed else ()) + ((tm,) if want_map else ())
    return res if len(res) > 1 else out
