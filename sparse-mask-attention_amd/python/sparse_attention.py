"""Sparse-mask attention: the user-facing Python API, unchanged from the reference.

Mirrors ``python/sparse_attention.py`` of the reference (line numbers below refer to it):

* ``sparse_attention(q, k, v, mask)``       :120-154  autograd-aware entry point
* ``sparse_attention_func(q, k, v, mask)``  :157-177  inference-only variant (no LSE, no graph)
* ``pack_mask(mask)``                       :184-201  bool [B,H,N,N] -> int32 [B,H,N,ceil(N/32)]
* ``SparseAttentionFunction``               :49-113   the autograd.Function behind the first
* ``sparse_attention_ref``                  :24-42    the plain-PyTorch statement of the operator
* ``generate_random_sparse_mask``           :204-211

``q, k, v`` are ``[B, H, N, D]`` fp16 / bf16 tensors on an MI355X, D = 64 as in the reference, 32 or
128 (other head dims up to 128 are zero-padded to the next of these, see below) (fp32 inputs are computed in
bf16 and returned as fp32, as in the reference :140-142,151-152); ``mask`` is a bool
``[B, H, N, N]`` tensor, True = attend.  Query rows that attend to nothing give zeros.

What differs from the reference, on purpose:

* The compute path is the HIP extension ``sparse_attn_cuda`` (same module name) and nothing else.
  Where the reference silently computes with PyTorch ops when the extension is missing or the
  tensors live on the CPU (:148-149, :65-74), this module raises ``RuntimeError``: a silent
  fallback would hide a broken build.  ``sparse_attention_ref`` stays available for callers who
  want the PyTorch formulation explicitly.
* ``q, k, v`` need not be contiguous: views whose last dimension is contiguous and whose other
  strides are multiples of 8 elements (a ``[B, N, H, D]`` buffer viewed as ``[B, H, N, D]``, slices
  of a fused qkv projection) go to the kernels as they are, where the reference would read them as
  if they were contiguous; anything else is copied with ``.contiguous()`` first.
* ``mask`` may be ``[1, 1, N, N]``, ``[B, 1, N, N]`` or ``[1, H, N, N]``: it is packed once at that
  size and shared between batch entries / heads by the kernels (the reference needs the expanded
  ``[B, H, N, N]`` tensor).  A mask passed as an ``expand``-ed view is recognised by its zero
  strides and treated the same way.
* Head dims: the kernels exist for 64 (the reference's only one), 32 and 128.  Any other D <= 128
  is computed exactly by zero-padding q, k, v to the next of these (the scores and the first D output
  columns do not change; the scale stays 1/sqrt(D)) at the price of the padding copies.
* The mask is not packed in a pass of its own: where the kernel's limits allow (any q, k, v the strided kernels take,
  N >= 16) one launch reads the bool mask itself and forms the packed words tile by
  tile, which is 15-35 % faster than pack + attention; under autograd the same launch also leaves
  the packed words behind for the backward.  Otherwise the mask is packed as the reference does.
  Results are bit-identical either way; both ways count any non-zero mask byte as True, so a bool
  tensor made by ``view`` from bytes other than 0 and 1 is read the same by both.
* Block-structured masks (sliding window, block-sparse, causal): ``tile_map(mask_packed)`` says
  which 64 x 64 blocks of the mask hold a set bit; given as ``tile_map=`` together with
  ``mask_packed=`` the forward neither loads nor computes the key tiles that hold none (the
  reference skips such a tile only after loading it, ``csrc/sparse_attention.cu:211,238-252``).
  Worth it for a mask that is used many times; ``tile_map`` returns None when too few visits would
  disappear for the walk to pay.
* ``.backward()`` works.  The reference calls a ``sparse_attn_cuda.backward`` that was never
  written (:91-94); here that function exists (two HIP kernels, dQ and dK/dV, from the saved
  log-sum-exp and the packed mask).  ``backward_recompute`` states the same gradients with PyTorch
  ops (the reference's own formulas, :97-111) for cross-checks.
"""
from __future__ import annotations

import math
import os
import sys

import torch
from torch.autograd import Function

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if _PKG_DIR not in sys.path:
    sys.path.insert(0, _PKG_DIR)

try:
    import sparse_attn_cuda  # pybind shim over libsma_hip.so, built in-tree by buildlib.py
    HAS_CUDA_EXT = True
    _EXT_ERROR = None
except ImportError as exc:  # the API stays importable; any compute call reports the cause
    sparse_attn_cuda = None
    HAS_CUDA_EXT = False
    _EXT_ERROR = exc


def _rows(t: torch.Tensor) -> torch.Tensor:
    """t itself if the kernels can address it (contiguous last dimension, the strides of the other
    dimensions multiples of 8 elements, 16-byte aligned storage), else a contiguous copy."""
    ok = (t.stride(-1) == 1 or t.size(-1) == 1) and t.data_ptr() % 16 == 0 and all(
        st % 8 == 0 for st, n in zip(t.stride()[:-1], t.shape[:-1]) if n > 1)
    return t if ok else t.contiguous()


def _require_ext(t: torch.Tensor) -> None:
    if not HAS_CUDA_EXT:
        raise RuntimeError(
            "the HIP extension sparse_attn_cuda is not built or failed to load "
            f"({_EXT_ERROR}); run `python setup.py build_ext --inplace` in {_PKG_DIR}")
    if not t.is_cuda:
        raise RuntimeError("sparse attention runs on the GPU only: move q, k, v and mask to the "
                           "device (sparse_attention_ref is the PyTorch formulation for any device)")


# ----------------------------------------------------------------------------------------------
# Plain-PyTorch statement of the operator (never called by the functions below)
# ----------------------------------------------------------------------------------------------

def sparse_attention_ref(q, k, v, mask):
    """softmax(mask ? q k^T / sqrt(D) : -inf) v with PyTorch ops, in the dtype of the inputs."""
    scale = 1.0 / math.sqrt(q.shape[-1])
    logits = (q @ k.transpose(-1, -2)) * scale
    logits = logits.masked_fill(mask.logical_not(), float("-inf"))
    probs = torch.nan_to_num(torch.softmax(logits, dim=-1), nan=0.0)   # empty rows -> zeros
    return probs @ v


# ----------------------------------------------------------------------------------------------
# autograd
# ----------------------------------------------------------------------------------------------

class SparseAttentionFunction(Function):
    """forward = fused HIP kernel (saves LSE); backward = the HIP dQ and dK/dV kernels.

    ``mask_packed`` may be None: the mask is then read as it is by the one-launch forward, which
    leaves the packed words the backward uses (and, with ``tile_map=True``, the mask's tile map) as
    by-products, or packed first where that kernel does not apply."""

    @staticmethod
    def forward(ctx, q, k, v, mask_packed, mask_bool, scale, seq_len, tile_map=None):
        _require_ext(q)
        B, H, N, _ = q.shape
        q, k, v = _rows(q), _rows(k), _rows(v)
        out = torch.empty_like(q)
        lse = torch.empty(B, H, N, device=q.device, dtype=torch.float32)
        if mask_packed is None:
            mask_bool = _unexpand(mask_bool)
            if sparse_attn_cuda.bool_mask_supported(q, k, v, mask_bool):
                mask_packed = torch.empty(mask_bool.shape[0], mask_bool.shape[1], N, (N + 31) // 32,
                                          device=q.device, dtype=torch.int32)
                # tile_map=True: the caller says the mask has empty 64 x 64 blocks; the same launch
                # then leaves the mask's tile map behind and the backward visits only the blocks
                # that hold something.  Not by default: a mask without empty blocks (any random one)
                # would pay for a by-product that nothing can use.
                if tile_map is True:
                    T = (N + 63) // 64
                    tile_map = torch.empty(mask_bool.shape[0], mask_bool.shape[1], T, 2, (T + 31) // 32,
                                           device=q.device, dtype=torch.int32)
                else:
                    tile_map = None
                sparse_attn_cuda.forward_bool_mask(q, k, v, mask_bool, out, lse, scale, True, mask_packed, tile_map)
                ctx.save_for_backward(q, k, v, out, lse, mask_packed)
                ctx.scale = scale
                ctx.tile_map = tile_map
                return out
            mask_packed = pack_mask(mask_bool)
            tile_map = sparse_attn_cuda.tile_map(mask_packed) if tile_map is True else None
        sparse_attn_cuda.forward(q, k, v, mask_packed, out, lse, scale, True, tile_map)
        ctx.save_for_backward(q, k, v, out, lse, mask_packed)
        ctx.scale = scale
        ctx.tile_map = tile_map
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, mask_packed = ctx.saved_tensors
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        # the call the reference makes at python/sparse_attention.py:91-94
        sparse_attn_cuda.backward(_rows(dout.to(q.dtype)), q, k, v, out, lse, mask_packed,
                                  dq, dk, dv, ctx.scale, getattr(ctx, "tile_map", None))
        return dq, dk, dv, None, None, None, None, None


def backward_recompute(q, k, v, out, lse, mask_bool, dout, scale):
    """The same gradients with PyTorch ops on the GPU from the saved log-sum-exp (the formulas of
    the reference's fallback, python/sparse_attention.py:97-111).  Not used by the autograd
    function; kept as a cross-check for users and tests."""
    qf, kf, vf, do = q.float(), k.float(), v.float(), dout.float()
    # p = exp(s - lse) on kept entries; rows that keep nothing have lse = -inf and p = 0.
    s = (qf @ kf.transpose(-1, -2)) * scale
    safe_lse = torch.where(torch.isinf(lse), torch.zeros_like(lse), lse).unsqueeze(-1)
    p = torch.exp(s - safe_lse).masked_fill(mask_bool.logical_not(), 0.0)
    dv = p.transpose(-1, -2) @ do
    dp = do @ vf.transpose(-1, -2)
    delta = (do * out.float()).sum(dim=-1, keepdim=True)      # = sum_j p_ij dp_ij
    ds = p * (dp - delta) * scale
    dq = ds @ kf
    dk = ds.transpose(-1, -2) @ qf
    return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype)


# ----------------------------------------------------------------------------------------------
# public entry points
# ----------------------------------------------------------------------------------------------

def _check_inputs(q, k, v, mask, mask_packed=None):
    assert q.shape == k.shape == v.shape, "q/k/v must have the same shape"
    B, H, N, _ = q.shape
    if mask_packed is not None:
        mp = tuple(mask_packed.shape)
        assert mask_packed.dtype == torch.int32 and len(mp) == 4 and mp[0] in (1, B) and mp[1] in (1, H) \
            and mp[2:] == (N, (N + 31) // 32), \
            "mask_packed must be the int32 [B or 1, H or 1, N, ceil(N/32)] result of pack_mask"
        assert mask_packed.device == q.device, "all tensors must be on the same device"
        return
    assert q.device == k.device == v.device == mask.device, "all tensors must be on the same device"
    assert mask.dtype == torch.bool, "mask must be a bool tensor"
    ms = tuple(mask.shape)
    assert len(ms) == 4 and ms[0] in (1, B) and ms[1] in (1, H) and ms[2:] == (N, N), \
        "mask must be [B or 1, H or 1, N, N]"


def _unexpand(mask: torch.Tensor) -> torch.Tensor:
    """The mask with its expanded (stride 0) batch / head extents taken back to 1: a mask given as
    ``m.expand(B, H, N, N)`` is read (or packed) once and shared, not B*H times."""
    if mask.size(0) > 1 and mask.stride(0) == 0:
        mask = mask[:1]
    if mask.size(1) > 1 and mask.stride(1) == 0:
        mask = mask[:, :1]
    return mask





def _pad_head_dim(q, k, v):
    """q, k, v with their head dim zero-padded to the next one the kernels have (32, 64 or 128)."""
    D = q.shape[-1]
    assert 1 <= D <= 128, "head_dim must be at most 128"
    Dk = 32 if D <= 32 else (64 if D <= 64 else 128)
    if D == Dk:
        return q, k, v
    pad = (0, Dk - D)
    return tuple(torch.nn.functional.pad(t, pad) for t in (q, k, v))


def sparse_attention(q, k, v, mask, mask_packed=None, tile_map=None):
    """Masked attention with autograd support.

    q, k, v: ``[B, H, N, D]`` (D = 32, 64 or 128; other D <= 128 are zero-padded) bf16 / fp16 / fp32;  mask: bool ``[B, H, N, N]``, True = keep
    (a leading extent of 1 shares the mask between batch entries / heads).
    Returns a tensor of q's shape and original dtype.

    ``mask_packed`` (optional, not in the reference): the result of ``pack_mask(mask)`` kept from an
    earlier call with the same mask; packing (as much HBM traffic as the attention itself at
    N = 512) is then skipped and ``mask`` may be None.  ``tile_map`` (optional): with ``mask_packed``,
    the result of ``tile_map(mask_packed)``; key tiles in which the mask keeps nothing are skipped.
    With a bool ``mask`` under autograd, ``tile_map=True`` says that the mask has empty 64 x 64 blocks:
    the forward then leaves the map behind for the backward (about 1 us at N = 512; off by default,
    because a mask without empty blocks gains nothing from it).
    """
    _check_inputs(q, k, v, mask, mask_packed)
    assert tile_map is None or tile_map is True or mask_packed is not None, "a tile_map tensor belongs to a mask_packed"
    assert not (tile_map is True and mask_packed is not None), "with mask_packed, pass the result of tile_map(mask_packed)"
    _require_ext(q)
    if not (torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)):
        # nothing will be differentiated: no LSE, and the mask can be read without packing it
        return sparse_attention_func(q, k, v, mask, mask_packed, tile_map)
    B, H, N, D = q.shape
    scale = 1.0 / math.sqrt(D)

    orig_dtype = q.dtype
    if orig_dtype == torch.float32:
        q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()

    q, k, v = _pad_head_dim(q, k, v)              # differentiable: the gradients are sliced back
    out = SparseAttentionFunction.apply(q, k, v, mask_packed, mask, scale, N, tile_map)[..., :D]

    if orig_dtype == torch.float32:
        out = out.float()
    return out


def sparse_attention_func(q, k, v, mask, mask_packed=None, tile_map=None):
    """Inference-only variant of :func:`sparse_attention`: no autograd graph, no LSE."""
    _check_inputs(q, k, v, mask, mask_packed)
    if tile_map is True:        # a hint for the backward only
        tile_map = None
    assert tile_map is None or mask_packed is not None, "tile_map belongs to a mask_packed"
    _require_ext(q)
    D = q.shape[-1]
    scale = 1.0 / math.sqrt(D)

    orig_dtype = q.dtype
    if orig_dtype == torch.float32:
        q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()

    with torch.no_grad():
        q, k, v = _pad_head_dim(q, k, v)
        q, k, v = _rows(q), _rows(k), _rows(v)
        if mask_packed is None:
            mask = _unexpand(mask)
            if sparse_attn_cuda.bool_mask_supported(q, k, v, mask):
                out = torch.empty_like(q)
                sparse_attn_cuda.forward_bool_mask(q, k, v, mask, out, None, scale, False)
                return (out[..., :D].float() if orig_dtype == torch.float32 else out[..., :D])
            mask_packed = pack_mask(mask)
        out = torch.empty_like(q)
        sparse_attn_cuda.forward(q, k, v, mask_packed, out, None, scale, False, tile_map)
        out = out[..., :D]

    if orig_dtype == torch.float32:
        out = out.float()
    return out


# ----------------------------------------------------------------------------------------------
# mask helpers
# ----------------------------------------------------------------------------------------------

def pack_mask(mask: torch.Tensor) -> torch.Tensor:
    """bool ``[B, H, N, N]`` -> bit-packed int32 ``[B, H, N, ceil(N/32)]`` (bit j of word w = column 32w+j).
    A mask shared between batch entries / heads is passed (and packed) as ``[1 or B, 1 or H, N, N]``."""
    _require_ext(mask)
    return sparse_attn_cuda.pack_mask(mask)


def tile_map(mask_packed: torch.Tensor, min_skip: float = 0.3):
    """Occupancy of the 64 x 64 blocks of a packed mask, for ``sparse_attention(..., mask_packed=,
    tile_map=)``: int32 ``[B, H, T, 2, ceil(T/32)]`` with T = ceil(N/64); per block of 64 query rows
    one bit per 64-key tile "some entry kept", then one bit per tile "every entry kept".

    Returns None when the map would not pay: the forward walks the key tiles per 128 query rows (two
    row blocks), and below ``min_skip`` (default 0.3) of those visits saved the walk costs what
    it saves (a causal mask at N = 256 skips 2 of 8 visits per head and runs no faster with the
    map).  ``min_skip=0`` returns the map whenever a single visit disappears.  Synchronises with the
    device once, to look at that; meant to be called once for a mask that is used many times."""
    _require_ext(mask_packed)
    tm = sparse_attn_cuda.tile_map(mask_packed)
    T = tm.shape[2]
    live = tm[:, :, :, 0, :]
    if T % 2:                                   # the last work-group has one row block only
        live = torch.cat([live, torch.zeros_like(live[:, :, :1])], dim=2)
    pairs = live[:, :, 0::2] | live[:, :, 1::2]             # what a work-group of 128 rows visits
    bits = (pairs.unsqueeze(-1) >> torch.arange(32, device=tm.device, dtype=torch.int32)) & 1
    visited = int(bits.sum().item())
    total = pairs.shape[0] * pairs.shape[1] * pairs.shape[2] * T
    skipped = total - visited
    return tm if skipped > 0 and skipped >= min_skip * total else None


def generate_random_sparse_mask(B, H, N, sparsity=0.75, device="cuda"):
    """Random mask whose entries are False (masked out) with probability ``sparsity``."""
    return torch.rand(B, H, N, N, device=device) > sparsity
