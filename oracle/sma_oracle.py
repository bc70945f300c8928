"""CPU oracle for the sparse-mask-attention hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, what the reference computes for the two steps of
its hot path.  Nothing in the shipped package imports it: only the test-suite, the
smoke check and the benchmark's CPU-baseline leg may call it, and only as the
checker that the HIP kernels are compared with.

Functions and the reference lines they follow (paths under the reference tree):

* ``pack_mask_ref``         bit format of ``csrc/sparse_attention.cu:549-568`` (bit j of
                            word w of a row is column 32*w+j, pad bits zero) with the
                            output dtype/shape of ``csrc/binding.cpp:54-57`` (int32,
                            ``[B,H,N,(N+31)//32]``).  Same format as the CPU fallback
                            ``python/sparse_attention.py:193-201``.
* ``pack_mask_loops``       the same format written as the literal per-bit triple loop,
                            for tiny inputs only (an independent second statement).
* ``unpack_mask_ref``       inverse, reading side ``csrc/sparse_attention.cu:284``
                            (``(word >> (col % 32)) & 1``).
* ``tile_map_ref``          which 64-key tiles hold a set mask bit for which block of 64 query rows, and
                            which hold nothing else: the block-level emptiness test of
                            ``csrc/sparse_attention.cu:238-252`` (there per 64 query rows, after the
                            tile has been loaded) stated over the whole mask; ``tile_map_loops`` is
                            the literal loop over blocks and entries, for tiny inputs.
* ``sparse_attention_ref``  the six ops of ``python/sparse_attention.py:29-42`` (twin:
                            ``run.py:158-165``): matmul, * 1/sqrt(D), masked_fill(~mask,-inf),
                            softmax, nan_to_num(nan=0), matmul.  Tests call it in fp32 on
                            up-cast inputs exactly as ``run.py:368`` does.
* ``lse_ref``               ``python/sparse_attention.py:72-74``: logsumexp of the masked,
                            scaled scores; -inf for a row with no key to attend to.
* ``attention_f64_loops``   float64 brute force over rows (numpy), tiny inputs only.

Pins (see tests/test_oracle.py): the pack format is pinned by ``numpy.packbits`` with
``bitorder='little'`` (library routine), by the literal loop, by known answers
(single bit at column c gives ``1 << (c % 32)`` in word ``c // 32``; all-True N=8 gives
0xFF) and by popcount / round-trip invariants.  The attention function is pinned by
closed forms: all-True mask equals dense softmax attention, a one-hot mask row returns
exactly that value row, an empty mask row returns zeros, q = 0 returns the mean of the
kept value rows, joint key permutation invariance, row independence, and the float64
brute force.  ``tile_map_ref`` is pinned by the literal loops, by known answers (all-True: every
tile live and full; all-False: nothing; a single True entry: one live bit, nothing full; a ragged
last tile is full when its valid entries are all True) and by the invariant that masking out every
tile it calls empty changes nothing.  ``lse_ref`` is pinned by ``scipy.special.logsumexp`` on the kept scores.
The reference ships no golden vectors for this path, so none are checked here.
"""
from __future__ import annotations

import math

import numpy as np
import torch


# ---------------------------------------------------------------------------
# mask packing
# ---------------------------------------------------------------------------

def tile_map_shape(N: int):
    """(blocks of 64 query rows, 2, words of 32 key tiles of 64 keys) per (batch entry, head)."""
    T = (N + 63) // 64
    return (T, 2, (T + 31) // 32)


def tile_map_ref(mask) -> np.ndarray:
    """uint32 ``[B,H,T,2,TW]``: bit t%32 of word t//32 of group 0 says that the 64 x 64 block (row
    block, key tile t) of the mask holds a True entry, of group 1 that it holds nothing but True entries
    (only rows and columns below N exist).  Bits of tiles that do not exist are zero."""
    m = _as_numpy_bool(mask)
    B, H, N, _ = m.shape
    QT, _, TW = tile_map_shape(N)
    T = (N + 63) // 64
    some = np.zeros((B, H, QT * 64, T * 64), dtype=bool)
    some[:, :, :N, :N] = m
    hole = np.zeros((B, H, QT * 64, T * 64), dtype=bool)
    hole[:, :, :N, :N] = ~m
    some = some.reshape(B, H, QT, 64, T, 64).any(axis=(3, 5))
    full = ~hole.reshape(B, H, QT, 64, T, 64).any(axis=(3, 5))
    out = np.zeros((B, H, QT, 2, TW * 32), dtype=bool)
    out[:, :, :, 0, :T] = some
    out[:, :, :, 1, :T] = full
    bits = np.packbits(out, axis=-1, bitorder="little")
    return np.ascontiguousarray(bits).view("<u4").reshape(B, H, QT, 2, TW)


def tile_map_loops(mask) -> np.ndarray:
    """The same as ``tile_map_ref`` as literal loops over blocks and their entries (tiny inputs)."""
    m = _as_numpy_bool(mask)
    B, H, N, _ = m.shape
    QT, _, TW = tile_map_shape(N)
    out = np.zeros((B, H, QT, 2, TW), dtype=np.uint32)
    for b in range(B):
        for h in range(H):
            for qt in range(QT):
                for t in range((N + 63) // 64):
                    any_set, all_set = False, True
                    for i in range(64 * qt, min(N, 64 * qt + 64)):
                        for j in range(64 * t, min(N, 64 * t + 64)):
                            if m[b, h, i, j]:
                                any_set = True
                            else:
                                all_set = False
                    if any_set:
                        out[b, h, qt, 0, t // 32] |= np.uint32(1 << (t % 32))
                    if all_set:
                        out[b, h, qt, 1, t // 32] |= np.uint32(1 << (t % 32))
    return out


def n_words(N: int) -> int:
    """Words per mask row: ``csrc/sparse_attention.cu:555``."""
    return (N + 31) // 32


def _as_numpy_bool(mask) -> np.ndarray:
    if isinstance(mask, torch.Tensor):
        mask = mask.detach().cpu().numpy()
    return np.ascontiguousarray(mask).astype(bool, copy=False)


def pack_mask_ref(mask) -> np.ndarray:
    """bool ``[B,H,N,N]`` -> int32 ``[B,H,N,ceil(N/32)]``, LSB-first, pad bits 0."""
    m = _as_numpy_bool(mask)
    assert m.ndim == 4 and m.shape[2] == m.shape[3], "mask must be [B,H,N,N]"
    B, H, N, _ = m.shape
    nw = n_words(N)
    padded = np.zeros((B, H, N, nw * 32), dtype=np.uint8)
    padded[..., :N] = m
    by = np.packbits(padded, axis=-1, bitorder="little")          # [B,H,N,nw*4] bytes
    words = by.reshape(B, H, N, nw, 4).astype(np.uint32)
    w = words[..., 0] | (words[..., 1] << 8) | (words[..., 2] << 16) | (words[..., 3] << 24)
    return w.astype(np.uint32).view(np.int32)


def pack_mask_loops(mask) -> np.ndarray:
    """Literal restatement of the per-word bit loop; O(B*H*N*N) Python, tiny inputs only."""
    m = _as_numpy_bool(mask)
    B, H, N, _ = m.shape
    nw = n_words(N)
    out = np.zeros((B, H, N, nw), dtype=np.uint32)
    for b in range(B):
        for h in range(H):
            for i in range(N):
                for w in range(nw):
                    acc = 0
                    for bit in range(32):
                        col = 32 * w + bit
                        if col < N and m[b, h, i, col]:
                            acc |= 1 << bit
                    out[b, h, i, w] = acc
    return out.view(np.int32)


def unpack_mask_ref(packed, N: int) -> np.ndarray:
    """int32/uint32 ``[B,H,N,nw]`` -> bool ``[B,H,N,N]``."""
    if isinstance(packed, torch.Tensor):
        packed = packed.detach().cpu().numpy()
    p = np.ascontiguousarray(packed).view(np.uint32)
    cols = np.arange(N)
    return ((p[..., cols // 32] >> (cols % 32).astype(np.uint32)) & 1).astype(bool)


# ---------------------------------------------------------------------------
# masked attention
# ---------------------------------------------------------------------------

def sparse_attention_ref(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                         mask: torch.Tensor, scale: float | None = None) -> torch.Tensor:
    """Masked softmax attention in the dtype given (tests pass fp32 up-casts).

    ``mask`` is bool ``[B,H,N,N]`` with True = attend.  Rows with no True give zeros.
    """
    D = q.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    s = torch.matmul(q, k.transpose(-2, -1)) * scale
    s = s.masked_fill(~mask, float("-inf"))
    p = torch.softmax(s, dim=-1)
    p = torch.nan_to_num(p, nan=0.0)
    return torch.matmul(p, v)


def lse_ref(q: torch.Tensor, k: torch.Tensor, mask: torch.Tensor,
            scale: float | None = None) -> torch.Tensor:
    """log-sum-exp over kept keys of the scaled scores, fp32 ``[B,H,N]``; -inf if none kept."""
    D = q.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    s = torch.matmul(q.float(), k.float().transpose(-2, -1)) * scale
    s = s.masked_fill(~mask, float("-inf"))
    return torch.logsumexp(s, dim=-1)


def sparse_attention_bwd_ref(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: torch.Tensor,
                             dout: torch.Tensor, scale: float | None = None, delta: torch.Tensor | None = None):
    """Gradients (dq, dk, dv) of sum(out * dout) for out = sparse_attention_ref(q, k, v, mask).

    The closed form of the reference's PyTorch fallback, python/sparse_attention.py:97-111:
    attn = softmax of the masked scaled scores (empty rows -> 0); dv = attn^T dout;
    dattn = dout v^T on kept entries; ds = attn * (dattn - rowsum(dattn * attn)) * scale;
    dq = ds k; dk = ds^T q.  Computed in the dtype given (tests pass fp32 or fp64 up-casts).

    `delta` ([B,H,N,1]), if given, stands in for rowsum(dattn * attn).  The two are equal in exact
    arithmetic when delta = sum_d dout * out (rowsum_j attn_ij dout_i.v_j = dout_i . out_i); a
    backward that forms delta from an `out` already rounded to 16 bits, as every flash-style backward
    does, computes exactly this function of that rounded `out`.
    """
    D = q.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    s = torch.matmul(q, k.transpose(-2, -1)) * scale
    s = s.masked_fill(~mask, float("-inf"))
    attn = torch.nan_to_num(torch.softmax(s, dim=-1), nan=0.0)
    dv = torch.matmul(attn.transpose(-2, -1), dout)
    dattn = torch.matmul(dout, v.transpose(-2, -1)).masked_fill(~mask, 0.0)
    if delta is None:
        delta = (dattn * attn).sum(dim=-1, keepdim=True)
    ds = attn * (dattn - delta) * scale
    dq = torch.matmul(ds, k)
    dk = torch.matmul(ds.transpose(-2, -1), q)
    return dq, dk, dv


def attention_f64_loops(q, k, v, mask, scale: float | None = None):
    """Row-by-row float64 brute force; returns (out, lse) as float64 numpy arrays."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    m = _as_numpy_bool(mask)
    B, H, N, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    out = np.zeros((B, H, N, D))
    lse = np.full((B, H, N), -np.inf)
    for b in range(B):
        for h in range(H):
            for i in range(N):
                keep = np.nonzero(m[b, h, i])[0]
                if keep.size == 0:
                    continue
                s = (k[b, h, keep] @ q[b, h, i]) * scale
                mx = s.max()
                e = np.exp(s - mx)
                out[b, h, i] = (e / e.sum()) @ v[b, h, keep]
                lse[b, h, i] = mx + math.log(e.sum())
    return out, lse


# ---------------------------------------------------------------------------
# timing helper for the benchmark's CPU-baseline leg
# ---------------------------------------------------------------------------

def time_cpu_reference(q, k, v, mask, reps: int = 3):
    """Median seconds of ``sparse_attention_ref`` on host cores (1 warm-up + reps)."""
    import time
    sparse_attention_ref(q, k, v, mask)
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        sparse_attention_ref(q, k, v, mask)
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2]
