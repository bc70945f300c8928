"""Two corners that ordinary random inputs do not reach.

* Mask bytes other than 0 and 1 (a bool tensor made by ``view`` from uint8 data): the packer and the
  forward that reads the boolean mask itself must agree that any non-zero byte means "attend",
  through the C ABI and through the Python API, and both must agree with the oracle.
* Rows whose largest score sits at an edge of the window inside which the kernel leaves its softmax
  reference point where it is, with a thousand keys at one per cent of the largest weight: the
  probabilities of those keys are then as small as the 16-bit format gets before the second
  product, and their rounding must not show in the result.
"""
import math

import numpy as np
import pytest
import torch

import _capi
from oracle import sma_oracle as O

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, {torch.float16: 1e-2, torch.bfloat16: 2e-2}


def _odd_byte_mask(B, H, N, g):
    """uint8 [B,H,N,N] with 70 % zeros and the rest drawn from 1, 2, 0x40, 0x80, 0xFF, viewed as bool."""
    pick = torch.tensor([1, 2, 0x40, 0x80, 0xFF], dtype=torch.uint8)
    vals = pick[torch.randint(0, 5, (B, H, N, N), generator=g)]
    raw = torch.where(torch.rand(B, H, N, N, generator=g) < 0.7, torch.zeros((), dtype=torch.uint8), vals)
    return raw


@pytest.mark.parametrize("N", [64, 100, 333])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_nonzero_mask_bytes_mean_attend_in_both_forward_paths(dev, N, dtype):
    g = torch.Generator().manual_seed(N)
    B, H = 2, 3
    raw = _odd_byte_mask(B, H, N, g)
    truth = raw != 0
    q, k, v = (torch.randn(B, H, N, 64, generator=g).to(dtype) for _ in range(3))
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    md = raw.to(dev).view(torch.bool)                      # storage keeps the odd bytes
    assert md.view(torch.uint8).max().item() == 0xFF
    # C ABI: the packer, then the two forwards
    packed = _capi.pack_mask(md)
    assert np.array_equal(packed.cpu().numpy(), O.pack_mask_ref(truth))
    want, want_lse = _capi.attn_fwd(qd, kd, vd, packed, want_lse=True)
    got, lse, words = _capi.attn_fwd_bool_mask(qd, kd, vd, md, want_lse=True, want_packed=True)
    torch.cuda.synchronize()
    assert torch.equal(words, packed)
    assert torch.equal(got, want) and torch.equal(lse, want_lse)
    ref = O.sparse_attention_ref(q.float(), k.float(), v.float(), truth)
    assert torch.allclose(got.float().cpu(), ref, atol=ATOL, rtol=RTOL[dtype])
    # Python API: one launch from the boolean mask against pack_mask + forward
    import importlib
    sa = importlib.import_module("python.sparse_attention")
    one = sa.sparse_attention_func(qd, kd, vd, md)
    two = sa.sparse_attention_func(qd, kd, vd, None, mask_packed=sa.pack_mask(md))
    torch.cuda.synchronize()
    assert torch.equal(one, two) and torch.equal(one, want)
    assert torch.allclose(one.float().cpu(), ref, atol=ATOL, rtol=RTOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("top_log2", [-7.9, -8.1, 7.9, 8.1, -3.0])
def test_row_maximum_at_the_edge_of_the_window(dev, dtype, top_log2):
    """Row i: one key with score top_log2 (in units of log2 of the weight) and N - 1 keys 100 times
    lighter.  |top_log2| just below 8 leaves the reference point at 0 (the weights are 2^-7.9 and
    2^-14.5: the bottom of fp16's normal range), just above 8 moves it."""
    N, D = 1024, 64
    g = torch.Generator().manual_seed(7)
    ln2 = math.log(2.0)
    # q = 8 e_0 so that (q . k) / sqrt(D) = k[0]
    q = torch.zeros(1, 2, N, D)
    q[..., 0] = 8.0
    k = torch.zeros(1, 2, N, D)
    k[..., 0] = (top_log2 - math.log2(100.0)) * ln2
    k[:, :, 5, 0] = top_log2 * ln2
    k[..., 1:] = torch.randn(1, 2, N, D - 1, generator=g) * 0.1    # orthogonal to q: no effect on the scores
    v = torch.randn(1, 2, N, D, generator=g)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    mask = torch.rand(1, 2, N, N, generator=g) < 0.97
    mask[..., 5] = True
    packed = torch.from_numpy(O.pack_mask_ref(mask)).to(dev)
    out, lse = _capi.attn_fwd(q.to(dev), k.to(dev), v.to(dev), packed, want_lse=True)
    fused = _capi.attn_fwd_bool_mask(q.to(dev), k.to(dev), v.to(dev), mask.to(dev))
    torch.cuda.synchronize()
    ref = O.sparse_attention_ref(q.float(), k.float(), v.float(), mask)
    # the light keys together weigh about ten times the heavy one: their rounding would show
    err = (out.float().cpu() - ref).abs().max().item()
    assert torch.allclose(out.float().cpu(), ref, atol=ATOL, rtol=RTOL[dtype]), f"max err {err:.3e}"
    assert torch.equal(fused, out)
    lse_ref = O.lse_ref(q.float(), k.float(), mask)
    assert torch.allclose(lse.cpu(), lse_ref, atol=2e-2, rtol=0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("step", [3.0, 12.0, 40.0, 200.0])
def test_scores_that_climb_from_tile_to_tile(dev, dtype, step):
    """The largest score of every row grows by `step` (log2 units of the weight) with each tile of 64
    keys, so that the kernel, which takes a row maximum only when the sum of a tile's weights tells
    it to, has to notice again and again (small steps stay inside what it tolerates for a while,
    large ones overflow the exponential itself).  Some rows meet their first kept key only in a
    late tile."""
    N, D = 448, 64
    g = torch.Generator().manual_seed(int(step))
    ln2 = math.log(2.0)
    q = torch.zeros(1, 2, N, D)
    q[..., 0] = 8.0                                              # (q . k) / sqrt(D) = k[0]
    k = torch.randn(1, 2, N, D, generator=g) * 0.2
    k[..., 0] = (torch.arange(N) // 64).float().view(1, 1, N) * step * ln2 + torch.randn(1, 2, N, generator=g)
    v = torch.randn(1, 2, N, D, generator=g)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    mask = torch.rand(1, 2, N, N, generator=g) < 0.3
    late = torch.arange(N) % 5 == 0                              # these rows keep nothing before key 200
    mask[:, :, late, :200] = False
    mask[:, :, 7, :] = False                                     # and one keeps nothing at all
    packed = torch.from_numpy(O.pack_mask_ref(mask)).to(dev)
    out, lse = _capi.attn_fwd(q.to(dev), k.to(dev), v.to(dev), packed, want_lse=True)
    fused = _capi.attn_fwd_bool_mask(q.to(dev), k.to(dev), v.to(dev), mask.to(dev))
    torch.cuda.synchronize()
    ref = O.sparse_attention_ref(q.float(), k.float(), v.float(), mask)
    assert torch.isfinite(out.float()).all()
    err = (out.float().cpu() - ref).abs().max().item()
    assert torch.allclose(out.float().cpu(), ref, atol=ATOL, rtol=RTOL[dtype]), f"max err {err:.3e}"
    assert torch.equal(fused, out)
    assert (out[:, :, 7] == 0).all() and (lse[:, :, 7] == -math.inf).all()
    lse_ref = O.lse_ref(q.float(), k.float(), mask)
    fin = torch.isfinite(lse_ref)
    # q is rounded to its 16-bit format once more after the scale has been folded into it, which
    # moves every score of a row, and with it lse, by up to half a unit in the last place
    eps = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    assert torch.allclose(lse.cpu()[fin], lse_ref[fin], atol=2e-2, rtol=eps)
