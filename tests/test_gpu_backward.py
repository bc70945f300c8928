"""GPU parity of sma_attn_bwd (through the C ABI) against the fp32 oracle's closed form.

The chain under test is the HIP forward (out, lse) followed by the HIP backward, on inputs whose
fp16 / bf16 values are also what the oracle sees.  Bar per gradient tensor g with reference r:
|g - r| <= 1e-4 + 1e-2 * max|r| + rtol * |r|, rtol = 1e-2 (fp16) / 2e-2 (bf16): probabilities and dS are
rounded to the 16-bit input format before the second matrix product, as in the forward.
"""
import math

import pytest
import torch

import _capi
import harness
from oracle import sma_oracle as O

pytestmark = pytest.mark.gpu

RTOL = {torch.float16: 1e-2, torch.bfloat16: 2e-2}


def _grads(q, k, v, do, mask, dev, scale=None):
    qd, kd, vd, dod = (t.to(dev) for t in (q, k, v, do))
    packed = torch.from_numpy(O.pack_mask_ref(mask)).to(dev)
    out, lse = _capi.attn_fwd(qd, kd, vd, packed, scale=scale, want_lse=True)
    dq, dk, dv, delta = _capi.attn_bwd(dod, qd, kd, vd, out, lse, packed, scale=scale)
    torch.cuda.synchronize()
    return dq.cpu(), dk.cpu(), dv.cpu(), delta.cpu(), out.cpu()


def _check(got, ref, dtype, what):
    got = got.float()
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    # 1e-4: floor for gradients that vanish identically (p = 1 rows), inputs are O(1)
    bound = 1e-4 + 1e-2 * ref.abs().max() + RTOL[dtype] * ref.abs()
    bad = (got - ref).abs() > bound
    assert not bad.any(), (f"{what}: {int(bad.sum())} elements out of tolerance, max err "
                           f"{(got - ref).abs().max():.3e} vs max|ref| {ref.abs().max():.3e}")


def _case(B, H, N, dtype, seed, keep=0.25, std=1.0):
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = ((torch.randn(B, H, N, 64, generator=g) * std).to(dtype) for _ in range(4))
    mask = torch.rand(B, H, N, N, generator=g) < keep
    return q, k, v, do, mask


def _compare(q, k, v, do, mask, dev, scale=None, tag=""):
    dq, dk, dv, delta, out = _grads(q, k, v, do, mask, dev, scale)
    rq, rk, rv = O.sparse_attention_bwd_ref(q.float(), k.float(), v.float(), mask, do.float(), scale=scale)
    _check(dq, rq, q.dtype, f"dq {tag}")
    _check(dk, rk, q.dtype, f"dk {tag}")
    _check(dv, rv, q.dtype, f"dv {tag}")
    ref_delta = (do.float() * out.float()).sum(-1)
    assert torch.allclose(delta, ref_delta, atol=1e-3 * max(1.0, float(ref_delta.abs().max())), rtol=1e-3)
    return dq, dk, dv


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N", [64, 128, 256, 512])
def test_random_masks(dev, dtype, N):
    _compare(*_case(2, 3, N, dtype, seed=N), dev, tag=f"N={N} {dtype}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N", [1, 2, 31, 33, 63, 65, 100, 127, 129, 200, 1000])
def test_ragged_lengths(dev, dtype, N):
    B, H = (1, 2) if N >= 200 else (2, 2)
    _compare(*_case(B, H, N, dtype, seed=1000 + N, keep=0.3, std=0.7), dev, tag=f"N={N} {dtype}")


def test_rows_and_keys_without_partners_get_zero_gradients(dev):
    q, k, v, do, mask = _case(1, 2, 192, torch.float16, seed=5)
    mask[:, :, 7, :] = False           # query row 7 keeps nothing
    mask[:, :, 130, :] = False
    mask[:, :, :, 9] = False           # nobody keeps key 9
    mask[:, :, :, 64:128] = False      # a whole key tile is unused
    dq, dk, dv = _compare(q, k, v, do, mask, dev, tag="empty rows/keys")
    assert (dq[:, :, 7] == 0).all() and (dq[:, :, 130] == 0).all()
    assert (dk[:, :, 9] == 0).all() and (dv[:, :, 9] == 0).all()
    assert (dk[:, :, 64:128] == 0).all() and (dv[:, :, 64:128] == 0).all()


def test_all_true_and_all_false(dev):
    q, k, v, do, mask = _case(1, 2, 160, torch.float16, seed=11)
    _compare(q, k, v, do, torch.ones_like(mask), dev, tag="all true")
    dq, dk, dv, _, _ = _grads(q, k, v, do, torch.zeros_like(mask), dev)
    assert (dq == 0).all() and (dk == 0).all() and (dv == 0).all()


def test_block_structured_and_causal_masks(dev):
    B, H, N = 1, 2, 384
    q, k, v, do, _ = _case(B, H, N, torch.float16, seed=21)
    g = torch.Generator().manual_seed(22)
    blocks = torch.rand(B, H, N // 64, N // 64, generator=g) > 0.6
    blocks |= torch.eye(N // 64, dtype=torch.bool)
    block_mask = blocks.repeat_interleave(64, -2).repeat_interleave(64, -1)
    _compare(q, k, v, do, block_mask, dev, tag="block64")
    causal = torch.tril(torch.ones(N, N, dtype=torch.bool)).expand(B, H, N, N) & (torch.rand(B, H, N, N, generator=g) > 0.5)
    causal = causal | torch.eye(N, dtype=torch.bool)
    _compare(q, k, v, do, causal, dev, tag="causal")


@pytest.mark.parametrize("scale", [1.0, 0.01, -0.125])
def test_scales(dev, scale):
    q, k, v, do, mask = _case(1, 2, 128, torch.float16, seed=31, std=0.5)
    _compare(q, k, v, do, mask, dev, scale=scale, tag=f"scale={scale}")


def test_one_hot_rows_have_closed_form(dev):
    # a row that keeps exactly one key j has p = 1 there: dq = 0, dv[j] collects dout, dk gets nothing
    N = 96
    q, k, v, do, _ = _case(1, 1, N, torch.float16, seed=41)
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(42))
    mask = torch.zeros(1, 1, N, N, dtype=torch.bool)
    mask[0, 0, torch.arange(N), perm] = True
    dq, dk, dv, _, _ = _grads(q, k, v, do, mask, dev)
    # p is 1 up to the rounding of lse and dP - delta vanishes up to the rounding of out
    assert dq.float().abs().max() < 2e-2 and dk.float().abs().max() < 2e-2
    expect = torch.zeros(N, 64)
    expect[perm] = do[0, 0].float()
    assert torch.allclose(dv[0, 0].float(), expect, atol=4e-3, rtol=4e-3)


def test_deterministic(dev):
    q, k, v, do, mask = _case(2, 2, 256, torch.bfloat16, seed=51)
    a = _grads(q, k, v, do, mask, dev)
    b = _grads(q, k, v, do, mask, dev)
    for x, y in zip(a[:3], b[:3]):
        assert torch.equal(x, y)


@pytest.mark.parametrize("name", ["C1", "C2", "C4"])
def test_baseline_workloads_subset(dev, name):
    # full-size launch; the oracle checks a seeded subset of heads
    w = harness.WORKLOADS[name]
    q, k, v, mask = harness.make_inputs(w, seed=42)
    do = (torch.randn(q.shape, generator=torch.Generator().manual_seed(43)) * 0.5).to(w.dtype)
    dq, dk, dv, _, _ = _grads(q, k, v, do, mask, dev)
    heads = [(0, 0), (w.B - 1, w.H - 1), (w.B // 2, w.H // 3)]
    for b, h in heads:
        sl = (slice(b, b + 1), slice(h, h + 1))
        rq, rk, rv = O.sparse_attention_bwd_ref(q[sl].float(), k[sl].float(), v[sl].float(), mask[sl], do[sl].float())
        _check(dq[sl], rq, w.dtype, f"{name} dq head {b},{h}")
        _check(dk[sl], rk, w.dtype, f"{name} dk head {b},{h}")
        _check(dv[sl], rv, w.dtype, f"{name} dv head {b},{h}")


def test_long_sequence(dev):
    N = 2304
    g = torch.Generator().manual_seed(77)
    q, k, v, do = ((torch.randn(1, 1, N, 64, generator=g) * 0.8).to(torch.float16) for _ in range(4))
    idx = torch.arange(N)
    mask = ((idx[:, None] - idx[None, :]).abs() < 150) & (torch.rand(N, N, generator=g) < 0.6)
    mask[:, 512:768] = False
    _compare(q, k, v, do, mask[None, None], dev, tag="N=2304")
