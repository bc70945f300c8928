"""Seeded random configurations of the whole operator (forward and backward through the strided
C entry points) against the oracle: head dim, dtype, extents, ragged lengths, layouts, shared masks,
mask structure and scale are drawn together, so that combinations no hand-written case names are
exercised.  Same bars as the dedicated tests at the API's scale 1/sqrt(D); a scale s times larger
sharpens the softmax and multiplies the effect of the 16-bit rounding of the inputs and of the
pre-scaled q, so the absolute and relative bars are multiplied by max(1, s) as well."""
import math
import random

import pytest
import torch

import _capi
from oracle import sma_oracle as O

pytestmark = pytest.mark.gpu

RTOL = {torch.float16: 1e-2, torch.bfloat16: 2e-2}


def _layout(t, kind, dev):
    """Device tensor with the values of t ([B,H,N,D]) stored in the given layout, viewed [B,H,N,D]."""
    td = t.to(dev)
    if kind == "dense":
        return td
    if kind == "bnhd":
        return td.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    if kind == "hbnd":
        return td.permute(1, 0, 2, 3).contiguous().permute(1, 0, 2, 3)
    if kind == "padded":
        store = torch.zeros(*t.shape[:3], t.shape[3] + 24, dtype=t.dtype, device=dev)
        store[..., :t.shape[3]] = td
        return store[..., :t.shape[3]]
    raise ValueError(kind)


def _mask(rng, g, Bm, Hm, N):
    kind = rng.choice(["random", "random", "dense", "causal", "block", "sparse_rows"])
    if kind == "random":
        return torch.rand(Bm, Hm, N, N, generator=g) < rng.choice([0.05, 0.25, 0.6])
    if kind == "dense":
        return torch.ones(Bm, Hm, N, N, dtype=torch.bool)
    if kind == "causal":
        return torch.tril(torch.ones(N, N, dtype=torch.bool)).expand(Bm, Hm, N, N).contiguous()
    if kind == "block":
        nb = -(-N // 32)
        blocks = torch.rand(Bm, Hm, nb, nb, generator=g) < 0.3
        return blocks.repeat_interleave(32, 2).repeat_interleave(32, 3)[:, :, :N, :N].contiguous()
    m = torch.rand(Bm, Hm, N, N, generator=g) < 0.3
    m[:, :, torch.rand(N, generator=g) < 0.3, :] = False          # many rows keep nothing
    return m


def _draw(seed):
    """The configuration that belongs to a seed: (D, dtype, B, H, N, Bm, Hm, scale, layouts, q, k, v, do, mask)."""
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    D = rng.choice([32, 64, 128])
    dtype = rng.choice([torch.float16, torch.bfloat16])
    B, H = rng.choice([(1, 1), (1, 3), (2, 2), (3, 1)])
    N = rng.choice([1, 7, 32, 63, 64, 65, 100, 127, 128, 129, 191, 192, 250, 320, 401])
    Bm, Hm = rng.choice([(B, H), (B, H), (1, 1), (B, 1), (1, H)])
    scale = rng.choice([None, None, 0.05, 0.3, -0.2])
    layouts = [rng.choice(["dense", "bnhd", "hbnd", "padded"]) for _ in range(8)]
    q, k, v, do = [torch.randn(B, H, N, D, generator=g).to(dtype) for _ in range(4)]
    mask = _mask(rng, g, Bm, Hm, N)
    return D, dtype, B, H, N, Bm, Hm, scale, layouts, q, k, v, do, mask


# Seeds outside the 40 below on which dq misses the ordinary bar (found by drawing some 63 000 more of
# them; all have N = 7, almost all are bf16): kept as a fixed list.
FLOOR_SEEDS = [8315, 15725, 23526, 54200, 101365]


@pytest.mark.parametrize("seed", FLOOR_SEEDS)
def test_backward_accuracy_floor_is_the_rounding_of_out(dev, seed):
    """The backward forms delta = sum_d dout * out from the forward's 16-bit `out` (as every flash-style
    backward does), so dS = p * (dP - delta) carries an absolute error of about (rounding of out) x
    |dout| whatever the size of the gradient; where the true gradient nearly cancels, that floor is
    what misses the ordinary bar.  Pinned here on the seeds that miss it: against the oracle's closed
    form with delta taken from the SAME rounded `out` (`delta=`, pinned in test_oracle.py) the kernels
    meet HALF the ordinary bar for dq, dk and dv (measured: at most 0.26 of it), where against the
    delta-free form dq or dk are at 1.04 to 14.9 times the bar.  If the misses had another cause,
    changing nothing but delta in the oracle would not remove them."""
    D, dtype, B, H, N, Bm, Hm, scale, layouts, q, k, v, do, mask = _draw(seed)
    tag = f"seed {seed}: D{D} {dtype} B{B} H{H} N{N} mask[{Bm},{Hm}] scale {scale}"
    print(tag, flush=True)
    qd, kd, vd, dod = (t.to(dev) for t in (q, k, v, do))
    packed = _capi.pack_mask(mask.to(dev))
    out, lse = _capi.attn_fwd_strided(qd, kd, vd, packed, scale=scale, want_lse=True)
    dq, dk, dv, _ = _capi.attn_bwd_strided(dod, qd, kd, vd, out, lse, packed, scale=scale)
    torch.cuda.synchronize()
    full = mask.expand(B, H, N, N)
    sharp = max(1.0, abs(scale) * math.sqrt(D)) if scale is not None else 1.0
    delta = (do.float() * out.float().cpu()).sum(dim=-1, keepdim=True)
    refs = O.sparse_attention_bwd_ref(q.float(), k.float(), v.float(), full, do.float(), scale=scale, delta=delta)
    plain = O.sparse_attention_bwd_ref(q.float(), k.float(), v.float(), full, do.float(), scale=scale)
    worst_plain = 0.0
    for name, got, want, want_plain in zip(("dq", "dk", "dv"), (dq, dk, dv), refs, plain):
        got = got.float().cpu()
        bound = 1e-4 + sharp * (1e-2 * want.abs().max() + RTOL[dtype] * want.abs())
        ratio = ((got - want).abs() / bound).max().item()
        assert ratio <= 0.5, f"{name} {tag}: {ratio:.2f} of the ordinary bar with delta from the rounded out"
        bound_plain = 1e-4 + sharp * (1e-2 * want_plain.abs().max() + RTOL[dtype] * want_plain.abs())
        worst_plain = max(worst_plain, ((got - want_plain).abs() / bound_plain).max().item())
    print(f"  against the delta-free form: {worst_plain:.2f} of the ordinary bar", flush=True)


@pytest.mark.parametrize("seed", range(40))
def test_random_configuration(dev, seed):
    D, dtype, B, H, N, Bm, Hm, scale, layouts, q, k, v, do, mask = _draw(seed)
    tag = f"seed {seed}: D{D} {dtype} B{B} H{H} N{N} mask[{Bm},{Hm}] scale {scale} layouts {layouts}"
    print(tag, flush=True)

    qd, kd, vd, dod = (_layout(t, l, dev) for t, l in zip((q, k, v, do), layouts[:4]))
    packed = _capi.pack_mask(mask.to(dev))
    assert torch.equal(packed.cpu(), torch.from_numpy(O.pack_mask_ref(mask)))
    out_view = _layout(torch.full((B, H, N, D), float("nan"), dtype=dtype), layouts[4], dev)
    out, lse = _capi.attn_fwd_strided(qd, kd, vd, packed, out=out_view, scale=scale, want_lse=True)
    grads = tuple(_layout(torch.full((B, H, N, D), float("nan"), dtype=dtype), l, dev) for l in layouts[5:8])
    dq, dk, dv, _ = _capi.attn_bwd_strided(dod, qd, kd, vd, out, lse, packed, grads=grads, scale=scale)
    torch.cuda.synchronize()

    # the same through the tile map, and (where it applies) through the one launch that reads the
    # boolean mask and leaves packed words and map behind: bit for bit what was computed above
    tm = _capi.tile_map(packed)
    assert torch.equal(tm.cpu(), torch.from_numpy(O.tile_map_ref(mask).view("int32"))), tag
    out_m, lse_m = _capi.attn_fwd_map_strided(qd, kd, vd, packed, tm, scale=scale, want_lse=True)
    assert torch.equal(out_m, out.contiguous()) and torch.equal(lse_m, lse), tag
    got_m = _capi.attn_bwd_map_strided(dod, qd, kd, vd, out, lse, packed, tm, scale=scale)
    for name, a, b_ in zip(("dq", "dk", "dv"), got_m, (dq, dk, dv)):
        assert torch.equal(a, b_.contiguous()), f"{name} with map {tag}"
    if N >= 16:
        qc, kc, vc = (t.contiguous() for t in (qd, kd, vd))
        out_b, lse_b, packed_b, tm_b = _capi.attn_fwd_bool_mask(qc, kc, vc, mask.to(dev), scale=scale, want_lse=True,
                                                                want_packed=True, want_map=True)
        assert torch.equal(packed_b, packed) and torch.equal(tm_b, tm), tag
        assert torch.equal(out_b, out.contiguous()) and torch.equal(lse_b, lse), tag
    torch.cuda.synchronize()

    full = mask.expand(B, H, N, N)
    sharp = max(1.0, abs(scale) * math.sqrt(D)) if scale is not None else 1.0
    ref = O.sparse_attention_ref(q.float(), k.float(), v.float(), full, scale=scale)
    assert torch.allclose(out.float().cpu(), ref, atol=1e-2 * sharp, rtol=RTOL[dtype] * sharp), tag
    empty = ~full.any(dim=-1)
    assert (out.cpu()[empty] == 0).all() and (lse.cpu()[empty] == -math.inf).all(), tag
    refs = O.sparse_attention_bwd_ref(q.float(), k.float(), v.float(), full, do.float(), scale=scale)
    for name, got, want in zip(("dq", "dk", "dv"), (dq, dk, dv), refs):
        got = got.float().cpu()
        assert torch.isfinite(got).all(), f"{name} {tag}"
        bound = 1e-4 + sharp * (1e-2 * want.abs().max() + RTOL[dtype] * want.abs())
        assert ((got - want).abs() <= bound).all(), f"{name} {tag}: max err {(got - want).abs().max():.3e}"
