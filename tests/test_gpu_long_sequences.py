"""Sequences with more than 32 and more than 64 key tiles (the tile map then has several words per
row block, and the backward's walk over row blocks several rounds): every path against the forward
and backward that visit every tile, bit for bit, and those against the oracle.  Seeded draws of
length, head dim, dtype, shared masks and mask structure."""
import random

import numpy as np
import pytest
import torch

import _capi
from oracle import sma_oracle as O

pytestmark = pytest.mark.gpu


def _mask(rng, g, Bm, Hm, N):
    kind = rng.choice(["blocks", "blocks", "sparse", "band"])
    if kind == "blocks":
        nb = -(-N // 64)
        blocks = torch.rand(Bm, Hm, nb, nb, generator=g) < rng.choice([0.02, 0.1])
        mask = blocks.repeat_interleave(64, 2).repeat_interleave(64, 3)[:, :, :N, :N].contiguous()
        if rng.random() < 0.5:
            mask &= torch.rand(Bm, Hm, N, N, generator=g) < 0.5
        return kind, mask
    if kind == "sparse":
        return kind, torch.rand(Bm, Hm, N, N, generator=g) < 0.0005
    i = torch.arange(N)
    return kind, ((i[:, None] - i[None, :]).abs() < rng.choice([10, 100])).expand(Bm, Hm, N, N).contiguous()


@pytest.mark.parametrize("seed", range(10))
def test_long_sequence_paths_agree(dev, seed):
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    N = rng.choice([2047, 2048, 2049, 2111, 2500, 3000, 4097, 4160, 4225])
    D = rng.choice([32, 64, 64, 128])
    dtype = rng.choice([torch.float16, torch.bfloat16])
    B, H = rng.choice([(1, 1), (1, 2), (2, 1)])
    Bm, Hm = rng.choice([(B, H), (1, 1)])
    kind, mask = _mask(rng, g, Bm, Hm, N)
    tag = f"seed {seed}: N{N} D{D} {dtype} B{B} H{H} mask[{Bm},{Hm}] {kind}"
    print(tag, flush=True)
    q, k, v, do = (torch.randn(B, H, N, D, generator=g).to(dtype).to(dev) for _ in range(4))
    md = mask.to(dev)
    packed, tm = _capi.pack_mask_map(md)
    assert np.array_equal(tm.cpu().numpy(), O.tile_map_ref(mask).view(np.int32)), tag
    out, lse = _capi.attn_fwd_strided(q, k, v, packed, want_lse=True)
    out_m, lse_m = _capi.attn_fwd_map_strided(q, k, v, packed, tm, want_lse=True)
    assert torch.equal(out_m, out) and torch.equal(lse_m, lse), tag
    out_b, lse_b, packed_b, tm_b = _capi.attn_fwd_bool_mask(q, k, v, md, want_lse=True, want_packed=True, want_map=True)
    assert torch.equal(out_b, out) and torch.equal(lse_b, lse), tag
    assert torch.equal(packed_b, packed) and torch.equal(tm_b, tm), tag
    grads = _capi.attn_bwd_strided(do, q, k, v, out, lse, packed)[:3]
    for name, a, b in zip(("dq", "dk", "dv"), _capi.attn_bwd_map_strided(do, q, k, v, out, lse, packed, tm), grads):
        assert torch.equal(a, b), f"{name} {tag}"
    torch.cuda.synchronize()

    full = mask.expand(B, H, N, N)
    rtol = 1e-2 if dtype == torch.float16 else 2e-2
    qf, kf, vf, dof = (t.float().cpu() for t in (q, k, v, do))
    assert torch.allclose(out.float().cpu(), O.sparse_attention_ref(qf, kf, vf, full), atol=1e-2, rtol=rtol), tag
    for name, got, want in zip(("dq", "dk", "dv"), grads, O.sparse_attention_bwd_ref(qf, kf, vf, full, dof)):
        got = got.float().cpu()
        bound = 1e-4 + 1e-2 * want.abs().max() + rtol * want.abs()
        assert ((got - want).abs() <= bound).all(), f"{name} {tag}: max err {(got - want).abs().max():.3e}"
