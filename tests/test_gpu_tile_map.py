"""GPU parity of the tile map (sma_tile_map, sma_pack_mask_map, and the one the forward from the
boolean mask leaves behind, sma_attn_fwd_bool_mask_map) against the oracle, bit for bit, and
of the forward that walks it (sma_attn_fwd_map): the same output and lse, bit for bit, as the forward
that visits every tile, on masks with empty blocks, empty block rows, full blocks and ragged
edges, at all head dims and both dtypes, and on the benchmark workloads at full size."""
import math

import numpy as np
import pytest
import torch

import _capi
import harness
from oracle import sma_oracle as O

pytestmark = pytest.mark.gpu


def _block_mask(B, H, N, g, keep=0.3, inner=1.0, bs=64):
    nb = (N + bs - 1) // bs
    blocks = torch.rand(B, H, nb, nb, generator=g) < keep
    m = blocks.repeat_interleave(bs, 2).repeat_interleave(bs, 3)[:, :, :N, :N].contiguous()
    if inner < 1.0:
        m &= torch.rand(B, H, N, N, generator=g) < inner
    return m


def _masks(N, g):
    yield "random 2 %", torch.rand(2, 2, N, N, generator=g) < 0.02
    yield "blocks of 64, some full", _block_mask(2, 2, N, g)
    yield "blocks of 64, thinned", _block_mask(2, 2, N, g, inner=0.5)
    yield "blocks of 32", _block_mask(2, 2, N, g, keep=0.15, bs=32)
    yield "causal", torch.tril(torch.ones(N, N, dtype=torch.bool)).expand(2, 2, N, N).contiguous()
    yield "all true", torch.ones(1, 2, N, N, dtype=torch.bool)
    yield "all false", torch.zeros(1, 2, N, N, dtype=torch.bool)
    band = (torch.arange(N)[:, None] - torch.arange(N)[None, :]).abs() < 40
    yield "band", band.expand(1, 2, N, N).contiguous()
    late = torch.zeros(1, 2, N, N, dtype=torch.bool)
    late[..., N - 1] = True                                       # only the last key: one live tile at the end
    yield "last key only", late


@pytest.mark.parametrize("N", [1, 17, 64, 65, 128, 129, 200, 256, 333, 512, 1000])
def test_tile_map_matches_the_oracle(dev, N):
    g = torch.Generator().manual_seed(N)
    for name, mask in _masks(N, g):
        packed, tm = _capi.pack_mask_map(mask.to(dev))
        torch.cuda.synchronize()
        want = O.tile_map_ref(mask).view(np.int32)
        assert np.array_equal(packed.cpu().numpy(), O.pack_mask_ref(mask)), (name, N)
        assert np.array_equal(tm.cpu().numpy(), want), (name, N)
        # the same from words that carry dirt in their pad bits
        if N % 32:
            dirty = packed.clone()
            dirty[..., -1] |= -(1 << (N % 32))
            assert np.array_equal(_capi.tile_map(dirty).cpu().numpy(), want), (name, N, "dirty pad bits")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("N", [16, 17, 63, 64, 65, 127, 128, 129, 200, 256, 333, 512, 640, 1000, 1152])
def test_forward_from_bool_mask_leaves_the_tile_map(dev, N, D, dtype):
    """The map that comes out of the one-launch forward equals the oracle's, with and without the
    packed words being asked for, and asking for it changes neither the output nor the lse."""
    g = torch.Generator().manual_seed(31 * N + D)
    q, k, v = (torch.randn(2, 2, N, D, generator=g).to(dtype).to(dev) for _ in range(3))
    for name, mask in _masks(N, g):
        B = mask.shape[0]
        qq, kk, vv = q[:B], k[:B], v[:B]
        m = mask.to(dev)
        want_out, want_lse = _capi.attn_fwd_bool_mask(qq, kk, vv, m, want_lse=True)
        out, lse, packed, tm = _capi.attn_fwd_bool_mask(qq, kk, vv, m, want_lse=True, want_packed=True, want_map=True)
        out2, tm2 = _capi.attn_fwd_bool_mask(qq, kk, vv, m, want_map=True)
        torch.cuda.synchronize()
        want = O.tile_map_ref(mask).view(np.int32)
        assert np.array_equal(tm.cpu().numpy(), want), (name, N, D, dtype)
        assert np.array_equal(tm2.cpu().numpy(), want), (name, N, D, dtype, "map only")
        assert np.array_equal(packed.cpu().numpy(), O.pack_mask_ref(mask)), (name, N, D, dtype)
        assert torch.equal(out, want_out) and torch.equal(lse, want_lse) and torch.equal(out2, want_out), (name, N, D)


def test_bool_mask_tile_map_of_a_shared_mask_and_of_odd_bytes(dev):
    g = torch.Generator().manual_seed(5)
    B, H, N = 3, 4, 300
    q, k, v = (torch.randn(B, H, N, 64, generator=g).half().to(dev) for _ in range(3))
    for shape in [(1, 1), (B, 1), (1, H), (B, H)]:
        mask = _block_mask(shape[0], shape[1], N, g, keep=0.3, inner=0.6)
        # bytes other than 0 and 1 count as set
        raw = mask.to(torch.uint8) * torch.randint(1, 256, mask.shape, generator=g, dtype=torch.int32).to(torch.uint8)
        out, packed, tm = _capi.attn_fwd_bool_mask(q, k, v, raw.to(dev).view(torch.bool), want_packed=True, want_map=True)
        torch.cuda.synchronize()
        assert np.array_equal(tm.cpu().numpy(), O.tile_map_ref(mask).view(np.int32)), shape
        assert np.array_equal(packed.cpu().numpy(), O.pack_mask_ref(mask)), shape
        assert torch.equal(_capi.tile_map(packed), tm), shape


def test_bool_mask_tile_map_with_more_than_32_key_tiles(dev):
    N = 64 * 33 + 5
    g = torch.Generator().manual_seed(11)
    mask = torch.rand(1, 2, N, N, generator=g) < 0.0005
    mask[0, 0, :64, 64 * 32: 64 * 33] = True
    mask[0, 1, 64 * 32:, :] = True                                    # full blocks up to the ragged corner
    q, k, v = (torch.randn(1, 2, N, 64, generator=g).half().to(dev) for _ in range(3))
    out, tm = _capi.attn_fwd_bool_mask(q, k, v, mask.to(dev), want_map=True)
    torch.cuda.synchronize()
    assert np.array_equal(tm.cpu().numpy(), O.tile_map_ref(mask).view(np.int32))


def test_tile_map_with_more_than_32_key_tiles(dev):
    N = 64 * 33 + 5
    g = torch.Generator().manual_seed(1)
    mask = torch.rand(1, 1, N, N, generator=g) < 0.0005
    mask[0, 0, :64, 64 * 32: 64 * 33] = True
    packed, tm = _capi.pack_mask_map(mask.to(dev))
    torch.cuda.synchronize()
    assert np.array_equal(tm.cpu().numpy(), O.tile_map_ref(mask).view(np.int32))
    q, k, v = (torch.randn(1, 1, N, 64, generator=g).half().to(dev) for _ in range(3))
    a, la = _capi.attn_fwd(q, k, v, packed, want_lse=True)
    b, lb = _capi.attn_fwd_map(q, k, v, packed, tm, want_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(a, b) and torch.equal(la, lb)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("N", [64, 200, 333, 512])
def test_forward_with_map_equals_forward_without(dev, N, D, dtype):
    g = torch.Generator().manual_seed(1000 * D + N)
    q, k, v = (torch.randn(2, 2, N, D, generator=g).to(dtype).to(dev) for _ in range(3))
    for name, mask in _masks(N, g):
        B, H = mask.shape[:2]
        packed, tm = _capi.pack_mask_map(mask.to(dev))
        qq, kk, vv = q[:B], k[:B], v[:B]
        want, want_lse = _capi.attn_fwd(qq, kk, vv, packed, want_lse=True)
        got, lse = _capi.attn_fwd_map(qq, kk, vv, packed, tm, want_lse=True)
        torch.cuda.synchronize()
        assert torch.equal(got, want) and torch.equal(lse, want_lse), (name, N, D, dtype)
        ref = O.sparse_attention_ref(qq.float().cpu(), kk.float().cpu(), vv.float().cpu(), mask)
        rtol = 1e-2 if dtype == torch.float16 else 2e-2
        assert torch.allclose(got.float().cpu(), ref, atol=1e-2, rtol=rtol), (name, N, D, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("N", [64, 200, 333, 512])
def test_backward_with_map_equals_backward_without(dev, N, D, dtype):
    g = torch.Generator().manual_seed(7000 * D + N)
    q, k, v, do = (torch.randn(2, 2, N, D, generator=g).to(dtype).to(dev) for _ in range(4))
    for name, mask in _masks(N, g):
        B, H = mask.shape[:2]
        packed, tm = _capi.pack_mask_map(mask.to(dev))
        qq, kk, vv, dd = q[:B], k[:B], v[:B], do[:B]
        out, lse = _capi.attn_fwd(qq, kk, vv, packed, want_lse=True)
        want = _capi.attn_bwd(dd, qq, kk, vv, out, lse, packed)[:3]
        got = _capi.attn_bwd_map(dd, qq, kk, vv, out, lse, packed, tm)
        torch.cuda.synchronize()
        for gname, a, b in zip(("dq", "dk", "dv"), got, want):
            assert torch.equal(a, b), (gname, name, N, D, dtype)


def test_backward_with_map_and_more_than_64_row_blocks(dev):
    N = 64 * 66 + 3
    g = torch.Generator().manual_seed(2)
    mask = torch.rand(1, 1, N, N, generator=g) < 0.0003
    mask[0, 0, 64 * 65:, :100] = True
    q, k, v, do = (torch.randn(1, 1, N, 64, generator=g).half().to(dev) for _ in range(4))
    packed, tm = _capi.pack_mask_map(mask.to(dev))
    out, lse = _capi.attn_fwd_map(q, k, v, packed, tm, want_lse=True)
    want = _capi.attn_bwd(do, q, k, v, out, lse, packed)[:3]
    got = _capi.attn_bwd_map(do, q, k, v, out, lse, packed, tm)
    torch.cuda.synchronize()
    for a, b in zip(got, want):
        assert torch.equal(a, b)


def test_shared_mask_and_strided_tensors(dev):
    g = torch.Generator().manual_seed(3)
    B, H, N = 3, 4, 300
    buf = torch.randn(B, N, 3, H, 64, generator=g).half().to(dev)
    q, k, v = (buf[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    for shape in [(1, 1), (B, 1), (1, H)]:
        mask = _block_mask(shape[0], shape[1], N, g, keep=0.3, inner=0.6)
        packed, tm = _capi.pack_mask_map(mask.to(dev))
        want = _capi.attn_fwd_strided(q, k, v, packed)
        got = _capi.attn_fwd_map_strided(q, k, v, packed, tm)
        torch.cuda.synchronize()
        assert torch.equal(got, want), shape
        ref = O.sparse_attention_ref(q.float().cpu(), k.float().cpu(), v.float().cpu(), mask.expand(B, H, N, N))
        assert torch.allclose(got.float().cpu(), ref, atol=1e-2, rtol=1e-2), shape


@pytest.mark.parametrize("name", ["C2", "C3", "C4", "C5"])
def test_benchmark_workloads_with_map(dev, name):
    w = harness.WORKLOADS[name]
    q, k, v, mask = harness.make_inputs(w, seed=42)
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    packed, tm = _capi.pack_mask_map(md)
    want, want_lse = _capi.attn_fwd(qd, kd, vd, packed, want_lse=True)
    got, lse = _capi.attn_fwd_map(qd, kd, vd, packed, tm, want_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(lse, want_lse)
    # the map itself, on the GPU: blocks with a set bit, blocks without a hole
    QT = T = (w.N + 63) // 64
    pad = torch.zeros(w.B, w.H, QT * 64, T * 64, dtype=torch.bool, device=dev)
    pad[:, :, :w.N, :w.N] = md
    some = pad.view(w.B, w.H, QT, 64, T, 64).any(dim=5).any(dim=3)
    pad.fill_(True)
    pad[:, :, :w.N, :w.N] = md
    full = pad.view(w.B, w.H, QT, 64, T, 64).all(dim=5).all(dim=3)
    bits = torch.arange(T, device=dev)
    words = tm.view(w.B, w.H, QT, 2, -1).long() & 0xFFFFFFFF
    got_some = ((words[:, :, :, 0, :].repeat_interleave(32, -1)[..., :T] >> (bits % 32)) & 1).bool()
    got_full = ((words[:, :, :, 1, :].repeat_interleave(32, -1)[..., :T] >> (bits % 32)) & 1).bool()
    assert torch.equal(got_some, some) and torch.equal(got_full, full)


def test_python_api_with_tile_map(dev):
    """tile_map() through the module: None for a mask without empty blocks; with a map, the forward
    (inference and autograd) gives bit for bit what it gives without, and gradients still flow."""
    import importlib
    sa = importlib.import_module("python.sparse_attention")
    g = torch.Generator().manual_seed(11)
    B, H, N = 2, 3, 320
    q, k, v = (torch.randn(B, H, N, 64, generator=g).half().to(dev) for _ in range(3))
    dense = (torch.rand(B, H, N, N, generator=g) < 0.3).to(dev)
    assert sa.tile_map(sa.pack_mask(dense)) is None
    mask = _block_mask(B, H, N, g, keep=0.3, inner=0.8).to(dev)
    packed = sa.pack_mask(mask)
    tm = sa.tile_map(packed)
    assert tm is not None and tuple(tm.shape) == (B, H, 5, 2, 1) and tm.dtype == torch.int32
    assert np.array_equal(tm.cpu().numpy(), O.tile_map_ref(mask.cpu()).view(np.int32))
    want = sa.sparse_attention_func(q, k, v, None, mask_packed=packed)
    got = sa.sparse_attention_func(q, k, v, None, mask_packed=packed, tile_map=tm)
    assert torch.equal(got, want)
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
    out = sa.sparse_attention(*leaves, None, mask_packed=packed, tile_map=tm)
    assert torch.equal(out.detach(), want)
    out.sum().backward()
    torch.cuda.synchronize()
    assert all(torch.isfinite(t.grad.float()).all() and t.grad.abs().sum() > 0 for t in leaves)
    plain = [t.clone().requires_grad_(True) for t in (q, k, v)]
    sa.sparse_attention(*plain, None, mask_packed=packed).sum().backward()
    torch.cuda.synchronize()
    assert all(torch.equal(a.grad, b.grad) for a, b in zip(leaves, plain))     # the backward walked the map too
    with pytest.raises(AssertionError):
        sa.sparse_attention_func(q, k, v, mask, tile_map=tm)          # a map without its packed mask
    with pytest.raises(RuntimeError):
        sa.sparse_attn_cuda.forward(q, k, v, packed, torch.empty_like(q), None, 0.125, False, tm[:, :, :4])
