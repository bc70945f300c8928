"""GPU parity of the strided entry points (sma_attn_fwd_strided / sma_attn_bwd_strided /
sma_attn_fwd_bool_mask_strided): tensors
that are views with explicit strides, and packed masks shared between batch entries and heads.

The reference reserves strides in its parameter block (csrc/sparse_attention.h:30-33) without ever
reading them, so its own tests hold nothing for this; the bar is that a strided call gives exactly
(bit for bit) what the dense entry point gives on a contiguous copy of the same data, and that the
dense result meets the oracle (checked here once more on the strided result).
"""
import pytest
import torch

import _capi
from oracle import sma_oracle as O

pytestmark = pytest.mark.gpu


def _inputs(B, H, N, dtype, seed, keep=0.3, n_tensors=3):
    g = torch.Generator().manual_seed(seed)
    ts = [torch.randn(B, H, N, 64, generator=g).to(dtype) for _ in range(n_tensors)]
    mask = torch.rand(B, H, N, N, generator=g) < keep
    return ts, mask


def _bnhd(t):
    """The same values stored as [B, N, H, D] (the layout a fused projection produces), viewed [B, H, N, D]."""
    return t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N", [64, 200, 512])
def test_forward_on_bnhd_views_equals_dense(dev, dtype, N):
    B, H = 2, 3
    (q, k, v), mask = _inputs(B, H, N, dtype, 100 + N)
    qd, kd, vd = (t.to(dev) for t in (q, k, v))
    packed = torch.from_numpy(O.pack_mask_ref(mask)).to(dev)
    want, want_lse = _capi.attn_fwd(qd, kd, vd, packed, want_lse=True)
    qs, ks, vs = (_bnhd(t) for t in (qd, kd, vd))
    assert not qs.is_contiguous()
    out_store = torch.full((B, N, H, 64), float("nan"), dtype=dtype, device=dev)
    got, lse = _capi.attn_fwd_strided(qs, ks, vs, packed, out=out_store.permute(0, 2, 1, 3), want_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(lse, want_lse)
    ref = O.sparse_attention_ref(q.float(), k.float(), v.float(), mask)
    assert torch.allclose(got.float().cpu(), ref, atol=1e-2, rtol=2e-2)


def test_forward_on_slices_of_a_fused_qkv_buffer(dev):
    """q, k, v as slices of one [B, N, 3, H, D] buffer; the gaps between rows must stay untouched."""
    B, H, N, dtype = 2, 4, 192, torch.float16
    (q, k, v), mask = _inputs(B, H, N, dtype, 7)
    qkv = torch.stack([q, k, v], dim=0).permute(1, 3, 0, 2, 4).contiguous().to(dev)   # [B,N,3,H,D]
    qs, ks, vs = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    packed = torch.from_numpy(O.pack_mask_ref(mask)).to(dev)
    # output rows padded to 96 elements: the 32 elements after each row are not the kernel's
    store = torch.full((B, H, N, 96), 7.0, dtype=dtype, device=dev)
    got = _capi.attn_fwd_strided(qs, ks, vs, packed, out=store[..., :64])
    want = _capi.attn_fwd(q.to(dev), k.to(dev), v.to(dev), packed)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert (store[..., 64:] == 7.0).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("N", [16, 100, 257, 512])
def test_forward_from_the_bool_mask_on_strided_views_equals_dense(dev, dtype, D, N):
    """The one launch that reads the boolean mask, on a [B,N,H,D] buffer viewed as [B,H,N,D] and on
    slices of a fused qkv buffer with padded output rows: bit for bit what the dense entry point gives
    on contiguous copies (output, lse, the packed words and the tile map it leaves behind), gaps
    between rows untouched."""
    B, H = 2, 3
    g = torch.Generator().manual_seed(1000 * D + N)
    q, k, v = (torch.randn(B, H, N, D, generator=g).to(dtype) for _ in range(3))
    mask = torch.rand(B, H, N, N, generator=g) < 0.3
    mask[:, :, :, N // 2:] &= torch.rand(B, H, 1, 1, generator=g) < 0.5          # some heads keep half the keys only
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    want, want_lse, want_packed, want_map = _capi.attn_fwd_bool_mask(qd, kd, vd, md, want_lse=True, want_packed=True,
                                                                     want_map=True)
    # [B, N, H, D] views, output stored [B, N, H, D] too
    qs, ks, vs = (_bnhd(t) for t in (qd, kd, vd))
    out_store = torch.full((B, N, H, D), float("nan"), dtype=dtype, device=dev)
    got, lse, packed, tm = _capi.attn_fwd_bool_mask_strided(qs, ks, vs, md, out=out_store.permute(0, 2, 1, 3),
                                                            want_lse=True, want_packed=True, want_map=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(lse, want_lse)
    assert torch.equal(packed, want_packed) and torch.equal(tm, want_map)
    # slices of one [B, N, 3, H, D] buffer, output rows padded by 32 elements
    qkv = torch.stack([qd, kd, vd], dim=0).permute(1, 3, 0, 2, 4).contiguous()
    qs, ks, vs = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    store = torch.full((B, H, N, D + 32), 7.0, dtype=dtype, device=dev)
    got = _capi.attn_fwd_bool_mask_strided(qs, ks, vs, md, out=store[..., :D])
    torch.cuda.synchronize()
    assert torch.equal(got, want) and (store[..., D:] == 7.0).all()
    ref = O.sparse_attention_ref(q.float(), k.float(), v.float(), mask)
    assert torch.allclose(got.float().cpu(), ref, atol=1e-2, rtol=2e-2)


def test_python_api_takes_strided_views_through_the_one_launch_path(dev):
    """sparse_attention_func / sparse_attention on [B,N,H,D] views: the module says the one-launch
    forward applies, and results (and gradients) are those of contiguous copies, bit for bit."""
    import importlib
    sa = importlib.import_module("python.sparse_attention")
    B, H, N = 2, 4, 200
    g = torch.Generator().manual_seed(77)
    q, k, v, do = (torch.randn(B, N, H, 64, generator=g).half().to(dev).permute(0, 2, 1, 3) for _ in range(4))
    mask = (torch.rand(B, H, N, N, generator=g) < 0.3).to(dev)
    assert not q.is_contiguous() and sa.sparse_attn_cuda.bool_mask_supported(q, k, v, mask)
    want = sa.sparse_attention_func(q.contiguous(), k.contiguous(), v.contiguous(), mask)
    assert torch.equal(sa.sparse_attention_func(q, k, v, mask), want)
    grads = []
    for conv in (lambda t: t, lambda t: t.contiguous()):
        leaves = [conv(t).clone().requires_grad_(True) for t in (q, k, v)]
        out = sa.sparse_attention(*leaves, mask)
        out.backward(conv(do))
        grads.append([out.detach()] + [t.grad for t in leaves])
    for a, b in zip(*grads):
        assert torch.equal(a, b)


@pytest.mark.parametrize("shape", ["11", "B1", "1H"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_shared_masks_forward_and_backward(dev, shape, dtype):
    """A mask [1,1,N,N], [B,1,N,N] or [1,H,N,N] is packed once and read by every batch entry / head;
    results equal those with the mask expanded to [B,H,N,N]."""
    B, H, N = 3, 4, 160
    Bm, Hm = (1 if shape[0] == "1" else B), (1 if shape[1] == "1" else H)
    (q, k, v, do), _ = _inputs(B, H, N, dtype, 31, n_tensors=4)
    g = torch.Generator().manual_seed(5)
    small = torch.rand(Bm, Hm, N, N, generator=g) < 0.3
    small[..., 7, :] = False                                   # one row that keeps nothing
    full = small.expand(B, H, N, N).contiguous()
    qd, kd, vd, dod = (t.to(dev) for t in (q, k, v, do))
    p_small = _capi.pack_mask(small.to(dev))
    p_full = _capi.pack_mask(full.to(dev))
    assert p_small.shape == (Bm, Hm, N, (N + 31) // 32)
    want, want_lse = _capi.attn_fwd(qd, kd, vd, p_full, want_lse=True)
    got, lse = _capi.attn_fwd_strided(qd, kd, vd, p_small, want_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(lse, want_lse)
    assert (got[:, :, 7] == 0).all()
    wq, wk, wv, wdelta = _capi.attn_bwd(dod, qd, kd, vd, want, want_lse, p_full)
    gq, gk, gv, gdelta = _capi.attn_bwd_strided(dod, qd, kd, vd, got, lse, p_small)
    torch.cuda.synchronize()
    assert torch.equal(gq, wq) and torch.equal(gk, wk) and torch.equal(gv, wv) and torch.equal(gdelta, wdelta)
    rq, rk, rv = O.sparse_attention_bwd_ref(q.float(), k.float(), v.float(), full, do.float())
    for got_g, ref_g in ((gq, rq), (gk, rk), (gv, rv)):
        bound = 1e-4 + 1e-2 * ref_g.abs().max() + 2e-2 * ref_g.abs()
        assert ((got_g.float().cpu() - ref_g).abs() <= bound).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N", [96, 333])
def test_backward_on_strided_views_equals_dense(dev, dtype, N):
    B, H = 2, 3
    (q, k, v, do), mask = _inputs(B, H, N, dtype, 900 + N, n_tensors=4)
    qd, kd, vd, dod = (t.to(dev) for t in (q, k, v, do))
    packed = torch.from_numpy(O.pack_mask_ref(mask)).to(dev)
    out, lse = _capi.attn_fwd(qd, kd, vd, packed, want_lse=True)
    want = _capi.attn_bwd(dod, qd, kd, vd, out, lse, packed)
    # every tensor in a different layout: [B,N,H,D] views, a padded-row view, a head-major view
    pad = torch.zeros(B, H, N, 128, dtype=dtype, device=dev)
    pad[..., :64] = dod
    gstore = [torch.full((B, N, H, 64), float("nan"), dtype=dtype, device=dev) for _ in range(2)]
    gk_store = torch.full((H, B, N, 64), float("nan"), dtype=dtype, device=dev)
    grads = (gstore[0].permute(0, 2, 1, 3), gk_store.permute(1, 0, 2, 3), gstore[1].permute(0, 2, 1, 3))
    got = _capi.attn_bwd_strided(pad[..., :64], _bnhd(qd), _bnhd(kd), _bnhd(vd), _bnhd(out), lse, packed, grads=grads)
    torch.cuda.synchronize()
    for g_, w_ in zip(got, want):
        assert torch.equal(g_, w_)


def test_stride_validation(dev):
    lib = _capi.load()
    B, H, N = 1, 2, 64
    q = torch.zeros(B, H, N, 64, dtype=torch.float16, device=dev)
    packed = torch.zeros(B, H, N, 2, dtype=torch.int32, device=dev)
    ok = _capi.SmaTensor.of(q)

    def call(tq=ok, msb=H * N * 2, msh=N * 2):
        return lib.sma_attn_fwd_strided(tq, ok, ok, packed.data_ptr(), msb, msh, ok, None, B, H, N, 64, 0.125,
                                        _capi.SMA_DTYPE_F16, None)

    assert call() == _capi.SMA_OK
    assert call(tq=_capi.SmaTensor(q.data_ptr(), H * N * 64, N * 64, 60)) == _capi.SMA_ERR_STRIDE     # rows misaligned
    assert call(tq=_capi.SmaTensor(q.data_ptr(), -8, N * 64, 64)) == _capi.SMA_ERR_STRIDE
    assert call(tq=_capi.SmaTensor(q.data_ptr(), 0, 0, 1 << 26)) == _capi.SMA_ERR_STRIDE              # slab beyond 2 GiB
    assert call(tq=_capi.SmaTensor(None, 0, 0, 64)) == _capi.SMA_ERR_NULL_POINTER
    assert call(msb=-1) == _capi.SMA_ERR_STRIDE
    torch.cuda.synchronize()
