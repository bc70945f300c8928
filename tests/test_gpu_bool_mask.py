"""GPU parity of sma_attn_fwd_bool_mask (the forward that reads the boolean mask itself) against
sma_pack_mask + sma_attn_fwd: the arithmetic is the same kernel, only the source of the mask words
differs, so the results must agree bit for bit; the pair is in turn checked against the oracle by
the other test files (and once more here)."""
import math

import pytest
import torch

import _capi
from oracle import sma_oracle as O

pytestmark = pytest.mark.gpu


def _inputs(B, H, N, D, dtype, seed, keep=0.25):
    g = torch.Generator().manual_seed(seed)
    q, k, v = [torch.randn(B, H, N, D, generator=g).to(dtype) for _ in range(3)]
    mask = torch.rand(B, H, N, N, generator=g) < keep
    return q, k, v, mask


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("N", [16, 17, 48, 64, 65, 79, 80, 100, 128, 144, 192, 250, 256, 400, 511, 512, 1000, 1001, 1008, 1024])
def test_equals_pack_then_attention(dev, dtype, D, N):
    B, H = 2, 3
    q, k, v, mask = _inputs(B, H, N, D, dtype, 300 + N + D)
    mask[0, 1, 5, :] = False                       # a row that keeps nothing
    mask[1, 2, :, N - 1] = False                   # a key nobody keeps
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    want, want_lse = _capi.attn_fwd(qd, kd, vd, _capi.pack_mask(md), want_lse=True)
    got, lse = _capi.attn_fwd_bool_mask(qd, kd, vd, md, want_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(lse, want_lse)
    ref = O.sparse_attention_ref(q.float(), k.float(), v.float(), mask)
    assert torch.allclose(got.float().cpu(), ref, atol=1e-2, rtol=2e-2)
    assert (got[0, 1, 5] == 0).all() and lse[0, 1, 5].item() == -math.inf


@pytest.mark.parametrize("kind", ["all_true", "all_false", "diag", "block64", "causal", "columns"])
def test_structured_masks(dev, kind):
    B, H, N, D, dtype = 1, 2, 320, 64, torch.float16
    q, k, v, _ = _inputs(B, H, N, D, dtype, 41)
    if kind == "all_true":
        mask = torch.ones(B, H, N, N, dtype=torch.bool)
    elif kind == "all_false":
        mask = torch.zeros(B, H, N, N, dtype=torch.bool)
    elif kind == "diag":
        mask = torch.eye(N, dtype=torch.bool).expand(B, H, N, N).contiguous()
    elif kind == "block64":
        g = torch.Generator().manual_seed(3)
        blocks = torch.rand(B, H, N // 64, N // 64, generator=g) < 0.3
        mask = blocks.repeat_interleave(64, dim=2).repeat_interleave(64, dim=3)
    elif kind == "causal":
        mask = torch.tril(torch.ones(N, N, dtype=torch.bool)).expand(B, H, N, N).contiguous()
    else:                                           # every key position in turn, one per row: bit order
        mask = torch.zeros(B, H, N, N, dtype=torch.bool)
        idx = torch.arange(N)
        mask[:, :, idx, (idx * 7 + 3) % N] = True
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    want = _capi.attn_fwd(qd, kd, vd, _capi.pack_mask(md))
    got = _capi.attn_fwd_bool_mask(qd, kd, vd, md)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    if kind == "columns":                           # one kept key per row: out is that row of v, exactly
        idx = torch.arange(N)
        assert torch.equal(got.cpu(), v[:, :, (idx * 7 + 3) % N])


@pytest.mark.parametrize("shape", ["11", "B1", "1H"])
def test_shared_masks(dev, shape):
    B, H, N, D = 3, 4, 128, 64
    Bm, Hm = (1 if shape[0] == "1" else B), (1 if shape[1] == "1" else H)
    q, k, v, _ = _inputs(B, H, N, D, torch.bfloat16, 52)
    g = torch.Generator().manual_seed(6)
    small = torch.rand(Bm, Hm, N, N, generator=g) < 0.3
    qd, kd, vd = (t.to(dev) for t in (q, k, v))
    want = _capi.attn_fwd(qd, kd, vd, _capi.pack_mask(small.expand(B, H, N, N).contiguous().to(dev)))
    got = _capi.attn_fwd_bool_mask(qd, kd, vd, small.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_scales_many_heads_and_long_rows(dev):
    q, k, v, mask = _inputs(1, 2, 256, 64, torch.float16, 61)
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    packed = _capi.pack_mask(md)
    for scale in (1.0, -0.3, 0.01):                 # scale 1 takes the post-multiplied exponent
        assert torch.equal(_capi.attn_fwd_bool_mask(qd, kd, vd, md, scale=scale),
                           _capi.attn_fwd(qd, kd, vd, packed, scale=scale))
    q, k, v, mask = _inputs(8, 40, 256, 64, torch.float16, 62)      # several rounds of work-groups
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    assert torch.equal(_capi.attn_fwd_bool_mask(qd, kd, vd, md), _capi.attn_fwd(qd, kd, vd, _capi.pack_mask(md)))
    q, k, v, mask = _inputs(1, 2, 2112, 64, torch.float16, 63, keep=0.1)
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    assert torch.equal(_capi.attn_fwd_bool_mask(qd, kd, vd, md), _capi.attn_fwd(qd, kd, vd, _capi.pack_mask(md)))
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [32, 64])
@pytest.mark.parametrize("N", [128, 384, 640, 1152, 2048])
def test_two_tiles_of_mask_bytes_per_request(dev, dtype, D, N):
    """With N a multiple of 128 and head dims up to 64 the kernel requests the mask bytes of two key
    tiles at once (whole 128-byte lines), unless the grid is a single round of work-groups in step
    (512 < B*H*ceil(N/128) <= 768 on this part, e.g. the headline workload, which
    test_benchmark_workloads_at_full_size runs).  Same arithmetic, so out and lse must be
    those of pack + attention bit for bit: with a mask per head, with one mask for all, with bytes
    other than 0 and 1, at an odd byte address, for a scale that takes the post-multiplied exponent,
    and through strided q, k, v, out.  (N = 1152 has an odd number of pairs' worth of 64-key tiles
    beyond a power of two; 2048 runs several rounds of work-groups.)"""
    B, H = 2, 3
    q, k, v, mask = _inputs(B, H, N, D, dtype, 900 + N + D, keep=0.2)
    mask[1, 0, 7, :] = False                       # a row that keeps nothing
    mask[0, 2, :, 0:128] = False                   # a pair of key tiles nobody in this head keeps
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    packed = _capi.pack_mask(md)
    for scale in (1.0, None):
        want, want_lse = _capi.attn_fwd(qd, kd, vd, packed, scale=scale, want_lse=True)
        got, lse = _capi.attn_fwd_bool_mask(qd, kd, vd, md, scale=scale, want_lse=True)
        torch.cuda.synchronize()
        assert torch.equal(got, want) and torch.equal(lse, want_lse), scale
    ref = O.sparse_attention_ref(q.float(), k.float(), v.float(), mask)
    assert torch.allclose(got.float().cpu(), ref, atol=1e-2, rtol=2e-2)
    assert (got[1, 0, 7] == 0).all() and lse[1, 0, 7].item() == -math.inf
    # one mask for every batch entry and head
    one = mask[:1, :1].contiguous().to(dev)
    want = _capi.attn_fwd(qd, kd, vd, _capi.pack_mask(one.expand(B, H, N, N).contiguous()))
    assert torch.equal(_capi.attn_fwd_bool_mask(qd, kd, vd, one), want)
    # bytes other than 0 and 1, at an odd address
    raw = torch.zeros(3 + mask.numel(), dtype=torch.uint8, device=dev)
    g = torch.Generator().manual_seed(N)
    values = torch.randint(1, 256, mask.shape, generator=g, dtype=torch.int32).to(torch.uint8)
    raw[3:].view(B, H, N, N).copy_((values * mask).to(dev))
    odd = raw[3:].view(B, H, N, N).view(torch.bool)
    assert odd.data_ptr() % 16 == (raw.data_ptr() + 3) % 16
    want, want_lse = _capi.attn_fwd(qd, kd, vd, packed, want_lse=True)
    got, lse = _capi.attn_fwd_bool_mask(qd, kd, vd, odd, want_lse=True)
    assert torch.equal(got, want) and torch.equal(lse, want_lse)
    # with the by-products asked for (what the training forward does): words and tile map as the packer makes them
    got, lse, words, tmap = _capi.attn_fwd_bool_mask(qd, kd, vd, md, want_lse=True, want_packed=True, want_map=True)
    want_words, want_map = _capi.pack_mask_map(md)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(lse, want_lse)
    assert torch.equal(words, want_words) and torch.equal(tmap, want_map)
    # strided q, k, v, out ([B,N,H,D] buffers)
    qs, ks, vs = (t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3) for t in (qd, kd, vd))
    out_view = torch.empty(B, N, H, D, dtype=dtype, device=dev).permute(0, 2, 1, 3)
    got = _capi.attn_fwd_bool_mask_strided(qs, ks, vs, md, out=out_view)
    torch.cuda.synchronize()
    assert torch.equal((got[0] if isinstance(got, tuple) else got).contiguous(), want)


def test_limits_are_reported(dev):
    q, k, v, mask = _inputs(1, 1, 15, 64, torch.float16, 70)                   # a row shorter than one 16-byte copy
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    assert _capi.attn_fwd_bool_mask(qd, kd, vd, md, expect=_capi.SMA_ERR_BAD_SHAPE) == _capi.SMA_ERR_BAD_SHAPE
    q, k, v, mask = _inputs(1, 1, 64, 96, torch.float16, 71)
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    assert _capi.attn_fwd_bool_mask(qd, kd, vd, md, expect=_capi.SMA_ERR_HEAD_DIM) == _capi.SMA_ERR_HEAD_DIM


@pytest.mark.parametrize("offset", [1, 2, 4, 8, 13])
def test_mask_at_any_byte_address(dev, offset):
    """The mask need not start on a 16-byte boundary, and it may end with its allocation's last
    byte: no copy reaches beyond it (every 16-byte copy that would is moved back)."""
    B, H, N, D = 2, 2, 200, 64
    q, k, v, mask = _inputs(B, H, N, D, torch.float16, 600 + offset)
    qd, kd, vd = (t.to(dev) for t in (q, k, v))
    buf = torch.ones(offset + mask.numel(), dtype=torch.bool, device=dev)
    md = buf[offset:].view(B, H, N, N)
    md.copy_(mask)
    assert md.data_ptr() % 16 == offset % 16 and md.is_contiguous()
    packed = _capi.pack_mask(md)
    assert torch.equal(packed.cpu(), torch.from_numpy(O.pack_mask_ref(mask)))
    got, lse, words = _capi.attn_fwd_bool_mask(qd, kd, vd, md, want_lse=True, want_packed=True)
    want, want_lse = _capi.attn_fwd(qd, kd, vd, packed, want_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(words, packed) and torch.equal(got, want) and torch.equal(lse, want_lse)


@pytest.mark.parametrize("shape", ["BH", "11", "B1", "1H"])
@pytest.mark.parametrize("N", [16, 35, 80, 128, 250, 400, 640, 1001, 1008, 1152])
def test_packed_words_are_left_behind(dev, N, shape):
    """packed_out receives exactly what sma_pack_mask writes (every word, pad bits zero), so that a
    backward can follow without a packing pass; shared masks are written once."""
    B, H, D = 2, 3, 64
    Bm, Hm = (1 if shape[0] == "1" else B), (1 if shape[1] == "1" else H)
    q, k, v, _ = _inputs(B, H, N, D, torch.float16, 80 + N)
    g = torch.Generator().manual_seed(N)
    mask = torch.rand(Bm, Hm, N, N, generator=g) < 0.3
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    out, lse, packed = _capi.attn_fwd_bool_mask(qd, kd, vd, md, want_lse=True, want_packed=True)
    torch.cuda.synchronize()
    assert torch.equal(packed.cpu(), torch.from_numpy(O.pack_mask_ref(mask)))
    want, want_lse = _capi.attn_fwd_strided(qd, kd, vd, packed, want_lse=True)
    assert torch.equal(out, want) and torch.equal(lse, want_lse)


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_benchmark_workloads_at_full_size(dev, name):
    """The five benchmark workloads, whole: identical to pack + attention
    (which the other files hold against the oracle at these sizes), words left behind identical to
    the packer's, and the oracle-free property that V = 1 gives exactly 1 on every non-empty row."""
    import harness
    w = harness.WORKLOADS[name]
    q, k, v, mask = harness.make_inputs(w, seed=42)
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    packed = _capi.pack_mask(md)
    want = _capi.attn_fwd(qd, kd, vd, packed)
    got, words = _capi.attn_fwd_bool_mask(qd, kd, vd, md, want_packed=True)
    assert torch.equal(got, want) and torch.equal(words, packed)
    ones = _capi.attn_fwd_bool_mask(qd, kd, torch.ones_like(vd), md)
    nonempty = md.any(dim=-1)
    assert (ones[nonempty] == 1).all() and (ones[~nonempty] == 0).all()
    torch.cuda.synchronize()


def test_every_length_up_to_512(dev):
    """All lengths from 16 to 512 (every size and alignment of last tile and of the rows' first
    bytes, with and without a second word, one to four work-groups per head), words included; one
    process, one launch pair per length."""
    for N in range(16, 513):
        q, k, v, mask = _inputs(1, 2, N, 64, torch.float16, 5000 + N, keep=0.2)
        qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
        packed = _capi.pack_mask(md)
        got, words = _capi.attn_fwd_bool_mask(qd, kd, vd, md, want_packed=True)
        assert torch.equal(words, packed), N
        assert torch.equal(got, _capi.attn_fwd(qd, kd, vd, packed)), N
        if N % 37 == 0:
            assert torch.equal(packed.cpu(), torch.from_numpy(O.pack_mask_ref(mask))), N
    torch.cuda.synchronize()


def test_mask_larger_than_4_GiB(dev):
    """Ten (b,h) masks of 21000 x 21000 bytes: 4.41 GB, so the offsets of the later ones need more than
    32 bits (those inside one mask stay below 2^31).  Identical to pack + attention everywhere; rows
    of the first and the last (b,h) against a float32 formulation with PyTorch ops on the device."""
    B, H, N, D = 2, 5, 21000, 64
    g = torch.Generator(device=dev).manual_seed(77)
    qd, kd, vd = [torch.randn(B, H, N, D, generator=g, device=dev).half() for _ in range(3)]
    md = torch.empty(B, H, N, N, dtype=torch.bool, device=dev)
    for b in range(B):
        for h in range(H):
            md[b, h] = torch.rand(N, N, generator=g, device=dev) < 0.05
    assert md.numel() > 2**32
    md[1, 4, N - 1, :] = False
    packed = _capi.pack_mask(md)
    want = _capi.attn_fwd(qd, kd, vd, packed)
    got, words = _capi.attn_fwd_bool_mask(qd, kd, vd, md, want_packed=True)
    torch.cuda.synchronize()
    assert torch.equal(words, packed) and torch.equal(got, want)
    rows = torch.tensor([0, 1, 127, 128, 10000, N - 2, N - 1], device=dev)
    for b, h in ((0, 0), (1, 4)):
        s = (qd[b, h, rows].float() @ kd[b, h].float().T) / math.sqrt(D)
        s = s.masked_fill(~md[b, h, rows], -math.inf)
        p = torch.softmax(s, dim=-1).nan_to_num(0.0)
        ref = p @ vd[b, h].float()
        assert torch.allclose(got[b, h, rows].float(), ref, atol=1e-2, rtol=1e-2), (b, h)
    assert (got[1, 4, N - 1] == 0).all()
