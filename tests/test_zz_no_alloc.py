"""sma_attn_bwd_static_ws (the backward whose workspace is a fixed array inside the library, for
callers that cannot allocate) against sma_attn_bwd with a caller-owned workspace: bit for bit the
same gradients, on two calls in a row of which the second is smaller (so it runs over what the
first left in the shared array), in both dtypes; and the size limit answers with an error."""
import ctypes

import pytest
import torch

import _capi
from oracle import sma_oracle as O

pytestmark = pytest.mark.gpu


def _problem(B, H, N, D, dtype, seed, dev):
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = (torch.randn(B, H, N, D, generator=g).to(dtype).to(dev) for _ in range(4))
    mask = torch.rand(B, H, N, N, generator=g) < 0.3
    mask[:, :, min(3, N - 1), :] = False                 # a row that keeps no key
    packed = torch.from_numpy(O.pack_mask_ref(mask)).to(dev)
    out, lse = _capi.attn_fwd(q, k, v, packed, want_lse=True)
    return do, q, k, v, out, lse, packed


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_two_calls_in_a_row_match_the_workspace_entry_point(dev, dtype):
    for seed, (B, H, N, D) in enumerate([(3, 4, 333, 64), (2, 2, 100, 64), (1, 3, 130, 128), (1, 1, 17, 32)]):
        args = _problem(B, H, N, D, dtype, 100 + seed, dev)
        print(f"static workspace backward: B={B} H={H} N={N} D={D} {dtype}", flush=True)
        want = _capi.attn_bwd(*args)[:3]
        got = _capi.attn_bwd_static_ws(*args)
        torch.cuda.synchronize()
        for g, w, name in zip(got, want, ("dq", "dk", "dv")):
            assert torch.isfinite(g.float()).all(), name
            assert torch.equal(g, w), f"{name} differs at B={B} H={H} N={N} D={D}"


def test_calls_allocate_no_device_memory(dev):
    """What the entry point is for: after the first call on a device (which looks the array's address
    up), a call leaves the device's free memory as it found it."""
    args = _problem(2, 2, 200, 64, torch.float16, 11, dev)
    lib = _capi.load()
    dq, dk, dv = (torch.empty_like(args[1]) for _ in range(3))
    p = [t.data_ptr() for t in args] + [dq.data_ptr(), dk.data_ptr(), dv.data_ptr()]
    call = lambda: lib.sma_attn_bwd_static_ws(*p, 2, 2, 200, 64, 0.125, _capi.SMA_DTYPE_F16, None)
    assert call() == _capi.SMA_OK
    torch.cuda.synchronize()
    first = dq.clone()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        assert call() == _capi.SMA_OK
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    assert torch.equal(dq, first)


def test_static_workspace_limit_and_empty_problem(dev):
    lib = _capi.load()
    args = _problem(1, 1, 64, 64, torch.float16, 7, dev)
    big = dict(B=1 << 10, H=1 << 5, N=64)                    # 2^21 rows: beyond the array
    p = [t.data_ptr() for t in args] + [args[1].data_ptr()] * 3
    st = lib.sma_attn_bwd_static_ws(*p, big["B"], big["H"], big["N"], 64, 0.125, _capi.SMA_DTYPE_F16, None)
    assert st == _capi.SMA_ERR_WORKSPACE
    assert lib.sma_strerror(st) not in (b"ok", b"unknown error code")
    st = lib.sma_attn_bwd_static_ws(*p, 0, 1, 64, 64, 0.125, _capi.SMA_DTYPE_F16, None)
    assert st == _capi.SMA_OK
    torch.cuda.synchronize()
