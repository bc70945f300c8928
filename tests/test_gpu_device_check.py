"""The library's one-time check that the device serves 8- and 16-byte loads from unaligned addresses
(the row packers and the forward that reads the boolean mask depend on it), and what happens on a
device where it does not: the packer switches to byte loads and gives the same words, the
one-launch forward refuses, and the Python API falls back to pack_mask + forward.  The verdict is
cached per process, so the second half runs in a child process that tells the library to assume a
device without unaligned access (no such device exists in this pool)."""
import os
import subprocess
import sys
import textwrap

import pytest
import torch

import _capi

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_this_device_serves_unaligned_loads(dev):
    lib = _capi.load()
    assert lib.sma_device_check(None) == _capi.SMA_OK
    assert lib.sma_device_check(None) == _capi.SMA_OK          # cached verdict, same answer
    assert lib.sma_strerror(_capi.SMA_ERR_DEVICE) not in (b"ok", b"unknown error code")


CHILD = textwrap.dedent("""
    import importlib, os, sys
    sys.path[:0] = [os.path.join(ROOT, "tests"), os.path.join(ROOT, "sparse-mask-attention_amd"), ROOT]
    import numpy as np, torch
    import _capi
    from oracle import sma_oracle as O
    lib = _capi.load()
    dev = torch.device("cuda:0")
    assert lib.sma_device_check(None) == _capi.SMA_ERR_DEVICE
    g = torch.Generator().manual_seed(5)
    for N in (8, 33, 100, 257, 1000):                 # rows that do not start 16-byte aligned: byte loads
        mask = torch.rand(2, 2, N, N, generator=g) < 0.3
        got = _capi.pack_mask(mask.to(dev))
        assert np.array_equal(got.cpu().numpy(), O.pack_mask_ref(mask)), N
    mask = torch.rand(1, 2, 96, 96, generator=g) < 0.3      # the aligned stream does not depend on it
    assert np.array_equal(_capi.pack_mask(mask.to(dev)).cpu().numpy(), O.pack_mask_ref(mask))
    q, k, v = (torch.randn(1, 2, 96, 64, generator=g).half().to(dev) for _ in range(3))
    out = torch.empty_like(q)
    st = lib.sma_attn_fwd_bool_mask(q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.to(dev).data_ptr(), 96 * 96 * 2, 96 * 96,
                                    out.data_ptr(), None, None, 1, 2, 96, 64, 0.125, 0, None)
    assert st == _capi.SMA_ERR_DEVICE
    sa = importlib.import_module("python.sparse_attention")
    assert not sa.sparse_attn_cuda.bool_mask_supported(q, k, v, mask.to(dev))
    got = sa.sparse_attention_func(q, k, v, mask.to(dev))          # falls back to pack_mask + forward
    want = O.sparse_attention_ref(q.float().cpu(), k.float().cpu(), v.float().cpu(), mask)
    assert torch.allclose(got.float().cpu(), want, atol=1e-2, rtol=1e-2)
    print("child ok")
""")


def test_fallbacks_on_a_device_without_unaligned_access(dev):
    env = dict(os.environ, SMA_ASSUME_NO_UNALIGNED_ACCESS="1")
    proc = subprocess.run([sys.executable, "-c", f"ROOT = {ROOT!r}\n" + CHILD], env=env, capture_output=True, text=True,
                          timeout=600)
    assert proc.returncode == 0 and "child ok" in proc.stdout, proc.stdout[-2000:] + proc.stderr[-4000:]
