"""GPU parity of sma_pack_mask (through the C ABI) against the oracle: bit-exact."""
import numpy as np
import pytest
import torch

import _capi
import harness
from oracle import sma_oracle as O

pytestmark = pytest.mark.gpu


def _check(mask_cpu, dev):
    got = _capi.pack_mask(mask_cpu.to(dev))
    torch.cuda.synchronize()
    assert got.dtype == torch.int32
    expect = O.pack_mask_ref(mask_cpu)
    assert got.shape == expect.shape
    assert np.array_equal(got.cpu().numpy(), expect)


@pytest.mark.parametrize("N", [1, 7, 8, 31, 32, 33, 63, 64, 65, 96, 100, 128, 250, 257, 512, 1000])
def test_random_masks_bit_exact(dev, N):
    g = torch.Generator().manual_seed(100 + N)
    _check(torch.rand(2, 3, N, N, generator=g) > 0.75, dev)


@pytest.mark.parametrize("N", [8, 32, 40, 64, 1000])
def test_all_true_all_false_and_single_bits(dev, N):
    _check(torch.ones(1, 2, N, N, dtype=torch.bool), dev)
    _check(torch.zeros(1, 2, N, N, dtype=torch.bool), dev)
    m = torch.zeros(1, 1, N, N, dtype=torch.bool)
    for c in {0, N - 1, min(31, N - 1), min(32, N - 1)}:
        m[0, 0, c % N, c] = True
    _check(m, dev)


def test_known_answer_words(dev):
    got = _capi.pack_mask(torch.ones(1, 1, 8, 8, dtype=torch.bool, device=dev)).cpu().numpy().view(np.uint32)
    assert (got == 0xFF).all()
    m = torch.zeros(1, 1, 64, 64, dtype=torch.bool)
    m[0, 0, 2, 31] = True
    m[0, 0, 3, 32] = True
    got = _capi.pack_mask(m.to(dev)).cpu().numpy()
    assert got[0, 0, 2, 0] == -2**31 and got[0, 0, 2, 1] == 0
    assert got[0, 0, 3, 0] == 0 and got[0, 0, 3, 1] == 1


def test_nonzero_bytes_count_as_true(dev):
    # storage of a bool tensor viewed from uint8 may hold values other than 0/1
    g = torch.Generator().manual_seed(5)
    for N in (64, 100):
        raw = torch.randint(0, 256, (1, 2, N, N), generator=g, dtype=torch.uint8)
        raw[torch.rand(1, 2, N, N, generator=g) > 0.3] = 0
        got = _capi.pack_mask(raw.to(dev).view(torch.bool))
        assert np.array_equal(got.cpu().numpy(), O.pack_mask_ref(raw.numpy() != 0))


def test_every_length_at_several_alignments(dev):
    """Rows of every length up to 140 bytes (and some long odd ones) starting 0, 1 and 5 bytes into
    an allocation that ends with the mask's last byte: every alignment of every row."""
    g = torch.Generator().manual_seed(8)
    for N in list(range(1, 141)) + [255, 511, 513, 999, 1001, 1031]:
        m = torch.rand(1, 2, N, N, generator=g) > 0.6
        want = O.pack_mask_ref(m)
        for off in (0, 1, 5):
            buf = torch.ones(off + m.numel(), dtype=torch.bool, device=dev)
            view = buf[off:].view(1, 2, N, N)
            view.copy_(m)
            assert np.array_equal(_capi.pack_mask(view).cpu().numpy(), want), (N, off)


def test_unaligned_base_pointer(dev):
    # a mask that starts 1 byte into an allocation takes the general (row) kernel
    g = torch.Generator().manual_seed(6)
    N = 64
    m = torch.rand(2, 2, N, N, generator=g) > 0.5
    buf = torch.zeros(m.numel() + 16, dtype=torch.bool, device=dev)
    view = buf[1:1 + m.numel()].view(2, 2, N, N)
    view.copy_(m)
    assert view.data_ptr() % 16 != 0
    got = _capi.pack_mask(view)
    assert np.array_equal(got.cpu().numpy(), O.pack_mask_ref(m))


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_benchmark_workloads_bit_exact_and_invariants(dev, name):
    w = harness.WORKLOADS[name]
    mask = harness.make_mask(w, torch.Generator().manual_seed(42))
    md = mask.to(dev)
    got = _capi.pack_mask(md)
    torch.cuda.synchronize()
    # full-size, size-independent properties evaluated on the GPU
    cols = torch.arange(w.N, device=dev)
    unpacked = ((got[..., cols // 32] >> (cols % 32)) & 1).bool()
    assert torch.equal(unpacked, md)                                   # unpack(pack(m)) == m
    tail = w.N % 32
    if tail:
        assert ((got[..., -1].to(torch.int64) & 0xFFFFFFFF) >> tail == 0).all()   # pad bits zero
    # and bit-exact against the oracle on the whole tensor
    assert np.array_equal(got.cpu().numpy(), O.pack_mask_ref(mask))
