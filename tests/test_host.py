"""CPU-only checks of the host side: the C ABI loads and exports what include/sma.h declares,
argument validation answers before anything touches a GPU, the Python API keeps the reference's
surface and refuses to compute anywhere but on the device, and the workloads have the documented
sizes."""
import ctypes
import os
import re
import sys

import numpy as np
import pytest
import torch

import _capi
import harness

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(capi):
    header = open(os.path.join(ROOT, "include", "sma.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(sma_[a-z_0-9]+)\s*\(", header))
    assert {"sma_version", "sma_strerror", "sma_pack_mask", "sma_attn_fwd", "sma_attn_bwd",
            "sma_attn_fwd_strided", "sma_attn_bwd_strided", "sma_attn_fwd_bool_mask"} <= declared
    for name in declared:
        assert hasattr(capi, name), f"{name} is declared in sma.h but not exported"
    assert capi.sma_version() >= 100
    assert capi.sma_strerror(0) == b"ok"
    for code in range(-10, 0):
        assert capi.sma_strerror(code) not in (b"ok", b"unknown error code")
    assert capi.sma_strerror(-99) == b"unknown error code"


def test_argument_validation_needs_no_gpu(capi):
    p = ctypes.c_void_p(0x1000)            # never dereferenced: every call below fails or is a no-op first
    f = capi.sma_attn_fwd
    ok_args = dict(B=1, H=1, N=64, D=64, scale=0.125, dtype=_capi.SMA_DTYPE_F16)

    def call(q=p, k=p, v=p, mp=p, out=p, lse=None, **kw):
        a = dict(ok_args, **kw)
        return f(q, k, v, mp, out, lse, a["B"], a["H"], a["N"], a["D"], a["scale"], a["dtype"], None)

    assert call(D=16) == _capi.SMA_ERR_HEAD_DIM
    assert call(D=96) == _capi.SMA_ERR_HEAD_DIM
    assert call(D=256) == _capi.SMA_ERR_HEAD_DIM
    assert call(dtype=2) == _capi.SMA_ERR_DTYPE
    assert call(B=-1) == _capi.SMA_ERR_BAD_SHAPE
    assert call(scale=float("nan")) == _capi.SMA_ERR_SCALE
    assert call(scale=float("inf")) == _capi.SMA_ERR_SCALE
    assert call(q=None) == _capi.SMA_ERR_NULL_POINTER
    assert call(out=None) == _capi.SMA_ERR_NULL_POINTER
    assert call(q=ctypes.c_void_p(0x1002)) == _capi.SMA_ERR_ALIGNMENT
    assert call(B=0) == _capi.SMA_OK and call(N=0) == _capi.SMA_OK          # empty problem: nothing to do
    assert call(B=1 << 20, H=1 << 12, N=64) == _capi.SMA_ERR_BAD_SHAPE      # index range
    assert call(B=1, H=1, N=200000) == _capi.SMA_ERR_BAD_SHAPE              # packed mask of one (b,h) beyond 4 GiB

    # a tile map is refused beyond the size the library can make one for, by every entry point that
    # takes one and before anything is written (N = 140000 is inside the packed-mask limit)
    assert capi.sma_attn_fwd_map(p, p, p, p, p, p, None, 1, 1, 140000, 64, 0.125, 0, None) == _capi.SMA_ERR_BAD_SHAPE
    assert capi.sma_attn_bwd_map(p, p, p, p, p, p, p, p, p, p, p, p, 1, 1, 140000, 64, 0.125, 0, None) == _capi.SMA_ERR_BAD_SHAPE
    assert capi.sma_pack_mask_map(p, p, p, 1, 1, 140000, None) == _capi.SMA_ERR_BAD_SHAPE
    assert capi.sma_tile_map(p, p, 1, 1, 140000, None) == _capi.SMA_ERR_BAD_SHAPE
    # the backward with the library's own workspace: what is wrong with the arguments is reported as
    # such, whatever the size; an empty problem is a no-op; only a valid call can be too large
    ws = capi.sma_attn_bwd_static_ws
    big = (1 << 10, 1 << 5, 64)            # 2^21 rows
    assert ws(*([p] * 10), *big, 96, 0.125, 0, None) == _capi.SMA_ERR_HEAD_DIM
    assert ws(*([p] * 10), *big, 64, 0.125, 7, None) == _capi.SMA_ERR_DTYPE
    assert ws(*([p] * 10), *big, 64, float("nan"), 0, None) == _capi.SMA_ERR_SCALE
    assert ws(*([p] * 10), -1, 1, 64, 64, 0.125, 0, None) == _capi.SMA_ERR_BAD_SHAPE
    assert ws(*([p] * 10), 0, 1, 64, 64, 0.125, 0, None) == _capi.SMA_OK
    assert ws(*([p] * 10), *big, 64, 0.125, 0, None) == _capi.SMA_ERR_WORKSPACE
    assert ws(*([p] * 10), 1 << 30, 1 << 30, 1 << 30, 64, 0.125, 0, None) == _capi.SMA_ERR_WORKSPACE   # no overflow on the way

    # strided entry point: the descriptor is checked before anything is launched
    fs = capi.sma_attn_fwd_strided
    T = _capi.SmaTensor

    def scall(q=T(0x1000, 4096, 4096, 64), msb=128, msh=128, **kw):
        a = dict(ok_args, **kw)
        t = T(0x1000, 4096, 4096, 64)
        return fs(q, t, t, p, msb, msh, t, None, a["B"], a["H"], a["N"], a["D"], a["scale"], a["dtype"], None)

    assert scall(D=96) == _capi.SMA_ERR_HEAD_DIM
    assert scall(q=T(0x1000, 4096, 4096, 60)) == _capi.SMA_ERR_STRIDE          # not a multiple of 8 elements
    assert scall(q=T(0x1000, 4096, -64, 64)) == _capi.SMA_ERR_STRIDE
    assert scall(q=T(0x1000, 0, 0, 1 << 25)) == _capi.SMA_ERR_STRIDE           # (N-1) * stride_n * 2 >= 2^31
    assert scall(q=T(None, 4096, 4096, 64)) == _capi.SMA_ERR_NULL_POINTER
    assert scall(q=T(0x1008, 4096, 4096, 64)) == _capi.SMA_ERR_ALIGNMENT
    assert scall(msh=-1) == _capi.SMA_ERR_STRIDE
    assert scall(q=None) == _capi.SMA_ERR_NULL_POINTER
    assert scall(B=0) == _capi.SMA_OK

    # an output whose rows would land on each other is refused; the same strides on an input are fine
    def ocall(out, q=T(0x1000, 4096, 4096, 64), **kw):
        a = dict(ok_args, **kw)
        return fs(q, q, q, p, 128, 128, out, None, a["B"], a["H"], a["N"], a["D"], a["scale"], a["dtype"], None)

    assert ocall(T(0x1000, 4096, 4096, 0)) == _capi.SMA_ERR_STRIDE              # every row at the same place
    assert ocall(T(0x1000, 4096, 4096, 32)) == _capi.SMA_ERR_STRIDE             # rows half on top of each other
    assert ocall(T(0x1000, 8192, 0, 64), H=2) == _capi.SMA_ERR_STRIDE           # both heads at the same place
    assert ocall(T(0x1000, 0, 4096, 64), B=2) == _capi.SMA_ERR_STRIDE           # both batch entries at the same place
    assert ocall(T(0x1000, 0, 0, 64), B=0, q=T(0x1000, 0, 0, 0)) == _capi.SMA_OK    # nothing to write

    # forward straight from the boolean mask: limits are reported, not worked around
    fb = capi.sma_attn_fwd_bool_mask

    def bcall(mask=p, msb=4096, msh=4096, **kw):
        a = dict(ok_args, **kw)
        return fb(p, p, p, mask, msb, msh, p, None, None, a["B"], a["H"], a["N"], a["D"], a["scale"], a["dtype"], None)

    assert bcall(D=96) == _capi.SMA_ERR_HEAD_DIM
    assert bcall(N=12) == _capi.SMA_ERR_BAD_SHAPE                             # shorter than one 16-byte copy
    assert bcall(N=46341) == _capi.SMA_ERR_BAD_SHAPE                          # N * N does not fit 31 bits
    assert bcall(mask=None) == _capi.SMA_ERR_NULL_POINTER
    assert bcall(msh=-24) == _capi.SMA_ERR_STRIDE
    assert bcall(dtype=5) == _capi.SMA_ERR_DTYPE
    assert bcall(B=0) == _capi.SMA_OK

    g = capi.sma_pack_mask
    assert g(None, p, 1, 1, 8, None) == _capi.SMA_ERR_NULL_POINTER
    assert g(p, None, 1, 1, 8, None) == _capi.SMA_ERR_NULL_POINTER
    assert g(p, p, 1, -2, 8, None) == _capi.SMA_ERR_BAD_SHAPE
    assert g(p, p, 0, 4, 8, None) == _capi.SMA_OK
    assert g(p, ctypes.c_void_p(0x1001), 1, 1, 8, None) == _capi.SMA_ERR_ALIGNMENT

    # extents whose products pass 2^63 are refused like any other index range, by every entry point
    huge = (1 << 31) - 1
    assert g(p, p, huge, huge, huge, None) == _capi.SMA_ERR_BAD_SHAPE
    assert capi.sma_tile_map(p, p, huge, huge, 64, None) == _capi.SMA_ERR_BAD_SHAPE
    assert capi.sma_pack_mask_map(p, p, p, huge, huge, 64, None) == _capi.SMA_ERR_BAD_SHAPE
    assert call(B=huge, H=huge, N=huge) == _capi.SMA_ERR_BAD_SHAPE
    assert bcall(B=huge, H=huge, N=1024) == _capi.SMA_ERR_BAD_SHAPE
    assert capi.sma_attn_bwd(*([p] * 11), huge, huge, 4096, 64, 0.125, 0, None) == _capi.SMA_ERR_BAD_SHAPE


def test_python_api_surface_and_loud_failure_off_gpu():
    import python as pkg
    assert set(pkg.__all__) == {"sparse_attention", "sparse_attention_func"}
    sa = sys.modules["python.sparse_attention"]
    for name in ("sparse_attention", "sparse_attention_func", "pack_mask", "sparse_attention_ref",
                 "SparseAttentionFunction", "generate_random_sparse_mask", "HAS_CUDA_EXT"):
        assert hasattr(sa, name), name
    assert sa.HAS_CUDA_EXT, f"extension did not import: {sa._EXT_ERROR}"
    import sparse_attn_cuda
    assert {"forward", "pack_mask"} <= set(dir(sparse_attn_cuda))
    q = torch.randn(1, 1, 8, 64)
    m = torch.ones(1, 1, 8, 8, dtype=torch.bool)
    for fn in (sa.sparse_attention, sa.sparse_attention_func):
        with pytest.raises(RuntimeError, match="GPU only"):
            fn(q, q, q, m)
    with pytest.raises(RuntimeError, match="GPU only"):
        sa.pack_mask(m)
    with pytest.raises(AssertionError):
        sa.sparse_attention(q, q, q, m.to(torch.uint8))
    with pytest.raises(AssertionError):
        sa.sparse_attention(q, q[:, :, :4], q, m)
    # the binding itself rejects host tensors with the reference's RuntimeError convention
    with pytest.raises(RuntimeError):
        sparse_attn_cuda.pack_mask(m)
    with pytest.raises(RuntimeError):
        sparse_attn_cuda.forward(q.half(), q.half(), q.half(), torch.zeros(1, 1, 8, 1, dtype=torch.int32),
                                 q.half(), None, 0.125, False)


def test_reference_formulation_kept_in_the_api_matches_the_oracle():
    from oracle import sma_oracle as O
    sa = sys.modules.get("python.sparse_attention") or __import__("python.sparse_attention")
    sa = sys.modules["python.sparse_attention"]
    q, k, v, mask = harness.make_inputs("C1", seed=1)
    mask[0, 0, 3, :] = False
    a = sa.sparse_attention_ref(q.float(), k.float(), v.float(), mask)
    b = O.sparse_attention_ref(q.float(), k.float(), v.float(), mask)
    assert torch.equal(a, b)


def test_workload_shapes_and_algorithmic_sizes():
    W = harness.WORKLOADS
    assert (W["C2"].B, W["C2"].H, W["C2"].N, W["C2"].D) == (16, 12, 512, 64)
    assert W["C2"].dense_flops == 12884901888
    assert W["C2"].attn_bytes == 56623104 and W["C2"].pack_bytes == 56623104
    assert W["C3"].attn_bytes == 125829120 and W["C3"].pack_bytes == 226492416
    assert W["C4"].attn_bytes == 81920000 and W["C4"].pack_bytes == 144384000
    assert W["C5"].attn_bytes == 142606336 and W["C5"].pack_bytes == 75497472
    q, k, v, m = harness.make_inputs("C1", seed=42)
    assert q.shape == (1, 2, 128, 64) and q.dtype == torch.float16 and m.dtype == torch.bool
    assert 0.2 < m.float().mean() < 0.3
    q2, _, _, m2 = harness.make_inputs("C1", seed=42)
    assert torch.equal(q, q2) and torch.equal(m, m2)                       # deterministic


def test_structured_masks():
    small = harness.Workload("blk", 1, 2, 256, 64, torch.float16, "block64", 0.25)
    m = harness.make_mask(small, torch.Generator().manual_seed(0))
    t = m.reshape(1, 2, 4, 64, 4, 64)
    per_block = t.float().mean(dim=(3, 5))
    assert ((per_block == 0) | (per_block == 1)).all()
    assert (torch.diagonal(per_block, dim1=2, dim2=3) == 1).all()
    rag = harness.Workload("rag", 1, 1, 100, 64, torch.bfloat16, "random_diag", 0.1, 0.5)
    m = harness.make_mask(rag, torch.Generator().manual_seed(0))
    assert torch.diagonal(m[0, 0]).all() and m.float().mean() < 0.2
    cau = harness.Workload("cau", 1, 1, 64, 64, torch.float16, "causal_random", 0.5)
    m = harness.make_mask(cau, torch.Generator().manual_seed(0))
    assert not torch.triu(m[0, 0], diagonal=1).any() and torch.diagonal(m[0, 0]).all()
    tf, pct = harness.compute_mfu(1.0, 16, 12, 512, 64, 2516.6)
    assert tf == pytest.approx(12.884901888) and pct == pytest.approx(100 * 12.884901888 / 2516.6)


def test_bench_passes_on_recorded_traffic_only_for_the_sources_it_was_recorded_for(tmp_path, monkeypatch):
    """bench.py cannot read HBM counters itself and quotes them from the summaries under profiles/;
    a summary made for other kernel sources than those in the tree must not be quoted."""
    sys.path.insert(0, ROOT)
    import bench
    csrc = tmp_path / "sparse-mask-attention_amd" / "csrc"
    csrc.mkdir(parents=True)
    for name in ("pack_mask.hip", "sma_internal.h"):
        (csrc / name).write_text("// " + name + "\n")
    monkeypatch.setattr(bench, "ROOT", str(tmp_path))
    digest = bench.source_digest("pack_mask_kernel")
    assert re.fullmatch(r"[0-9a-f]{16}", digest)
    prof = tmp_path / "profiles"
    prof.mkdir()
    (prof / "pack_mask_kernel_C2.txt").write_text(
        f"kernel sources (...), sources sha256/16: {digest}\n  traffic per launch 56.65 MB vs algorithmic 56.62 MB\n")
    assert bench.measured_traffic("C2", "pack_mask_kernel") == 56650000
    assert bench.measured_traffic("C3", "pack_mask_kernel") is None            # no summary
    (csrc / "pack_mask.hip").write_text("// changed\n")
    assert bench.measured_traffic("C2", "pack_mask_kernel") is None            # recorded for other code
