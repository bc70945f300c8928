#!/usr/bin/env python3
"""Command-line harness:  python run.py --mode {correctness,perf,all}

Counterpart of the reference's run.py (argparse at run.py:804-818) for the MI355X build, without
its competitor baselines (Triton, cuDNN, FlashInfer, flash-attn):

* correctness  the reference's acceptance run (run.py:349-404): fp16, B=2, H=4, D=64, 75 % random
               sparsity, N in {64,128,256,512}, max |out - fp32 PyTorch formulation| < 1e-2, and the
               fully-masked-row case (N=8, row 0 masked) which must contain no NaN;
* perf         the N-sweep at B=16 and the B-sweep at N=512 (run.py:410-450), H=12, D=64, fp16,
               75 % sparsity; every latency covers what the reference's covers, boolean mask in and
               output out (there: pack_mask + allocation + forward; here: allocation + the one
               launch that reads the boolean mask, with the reference's three calls in a second
               column), 10 warm-up and 50 timed calls between stream events (run.py:172-183), with
               dense-equivalent TFLOP/s and percent of the MI355X dense FP16 MFMA peak.

Inputs are generated on the CPU from an explicit seed and moved to the GPU.  The PyTorch
formulation used as the yardstick here is python/sparse_attention.py::sparse_attention_ref, run on
the GPU in fp32; it is a check for users, the test-suite has its own CPU oracle.
"""
import argparse
import importlib
import math
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)

import harness  # noqa: E402

sa = importlib.import_module("python.sparse_attention")


def sparse_attention_hip_two_launches(q, k, v, mask):
    """pack_mask + allocation + forward: the reference's sequence of calls (run.py:147-155)."""
    import sparse_attn_cuda as ext
    packed = ext.pack_mask(mask)
    out = torch.empty_like(q)
    ext.forward(q, k, v, packed, out, None, 1.0 / math.sqrt(q.shape[-1]), False)
    return out


def sparse_attention_hip_fwd(q, k, v, mask):
    """Boolean mask in, output out: allocation + the forward that reads the boolean mask itself
    where it applies (contiguous q, k, v, N >= 16), else the two launches above."""
    import sparse_attn_cuda as ext
    if not ext.bool_mask_supported(q, k, v, mask):
        return sparse_attention_hip_two_launches(q, k, v, mask)
    out = torch.empty_like(q)
    ext.forward_bool_mask(q, k, v, mask, out, None, 1.0 / math.sqrt(q.shape[-1]), False)
    return out


def sdpa_bool_mask(q, k, v, mask):
    """PyTorch's own fused attention with the same bool mask (True = attend): the on-box
    competitor column, as the reference compares against library kernels (run.py:514-523)."""
    return torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask)


def _inputs(B, H, N, seed, device):
    g = torch.Generator().manual_seed(seed)
    q, k, v = [torch.randn(B, H, N, 64, generator=g).half().to(device) for _ in range(3)]
    mask = harness.generate_mask(B, H, N, 0.75, generator=g).to(device)
    return q, k, v, mask


def run_correctness(device):
    print("=" * 56 + "\ncorrectness (fp16, B=2, H=4, D=64, sparsity 0.75, tol 1e-2)\n" + "=" * 56)
    ok = True
    for N in (64, 128, 256, 512):
        q, k, v, mask = _inputs(2, 4, N, 42, device)
        ref = sa.sparse_attention_ref(q.float(), k.float(), v.float(), mask)
        out = sparse_attention_hip_fwd(q, k, v, mask).float()
        d = (out - ref).abs()
        passed = d.max().item() < 1e-2
        ok &= passed
        print(f"  N={N:4d}  max_diff={d.max().item():.6f}  mean_diff={d.mean().item():.6f}  [{'PASS' if passed else 'FAIL'}]")
    q, k, v, _ = _inputs(1, 1, 8, 7, device)
    mask = torch.ones(1, 1, 8, 8, dtype=torch.bool, device=device)
    mask[:, :, 0, :] = False
    out = sparse_attention_hip_fwd(q, k, v, mask)
    nan_ok = not torch.isnan(out).any().item() and (out[0, 0, 0] == 0).all().item()
    ok &= nan_ok
    print(f"  fully masked row: no NaN, zeros  [{'PASS' if nan_ok else 'FAIL'}]")
    print("\nresult:", "all passed" if ok else "FAILURES", "\n")
    return ok


def run_perf(device):
    peak = harness.MI355X_MFMA_F16_TFLOPS
    print("=" * 56 + f"\nperformance (fp16, H=12, D=64, sparsity 0.75; peak {peak} TFLOP/s)\n" + "=" * 56)
    print("\n[sequence length sweep]  B=16")
    print(f"  {'N':>6}  {'latency(ms)':>12}  {'TFLOPS':>8}  {'MFU%':>7}  {'pack+fwd(ms)':>13}  {'torch SDPA(ms)':>15}  {'speed-up':>8}")
    for N in (64, 128, 256, 512, 1024):
        q, k, v, mask = _inputs(16, 12, N, 1, device)
        lat = harness.measure_latency(lambda: sparse_attention_hip_fwd(q, k, v, mask))
        two = harness.measure_latency(lambda: sparse_attention_hip_two_launches(q, k, v, mask))
        tf, mfu = harness.compute_mfu(lat, 16, 12, N, 64, peak)
        ref = harness.measure_latency(lambda: sdpa_bool_mask(q, k, v, mask))
        print(f"  {N:>6}  {lat:>12.4f}  {tf:>8.2f}  {mfu:>7.1f}%  {two:>13.4f}  {ref:>15.4f}  {ref / lat:>7.1f}x")
    print("\n[batch size sweep]  N=512")
    print(f"  {'B':>6}  {'latency(ms)':>12}  {'TFLOPS':>8}  {'MFU%':>7}  {'pack+fwd(ms)':>13}  {'seq/s':>10}")
    for B in (1, 4, 8, 16, 32, 64):
        q, k, v, mask = _inputs(B, 12, 512, 2, device)
        lat = harness.measure_latency(lambda: sparse_attention_hip_fwd(q, k, v, mask))
        two = harness.measure_latency(lambda: sparse_attention_hip_two_launches(q, k, v, mask))
        tf, mfu = harness.compute_mfu(lat, B, 12, 512, 64, peak)
        print(f"  {B:>6}  {lat:>12.4f}  {tf:>8.2f}  {mfu:>7.1f}%  {two:>13.4f}  {B / (lat / 1e3):>10.0f}")
    print()


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--mode", choices=["correctness", "perf", "all"], default="all")
    args = ap.parse_args()
    if not sa.HAS_CUDA_EXT:
        sys.exit(f"HIP extension missing: {sa._EXT_ERROR}")
    if not torch.cuda.is_available():
        sys.exit("no GPU visible")
    device = torch.device("cuda:0")
    print(f"GPU: {torch.cuda.get_device_name(0)}")
    ok = True
    if args.mode in ("correctness", "all"):
        ok = run_correctness(device)
    if args.mode in ("perf", "all"):
        run_perf(device)
    sys.exit(0 if ok else 1)


if __name__ == "__main__":
    main()
