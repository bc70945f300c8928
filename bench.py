#!/usr/bin/env python3
"""Benchmark of the sparse-mask attention hot path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input, as the reference times it
(run.py:147-155, :172-183): boolean mask in, attention output out, called through the
`sparse_attn_cuda` module with all inputs already resident in HBM.  The reference needs two
launches for it (pack_mask, then the fused forward); here the step is: allocate out -> ONE launch
that reads the boolean mask itself (forward_bool_mask), where the kernel's limits allow (N >= 16),
else pack_mask -> allocate out -> forward.  The two-launch step is
timed as well and reported beside it.  The headline value is dense-equivalent TFLOP/s,
4*B*H*N*N*D per step whatever the sparsity (run.py:198-203).

Prints ONE JSON line.  Besides the whole-step figure it carries
  roofline      the dominant kernel of the step alone, from stream-event timing of back-to-back
                launches on the launch stream: the forward that reads the boolean mask or, where
                that does not apply, the packed-mask forward.  `frac` is the fraction of the dense
                FP16/BF16 MFMA peak in dense-equivalent FLOP (the figure the target is written in);
                the HBM side is in `hbm_*` (100.7 MB of compulsory traffic for 12.9 GFLOP on the
                headline workload, 128 FLOP/B: below the ridge at 315);
  roofline_attn the packed-mask forward kernel alone against the MFMA peak (with the tile map of the
                mask where walking it saves enough visits to pay);
  roofline_pack the packer alone against the HBM peak;
  roofline_bwd  the backward (its two kernels, one call) against the MFMA peak, 2.5 x the forward's FLOP;
  cpu_baseline  the oracle's PyTorch formulation of the same workload on the host cores.
Every roofline carries two timings.  The plain ones repeat the launch on the same tensors, as the
reference's protocol does (run.py:172-183): the working set of the headline workload (57 to 101 MB)
then stays in the 256 MB last-level cache between launches, and the "HBM" fractions computed from it
are fractions of the HBM peak served partly from that cache.  The `*_cold` ones rotate through
enough distinct copies of all tensors (more than 512 MB in total) that every launch finds none of
its data cached: those are HBM figures.
"""
import argparse
import ctypes
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "sparse-mask-attention_amd")
for p in (PKG, ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)

# Published figure for exactly this metric and configuration (pack_mask included in the timing):
# 27.66 dense-equivalent TFLOP/s on an RTX 3080, reference README.md:13.
PUBLISHED_TFLOPS = {"C2": 27.66}


def event_time_ms(fn, warmup, repeat, torch):
    """Mean ms per call of `repeat` back-to-back calls between two events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(repeat):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / repeat


def settle(fn, torch, ms=60.0):
    """Run fn back to back for `ms` milliseconds, untimed: after the host-side pauses between the
    sections of this script (building tensors on the CPU, copies) the device needs tens of
    milliseconds of work to be back at the clock it keeps under load."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < ms * 1e-3:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def cold_time_ms(make_call, n_sets, warmup, repeat, torch):
    """Mean ms per call when consecutive calls use different copies of every tensor: make_call(i)
    returns the call for copy i, n_sets copies exceed the caches, so no call finds its inputs (or
    the lines of its outputs) resident."""
    calls = [make_call(i) for i in range(n_sets)]
    for i in range(max(warmup, n_sets)):
        calls[i % n_sets]()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(repeat):
        calls[i % n_sets]()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / repeat


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


# The source files each profiled kernel is compiled from: a counter summary under profiles/ records
# their digest, so that a figure recorded for other code than the one that runs now is not passed on.
KERNEL_SOURCES = {
    "attn_fwd_kernel": ("attn_fwd.hip", "attn_common.h", "sma_internal.h"),
    "attn_fwd_bool_mask_kernel": ("attn_fwd.hip", "attn_common.h", "sma_internal.h"),
    "pack_mask_kernel": ("pack_mask.hip", "sma_internal.h"),
    "attn_bwd_dq_kernel": ("attn_bwd.hip", "attn_common.h", "sma_internal.h"),
    "attn_bwd_dkv_kernel": ("attn_bwd.hip", "attn_common.h", "sma_internal.h"),
}


def source_digest(kernel):
    """First 16 hex digits of the SHA-256 of the kernel's source files, in the order listed."""
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES[kernel]:
        with open(os.path.join(ROOT, "sparse-mask-attention_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def roofline_ceiling(flops, algorithmic_bytes, achieved_tflops):
    """Where a kernel sits on the roofline: its FLOP per algorithmic byte against the machine's
    balance (MFMA peak / HBM peak), the ceiling the model gives it (the lower of the MFMA peak and
    FLOP-per-byte x HBM peak) and the fraction of that ceiling it reaches.  `frac` of the roofline
    objects stays the fraction of the MFMA peak whichever side the kernel is on."""
    import harness
    balance = harness.MI355X_MFMA_F16_TFLOPS * 1e3 / harness.MI355X_HBM_GBPS
    ai = flops / algorithmic_bytes
    ceiling = min(harness.MI355X_MFMA_F16_TFLOPS, ai * harness.MI355X_HBM_GBPS / 1e3)
    return {"flop_per_byte": round(ai, 1), "machine_balance_flop_per_byte": round(balance, 1),
            "ceiling_side": "hbm" if ai < balance else "mfma", "ceiling_tflops": round(ceiling, 1),
            "frac_of_ceiling": round(achieved_tflops / ceiling, 4)}


def measured_traffic(workload, *kernels):
    """HBM bytes per launch (summed over `kernels`) from the committed rocprofv3 counter summaries
    of this workload (FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for a
    plain copy of known size).  Counters cannot be read from inside this process, so the figure is
    the recorded one, not a live one: None when a summary for this workload is not there, or when
    it was recorded for other kernel sources than the ones in the tree now."""
    import re
    total = 0
    for kernel in kernels:
        path = os.path.join(ROOT, "profiles", f"{kernel}_{workload}.txt")
        try:
            text = open(path).read()
        except OSError:
            return None
        m = re.search(r"traffic per launch ([0-9.]+) MB", text)
        d = re.search(r"sources sha256/16: ([0-9a-f]{16})", text)
        try:
            current = source_digest(kernel)
        except OSError:
            return None
        if not m or not d or d.group(1) != current:
            return None
        total += int(float(m.group(1)) * 1e6)
    return total


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="C2", choices=["C1", "C2", "C3", "C4", "C5"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--precondition-ms", type=float, default=200.0,
                    help="run the step untimed for this long before the warm-up steps, so that the timed steps "
                         "see the clock the device settles at rather than its ramp after idling")
    ap.add_argument("--only", default=None,
                    choices=["packed", "packed_map", "fused", "fused_training", "pack", "bwd", "bwd_map"],
                    help="launch ONE kind of kernel back to back (--warmup, then --steps launches), print its "
                         "mean time and exit: packed = packed-mask forward over all tiles, packed_map = the same "
                         "walking the mask's tile map, fused = forward from the boolean mask, fused_training = "
                         "the same leaving lse, packed words and tile map behind, pack = the packer, bwd / "
                         "bwd_map = the backward without / with the tile map.  For rocprofv3 runs whose "
                         "per-kernel averages must not blend launch contexts.")
    ap.add_argument("--ramp", action="store_true",
                    help="instead of the benchmark: time the step in consecutive blocks from the first launch after "
                         "idling (10 blocks of 20 steps, then 50 of 200) and print one line per block; shows the "
                         "clock ramp that --precondition-ms skips")
    ap.add_argument("--calib-copy-mib", type=int, default=0,
                    help="also run one plain device-to-device copy of this many MiB (a traffic yardstick "
                         "for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; every (b,h) pair is independent, so more "
                 "GPUs would each take a slice of the batch with no exchange. Use --gpus 1.")

    import torch
    import harness
    sa = importlib.import_module("python.sparse_attention")
    if not sa.HAS_CUDA_EXT:
        sys.exit(f"bench.py: HIP extension missing ({sa._EXT_ERROR}); run __graft_entry__.build()")
    import sparse_attn_cuda as ext
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")

    w = harness.WORKLOADS[args.workload]
    q, k, v, mask = harness.make_inputs(w, seed=42)
    qd, kd, vd, md = (t.to(dev) for t in (q, k, v, mask))
    scale = 1.0 / (w.D ** 0.5)

    if args.calib_copy_mib > 0:
        src = torch.zeros(args.calib_copy_mib << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.only:
        packed = ext.pack_mask(md)
        out = torch.empty_like(qd)
        full_map = ext.tile_map(packed)         # the map itself, whether or not walking it pays
        lse = torch.empty(w.B, w.H, w.N, dtype=torch.float32, device=dev)
        if args.only in ("bwd", "bwd_map"):
            ext.forward(qd, kd, vd, packed, out, lse, scale, True)
            dout = torch.randn(qd.shape, generator=torch.Generator().manual_seed(43)).to(qd.dtype).to(dev)
            dq, dk, dv = (torch.empty_like(qd) for _ in range(3))
        packed2, map2 = torch.empty_like(packed), torch.empty_like(full_map)
        fn = {
            "packed": lambda: ext.forward(qd, kd, vd, packed, out, None, scale, False),
            "packed_map": lambda: ext.forward(qd, kd, vd, packed, out, None, scale, False, full_map),
            "fused": lambda: ext.forward_bool_mask(qd, kd, vd, md, out, None, scale, False),
            "fused_training": lambda: ext.forward_bool_mask(qd, kd, vd, md, out, lse, scale, True, packed2, map2),
            "pack": lambda: ext.pack_mask(md),
            "bwd": lambda: ext.backward(dout, qd, kd, vd, out, lse, packed, dq, dk, dv, scale),
            "bwd_map": lambda: ext.backward(dout, qd, kd, vd, out, lse, packed, dq, dk, dv, scale, full_map),
        }[args.only]
        t_pre = time.perf_counter()          # to the device's steady clock first, as for the whole line
        while time.perf_counter() - t_pre < args.precondition_ms * 1e-3:
            for _ in range(50):
                fn()
            torch.cuda.synchronize()
        ms = event_time_ms(fn, args.warmup, args.steps, torch)
        print(json.dumps({"only": args.only, "workload": w.name, "launches": args.steps, "ms": round(ms, 5)}), flush=True)
        return

    def step_two_launches():
        packed = ext.pack_mask(md)
        out = torch.empty_like(qd)
        ext.forward(qd, kd, vd, packed, out, None, scale, False)
        return out

    def step_one_launch():
        out = torch.empty_like(qd)
        ext.forward_bool_mask(qd, kd, vd, md, out, None, scale, False)
        return out

    one_launch = bool(ext.bool_mask_supported(qd, kd, vd, md))
    step = step_one_launch if one_launch else step_two_launches

    def wall_ms(fn):
        """W untimed, K timed calls, synchronize on both sides."""
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps

    if args.ramp:
        torch.cuda.synchronize()
        time.sleep(0.5)                      # idle first
        t00 = time.perf_counter()
        for blk in range(60):
            n = 20 if blk < 10 else 200
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                step()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            print(json.dumps({"block": blk, "steps": n, "starts_at_ms": round((t0 - t00) * 1e3, 2),
                              "us_per_step": round((t1 - t0) * 1e6 / n, 2)}), flush=True)
        return

    # Before anything is timed the device is brought to its steady clock: for the first 25-30 ms of
    # work after idling the part runs this step 5 to 25 % slower than it then settles at (measured:
    # 23-26 us per step during the first 10 ms, 20.7 us from 30 ms on), and W warm-up steps of 23 us
    # end long before that.  The warm-up and the K timed steps follow immediately.
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < args.precondition_ms * 1e-3:
        for _ in range(50):
            step()
        torch.cuda.synchronize()
    two_launch_ms = wall_ms(step_two_launches)
    ms_per_step = wall_ms(step) if one_launch else two_launch_ms
    value = w.dense_flops / (ms_per_step * 1e-3) / 1e12

    # ---- the two kernels on their own: back-to-back launches between stream events ----
    packed = ext.pack_mask(md)
    tmap = sa.tile_map(packed)          # None unless walking the map would save enough visits to pay
    out = torch.empty_like(qd)
    reps = max(200, args.steps)          # a burst of at least 4 ms: shorter ones are timed on the clock ramp after the preceding synchronisation
    # the packer through the C ABI into a preallocated buffer (no allocator in the loop)
    lib = ctypes.CDLL(os.path.join(PKG, "libsma_hip.so"))
    lib.sma_pack_mask.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                  ctypes.c_int, ctypes.c_void_p]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    lse_t = torch.empty(w.B, w.H, w.N, dtype=torch.float32, device=dev)
    packed_t = torch.empty_like(packed)
    kernels = {
        "attn": lambda: ext.forward(qd, kd, vd, packed, out, None, scale, False, tmap),
        "pack": lambda: lib.sma_pack_mask(md.data_ptr(), packed_t.data_ptr(), w.B, w.H, w.N, stream),
        "api": lambda: sa.sparse_attention_func(qd, kd, vd, md),
    }
    if tmap is not None:
        kernels["attn_nomap"] = lambda: ext.forward(qd, kd, vd, packed, out, None, scale, False)
    if one_launch:
        kernels["fused"] = lambda: ext.forward_bool_mask(qd, kd, vd, md, out, None, scale, False)
        # the same launch as autograd makes it: with the lse, and leaving the packed words behind
        kernels["fused_training"] = lambda: ext.forward_bool_mask(qd, kd, vd, md, out, lse_t, scale, True, packed_t)
    # Three rounds over all of them, the median round of each: what a kernel is timed after (the
    # clock the part has settled at, what the caches hold) moves a single measurement by several
    # per cent, and differences between these kernels are read off this line.
    timings = {name: [] for name in kernels}
    settle(kernels["attn"], torch)
    for rnd in range(3):
        for name, fn in kernels.items():
            timings[name].append(event_time_ms(fn, 10, reps, torch))
    med = {name: sorted(v)[1] for name, v in timings.items()}
    attn_ms, pack_ms, api_ms = med["attn"], med["pack"], med["api"]
    attn_nomap_ms = med.get("attn_nomap", attn_ms)
    fused_ms, fused_training_ms = med.get("fused"), med.get("fused_training")
    del lse_t, packed_t
    # the backward (dQ kernel, then dK/dV kernel) on the forward's saved out and lse
    lse = torch.empty(w.B, w.H, w.N, dtype=torch.float32, device=dev)
    ext.forward(qd, kd, vd, packed, out, lse, scale, True)
    dout = torch.randn(qd.shape, generator=torch.Generator().manual_seed(43)).to(qd.dtype).to(dev)
    dq, dk, dv = (torch.empty_like(qd) for _ in range(3))
    bwd_call = lambda: ext.backward(dout, qd, kd, vd, out, lse, packed, dq, dk, dv, scale, tmap)
    settle(bwd_call, torch)
    bwd_ms = sorted(event_time_ms(bwd_call, 5, reps, torch) for _ in range(3))[1]
    bwd_tflops = w.bwd_dense_flops / (bwd_ms * 1e-3) / 1e12

    # ---- the same kernels with nothing cached: rotate through copies of every tensor (> 512 MB) ----
    set_bytes = 4 * qd.numel() * qd.element_size() + md.numel() + packed.numel() * 4
    n_sets = max(3, -(-(640 << 20) // set_bytes))
    copies = [(qd.clone(), kd.clone(), vd.clone(), md.clone(), packed.clone(), torch.empty_like(qd))
              for _ in range(n_sets)]
    settle(kernels["attn"], torch)
    attn_cold_ms = cold_time_ms(lambda i: (lambda c=copies[i]: ext.forward(c[0], c[1], c[2], c[4], c[5], None, scale,
                                                                            False, tmap)), n_sets, 10, reps, torch)
    pack_cold_ms = cold_time_ms(lambda i: (lambda c=copies[i]: lib.sma_pack_mask(c[3].data_ptr(), c[4].data_ptr(),
                                                                                 w.B, w.H, w.N, stream)),
                                n_sets, 10, reps, torch)
    fused_cold_ms = None
    if one_launch:
        fused_cold_ms = cold_time_ms(lambda i: (lambda c=copies[i]: ext.forward_bool_mask(c[0], c[1], c[2], c[3], c[5],
                                                                                          None, scale, False)),
                                     n_sets, 10, reps, torch)
    del copies

    # FLOP the kernel really executes: 32-row x 64-key blocks of the mask that hold a set bit
    # (a wavefront skips the others), 4*32*64*D each, so that skipping is not mistaken for MFMA speed
    Np32, Np64 = -(-w.N // 32) * 32, -(-w.N // 64) * 64
    mp = torch.zeros(w.B, w.H, Np32, Np64, dtype=torch.bool, device=dev)
    mp[:, :, :w.N, :w.N] = md
    live = int(mp.view(w.B, w.H, Np32 // 32, 32, Np64 // 64, 64).any(dim=5).any(dim=3).sum().item())
    executed_flops = live * 4 * 32 * 64 * w.D
    del mp
    attn_tflops = w.dense_flops / (attn_ms * 1e-3) / 1e12
    pack_gbps = w.pack_bytes / (pack_ms * 1e-3) / 1e9
    result = {
        "metric": "dense_equiv_tflops_sparse_attention_fwd_incl_pack_mask",
        "value": round(value, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": (round(value / PUBLISHED_TFLOPS[w.name], 3) if w.name in PUBLISHED_TFLOPS else None),
        "vs_baseline_note": "the published figure is the reference's kernel on an RTX 3080 (README.md:13): other hardware",
        "dtype": "fp16" if w.dtype == torch.float16 else "bf16",
        "data": "synthetic",
        "preconditioning": f"{args.precondition_ms:.0f} ms of the same step, untimed, before the {args.warmup} warm-up steps "
                           "(the device's clock ramps for ~30 ms after idling)",
        "config": {"workload": f"{w.name}: B={w.B} H={w.H} N={w.N} D={w.D} {w.mask_kind} mask keep_p={w.keep_prob}",
                   "step": ("torch.empty_like + forward_bool_mask via sparse_attn_cuda (bool mask in, one launch, no LSE)"
                            if one_launch else
                            "pack_mask + torch.empty_like + forward via sparse_attn_cuda (no LSE)"),
                   "dense_equiv_flop_per_step": w.dense_flops},
        "step_pack_then_attention_ms": round(two_launch_ms, 5),
        "step_pack_then_attention_tflops": round(w.dense_flops / (two_launch_ms * 1e-3) / 1e12, 3),
        "kernel_timing": "stream events around back-to-back launches; three rounds over all kernels, median round of each",
        "attn_kernel_ms": round(attn_ms, 5),
        "attn_kernel_without_tile_map_ms": round(attn_nomap_ms, 5),
        "attn_kernel_cold_ms": round(attn_cold_ms, 5),
        "pack_kernel_cold_ms": round(pack_cold_ms, 5),
        "cold_sets": n_sets,
        "attn_kernel_tflops": round(attn_tflops, 2),
        "attn_kernel_hbm_gbps": round(w.attn_bytes / (attn_ms * 1e-3) / 1e9, 1),
        "attn_kernel_executed_tflops": round(executed_flops / (attn_ms * 1e-3) / 1e12, 2),
        "attn_live_block_fraction": round(executed_flops / w.dense_flops, 4) if w.N % 64 == 0 else None,
        "pack_kernel_ms": round(pack_ms, 5),
        "backward_ms": round(bwd_ms, 5),
        "api_sparse_attention_func_ms": round(api_ms, 5),
        "roofline_attn": {"kernel": "attn_fwd_kernel (packed mask" + (", tile map)" if tmap is not None else ")"),
                          "bound": "mfma", "achieved": round(attn_tflops, 2),
                          "peak": harness.MI355X_MFMA_F16_TFLOPS, "unit": "TFLOP/s",
                          "frac": round(attn_tflops / harness.MI355X_MFMA_F16_TFLOPS, 4),
                          "frac_cold": round(w.dense_flops / (attn_cold_ms * 1e-3) / 1e12 / harness.MI355X_MFMA_F16_TFLOPS, 4),
                          "hbm_gbps": round(w.attn_bytes / (attn_ms * 1e-3) / 1e9, 1),
                          "hbm_frac": round(w.attn_bytes / (attn_ms * 1e-3) / 1e9 / harness.MI355X_HBM_GBPS, 4),
                          "hbm_frac_cold": round(w.attn_bytes / (attn_cold_ms * 1e-3) / 1e9 / harness.MI355X_HBM_GBPS, 4),
                          "traffic": measured_traffic(w.name, "attn_fwd_kernel"), "algorithmic_bytes": w.attn_bytes},
        "roofline_pack": {"kernel": "pack_flat_kernel" if w.N % 32 == 0 else ("pack_row_kernel" if w.N >= 8 else "pack_short_rows_kernel"),
                          "bound": "hbm", "achieved": round(pack_gbps, 1), "peak": harness.MI355X_HBM_GBPS,
                          "unit": "GB/s", "frac": round(pack_gbps / harness.MI355X_HBM_GBPS, 4),
                          "frac_cold": round(w.pack_bytes / (pack_cold_ms * 1e-3) / 1e9 / harness.MI355X_HBM_GBPS, 4),
                          "cache_note": "frac: same mask every launch (last-level cache warm); frac_cold: HBM",
                          "traffic": measured_traffic(w.name, "pack_mask_kernel"), "algorithmic_bytes": w.pack_bytes},
        "roofline_bwd": {"kernel": "attn_bwd_dq_kernel + attn_bwd_dkv_kernel", "bound": "mfma",
                         "achieved": round(bwd_tflops, 2), "peak": harness.MI355X_MFMA_F16_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(bwd_tflops / harness.MI355X_MFMA_F16_TFLOPS, 4),
                         "traffic": measured_traffic(w.name, "attn_bwd_dq_kernel", "attn_bwd_dkv_kernel"), "algorithmic_bytes": w.bwd_bytes},
    }

    result["roofline_attn"].update(roofline_ceiling(w.dense_flops, w.attn_bytes, attn_tflops))
    if one_launch:
        gbps = w.fused_bytes / (fused_ms * 1e-3) / 1e9
        tfl = w.dense_flops / (fused_ms * 1e-3) / 1e12
        result["fused_kernel_ms"] = round(fused_ms, 5)
        result["fused_kernel_with_lse_and_packed_words_ms"] = round(fused_training_ms, 5)
        cold_gbps = w.fused_bytes / (fused_cold_ms * 1e-3) / 1e9
        cold_tfl = w.dense_flops / (fused_cold_ms * 1e-3) / 1e12
        result["fused_kernel_cold_ms"] = round(fused_cold_ms, 5)
        result["roofline"] = {"kernel": "attn_fwd_kernel (boolean mask in)", "bound": "mfma", "achieved": round(tfl, 2),
                              "peak": harness.MI355X_MFMA_F16_TFLOPS, "unit": "TFLOP/s",
                              "frac": round(tfl / harness.MI355X_MFMA_F16_TFLOPS, 4),
                              "frac_cold": round(cold_tfl / harness.MI355X_MFMA_F16_TFLOPS, 4),
                              "traffic": measured_traffic(w.name, "attn_fwd_bool_mask_kernel"),
                              "algorithmic_bytes": w.fused_bytes,
                              "flop_per_byte": round(w.dense_flops / w.fused_bytes, 1),
                              "hbm_gbps": round(gbps, 1),
                              "hbm_frac": round(gbps / harness.MI355X_HBM_GBPS, 4),
                              "hbm_frac_cold": round(cold_gbps / harness.MI355X_HBM_GBPS, 4),
                              "cache_note": "frac / hbm_frac: same tensors every launch, working set inside the 256 MB "
                                            "last-level cache (the reference's protocol); *_cold: rotating copies, "
                                            "every launch reads from HBM"}
        result["roofline"].update(roofline_ceiling(w.dense_flops, w.fused_bytes, tfl))
    else:
        result["roofline"] = dict(result["roofline_attn"])

    # ---- what this GPU sustains on a pure stream of the kernels' MFMA, and at what clock ----
    # (benchmark infrastructure in a library of its own, benchprobe/mfma_probe.h: not part of libsma_hip.so)
    probe_lib = ctypes.CDLL(os.path.join(PKG, "libsma_probe.so"))
    probe_lib.sma_probe_mfma_stream.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    n_cu = torch.cuda.get_device_properties(0).multi_processor_count
    stamps = torch.zeros(2 * n_cu, dtype=torch.int64, device=dev)
    probe = {}
    for label, rnd in (("zero_operands", 0), ("random_operands", 1)):
        iters = 20000
        probe_lib.sma_probe_mfma_stream(rnd, 2000, n_cu, stamps.data_ptr(), stream)
        ms = event_time_ms(lambda: probe_lib.sma_probe_mfma_stream(rnd, iters, n_cu, stamps.data_ptr(), stream), 1, 3, torch)
        st = stamps.view(n_cu, 2).double().cpu()
        flops = n_cu * 12 * 8 * iters * 2.0 * 32 * 32 * 16
        probe[label] = {"tflops": round(flops / (ms * 1e-3) / 1e12, 1),
                        "shader_clock_ghz": round(float((st[:, 0] / (st[:, 1] * 10.0)).mean()), 3)}
    result["mfma_stream_probe"] = dict(
        probe, note="pure stream of v_mfma_f32_32x32x16_f16, three wavefronts per SIMD on every CU; the data-sheet "
                    "peak (2516.6 TFLOP/s) assumes 2.4 GHz, the part lowers its clock under MFMAs on real data")
    sustained = probe["random_operands"]["tflops"]
    for key in ("roofline", "roofline_attn", "roofline_bwd"):
        result[key]["frac_of_sustained_mfma"] = round(result[key]["achieved"] / sustained, 4)

    if not args.no_cpu_baseline:
        from oracle import sma_oracle
        import numpy as np
        threads = torch.get_num_threads()
        sec = sma_oracle.time_cpu_reference(q.float(), k.float(), v.float(), mask, reps=3)
        # the input dtype as it is (what the reference's run.py:461 times as "PyTorch Ref")
        sec_native = sma_oracle.time_cpu_reference(q, k, v, mask, reps=3)
        # the CPU bit-packer: numpy.packbits(bitorder="little") on the whole mask
        m_np = mask.numpy()
        ts = []
        for _ in range(4):
            t0 = time.perf_counter()
            sma_oracle.pack_mask_ref(m_np)
            ts.append(time.perf_counter() - t0)
        sec_pack = sorted(ts[1:])[1]
        result["cpu_baseline"] = {
            "value": round(w.dense_flops / sec / 1e12, 5), "unit": "TFLOP/s", "cores": threads,
            "kind": "port", "ms": round(sec * 1e3, 2), "cpu": cpu_model(),
            "sample": f"whole {w.name} workload, fp32 PyTorch formulation of the oracle on the host CPU, "
                      f"median of 3 after 1 warm-up, torch threads={threads}, os.cpu_count()={os.cpu_count()}",
            "variants": {
                "native_dtype": {"value": round(w.dense_flops / sec_native / 1e12, 5), "unit": "TFLOP/s",
                                 "ms": round(sec_native * 1e3, 2), "cores": threads,
                                 "sample": f"the same in the inputs' own dtype ({'fp16' if w.dtype == torch.float16 else 'bf16'}), "
                                           "whole workload, median of 3"},
                "pack_mask": {"value": round(w.pack_bytes / sec_pack / 1e9, 3), "unit": "GB/s",
                              "ms": round(sec_pack * 1e3, 2), "cores": 1,
                              "sample": "numpy.packbits(bitorder='little') of the whole mask (the oracle's packer), "
                                        "median of 3 after 1 warm-up, one thread"}}}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
