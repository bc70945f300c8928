"""Workloads and timing protocol for sparse-mask attention on MI355X.

The counterpart of the reference's ``run.py`` harness, reduced to what the hot path needs:

* the five benchmark configurations (inputs are generated on the CPU from an explicit
  ``torch.Generator`` seed, in the fixed order q, k, v, mask, so that every machine sees the same
  tensors; the reference seeds the CUDA generator, ``run.py:361-365``, which no other device can
  reproduce);
* ``generate_mask``     random mask of a given sparsity, ``run.py:168-169``;
* ``measure_latency``   10 warm-up calls, then 50 back-to-back calls between two stream events,
                        mean milliseconds, ``run.py:172-183``;
* ``compute_mfu``       dense-equivalent FLOPs ``4*B*H*N*N*D`` whatever the sparsity,
                        ``run.py:198-203``.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

# Dense FP16/BF16 MFMA peak of one MI355X: 256 CUs x 4096 FLOP/clk x 2.4 GHz.
MI355X_MFMA_F16_TFLOPS = 2516.6
# HBM3E peak of one MI355X.
MI355X_HBM_GBPS = 8000.0


@dataclass(frozen=True)
class Workload:
    name: str
    B: int
    H: int
    N: int
    D: int
    dtype: torch.dtype
    mask_kind: str          # "random" | "block64" | "random_diag" | "causal_random"
    keep_prob: float
    qkv_std: float = 1.0

    @property
    def n_words(self) -> int:
        return (self.N + 31) // 32

    @property
    def dense_flops(self) -> int:
        return 4 * self.B * self.H * self.N * self.N * self.D

    @property
    def attn_bytes(self) -> int:
        """Algorithmic bytes of one attention launch: q, k, v, out (2 B/element) + packed mask."""
        return 4 * self.B * self.H * self.N * self.D * 2 + 4 * self.B * self.H * self.N * self.n_words

    @property
    def fused_bytes(self) -> int:
        """Algorithmic bytes of the forward that reads the boolean mask itself: q, k, v, out and one
        byte per score."""
        return 4 * self.B * self.H * self.N * self.D * 2 + self.B * self.H * self.N * self.N

    @property
    def bwd_dense_flops(self) -> int:
        """Dense-equivalent FLOP of the backward, by the usual convention 2.5 x the forward: the five
        N x N x D products dV, dP, dQ, dK and the recomputed S (what the kernels execute is seven,
        S and dP are formed in both)."""
        return 10 * self.B * self.H * self.N * self.N * self.D

    @property
    def bwd_bytes(self) -> int:
        """Algorithmic bytes of one backward (both launches): the dQ kernel reads q, k, v, dout, out,
        the mask and lse and writes dq and delta; the dK/dV kernel reads q, k, v, dout, the mask, lse
        and delta and writes dk and dv."""
        mat = self.B * self.H * self.N * self.D * 2
        mask = 4 * self.B * self.H * self.N * self.n_words
        vec = 4 * self.B * self.H * self.N
        return (6 * mat + mask + 2 * vec) + (6 * mat + mask + 2 * vec)

    @property
    def pack_bytes(self) -> int:
        """Algorithmic bytes of one pack_mask launch: one byte in per entry + the words out."""
        return self.B * self.H * self.N * self.N + 4 * self.B * self.H * self.N * self.n_words


WORKLOADS = {
    # tiny CPU-runnable case
    "C1": Workload("C1", 1, 2, 128, 64, torch.float16, "random", 0.25),
    # headline shape
    "C2": Workload("C2", 16, 12, 512, 64, torch.float16, "random", 0.25),
    # 64x64 block-structured mask: diagonal blocks kept, off-diagonal kept with p = 0.25
    "C3": Workload("C3", 16, 12, 1024, 64, torch.float16, "block64", 0.25),
    # bf16, ragged length, 90 % sparse, diagonal forced
    "C4": Workload("C4", 8, 16, 1000, 64, torch.bfloat16, "random_diag", 0.10, 0.5),
    # causal AND Bernoulli(0.5), diagonal forced
    "C5": Workload("C5", 64, 16, 256, 64, torch.float16, "causal_random", 0.5),
}


def generate_mask(B, H, N, sparsity=0.75, device="cpu", generator=None):
    """bool [B,H,N,N]; an entry is True (attend) with probability 1 - sparsity."""
    return torch.rand(B, H, N, N, device=device, generator=generator) > sparsity


def make_mask(w: Workload, generator: torch.Generator) -> torch.Tensor:
    B, H, N = w.B, w.H, w.N
    if w.mask_kind == "random":
        return generate_mask(B, H, N, 1.0 - w.keep_prob, generator=generator)
    if w.mask_kind == "block64":
        nb = (N + 63) // 64
        blocks = torch.rand(B, H, nb, nb, generator=generator) > (1.0 - w.keep_prob)
        blocks |= torch.eye(nb, dtype=torch.bool)
        full = blocks.repeat_interleave(64, dim=2).repeat_interleave(64, dim=3)
        return full[:, :, :N, :N].contiguous()
    if w.mask_kind == "random_diag":
        m = generate_mask(B, H, N, 1.0 - w.keep_prob, generator=generator)
        return m | torch.eye(N, dtype=torch.bool)
    if w.mask_kind == "causal_random":
        m = generate_mask(B, H, N, 1.0 - w.keep_prob, generator=generator)
        m &= torch.tril(torch.ones(N, N, dtype=torch.bool))
        return m | torch.eye(N, dtype=torch.bool)
    raise ValueError(w.mask_kind)


def make_inputs(w: Workload | str, seed: int = 42, device="cpu"):
    """q, k, v (w.dtype) and mask (bool) for a workload, generated on the CPU, then moved."""
    if isinstance(w, str):
        w = WORKLOADS[w]
    g = torch.Generator().manual_seed(seed)
    shape = (w.B, w.H, w.N, w.D)
    q = (torch.randn(shape, generator=g) * w.qkv_std).to(w.dtype)
    k = (torch.randn(shape, generator=g) * w.qkv_std).to(w.dtype)
    v = (torch.randn(shape, generator=g) * w.qkv_std).to(w.dtype)
    mask = make_mask(w, g)
    return tuple(t.to(device) for t in (q, k, v, mask))


def measure_latency(fn, warmup: int = 10, repeat: int = 50) -> float:
    """Mean milliseconds per call over `repeat` back-to-back calls on the current stream."""
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


def compute_mfu(latency_ms, B, H, N, D, peak_tflops=MI355X_MFMA_F16_TFLOPS):
    """(dense-equivalent TFLOP/s, percent of peak) for one forward of the given shape."""
    flops = 4 * B * H * N * N * D
    tflops = flops / (latency_ms * 1e-3) / 1e12
    return tflops, 100.0 * tflops / peak_tflops
