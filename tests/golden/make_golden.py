"""Writes tests/golden/c1_fp16.npz: the tiny configuration (B=1, H=2, N=128, D=64, fp16, 75 % random
sparsity, seed 42) with what the CPU oracle computes for it.

The reference ships no golden vectors for this path, and its Python file was not imported to make
these: the expected values come from oracle/sma_oracle.py, whose functions are pinned by
tests/test_oracle.py.  The fixture freezes inputs and expected outputs so that neither a change of
the oracle nor of the random generator can go unnoticed.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "sparse-mask-attention_amd"))

import harness  # noqa: E402
from oracle import sma_oracle as O  # noqa: E402


def main():
    q, k, v, mask = harness.make_inputs("C1", seed=42)
    mask = mask.clone()
    mask[0, 1, 17, :] = False                     # one query row that keeps nothing
    out = O.sparse_attention_ref(q.float(), k.float(), v.float(), mask)
    lse = O.lse_ref(q, k, mask)
    # backward: a fixed upstream gradient and the closed-form gradients of the oracle
    import torch
    dout = (torch.randn(q.shape, generator=torch.Generator().manual_seed(43)) * 0.5).to(q.dtype)
    dq, dk, dv = O.sparse_attention_bwd_ref(q.float(), k.float(), v.float(), mask, dout.float())
    np.savez_compressed(
        os.path.join(os.path.dirname(os.path.abspath(__file__)), "c1_fp16.npz"),
        q=q.numpy().view(np.uint16), k=k.numpy().view(np.uint16), v=v.numpy().view(np.uint16),
        mask_bits=np.packbits(mask.numpy(), axis=-1),           # MSB-first numpy default, storage only
        packed=O.pack_mask_ref(mask), out=out.numpy(), lse=lse.numpy(),
        dout=dout.numpy().view(np.uint16), dq=dq.numpy(), dk=dk.numpy(), dv=dv.numpy())


if __name__ == "__main__":
    main()
