"""The committed fixture tests/golden/c1_fp16.npz against the oracle (CPU) and the HIP path (GPU)."""
import os

import numpy as np
import pytest
import torch

from oracle import sma_oracle as O
from oracle import sma_oracle_c as OC

HERE = os.path.dirname(os.path.abspath(__file__))


def _load():
    z = np.load(os.path.join(HERE, "golden", "c1_fp16.npz"))
    q, k, v = (torch.from_numpy(z[n].view(np.float16).copy()) for n in ("q", "k", "v"))
    mask = torch.from_numpy(np.unpackbits(z["mask_bits"], axis=-1).astype(bool))
    return q, k, v, mask, z


def test_oracle_reproduces_the_fixture():
    q, k, v, mask, z = _load()
    assert mask.shape == (1, 2, 128, 128) and not mask[0, 1, 17].any()
    assert np.array_equal(O.pack_mask_ref(mask), z["packed"])
    assert np.array_equal(OC.pack_mask(mask.numpy()), z["packed"])
    out = O.sparse_attention_ref(q.float(), k.float(), v.float(), mask).numpy()
    assert np.allclose(out, z["out"], atol=1e-6, rtol=1e-5)
    c_out, c_lse = OC.attn_fwd(q.float().numpy(), k.float().numpy(), v.float().numpy(), mask.numpy(), 0.125)
    assert np.allclose(c_out, z["out"], atol=2e-6, rtol=1e-5)
    fin = np.isfinite(z["lse"])
    assert np.allclose(c_lse[fin], z["lse"][fin], atol=1e-5) and (c_lse[~fin] == -np.inf).all()
    assert (~fin).sum() == 1 and (z["out"][0, 1, 17] == 0).all()
    dout = torch.from_numpy(z["dout"].view(np.float16).copy())
    grads = O.sparse_attention_bwd_ref(q.float(), k.float(), v.float(), mask, dout.float())
    for got, name in zip(grads, ("dq", "dk", "dv")):
        assert np.allclose(got.numpy(), z[name], atol=1e-6, rtol=1e-5), name
    assert (z["dq"][0, 1, 17] == 0).all()


@pytest.mark.gpu
def test_hip_path_matches_the_fixture(dev):
    import _capi
    q, k, v, mask, z = _load()
    packed = _capi.pack_mask(mask.to(dev))
    assert np.array_equal(packed.cpu().numpy(), z["packed"])
    out, lse = _capi.attn_fwd(q.to(dev), k.to(dev), v.to(dev), packed, want_lse=True)
    torch.cuda.synchronize()
    assert torch.allclose(out.float().cpu(), torch.from_numpy(z["out"]), atol=1e-2, rtol=1e-2)
    fin = np.isfinite(z["lse"])
    assert np.allclose(lse.cpu().numpy()[fin], z["lse"][fin], atol=2e-3)
    assert (lse.cpu().numpy()[~fin] == -np.inf).all()
    assert (out[0, 1, 17] == 0).all()


@pytest.mark.gpu
def test_hip_backward_matches_the_fixture(dev):
    import _capi
    q, k, v, mask, z = _load()
    dout = torch.from_numpy(z["dout"].view(np.float16).copy())
    packed = _capi.pack_mask(mask.to(dev))
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    out, lse = _capi.attn_fwd(qd, kd, vd, packed, want_lse=True)
    dq, dk, dv, _ = _capi.attn_bwd(dout.to(dev), qd, kd, vd, out, lse, packed)
    torch.cuda.synchronize()
    for got, name in ((dq, "dq"), (dk, "dk"), (dv, "dv")):
        ref = torch.from_numpy(z[name])
        bound = 1e-4 + 1e-2 * ref.abs().max() + 1e-2 * ref.abs()
        assert ((got.float().cpu() - ref).abs() <= bound).all(), name
    assert (dq[0, 1, 17] == 0).all()
