"""Pins of the CPU oracle (no GPU): library routines, known answers, closed forms, brute force.

The reference ships no golden vectors for this path (its only checks are tolerance runs against
its own PyTorch formulation on CUDA-seeded inputs, run.py:355-376 and :387-396), so the oracle is
pinned by what the format and the mathematics fix.  Each test is chosen so that a plausible slip
(MSB-first bits, wrong word order, non-zero pad bits, a transposed operand, a missing scale, a
wrong empty-row convention) fails it.
"""
import math

import numpy as np
import pytest
import scipy.special
import torch

from oracle import sma_oracle as O
from oracle import sma_oracle_c as OC


# ---------------------------------------------------------------- pack format

def test_pack_single_bit_known_answers():
    N = 70
    for c in (0, 1, 31, 32, 33, 63, 64, 69):
        m = np.zeros((1, 1, N, N), dtype=bool)
        m[0, 0, 5, c] = True
        p = O.pack_mask_ref(m).view(np.uint32)
        assert p.shape == (1, 1, N, 3)
        expect = np.zeros((N, 3), dtype=np.uint32)
        expect[5, c // 32] = np.uint32(1) << np.uint32(c % 32)
        assert np.array_equal(p[0, 0], expect), c
    # column 31 sets the sign bit of the int32 word, as `int32 << 31` does in the reference's
    # CPU fallback (python/sparse_attention.py:195-200)
    m = np.zeros((1, 1, 32, 32), dtype=bool)
    m[0, 0, 0, 31] = True
    assert O.pack_mask_ref(m)[0, 0, 0, 0] == -2**31


def test_pack_all_true_tail_words():
    p = O.pack_mask_ref(np.ones((1, 1, 8, 8), dtype=bool)).view(np.uint32)
    assert p.shape == (1, 1, 8, 1) and (p == 0xFF).all()
    p = O.pack_mask_ref(np.ones((1, 2, 1000, 1000), dtype=bool)).view(np.uint32)
    assert p.shape == (1, 2, 1000, 32)
    assert (p[..., :31] == 0xFFFFFFFF).all() and (p[..., 31] == 0xFF).all()   # 1000 = 31*32 + 8
    assert O.pack_mask_ref(np.ones((1, 1, 33, 33), dtype=bool)).dtype == np.int32


@pytest.mark.parametrize("N", [1, 8, 31, 32, 33, 64, 100])
def test_pack_three_statements_agree(N):
    rng = np.random.default_rng(N)
    m = rng.random((2, 3, N, N)) > 0.6
    a = O.pack_mask_ref(m)
    assert np.array_equal(a, O.pack_mask_loops(m))       # literal bit loop (Python)
    assert np.array_equal(a, OC.pack_mask(m))            # literal bit loop (C)


@pytest.mark.parametrize("N", [8, 33, 64, 257, 1000])
def test_pack_invariants(N):
    rng = np.random.default_rng(7 * N)
    m = rng.random((1, 2, N, N)) > 0.75
    p = O.pack_mask_ref(m)
    assert np.array_equal(O.unpack_mask_ref(p, N), m)                       # round trip
    bits = np.unpackbits(p.view(np.uint8), bitorder="little").sum()
    assert bits == m.sum()                                                  # popcount, pad bits 0
    tail = N % 32
    if tail:
        assert (p.view(np.uint32)[..., -1] >> np.uint32(tail) == 0).all()


def test_pack_accepts_torch_and_matches_reference_cpu_formula():
    # the reference's CPU fallback builds words with `|= mask[..., col].int() << bit`
    g = torch.Generator().manual_seed(3)
    m = torch.rand(1, 2, 40, 40, generator=g) > 0.5
    nw = 2
    expect = torch.zeros(1, 2, 40, nw, dtype=torch.int32)
    for col in range(40):
        expect[..., col // 32] |= m[..., col].int() << (col % 32)
    assert np.array_equal(O.pack_mask_ref(m), expect.numpy())


# ---------------------------------------------------------------- attention

def _rand(B, H, N, D, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(B, H, N, D, generator=g).to(dtype).float() for _ in range(3)]


def test_all_true_mask_is_dense_attention():
    q, k, v = _rand(2, 3, 50, 64, 0)
    mask = torch.ones(2, 3, 50, 50, dtype=torch.bool)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v)
    assert torch.allclose(O.sparse_attention_ref(q, k, v, mask), ref, atol=1e-5, rtol=1e-5)


def test_bool_mask_matches_sdpa_on_nonempty_rows():
    q, k, v = _rand(1, 2, 40, 64, 1)
    g = torch.Generator().manual_seed(11)
    mask = (torch.rand(1, 2, 40, 40, generator=g) > 0.75) | torch.eye(40, dtype=torch.bool)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask)   # True = keep
    assert torch.allclose(O.sparse_attention_ref(q, k, v, mask), ref, atol=1e-5, rtol=1e-5)


def test_one_hot_rows_return_the_selected_value_row():
    q, k, v = _rand(1, 1, 16, 64, 2)
    perm = torch.randperm(16, generator=torch.Generator().manual_seed(5))
    mask = torch.zeros(1, 1, 16, 16, dtype=torch.bool)
    mask[0, 0, torch.arange(16), perm] = True
    out = O.sparse_attention_ref(q, k, v, mask)
    assert torch.equal(out[0, 0], v[0, 0, perm])       # a transposed mask would give v[inverse perm]


def test_empty_rows_give_zeros_and_minus_inf_lse():
    q, k, v = _rand(1, 1, 8, 64, 3)
    mask = torch.ones(1, 1, 8, 8, dtype=torch.bool)
    mask[0, 0, 0, :] = False                            # the reference's own case, run.py:387-396
    out = O.sparse_attention_ref(q, k, v, mask)
    assert not torch.isnan(out).any()
    assert torch.equal(out[0, 0, 0], torch.zeros(64))
    lse = O.lse_ref(q, k, mask)
    assert lse[0, 0, 0] == -math.inf and torch.isfinite(lse[0, 0, 1:]).all()


def test_zero_queries_give_mean_of_kept_values():
    _, k, v = _rand(1, 2, 30, 64, 4)
    q = torch.zeros(1, 2, 30, 64)
    g = torch.Generator().manual_seed(9)
    mask = (torch.rand(1, 2, 30, 30, generator=g) > 0.5) | torch.eye(30, dtype=torch.bool)
    out = O.sparse_attention_ref(q, k, v, mask)
    w = mask.float() / mask.float().sum(-1, keepdim=True)
    assert torch.allclose(out, w @ v, atol=1e-6, rtol=1e-5)


def test_scale_is_one_over_sqrt_d_and_enters_the_scores():
    # two keys, scores differ by a known amount: softmax weights have a closed form
    D = 64
    q = torch.zeros(1, 1, 2, D); q[..., 0] = 8.0
    k = torch.zeros(1, 1, 2, D); k[0, 0, 1, 0] = 1.0      # scores (0, 8) -> scaled (0, 1)
    v = torch.zeros(1, 1, 2, D); v[0, 0, 0, 0] = 1.0; v[0, 0, 1, 1] = 1.0
    mask = torch.ones(1, 1, 2, 2, dtype=torch.bool)
    out = O.sparse_attention_ref(q, k, v, mask)
    p1 = math.e / (1.0 + math.e)
    assert out[0, 0, 0, 1].item() == pytest.approx(p1, rel=1e-6)
    assert out[0, 0, 0, 0].item() == pytest.approx(1.0 - p1, rel=1e-6)
    assert O.lse_ref(q, k, mask)[0, 0, 0].item() == pytest.approx(math.log(1.0 + math.e), rel=1e-6)


def test_key_permutation_invariance_and_row_independence():
    q, k, v = _rand(1, 2, 24, 64, 5)
    g = torch.Generator().manual_seed(13)
    mask = (torch.rand(1, 2, 24, 24, generator=g) > 0.6) | torch.eye(24, dtype=torch.bool)
    out = O.sparse_attention_ref(q, k, v, mask)
    perm = torch.randperm(24, generator=g)
    out_p = O.sparse_attention_ref(q, k[:, :, perm], v[:, :, perm], mask[:, :, :, perm])
    assert torch.allclose(out, out_p, atol=1e-6, rtol=1e-5)
    mask2 = mask.clone()
    mask2[:, :, 7, :] = ~mask2[:, :, 7, :]
    out2 = O.sparse_attention_ref(q, k, v, mask2)
    keep = torch.arange(24) != 7
    assert torch.equal(out[:, :, keep], out2[:, :, keep])


@pytest.mark.parametrize("N", [8, 33, 70])
def test_torch_numpy_and_c_statements_agree(N):
    q, k, v = _rand(1, 2, N, 64, 6 + N, dtype=torch.float16)
    g = torch.Generator().manual_seed(17)
    mask = torch.rand(1, 2, N, N, generator=g) > 0.75
    mask[0, 0, 1, :] = False
    scale = 1.0 / 8.0
    a = O.sparse_attention_ref(q, k, v, mask).numpy()
    b, lse_b = O.attention_f64_loops(q.numpy(), k.numpy(), v.numpy(), mask)
    c, lse_c = OC.attn_fwd(q.numpy(), k.numpy(), v.numpy(), mask.numpy(), scale)
    assert np.allclose(a, b, atol=2e-6, rtol=1e-5)
    assert np.allclose(c, b, atol=2e-6, rtol=1e-5)
    lse_a = O.lse_ref(q, k, mask).numpy()
    assert np.allclose(lse_a, lse_b, atol=1e-5, equal_nan=False)
    assert np.allclose(lse_c, lse_b, atol=1e-5)
    assert lse_a[0, 0, 1] == -np.inf and lse_c[0, 0, 1] == -np.inf


def test_lse_matches_scipy_logsumexp():
    q, k, _ = _rand(1, 1, 12, 64, 8)
    g = torch.Generator().manual_seed(19)
    mask = (torch.rand(1, 1, 12, 12, generator=g) > 0.5) | torch.eye(12, dtype=torch.bool)
    s = (q[0, 0] @ k[0, 0].T).numpy() / 8.0
    expect = np.array([scipy.special.logsumexp(s[i][mask[0, 0, i].numpy()]) for i in range(12)])
    assert np.allclose(O.lse_ref(q, k, mask)[0, 0].numpy(), expect, atol=1e-5)


# ---------------------------------------------------------------------------
# backward: the closed form against automatic differentiation and finite differences
# ---------------------------------------------------------------------------

def _bwd_case(B, H, N, seed, keep=0.3, empty_row=True):
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = (torch.randn(B, H, N, 64, generator=g, dtype=torch.float64) for _ in range(4))
    mask = torch.rand(B, H, N, N, generator=g) < keep
    if empty_row and N > 2:
        mask[:, :, 1, :] = False          # a row that keeps nothing
        mask[:, :, :, 2] = False          # a key that nobody keeps
    return q, k, v, do, mask


@pytest.mark.parametrize("N", [1, 7, 33, 64])
def test_backward_closed_form_equals_autograd(N):
    q, k, v, do, mask = _bwd_case(2, 2, N, seed=100 + N)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = O.sparse_attention_ref(qa, ka, va, mask)
    out.backward(do)
    dq, dk, dv = O.sparse_attention_bwd_ref(q, k, v, mask, do)
    for got, ref in ((dq, qa.grad), (dk, ka.grad), (dv, va.grad)):
        assert torch.allclose(got, ref, atol=1e-12, rtol=1e-10)
    if N > 2:
        assert (dq[:, :, 1] == 0).all()                       # empty row: no gradient to its query
        assert (dk[:, :, 2] == 0).all() and (dv[:, :, 2] == 0).all()   # unused key: none either


def test_backward_closed_form_equals_finite_differences():
    q, k, v, do, mask = _bwd_case(1, 1, 5, seed=7, keep=0.6, empty_row=False)
    scale = 0.37
    dq, dk, dv = O.sparse_attention_bwd_ref(q, k, v, mask, do, scale=scale)
    f = lambda q_, k_, v_: (O.sparse_attention_ref(q_, k_, v_, mask, scale=scale) * do).sum().item()
    h = 1e-6
    for t, grad in ((q, dq), (k, dk), (v, dv)):
        for idx in [(0, 0, 0, 0), (0, 0, 3, 17), (0, 0, 4, 63)]:
            tp, tm = t.clone(), t.clone()
            tp[idx] += h
            tm[idx] -= h
            args_p = [tp if x is t else x for x in (q, k, v)]
            args_m = [tm if x is t else x for x in (q, k, v)]
            fd = (f(*args_p) - f(*args_m)) / (2 * h)
            assert abs(fd - grad[idx].item()) < 1e-6 * max(1.0, abs(fd))


def test_backward_all_true_mask_equals_dense_sdpa_autograd():
    q, k, v, do, _ = _bwd_case(1, 2, 16, seed=3)
    mask = torch.ones(1, 2, 16, 16, dtype=torch.bool)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    torch.nn.functional.scaled_dot_product_attention(qa, ka, va).backward(do)
    dq, dk, dv = O.sparse_attention_bwd_ref(q, k, v, mask, do)
    for got, ref in ((dq, qa.grad), (dk, ka.grad), (dv, va.grad)):
        assert torch.allclose(got, ref, atol=1e-10, rtol=1e-8)


def test_backward_with_delta_given_is_the_delta_free_form():
    """`delta=` only replaces rowsum(dattn * attn): with delta = sum_d dout * out of the exact `out` the
    gradients are those of the delta-free form (fp64), and a perturbed delta moves dq and dk by
    exactly attn * (-perturbation) * scale pushed through the last two products, dv not at all."""
    q, k, v, do, mask = _bwd_case(2, 2, 33, seed=55)
    scale = 0.21
    out = O.sparse_attention_ref(q, k, v, mask, scale=scale)
    delta = (do * out).sum(dim=-1, keepdim=True)
    plain = O.sparse_attention_bwd_ref(q, k, v, mask, do, scale=scale)
    given = O.sparse_attention_bwd_ref(q, k, v, mask, do, scale=scale, delta=delta)
    for a, b in zip(plain, given):
        assert torch.allclose(a, b, atol=1e-12, rtol=1e-10)
    eps = torch.randn(2, 2, 33, 1, generator=torch.Generator().manual_seed(56), dtype=torch.float64) * 1e-3
    moved = O.sparse_attention_bwd_ref(q, k, v, mask, do, scale=scale, delta=delta + eps)
    s = (q @ k.transpose(-1, -2)) * scale
    attn = torch.nan_to_num(torch.softmax(s.masked_fill(~mask, float("-inf")), dim=-1), nan=0.0)
    dds = attn * (-eps) * scale
    assert torch.allclose(moved[0] - plain[0], dds @ k, atol=1e-12)
    assert torch.allclose(moved[1] - plain[1], dds.transpose(-1, -2) @ q, atol=1e-12)
    assert torch.equal(moved[2], plain[2])


# ---------------------------------------------------------------------------
# tile map
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("N", [1, 63, 64, 65, 127, 128, 129, 200, 333])
def test_tile_map_equals_literal_loops(N):
    g = torch.Generator().manual_seed(N)
    mask = torch.rand(1, 2, N, N, generator=g) < 0.02            # sparse enough for empty blocks
    mask[0, 0, : min(N, 64), : min(N, 64)] = True                # and one full block
    assert np.array_equal(O.tile_map_ref(mask), O.tile_map_loops(mask))


def test_tile_map_known_answers():
    N = 200                                                      # 4 row blocks, 4 key tiles (last: 8 wide)
    assert O.tile_map_shape(N) == (4, 2, 1)
    ones = O.tile_map_ref(torch.ones(1, 1, N, N, dtype=torch.bool))
    assert (ones == 0xF).all()                                   # four tiles live and full, the ragged ones too
    zeros = O.tile_map_ref(torch.zeros(1, 1, N, N, dtype=torch.bool))
    assert (zeros == 0).all()
    one = torch.zeros(1, 1, N, N, dtype=torch.bool)
    one[0, 0, 130, 70] = True                                    # row block 2, key tile 1
    m = O.tile_map_ref(one)
    assert m[0, 0, 2, 0, 0] == 2 and m.sum() == 2                # one live bit, nothing full
    hole = torch.ones(1, 1, N, N, dtype=torch.bool)
    hole[0, 0, 5, 199] = False                                   # row block 0, key tile 3
    m = O.tile_map_ref(hole)
    assert m[0, 0, 0, 0, 0] == 0xF and m[0, 0, 0, 1, 0] == 0x7 and m[0, 0, 1, 1, 0] == 0xF
    # more than 32 key tiles: a second word
    N = 64 * 33
    assert O.tile_map_shape(N) == (33, 2, 2)
    last = torch.zeros(1, 1, N, N, dtype=torch.bool)
    last[0, 0, 0, N - 1] = True
    m = O.tile_map_ref(last)
    assert m[0, 0, 0, 0, 1] == 1 and m[0, 0, 0, 0, 0] == 0 and m.sum() == 1


def test_tiles_called_empty_do_not_matter():
    """Clearing what the map calls empty changes nothing, and every block it calls full is all True."""
    g = torch.Generator().manual_seed(5)
    N = 300
    blocks = torch.rand(1, 2, 5, 5, generator=g) < 0.4
    mask = blocks.repeat_interleave(64, 2).repeat_interleave(64, 3)[:, :, :N, :N] & (torch.rand(1, 2, N, N, generator=g) < 0.7)
    mask[0, 1, 128:192, 64:128] = True
    m = O.tile_map_ref(mask)
    QT, _, TW = O.tile_map_shape(N)
    kept = torch.zeros_like(mask)
    for h in range(2):
        for qt in range(QT):
            for t in range((N + 63) // 64):
                live = (int(m[0, h, qt, 0, t // 32]) >> (t % 32)) & 1
                full = (int(m[0, h, qt, 1, t // 32]) >> (t % 32)) & 1
                blk = mask[0, h, 64 * qt:64 * qt + 64, 64 * t:64 * t + 64]
                if live:
                    kept[0, h, 64 * qt:64 * qt + 64, 64 * t:64 * t + 64] = blk
                if full:
                    assert blk.all() and live
    assert torch.equal(kept, mask)
    assert (int(m[0, 1, 2, 1, 0]) >> 1) & 1
