"""CPU checks of address arithmetic that a GPU run cannot judge (an over-read of a few bytes usually
lands in mapped memory).  First, the forward that reads the boolean mask
(csrc/attn_fwd.hip, issue_mask / mask_words): restated here with numpy for every lane of every wave,
so that for every sequence length
  * each lane offset is a non-negative 32-bit number (the hardware adds it unsigned to the base),
  * each 16-byte copy lies inside the N*N bytes of its (b,h) mask (nothing before the first or
    after the last byte is read),
  * the chunk a lane converts holds the 16 columns it stands for, or, for the chunk that contains
    the row's end, those columns after the right shift the kernel applies.
Second, the same forward when it requests two tiles' bytes at once; third, the packer's row loads
(csrc/pack_mask.hip), further down."""
import numpy as np
import pytest

BM, BN = 128, 64


def _check(N):
    T = (N + BN - 1) // BN
    ragged = N % BN != 0
    qtiles = (N + BM - 1) // BM
    lane = np.arange(64)
    for qt in {0, qtiles - 1}:
        for wave in range(4):
            for x in {0, T - 2, T - 1} & set(range(T)):
                base = x * BN
                for j in range(2):
                    row = 16 * j + (lane >> 2)
                    grow = qt * BM + wave * 32 + row
                    grow = np.where(grow < N, grow, N - 1).astype(np.int64)
                    chunk = ((lane & 3) ^ ((row >> 2) & 3)) << 4
                    voff = grow * N + chunk
                    src = base
                    row_end = N - x * BN
                    if ragged and x == T - 1:
                        back = 16 if x > 0 else 0
                        src -= back
                        voff = voff + back
                        voff = np.where(chunk + 16 > row_end, voff - (chunk + 16 - row_end), voff)
                    assert src >= 0 and (voff >= 0).all() and (voff < 2**32).all(), (N, x)
                    addr = src + voff
                    assert (addr >= 0).all() and (addr + 16 <= N * N).all(), (N, x)
                    col0 = addr - grow * N                      # first column the copy holds
                    want0 = x * BN + chunk
                    whole = want0 + 16 <= N
                    assert (col0[whole] == want0[whole]).all(), (N, x)
                    part = (want0 < N) & ~whole                 # the chunk that holds the row's end
                    shift = (16 - (row_end & 15)) & 15
                    assert ((chunk[part] >> 4) == (row_end >> 4)).all() and (col0[part] + shift == want0[part]).all(), (N, x)


def test_every_length_up_to_1100():
    for N in range(16, 1101):
        _check(N)


@pytest.mark.parametrize("N", [2047, 4095, 8191, 46340])
def test_long_rows(N):
    _check(N)


def _check_pairs(N):
    """The same forward when it requests the bytes of two key tiles at once (attn_fwd.hip,
    issue_mask_pair / mask_words with pair_half; N a multiple of 128): restated for every lane of
    every wave and every pair, so that each 16-byte copy lies inside the row it is meant for, every
    chunk of the pair lands exactly once in the wave's 4 KiB, and the two chunks a lane reads for a
    tile are the 32 columns it stands for."""
    assert N % 128 == 0
    qtiles = N // BM
    lane = np.arange(64)
    for qt in {0, qtiles - 1}:
        for wave in range(4):
            for p in {0, N // 128 - 1}:
                lds = np.full((32, 8), -1, dtype=np.int64)        # [row][position] -> first column held
                r = lane >> 3
                voff0 = (qt * BM + wave * 32 + r).astype(np.int64) * N + (((lane & 7) ^ (r >> 1)) << 4)
                for j in range(4):
                    voff = voff0 ^ 64 if j & 1 else voff0
                    assert (voff >= 0).all() and (voff < 2**32).all()
                    addr = p * 128 + 8 * j * N + voff
                    row = 8 * j + r
                    grow = qt * BM + wave * 32 + row
                    col0 = addr - grow.astype(np.int64) * N
                    assert (col0 >= p * 128).all() and (col0 + 16 <= (p + 1) * 128).all(), (N, p, j)
                    assert (grow < N).all() and (addr + 16 <= N * N).all()
                    dst = j * 1024 + lane * 16                      # byte in the wave's 4 KiB
                    assert ((dst >> 7) == row).all()
                    lds[row, (dst >> 4) & 7] = col0
                assert (lds >= 0).all()
                for half in range(2):                               # which tile of the pair
                    for l32 in range(32):
                        for hh in range(2):
                            psw = (l32 >> 1) & 7
                            for k in range(2):
                                pos = (4 * half + 2 * hh + k) ^ psw
                                assert lds[l32, pos] == p * 128 + half * 64 + 32 * hh + 16 * k, (N, p, half, l32, hh, k)


def test_pairs_of_tiles():
    for N in (128, 640, 768, 1024, 2048, 4096, 46336):
        _check_pairs(N)


def _check_packer_row(N, lanes_per_row=64):
    """csrc/pack_mask.hip, pack_row_kernel / pack_few_lanes_per_row_kernel: lane l of a segment takes
    the 8 bytes at column 8l, or the row's last 8 bytes shifted down when those would cross the
    row's end; restated with numpy on one row of distinct bits."""
    rng = np.random.default_rng(N)
    row = rng.integers(0, 2, N).astype(np.uint8)
    nw = (N + 31) // 32
    words = np.zeros(nw, dtype=np.uint64)
    seg_bytes = 8 * lanes_per_row
    for seg in range((N + seg_bytes - 1) // seg_bytes):
        for lane in range(lanes_per_row):
            col = seg * seg_bytes + lane * 8
            start = col if col + 8 <= N else N - 8
            assert 0 <= start and start + 8 <= N, (N, col)           # the load stays inside the row
            v = int.from_bytes(row[start:start + 8].tobytes(), "little")
            if col + 8 > N:
                v = v >> (8 * (col + 8 - N)) if col < N else 0
            bits = sum(((v >> (8 * i)) & 1) << i for i in range(8))
            w = col // 32
            if w < nw:
                words[w] |= np.uint64(bits << (8 * (lane & 3)))
    want = np.zeros(nw, dtype=np.uint64)
    for c in range(N):
        want[c // 32] |= np.uint64(int(row[c]) << (c % 32))
    assert (words == want).all(), N


def test_packer_row_loads_stay_inside_the_row_and_place_every_bit():
    for N in list(range(8, 600)) + [999, 1000, 1001, 1023, 1025, 2047]:
        _check_packer_row(N)
    for N in range(8, 257):                                  # the kernel with fewer lanes per row
        lanes = 4
        while 8 * lanes < N:
            lanes *= 2
        _check_packer_row(N, lanes)
