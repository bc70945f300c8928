// Masked-attention backward for gfx950 (MI355X), head_dim 32, 64 or 128, fp16 / bf16, fp32 accumulate.
//
// The reference declares a backward launcher (csrc/sparse_attention.h:57-64) and its Python API
// calls sparse_attn_cuda.backward (python/sparse_attention.py:91-94), but neither was ever
// written; the formulas are those of its PyTorch fallback (python/sparse_attention.py:97-111):
//
//     P  = exp(scale * Q K^T - lse) on kept entries, 0 elsewhere      (lse saved by the forward)
//     dV = P^T dO          dP = dO V^T          delta_i = sum_d dO_id O_id  (= sum_j P_ij dP_ij)
//     dS = P o (dP - delta) * scale             dQ = dS K            dK = dS^T Q
//
// Two kernels, no atomics, bit-reproducible:
//
//   attn_bwd_dq_kernel   one work-group = 128 query rows, walks the key tiles exactly like the
//                        forward: S^T = K Q^T and dP^T = V dO^T on the MFMA (lane = query row, so
//                        lse and delta are per-lane scalars and the mask enters as the accumulator's
//                        initial value), dS^T packed to 16 bit is the B operand of dQ^T += K^T dS^T
//                        (K^T by transposing LDS reads).  Also writes delta to the workspace.
//   attn_bwd_dkv_kernel  one work-group = 128 keys (lane = key), walks the query tiles:
//                        S = Q K^T and dP = dO V^T with K, V fragments held in registers; -lse and
//                        -delta of the tile's rows are read from LDS (broadcast reads) straight
//                        into the accumulators as their initial values, so the products leave
//                        s - lse and dP - delta; the mask bit of (row, key) is bit (key % 32) of the
//                        row's word; P and dS packed to 16 bit are the B operands of
//                        dV^T += dO^T P and dK^T += Q^T dS.  The loop over the query tiles is
//                        unrolled by the two ring stages, so every LDS address in it is a
//                        register plus an immediate.
//
// Tiles (64 rows x 64 x 16 bit) are copied global -> LDS by global_load_lds_dwordx4 into two
// stages, one tile ahead; the 16-byte chunks of a row are XOR-swizzled with bitrev3((row >> 1) & 7),
// which keeps both the row reads (ds_read_b128) and the transposing reads (ds_read_b64_tr_b16) of
// the same tile free of bank conflicts.
//
// Head dim 128 (NH = 2) is handled as two column halves of 64: every streamed matrix is kept in LDS
// as two 64-column tiles, the products that contract over the head dim (S, dP) run over both
// halves, the others (dQ, dK, dV) fill one pair of accumulators per half.  The dK/dV kernel would
// need 128 accumulator registers for that; it is therefore launched twice, once for dK and once
// for dV (S is formed in both).  Head dim 32 uses half a tile: the copies fill the upper half of
// every LDS row with a second copy of the lower half (global chunk index & 3), which is never read;
// contractions over the head dim take two MFMA steps and the outputs have one 32-column block.
#include "attn_common.h"

namespace sma {
namespace {

constexpr int HD = 64;             // columns of one LDS tile: the head dim, or one half of a head dim of 128
constexpr int BM = 128;            // rows (queries or keys) per work-group
constexpr int BN = 64;             // rows per streamed tile
constexpr int NTHREADS = 256;
constexpr int TILE_BYTES = BN * HD * 2;
constexpr int NSTAGE = 2;
constexpr int AUX_BYTES = 2048;                             // small per-tile data of a stage
constexpr float LOG2E = 1.4426950408889634f;

// LDS map (bytes) for head dim 64 * NH: a stage holds the NH column halves of the first streamed
// matrix, then those of the second.
template <int NH> struct Cfg {
    static constexpr int STAGE_BYTES = 2 * NH * TILE_BYTES;
    static constexpr int OFF_B = NH * TILE_BYTES;           // second matrix inside a stage
    static constexpr int OFF_AUX = NSTAGE * STAGE_BYTES;
    static constexpr int OFF_LUT = OFF_AUX + NSTAGE * AUX_BYTES;
    static constexpr int LDS_BYTES = OFF_LUT + 256;
};

// Per-lane constants of the tile copies: wave w copies row blocks 2w and 2w+1 (8 rows each) of a
// 64-row tile; lane i fills LDS chunk (row 8*blk + i/8, position i%8) with global chunk
// position ^ bitrev3((row >> 1) & 7).
struct TileCopy {
    uint32_t chunk[2];      // byte offset of the lane's global chunk inside its row
    int row[2];
};
__device__ __forceinline__ TileCopy make_tile_copy(int wave, int lane, int chunk_mask)
{
    TileCopy c;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int row = 8 * (2 * wave + j) + (lane >> 3);
        const int pos = lane & 7;
        c.row[j] = row;
        c.chunk[j] = (uint32_t)(((pos ^ bitrev3((row >> 1) & 7)) & chunk_mask) << 4);
    }
    return c;
}
// Copy the tile whose first row is row r0 of the N-row matrix `mat` (row stride sn elements, below
// 2^23); rows >= N re-read row N-1 (they are zeroed after landing).
template <int NH>
__device__ __forceinline__ void issue_tile(uint32_t dst, const uint16_t *mat, uint32_t sn, int r0,
                                           int N, const TileCopy &c, int wave)
{
    const uint16_t *src = mat + (size_t)r0 * sn;
    const int last = N - 1 - r0;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int r = c.row[j] < last ? c.row[j] : last;
        const uint32_t voff = __umul24(r, 2u * sn) + c.chunk[j];
        async_copy_b128(dst + wave * 2048 + j * 1024, src, voff);
        if constexpr (NH == 2) async_copy_b128(dst + TILE_BYTES + wave * 2048 + j * 1024, src + HD, voff);
    }
}
// Zero the rows >= N of the `parts` consecutive 64-column tiles that start at dst.
__device__ __forceinline__ void zero_tile_tail(uint32_t dst, int parts, int r0, int N, const TileCopy &c,
                                               int wave, int lane)
{
#pragma unroll
    for (int j = 0; j < 2; ++j)
        if (r0 + c.row[j] >= N) {
            const u32x4 z = {0u, 0u, 0u, 0u};
            for (int part = 0; part < parts; ++part)
                *(LDS_PTR(u32x4))(uintptr_t)(dst + part * TILE_BYTES + wave * 2048 + j * 1024 + lane * 16) = z;
        }
}

// Per-lane LDS read offsets inside a tile (add the tile's base and 4096 per block of 32 rows).
//   rowaddr[s]       ds_read_b128: row l32, columns 16s + 8hh .. +7          (A operand, k-step s)
//   traddr[dblk][x]  ds_read_b64_tr_b16: rows 8x + 4hh + (i >> 2) (+16u), columns 32dblk + 16G +
//                    4(i & 3) .. +3, i = lane % 16, G = (lane % 32) / 16     (A operand = tile^T)
struct TileRead {
    uint32_t rowaddr[4];
    uint32_t traddr[2][2];
};
__device__ __forceinline__ TileRead make_tile_read(int lane)
{
    TileRead r;
    const int l32 = lane & 31, hh = lane >> 5;
    const int fk = bitrev3((l32 >> 1) & 7);
#pragma unroll
    for (int s = 0; s < 4; ++s) r.rowaddr[s] = (uint32_t)(l32 * 128 + (((2 * s + hh) ^ fk) << 4));
    const int i16 = lane & 15, G = l32 >> 4;
    const int r3 = 4 * hh + (i16 >> 2);
#pragma unroll
    for (int x = 0; x < 2; ++x) {
        const int row = 8 * x + r3;
        const int fr = bitrev3((row >> 1) & 7);
#pragma unroll
        for (int dblk = 0; dblk < 2; ++dblk) {
            const int chunk = 4 * dblk + 2 * G + ((i16 & 3) >> 1);
            r.traddr[dblk][x] = (uint32_t)(row * 128 + ((chunk ^ fr) << 4) + ((i16 & 1) << 3));
        }
    }
    return r;
}

// 16 bytes (8 elements) of row `row` (row stride sn elements) at element offset `col`.
__device__ __forceinline__ u32x4 load_frag(const uint16_t *mat, int sn, int row, int col)
{
    return *reinterpret_cast<const u32x4 *>(mat + (size_t)row * sn + col);
}

// ------------------------------------------------------------------------------------------------
// dQ (and delta)
// ------------------------------------------------------------------------------------------------
template <bool BF16, int HDIM>
__global__ __launch_bounds__(NTHREADS, HDIM == 128 ? 2 : 3) void attn_bwd_dq_kernel(const AttnBwdArgs a)
{
    using E = Elem<BF16>;
    constexpr int NH = HDIM == 128 ? 2 : 1;       // 64-column tiles per matrix
    constexpr int KS = HDIM / 16;                 // MFMA steps of a contraction over the head dim
    constexpr int OB = HDIM / 32;                 // 32-column accumulator blocks of an output
    constexpr int CHM = HDIM == 32 ? 3 : 7;       // 16-byte chunks per global row, minus one
    using C = Cfg<NH>;
    constexpr int STAGE_BYTES = C::STAGE_BYTES, OFF_AUX = C::OFF_AUX, OFF_LUT = C::OFF_LUT;
    __shared__ __attribute__((aligned(1024))) unsigned char smem[C::LDS_BYTES];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(LDS_PTR(unsigned char))smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, hh = lane >> 5;
    const int nid = renumber_block();
    const int bh = (int)fastdiv((uint32_t)nid, a.div_qtiles);
    const int qt = nid - bh * a.qtiles;
    const int N = a.N, nw = (N + 31) >> 5;
    const int T = (N + BN - 1) / BN;
    const bool ragged = (N & (BN - 1)) != 0;
    const float pm = a.post_mul;

    const int bi = (int)fastdiv((uint32_t)bh, a.div_H), hi = bh - bi * a.H;
    const uint16_t *kb = slab(a.k, bi, hi), *vb = slab(a.v, bi, hi);
    const uint16_t *qb = slab(a.q, bi, hi), *dob = slab(a.dout, bi, hi), *ob = slab(a.out, bi, hi);
    const uint32_t *mb = slab(a.mask, bi, hi);

    // ---- this lane's query row: q^T and dO^T fragments (B operands), delta, lse ----
    const int qrow = qt * BM + wave * 32 + l32;
    const int qr = qrow < N ? qrow : N - 1;
    u32x4 qf[KS], dof[KS];
    float delta = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int col = 16 * s + 8 * hh;
        u32x4 tq = load_frag(qb, a.q.sn, qr, col);
        const u32x4 td = load_frag(dob, a.dout.sn, qr, col);
        const u32x4 to = load_frag(ob, a.out.sn, qr, col);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            delta += E::up1((uint16_t)(td[i] & 0xffffu)) * E::up1((uint16_t)(to[i] & 0xffffu)) +
                     E::up1((uint16_t)(td[i] >> 16)) * E::up1((uint16_t)(to[i] >> 16));
            const float lo = E::up1((uint16_t)(tq[i] & 0xffffu)) * a.q_scale;
            const float hi = E::up1((uint16_t)(tq[i] >> 16)) * a.q_scale;
            tq[i] = (uint32_t)E::cvt1(lo) | ((uint32_t)E::cvt1(hi) << 16);
        }
        qf[s] = tq;
        dof[s] = td;
    }
    delta = xhalf_sum(delta);
    if (qrow < N && hh == 0) a.delta[(size_t)bh * N + qrow] = delta;
    const float lse_row = a.lse[(size_t)bh * N + qr];
    // p = exp2(pm * s - L); rows that kept nothing (lse = -inf) and rows beyond N get L = +inf
    const float L = (qrow >= N || lse_row == -__builtin_inff()) ? __builtin_inff() : lse_row * LOG2E;

    // ---- copies ----
    const TileCopy tc = make_tile_copy(wave, lane, CHM);
    const TileRead tr = make_tile_read(lane);
    const int mrow = qt * BM + wave * 32 + (lane >> 1);
    const uint32_t m_voff = (uint32_t)(((size_t)(mrow < N ? mrow : N - 1) * nw + (lane & 1)) * 4);
    auto issue = [&](int t, int st) {
        uint32_t voff = m_voff;
        if (2 * t + 1 >= nw) voff -= (lane & 1) * 4;          // odd word count: re-read the last word
        async_copy_b32(lds0 + OFF_AUX + st * AUX_BYTES + wave * 256, mb + 2 * t, voff);
        issue_tile<NH>(lds0 + st * STAGE_BYTES, kb, a.k.sn, t * BN, N, tc, wave);
        issue_tile<NH>(lds0 + st * STAGE_BYTES + C::OFF_B, vb, a.v.sn, t * BN, N, tc, wave);
    };
    // With a tile map only the key tiles that hold a set mask bit for this work-group's rows are
    // visited (the map has one row of "live" bits per block of 64 query rows: two of them are ORed);
    // without one, all.  Wave-uniform walk over the set bits, a word (32 tiles) at a time.
    const int TW = (T + 31) >> 5;
    const uint32_t *mapw = nullptr, *mapw2 = nullptr;
    if (a.tile_map != nullptr) {
        mapw = a.tile_map + bi * a.map_sb + hi * a.map_sh + (size_t)(2 * qt) * 2 * TW;
        mapw2 = (2 * qt + 1 < T) ? mapw + 2 * TW : mapw;
    }
    int cur_w = -1;
    uint32_t live_w = 0u;
    auto next_tile = [&]() __attribute__((always_inline)) -> int {     // next live tile, T if there is none
        while (live_w == 0u) {
            if (++cur_w >= TW) return T;
            uint32_t lv = 0xffffffffu;
            if (mapw != nullptr) lv = __builtin_amdgcn_readfirstlane(mapw[cur_w] | mapw2[cur_w]);
            if (cur_w == TW - 1 && (T & 31) != 0) lv &= (1u << (T & 31)) - 1u;
            live_w = lv;
        }
        const int b = __builtin_ctz(live_w);
        live_w &= live_w - 1u;
        return 32 * cur_w + b;
    };
    const int t_first = next_tile();
    if (t_first < T) issue(t_first, 0);
    if (tid < 64)
        reinterpret_cast<float *>(smem + OFF_LUT)[tid] = (((tid >> 2) >> (tid & 3)) & 1) ? 0.f : -__builtin_inff();

    f32x16 oacc[OB];                    // [2 * half + dblk]: 32 columns of dQ each
#pragma unroll
    for (int b = 0; b < OB; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[b][i] = 0.f;
    const uint32_t lut_addr = lds0 + OFF_LUT;
    const uint32_t nib_shift = 4u - 4u * hh;

    int st = 1;
    for (int t = t_first, t_next; t < T; t = t_next) {
        t_next = next_tile();
        st ^= 1;                  // the visits alternate between the two stages
        const uint32_t so = lds0 + st * STAGE_BYTES;
        WAIT_VMCNT(0);
        if (ragged && t == T - 1) zero_tile_tail(so, 2 * NH, t * BN, N, tc, wave, lane);
        __syncthreads();          // tile t of every wave landed; the other stage is free
        if (t_next < T) issue(t_next, st ^ 1);

        u32x2 w2 = lds_read_b64(lds0 + OFF_AUX + st * AUX_BYTES + wave * 256 + l32 * 8);
        if (t == T - 1) { w2.x &= a.last_mask0; w2.y &= a.last_mask1; }
        if (__builtin_amdgcn_ballot_w64((w2.x | w2.y) != 0u) == 0ull) continue;

        // Per block of 32 keys: S^T (mask bias as initial value) and dP^T, element [4g+j] <-> key
        // 32blk + 8g + 4hh + j, then dS^T / scale = P^T o (dP^T - delta), packed as B operands.
        uint32_t pb[2][2][4];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            f32x16 sacc, dacc;
            const uint32_t wa = (blk == 0 ? w2.x : w2.y) << nib_shift;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x4 b = lds_read_b128(lut_addr + ((wa >> (8 * g)) & 0xF0u));
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    sacc[4 * g + j] = __builtin_bit_cast(float, (uint32_t)b[j]);
                    dacc[4 * g + j] = 0.f;
                }
            }
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const uint32_t ra = tr.rowaddr[s & 3] + so + (s >> 2) * TILE_BYTES + 4096 * blk;
                sacc = E::mfma(lds_read_b128(ra), qf[s], sacc);
                dacc = E::mfma(lds_read_b128(ra + C::OFF_B), dof[s], dacc);
            }
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int e = 8 * u + 2 * i;
                    const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[e], pm, -L));
                    const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[e + 1], pm, -L));
                    pb[blk][u][i] = E::pack2_rne(p0 * (dacc[e] - delta), p1 * (dacc[e + 1] - delta));
                }
        }
        // dQ^T += K^T dS^T
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const u32x4 pv = {pb[blk][u][0], pb[blk][u][1], pb[blk][u][2], pb[blk][u][3]};
                const uint32_t off = so + 4096 * blk + 2048 * u;
#pragma unroll
                for (int b = 0; b < OB; ++b) {
                    const uint32_t ko = off + (b >> 1) * TILE_BYTES;
                    const u32x2 lo = lds_read_tr16_b64(tr.traddr[b & 1][0] + ko);
                    const u32x2 hi = lds_read_tr16_b64(tr.traddr[b & 1][1] + ko);
                    const u32x4 va = {lo.x, lo.y, hi.x, hi.y};
                    oacc[b] = E::mfma(va, pv, oacc[b]);
                }
            }
    }
    WAIT_VMCNT(0);
    __syncthreads();              // every wave is done reading the stages
    const int row0 = qt * BM + wave * 32;
    if (row0 < N) {
        uint16_t *dst = slab(a.dq, bi, hi) + (size_t)row0 * a.dq.sn;
        if constexpr (HDIM == 32) {
            store_block<BF16, 32>(oacc[0], oacc[0], a.scale, lds0 + wave * 4096, dst, a.dq.sn, row0, N, lane);
        } else {
#pragma unroll
            for (int half = 0; half < NH; ++half)
                store_block<BF16>(oacc[2 * half], oacc[2 * half + 1], a.scale, lds0 + wave * 4096,
                                  dst + half * HD, a.dq.sn, row0, N, lane);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// dK and dV
// ------------------------------------------------------------------------------------------------
// DK / DV: which of the two gradients this instance produces (both for head dim 64; one per launch
// for head dim 128, where both sets of accumulators do not fit the register file).
template <bool BF16, int HDIM, bool DK, bool DV, bool POSTMUL>
__global__ __launch_bounds__(NTHREADS, 2) void attn_bwd_dkv_kernel(const AttnBwdArgs a)
{
    using E = Elem<BF16>;
    constexpr int NH = HDIM == 128 ? 2 : 1;
    constexpr int KS = HDIM / 16;
    constexpr int OB = HDIM / 32;
    constexpr int CHM = HDIM == 32 ? 3 : 7;
    using C = Cfg<NH>;
    constexpr int STAGE_BYTES = C::STAGE_BYTES, OFF_AUX = C::OFF_AUX;
    __shared__ __attribute__((aligned(1024))) unsigned char smem[C::LDS_BYTES];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(LDS_PTR(unsigned char))smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, hh = lane >> 5;
    const int nid = renumber_block();
    const int bh = (int)fastdiv((uint32_t)nid, a.div_qtiles);
    const int kt = nid - bh * a.qtiles;
    const int N = a.N, nw = (N + 31) >> 5;
    const int T = (N + BN - 1) / BN;
    const bool ragged = (N & (BN - 1)) != 0;
    const float pm = POSTMUL ? a.post_mul : 1.0f;
    const float lse_mul = -LOG2E / pm;                // pm is a power of two: exact

    const int bi = (int)fastdiv((uint32_t)bh, a.div_H), hi = bh - bi * a.H;
    const uint16_t *qb = slab(a.q, bi, hi), *dob = slab(a.dout, bi, hi);
    const uint16_t *kb = slab(a.k, bi, hi), *vb = slab(a.v, bi, hi);
    const uint32_t *mb = slab(a.mask, bi, hi);
    const float *lse_b = a.lse + (size_t)bh * N, *delta_b = a.delta + (size_t)bh * N;

    // ---- this lane's key: K^T (scaled) and V^T fragments, B operands ----
    const int key0 = kt * BM + wave * 32;
    const bool wave_valid = key0 < N;                 // wave-uniform: some key of this wave exists
    const int key = key0 + l32;
    const int kr = key < N ? key : N - 1;
    const uint32_t key_ok = key < N ? 0xffffffffu : 0u;
    const uint32_t key_w = key < N ? 1u : 0u;         // width of the bit field that holds this key's mask bit
    const int wi = (key0 >> 5) < nw ? (key0 >> 5) : nw - 1;     // this wave's mask word of a row
    u32x4 kf[KS], vf[DK ? KS : 1];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int col = 16 * s + 8 * hh;
        u32x4 tk = load_frag(kb, a.k.sn, kr, col);
        if constexpr (DK) vf[s] = load_frag(vb, a.v.sn, kr, col);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float lo = E::up1((uint16_t)(tk[i] & 0xffffu)) * a.q_scale;
            const float hi = E::up1((uint16_t)(tk[i] >> 16)) * a.q_scale;
            tk[i] = (uint32_t)E::cvt1(lo) | ((uint32_t)E::cvt1(hi) << 16);
        }
        kf[s] = tk;
    }

    // ---- copies: Q tile, dO tile; per wave its mask word of the 64 rows; lse (wave 0), delta (wave 1)
    const TileCopy tc = make_tile_copy(wave, lane, CHM);
    const TileRead tr = make_tile_read(lane);
    auto issue = [&](int t, int st) {
        const int r0 = t * BN;
        const int row = r0 + lane < N ? r0 + lane : N - 1;
        const uint32_t aux = lds0 + OFF_AUX + st * AUX_BYTES;
        async_copy_b32(aux + wave * 256, mb + wi, (uint32_t)((size_t)row * nw * 4));
        if (wave == 0) async_copy_b32(aux + 1024, lse_b, (uint32_t)(row * 4));
        if (wave == 1) async_copy_b32(aux + 1280, delta_b, (uint32_t)(row * 4));
        issue_tile<NH>(lds0 + st * STAGE_BYTES, qb, a.q.sn, r0, N, tc, wave);
        issue_tile<NH>(lds0 + st * STAGE_BYTES + C::OFF_B, dob, a.dout.sn, r0, N, tc, wave);
    };
    // With a tile map only the blocks of 64 query rows in which the mask keeps something for this
    // work-group's 128 keys (its two key tiles 2kt, 2kt+1: neighbouring bits of one word of the
    // row block's "live" bits) are visited: lane r of a wavefront looks at row block 64c + r, a
    // ballot turns the 64 answers into the bits that are walked.  Every wavefront does the same.
    const int TW = (T + 31) >> 5;
    const uint32_t *mapc = a.tile_map != nullptr
        ? a.tile_map + bi * a.map_sb + hi * a.map_sh + ((2 * kt) >> 5) : nullptr;
    int cur_c = -1;
    unsigned long long live_c = 0ull;
    auto next_tile = [&]() __attribute__((always_inline)) -> int {     // next live row block, T if there is none
        while (live_c == 0ull) {
            if (64 * ++cur_c >= T) return T;
            const int r = 64 * cur_c + lane;
            bool lv = r < T;
            if (mapc != nullptr && lv) lv = ((mapc[(size_t)r * 2 * TW] >> ((2 * kt) & 31)) & 3u) != 0u;
            live_c = __builtin_amdgcn_ballot_w64(lv);
        }
        const int b = __builtin_ctzll(live_c);
        live_c &= live_c - 1ull;
        return 64 * cur_c + b;
    };
    const int t_first = next_tile();
    if (t_first < T) issue(t_first, 0);

    f32x16 dkacc[DK ? OB : 1], dvacc[DV ? OB : 1];      // [2 * half + dblk]: 32 columns each
#pragma unroll
    for (int b = 0; b < OB; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if constexpr (DK) dkacc[b][i] = 0.f;
            if constexpr (DV) dvacc[b][i] = 0.f;
        }

    // one q tile; the ring stage is a compile-time constant so that every LDS address of the body is
    // a register plus an immediate
    auto tile = [&](int t, int t_next, auto st_c) __attribute__((always_inline)) {
        constexpr int st = decltype(st_c)::value;
        const uint32_t so = lds0 + st * STAGE_BYTES;
        const uint32_t aux = lds0 + OFF_AUX + st * AUX_BYTES;
        WAIT_VMCNT(0);
        if (wave == 0) {
            // lse of the tile's rows -> what the score accumulators start from, -lse * log2(e) / pm, so
            // that exp2(pm * accumulator) is the probability; rows that kept nothing or lie beyond N
            // -> -inf (probability 0)
            const uint32_t p = aux + 1024 + lane * 4;
            const float l = *(LDS_PTR(float))(uintptr_t)p;
            const bool dead = (t * BN + lane >= N) || (l == -__builtin_inff());
            *(LDS_PTR(float))(uintptr_t)p = dead ? -__builtin_inff() : l * lse_mul;
        }
        if (wave == 1) {
            // -delta: the dP accumulators start from it
            const uint32_t p = aux + 1280 + lane * 4;
            *(LDS_PTR(float))(uintptr_t)p = -*(LDS_PTR(float))(uintptr_t)p;
        }
        if (ragged && t == T - 1) zero_tile_tail(so, 2 * NH, t * BN, N, tc, wave, lane);
        __syncthreads();
        if (t_next < T) issue(t_next, st ^ 1);
        if (!wave_valid) return;

#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            // element 4g+j of an accumulator <-> query row 32blk + 8g + 4hh + j of the tile
            const uint32_t rsel = (uint32_t)((32 * blk + 4 * hh) * 4);
            u32x4 mw[4];
            uint32_t any = 0u;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                mw[g] = lds_read_b128(aux + wave * 256 + rsel + 32 * g);
                any |= mw[g].x | mw[g].y | mw[g].z | mw[g].w;
            }
            if (__builtin_amdgcn_ballot_w64((((any >> l32) & 1u) & key_ok) != 0u) == 0ull) continue;

            // the accumulators start from the rows' -lse (scaled) and -delta, read straight into them:
            // the products then leave s - lse and dP - delta, with no subtraction per element
            f32x16 sacc, dacc;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x4 Lr = lds_read_b128(aux + 1024 + rsel + 32 * g);
                u32x4 Dr = {0u, 0u, 0u, 0u};
                if constexpr (DK) Dr = lds_read_b128(aux + 1280 + rsel + 32 * g);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    sacc[4 * g + j] = __builtin_bit_cast(float, (uint32_t)Lr[j]);
                    dacc[4 * g + j] = __builtin_bit_cast(float, (uint32_t)Dr[j]);
                }
            }
#pragma unroll
            for (int s = 0; s < KS; ++s)
                sacc = E::mfma(lds_read_b128(tr.rowaddr[s & 3] + so + (s >> 2) * TILE_BYTES + 4096 * blk), kf[s], sacc);
            if constexpr (DK) {
#pragma unroll
                for (int s = 0; s < KS; ++s)
                    dacc = E::mfma(lds_read_b128(tr.rowaddr[s & 3] + so + C::OFF_B + (s >> 2) * TILE_BYTES + 4096 * blk),
                                   vf[s], dacc);
            }

            uint32_t pp[2][4] = {}, ps[2][4] = {};       // the one a single-gradient instance leaves unused is dropped
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float p[4], d[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t keep = (uint32_t)__builtin_amdgcn_sbfe((int)mw[g][j], (uint32_t)l32, key_w);
                    const float e = __builtin_amdgcn_exp2f(POSTMUL ? sacc[4 * g + j] * pm : sacc[4 * g + j]);
                    p[j] = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, e) & keep);
                    d[j] = p[j] * dacc[4 * g + j];
                }
                // elements 4g .. 4g+3 are pairs (2i, 2i+1) with i = 2(g & 1), 2(g & 1) + 1 of u = g >> 1
                if constexpr (DV) {
                    pp[g >> 1][2 * (g & 1)] = E::pack2_rne(p[0], p[1]);
                    pp[g >> 1][2 * (g & 1) + 1] = E::pack2_rne(p[2], p[3]);
                }
                if constexpr (DK) {
                    ps[g >> 1][2 * (g & 1)] = E::pack2_rne(d[0], d[1]);
                    ps[g >> 1][2 * (g & 1) + 1] = E::pack2_rne(d[2], d[3]);
                }
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const u32x4 bp = {pp[u][0], pp[u][1], pp[u][2], pp[u][3]};
                const u32x4 bs = {ps[u][0], ps[u][1], ps[u][2], ps[u][3]};
                const uint32_t off = so + 4096 * blk + 2048 * u;
#pragma unroll
                for (int b = 0; b < OB; ++b) {
                    const uint32_t ho = off + (b >> 1) * TILE_BYTES;
                    if constexpr (DK) {                              // dK^T += Q^T dS
                        const u32x2 qlo = lds_read_tr16_b64(tr.traddr[b & 1][0] + ho);
                        const u32x2 qhi = lds_read_tr16_b64(tr.traddr[b & 1][1] + ho);
                        const u32x4 qa = {qlo.x, qlo.y, qhi.x, qhi.y};
                        dkacc[b] = E::mfma(qa, bs, dkacc[b]);
                    }
                    if constexpr (DV) {                              // dV^T += dO^T P
                        const u32x2 dlo = lds_read_tr16_b64(tr.traddr[b & 1][0] + ho + C::OFF_B);
                        const u32x2 dhi = lds_read_tr16_b64(tr.traddr[b & 1][1] + ho + C::OFF_B);
                        const u32x4 da = {dlo.x, dlo.y, dhi.x, dhi.y};
                        dvacc[b] = E::mfma(da, bp, dvacc[b]);
                    }
                }
            }
        }
    };
    for (int t = t_first; t < T;) {
        const int tn = next_tile();
        tile(t, tn, std::integral_constant<int, 0>{});
        if (tn >= T) break;
        t = next_tile();
        tile(tn, t, std::integral_constant<int, 1>{});
    }
    WAIT_VMCNT(0);
    __syncthreads();
    if (wave_valid) {
        uint16_t *dk_dst = slab(a.dk, bi, hi) + (size_t)key0 * a.dk.sn;
        uint16_t *dv_dst = slab(a.dv, bi, hi) + (size_t)key0 * a.dv.sn;
        if constexpr (HDIM == 32) {
            if constexpr (DK) store_block<BF16, 32>(dkacc[0], dkacc[0], a.scale, lds0 + wave * 4096, dk_dst, a.dk.sn, key0, N, lane);
            if constexpr (DV) store_block<BF16, 32>(dvacc[0], dvacc[0], 1.0f, lds0 + wave * 4096, dv_dst, a.dv.sn, key0, N, lane);
        } else {
#pragma unroll
            for (int half = 0; half < NH; ++half) {
                if constexpr (DK)
                    store_block<BF16>(dkacc[2 * half], dkacc[2 * half + 1], a.scale, lds0 + wave * 4096,
                                      dk_dst + half * HD, a.dk.sn, key0, N, lane);
                if constexpr (DV)
                    store_block<BF16>(dvacc[2 * half], dvacc[2 * half + 1], 1.0f, lds0 + wave * 4096,
                                      dv_dst + half * HD, a.dv.sn, key0, N, lane);
            }
        }
    }
}

// Launches the dK/dV instance for (dtype, head dim, gradients) with or without the post-multiplier.
template <bool BF16, int HDIM, bool DK, bool DV>
void launch_dkv(bool postmul, dim3 grid, dim3 block, hipStream_t stream, const AttnBwdArgs &a)
{
    if (postmul)
        hipLaunchKernelGGL((attn_bwd_dkv_kernel<BF16, HDIM, DK, DV, true>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((attn_bwd_dkv_kernel<BF16, HDIM, DK, DV, false>), grid, block, 0, stream, a);
}

}  // namespace

hipError_t launch_attn_bwd(const AttnBwdArgs &args, bool bf16, hipStream_t stream)
{
    AttnBwdArgs a = args;
    a.div_qtiles = make_fastdiv((uint32_t)a.qtiles);
    a.div_H = make_fastdiv((uint32_t)a.H);
    const long long groups = (long long)a.BH * a.qtiles;
    if (groups == 0) return hipSuccess;
    const dim3 grid((unsigned)groups), block(NTHREADS);
    const bool postmul = a.post_mul != 1.0f;       // exp2(pm * s) needs its multiplication only then
    // dQ first: it also fills the delta workspace that the dK/dV kernel reads (same stream).
    if (a.D == 2 * HD) {
        if (bf16) {
            hipLaunchKernelGGL((attn_bwd_dq_kernel<true, 128>), grid, block, 0, stream, a);
            launch_dkv<true, 128, true, false>(postmul, grid, block, stream, a);
            launch_dkv<true, 128, false, true>(postmul, grid, block, stream, a);
        } else {
            hipLaunchKernelGGL((attn_bwd_dq_kernel<false, 128>), grid, block, 0, stream, a);
            launch_dkv<false, 128, true, false>(postmul, grid, block, stream, a);
            launch_dkv<false, 128, false, true>(postmul, grid, block, stream, a);
        }
    } else if (a.D == HD) {
        if (bf16) {
            hipLaunchKernelGGL((attn_bwd_dq_kernel<true, 64>), grid, block, 0, stream, a);
            launch_dkv<true, 64, true, true>(postmul, grid, block, stream, a);
        } else {
            hipLaunchKernelGGL((attn_bwd_dq_kernel<false, 64>), grid, block, 0, stream, a);
            launch_dkv<false, 64, true, true>(postmul, grid, block, stream, a);
        }
    } else {
        if (bf16) {
            hipLaunchKernelGGL((attn_bwd_dq_kernel<true, 32>), grid, block, 0, stream, a);
            launch_dkv<true, 32, true, true>(postmul, grid, block, stream, a);
        } else {
            hipLaunchKernelGGL((attn_bwd_dq_kernel<false, 32>), grid, block, 0, stream, a);
            launch_dkv<false, 32, true, true>(postmul, grid, block, stream, a);
        }
    }
    return hipGetLastError();
}

}  // namespace sma
