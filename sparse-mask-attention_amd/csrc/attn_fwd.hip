// Fused masked-attention forward for gfx950 (MI355X), head_dim 64, fp16 / bf16, fp32 accumulate.
//
// Stands in for sparse_attn_wmma_full_fp16 (csrc/sparse_attention.cu:82-412 of the reference) and
// for its scalar bf16 kernel (csrc/sparse_attention.cu:418-543); the design below is specific to
// CDNA4 and shares nothing with either beyond the function computed.
//
// Work decomposition
//   work-group  = 4 wavefronts = 128 query rows of one (b,h); it walks the keys in tiles of 64.
//                 Three work-groups fit a CU (<= 168 VGPRs, ~42 KB LDS each): one wavefront of
//                 each per SIMD, so that the softmax VALU work of one overlaps the MFMAs of another.
//   wavefront   = 32 query rows.  It computes S^T = K_tile (64x64) * Q^T (64x32) with eight
//                 v_mfma_f32_32x32x16, so every lane owns ONE query row (lane % 32) and 32 of the
//                 tile's 64 keys: the online softmax is a per-lane register loop plus a single
//                 exchange between lane l and lane l+32 (v_permlane32_swap).  P^T is already in
//                 the B-operand layout of O^T += V^T * P^T (eight more MFMAs): probabilities never
//                 leave registers.
//   K/V tiles   = copied global -> LDS by global_load_lds_dwordx4 (no VGPR staging), two stages.
//                 Rows are 128 B; the 16-byte chunks of a row are XOR-swizzled (the permutation is
//                 applied to the global address of each lane, the LDS side of such a load is always
//                 linear) so that K's ds_read_b128 (32 consecutive rows, same column) and V's
//                 ds_read_b64_tr_b16 (transposing read: 8 consecutive rows x 64 B) are free of bank
//                 conflicts on the 64-bank LDS.
//   mask        = the work-group's packed words for 512 keys at a time are staged in LDS.  A lane
//                 reads the two words of its query row for the tile; each nibble of a word selects
//                 one of 16 rows of a small LDS table holding four floats that are 0 (keep) or -inf
//                 (drop); one ds_read_b128 of that row initialises four accumulator registers of
//                 the QK^T MFMA, which then adds the scores on top.  Masking costs no VALU work per
//                 score.
//   skipping    = per 512-key chunk the work-group builds a bitmap of the tiles in which at least
//                 one of its mask bits is set: other tiles are never loaded; and a wavefront whose
//                 own 32x64 block of bits is empty skips its GEMMs and softmax for that tile.
//   rescaling   = the running maximum is only raised (and O, l rescaled) when some row's new
//                 maximum exceeds the one in use by more than 2^8 after scaling: probabilities stay
//                 below 256, far inside fp16/bf16 range, and most tiles skip the 32 multiplies.
#include "sma_internal.h"

namespace sma {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define LDS_PTR(T) __attribute__((address_space(3))) T *
#define GLOBAL_PTR(T) __attribute__((address_space(1))) T *

constexpr int HD = 64;             // head dim
constexpr int BM = 128;            // query rows per work-group
constexpr int BN = 64;             // keys per tile
constexpr int NTHREADS = 256;
constexpr int TILE_BYTES = BN * HD * 2;          // 8 KiB, rows of 128 B
constexpr int MCHUNK = 16;         // mask words staged per query row (= 512 keys = 8 tiles)
constexpr int MPITCH = 18;         // LDS row pitch of the mask stage, in words (bank spread)
constexpr float RESCALE_LOG2 = 8.0f;

// LDS map (bytes)
constexpr int OFF_K = 0;                          // 2 stages x 8 KiB
constexpr int OFF_V = 2 * TILE_BYTES;             // 2 stages x 8 KiB
constexpr int OFF_LUT = 4 * TILE_BYTES;           // 16 x 16 B
constexpr int OFF_MASK = OFF_LUT + 256;           // 128 x 18 words
constexpr int OFF_LIVE = OFF_MASK + BM * MPITCH * 4;
constexpr int LDS_BYTES = OFF_LIVE + 16;

template <bool BF16> struct Elem;

template <> struct Elem<false> {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    // Two probabilities -> one packed register (round toward zero); the row sum below is taken
    // over the SAME rounded values, so numerator and denominator stay consistent.
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
    }
    static __device__ __forceinline__ float add2(uint32_t p, float acc) {
        const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, p), ones, acc, false);
    }
    static __device__ __forceinline__ uint16_t cvt1(float a) {
        return __builtin_bit_cast(uint16_t, (_Float16)a);
    }
};

template <> struct Elem<true> {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        bf16x2 v = {(__bf16)a, (__bf16)b};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float add2(uint32_t p, float acc) {
        const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, p), ones, acc, false);
    }
    static __device__ __forceinline__ uint16_t cvt1(float a) {
        return __builtin_bit_cast(uint16_t, (__bf16)a);
    }
};

// max / sum of a value with its partner in the other lane half (lane l <-> lane l ^ 32).
// v_permlane32_swap(a, b) returns {own a | partner's b, partner's a | own b} for lanes < 32 | >= 32.
__device__ __forceinline__ float xhalf_max(float x) {
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x) {
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr) {
    return *(LDS_PTR(const u32x4))(uintptr_t)addr;
}
// Transposing LDS read: within each group of 16 lanes, lane i receives element (i % 4) of the
// 8-byte rows addressed by lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4 of the group.
__device__ __forceinline__ u32x2 lds_read_tr16_b64(uint32_t addr) {
    const i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(i16x4))(uintptr_t)addr);
    return __builtin_bit_cast(u32x2, v);
}

template <bool BF16>
__global__ __launch_bounds__(NTHREADS, 3) void attn_fwd_kernel(const AttnArgs a)
{
    using E = Elem<BF16>;
    __shared__ __attribute__((aligned(1024))) unsigned char smem[LDS_BYTES];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(LDS_PTR(unsigned char))smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hh = lane >> 5;

    // Work-groups are handed to the 8 XCDs round-robin by linear id.  Renumber so that each XCD
    // (own L2) owns a contiguous range of (b,h) pairs and the query tiles of one (b,h) are
    // dispatched next to each other: K and V of a head are then fetched into one L2 only.
    int nid;
    {
        const int total = gridDim.x, bid = blockIdx.x;
        const int xcd = bid & 7, j = bid >> 3;
        const int base = total >> 3, rem = total & 7;
        nid = xcd * base + (xcd < rem ? xcd : rem) + j;
    }
    const int bh = nid / a.qtiles;
    const int qt = nid - bh * a.qtiles;
    const int N = a.N, nw = a.nw;

    const uint16_t *qb = a.q + (size_t)bh * N * HD;
    const uint16_t *kb = a.k + (size_t)bh * N * HD;
    const uint16_t *vb = a.v + (size_t)bh * N * HD;
    const uint32_t *mb = a.mask_packed + (size_t)bh * N * nw;

    // ---- table for the mask: entry n (16 B) holds four floats, float j = bit j of n ? 0 : -inf ----
    if (tid < 64)
        reinterpret_cast<float *>(smem + OFF_LUT)[tid] = ((tid >> 2) >> (tid & 3)) & 1 ? 0.f : -__builtin_inff();

    // ---- Q^T as MFMA B operands: lane holds query row l32, d = 16*s + 8*hh .. +7 ----
    const int qrow = qt * BM + wave * 32 + l32;
    u32x4 qf[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        u32x4 t = {0u, 0u, 0u, 0u};
        if (qrow < N) t = *reinterpret_cast<const u32x4 *>(qb + (size_t)qrow * HD + 16 * s + 8 * hh);
        qf[s] = t ^ a.qsign;
    }

    // ---- global -> LDS copy of a K/V tile -------------------------------------------------------
    // One global_load_lds_dwordx4 moves 64 x 16 B into 1 KiB of consecutive LDS (lane i -> +16 i),
    // i.e. 8 tile rows.  Wave w issues the row blocks 2w and 2w+1 of K and of V.  Lane i fills LDS
    // chunk (row = 8*blk + i/8, position i%8) with the global chunk  position ^ swz(row).
    //   K: swz(row) = (row >> 1) & 7               V: swz(row) = bit-reverse3((row >> 1) & 7)
    int g_off_k[2], g_off_v[2];          // element offsets inside a tile of this lane's source chunk
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int row = 8 * (2 * wave + j) + (lane >> 3);
        const int pos = lane & 7;
        const int f = (row >> 1) & 7;
        const int fr = ((f & 1) << 2) | (f & 2) | (f >> 2);
        g_off_k[j] = row * HD + ((pos ^ f) << 3);
        g_off_v[j] = row * HD + ((pos ^ fr) << 3);
    }
    auto issue_tile = [&](int t, int stage) {
        const int key0 = t * BN;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int row = 8 * (2 * wave + j) + (lane >> 3);
            const uint32_t blk_off = (uint32_t)(stage * TILE_BYTES + (2 * wave + j) * 1024);
            if (key0 + row < N) {
                __builtin_amdgcn_global_load_lds(
                    (GLOBAL_PTR(const void))(kb + (size_t)key0 * HD + g_off_k[j]),
                    (LDS_PTR(void))(uintptr_t)(lds0 + OFF_K + blk_off), 16, 0, 0);
                __builtin_amdgcn_global_load_lds(
                    (GLOBAL_PTR(const void))(vb + (size_t)key0 * HD + g_off_v[j]),
                    (LDS_PTR(void))(uintptr_t)(lds0 + OFF_V + blk_off), 16, 0, 0);
            } else {            // keys beyond N (last tile only): zero rows
                const u32x4 z = {0u, 0u, 0u, 0u};
                *(LDS_PTR(u32x4))(uintptr_t)(lds0 + OFF_K + blk_off + lane * 16) = z;
                *(LDS_PTR(u32x4))(uintptr_t)(lds0 + OFF_V + blk_off + lane * 16) = z;
            }
        }
    };

    // ---- per-lane LDS read addresses (stage 0), all other offsets are immediates ----
    // K operand (blk, s): row 32*blk + l32, chunk 2s + hh      -> kaddr[s] + 4096*blk
    // V operand (dblk, blk, u, x): 8-byte unit read by ds_read_b64_tr_b16, see lds_read_tr16_b64:
    //   lane supplies row 32blk + 16u + 8x + 4hh + (i >> 2), columns 32dblk + 16G + 4(i & 3) .. +3
    //   with i = lane % 16, G = (lane % 32) / 16             -> vaddr[dblk][x] + 4096*blk + 2048*u
    uint32_t kaddr[4], vaddr[2][2];
    {
        const int fk = (l32 >> 1) & 7;
#pragma unroll
        for (int s = 0; s < 4; ++s)
            kaddr[s] = lds0 + OFF_K + l32 * 128 + (((2 * s + hh) ^ fk) << 4);
        const int i16 = lane & 15, G = l32 >> 4;
        const int r3 = 4 * hh + (i16 >> 2);
#pragma unroll
        for (int x = 0; x < 2; ++x) {
            const int row = 8 * x + r3;
            const int f = (row >> 1) & 7;
            const int fr = ((f & 1) << 2) | (f & 2) | (f >> 2);
#pragma unroll
            for (int dblk = 0; dblk < 2; ++dblk) {
                const int chunk = 4 * dblk + 2 * G + ((i16 & 3) >> 1);
                vaddr[dblk][x] = lds0 + OFF_V + row * 128 + ((chunk ^ fr) << 4) + ((i16 & 1) << 3);
            }
        }
    }
    const uint32_t maddr = lds0 + OFF_MASK + (wave * 32 + l32) * (MPITCH * 4);
    const uint32_t lut_addr = lds0 + OFF_LUT;
    const uint32_t nib_shift = 4u - 4u * hh;

    // Packed mask words of the work-group's 128 rows for keys [512*chunk, 512*chunk + 512).
    auto stage_mask = [&](int chunk) {
#pragma unroll
        for (int i = 0; i < (BM * MCHUNK) / NTHREADS; ++i) {
            const int idx = i * NTHREADS + tid;
            const int row = idx >> 4, wi = idx & 15;
            const int gw = chunk * MCHUNK + wi, grow = qt * BM + row;
            uint32_t w = 0u;
            if (grow < N && gw < nw) {
                w = mb[(size_t)grow * nw + gw];
                if (gw == nw - 1) w &= a.tail_mask;
            }
            reinterpret_cast<uint32_t *>(smem + OFF_MASK)[row * MPITCH + wi] = w;
        }
    };

    // ---- running state: one query row per lane (both lane halves hold the same maximum) ----
    f32x16 oacc[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) { oacc[0][i] = 0.f; oacc[1][i] = 0.f; }
    float m_ref = -__builtin_inff();   // maximum in use, raw (unscaled) score units
    float mc = 0.f;                    // (m_ref == -inf ? 0 : m_ref) * c
    float l_run = 0.f;                 // this lane's share of the running denominator
    const float c = a.c;

    auto compute_tile = [&](int t, int stage) {
        const u32x2 w2 = *(LDS_PTR(const u32x2))(uintptr_t)(maddr + 8 * (t & 7));
        if (__builtin_amdgcn_ballot_w64((w2.x | w2.y) != 0u) == 0ull) return;
        const uint32_t so = (uint32_t)stage * TILE_BYTES;
        // ---- S^T = bias + K * Q^T : sacc[blk][4g+j] = score(key 32blk + 8g + 4hh + j, query l32) ----
        f32x16 sacc[2];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const uint32_t wa = (blk == 0 ? w2.x : w2.y) << nib_shift;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x4 b = lds_read_b128(lut_addr + ((wa >> (8 * g)) & 0xF0u));
#pragma unroll
                for (int j = 0; j < 4; ++j) sacc[blk][4 * g + j] = __builtin_bit_cast(float, (uint32_t)b[j]);
            }
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
                const u32x4 ka = lds_read_b128(kaddr[s] + so + 4096 * blk);
                sacc[blk] = E::mfma(ka, qf[s], sacc[blk]);
            }
        // ---- row max over this tile; raise the maximum in use only when it pays ----
        float mx = -__builtin_inff();
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int i = 0; i < 16; ++i) mx = __builtin_fmaxf(mx, sacc[blk][i]);
        mx = xhalf_max(mx);
        const bool grow = (mx - m_ref) * c > RESCALE_LOG2;      // -inf - -inf = NaN -> false
        if (__builtin_amdgcn_ballot_w64(grow) != 0ull) {
            const float m_new = __builtin_fmaxf(m_ref, mx);
            const float m_use = (m_new == -__builtin_inff()) ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f((m_ref - m_use) * c);   // m_ref = -inf -> 0
            m_ref = m_new;
            mc = m_use * c;
            l_run *= alpha;
#pragma unroll
            for (int i = 0; i < 16; ++i) { oacc[0][i] *= alpha; oacc[1][i] *= alpha; }
        }
        // ---- probabilities, packed as the B operands of the PV product ----
        uint32_t pb[2][2][4];
        float lsum = 0.f;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[blk][8 * u + 2 * i], c, -mc));
                    const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[blk][8 * u + 2 * i + 1], c, -mc));
                    const uint32_t pk = E::pack2(p0, p1);
                    pb[blk][u][i] = pk;
                    lsum = E::add2(pk, lsum);
                }
        l_run += lsum;
        // ---- O^T += V^T * P^T : oacc[dblk][4g+j] = out(query l32, d = 32dblk + 8g + 4hh + j) ----
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const u32x4 pv = {pb[blk][u][0], pb[blk][u][1], pb[blk][u][2], pb[blk][u][3]};
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk) {
                    const uint32_t off = so + 4096 * blk + 2048 * u;
                    const u32x2 lo = lds_read_tr16_b64(vaddr[dblk][0] + off);
                    const u32x2 hi = lds_read_tr16_b64(vaddr[dblk][1] + off);
                    const u32x4 va = {lo.x, lo.y, hi.x, hi.y};
                    oacc[dblk] = E::mfma(va, pv, oacc[dblk]);
                }
            }
    };

    // ---- main loop: 512-key chunks of the mask, live 64-key tiles inside a chunk ----
    const int T = (N + BN - 1) / BN;
    const int n_chunks = (T + 7) >> 3;
    uint32_t *s_live = reinterpret_cast<uint32_t *>(smem + OFF_LIVE);
    for (int chunk = 0; chunk < n_chunks; ++chunk) {
        stage_mask(chunk);
        if (tid == 0) *s_live = 0u;
        __syncthreads();
        {   // which of the chunk's 8 tiles hold a set bit in any of the work-group's 128 rows
            uint32_t bits = 0u;
#pragma unroll
            for (int tt = 0; tt < 8; ++tt) {
                const u32x2 w2 = *(LDS_PTR(const u32x2))(uintptr_t)(maddr + 8 * tt);
                if (__builtin_amdgcn_ballot_w64((w2.x | w2.y) != 0u) != 0ull) bits |= 1u << tt;
            }
            if (lane == 0 && bits != 0u) atomicOr(s_live, bits);
        }
        __syncthreads();
        uint32_t live = __builtin_amdgcn_readfirstlane(*s_live);
        int stage = 0;
        if (live != 0u) issue_tile(8 * chunk + __builtin_ctz(live), stage);
        while (live != 0u) {
            const int t = 8 * chunk + __builtin_ctz(live);
            live &= live - 1u;
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();               // tile t is in LDS; everyone is done with the other stage
            if (live != 0u) issue_tile(8 * chunk + __builtin_ctz(live), stage ^ 1);
            compute_tile(t, stage);
            stage ^= 1;
        }
        __syncthreads();                   // all reads of this chunk's mask words and tiles are done
    }

    // ---- epilogue ----
    const float l_tot = xhalf_sum(l_run);
    const float inv = (l_tot > 0.f) ? 1.0f / l_tot : 0.f;
    if (qrow < N) {
        uint16_t *ob = a.out + ((size_t)bh * N + qrow) * HD;
#pragma unroll
        for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const uint32_t lo = (uint32_t)E::cvt1(oacc[dblk][4 * g + 0] * inv) |
                                    ((uint32_t)E::cvt1(oacc[dblk][4 * g + 1] * inv) << 16);
                const uint32_t hi = (uint32_t)E::cvt1(oacc[dblk][4 * g + 2] * inv) |
                                    ((uint32_t)E::cvt1(oacc[dblk][4 * g + 3] * inv) << 16);
                u32x2 o = {lo, hi};
                *reinterpret_cast<u32x2 *>(ob + 32 * dblk + 8 * g + 4 * hh) = o;
            }
        if (a.lse != nullptr && hh == 0) {
            // m_ref * |scale| is the scaled maximum in use; l_tot sums exp(scaled score - that)
            a.lse[(size_t)bh * N + qrow] =
                (l_tot > 0.f) ? mc * 0.6931471805599453f + __builtin_logf(l_tot) : -__builtin_inff();
        }
    }
}

}  // namespace

hipError_t launch_attn_fwd(const AttnArgs &a, bool bf16, hipStream_t stream)
{
    const long long groups = (long long)a.BH * a.qtiles;
    if (groups == 0) return hipSuccess;
    const dim3 grid((unsigned)groups), block(NTHREADS);
    if (bf16)
        hipLaunchKernelGGL(attn_fwd_kernel<true>, grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL(attn_fwd_kernel<false>, grid, block, 0, stream, a);
    return hipGetLastError();
}

}  // namespace sma
