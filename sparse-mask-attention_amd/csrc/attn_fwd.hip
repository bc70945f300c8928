// Fused masked-attention forward for gfx950 (MI355X), head_dim 64, fp16 / bf16, fp32 accumulate.
//
// Stands in for sparse_attn_wmma_full_fp16 (csrc/sparse_attention.cu:82-412 of the reference) and
// for its scalar bf16 kernel (csrc/sparse_attention.cu:418-543); the design below is specific to
// CDNA4 and shares nothing with either beyond the function computed.
//
// Work decomposition
//   work-group  = 4 wavefronts = 128 query rows of one (b,h); it walks the keys in tiles of 64.
//   wavefront   = 32 query rows.  It computes S^T = K_tile (64x64) * Q^T (64x32) with eight
//                 v_mfma_f32_32x32x16, so that every lane owns ONE query row (lane % 32) and 32
//                 of the tile's 64 keys: the online softmax is a per-lane register loop plus a
//                 single exchange between lane l and lane l+32.
//                 P^T is already in the B-operand layout of O^T += V^T * P^T (eight more MFMAs):
//                 probabilities never leave registers.
//   LDS         = double-buffered K tile [key][d] and V tile stored transposed [d][key] (both
//                 padded to a 72-element pitch: 16-byte reads by 16 consecutive rows hit disjoint
//                 banks), plus the work-group's packed mask words for 512 keys at a time.
//   mask        = lane (query row) reads its two words of the tile from LDS; bit 8g+4h+j of a
//                 word belongs to accumulator register 4g+j of lane-half h.
//   skipping    = a wavefront whose 32x64 block of mask bits is all zero skips both GEMMs and
//                 the softmax for that tile.
#include "sma_internal.h"

namespace sma {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int HD = 64;            // head dim
constexpr int BM = 128;           // query rows per work-group
constexpr int BN = 64;            // keys per tile
constexpr int NTHREADS = 256;
constexpr int PITCH = 72;         // LDS row pitch of the K and V^T tiles, in 16-bit elements
constexpr int MCHUNK = 16;        // mask words staged per query row (= 512 keys = 8 tiles)
constexpr int MPITCH = 18;        // LDS row pitch of the mask stage, in words
constexpr uint32_t NEG_INF_BITS = 0xff800000u;

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

// Exchange a value between lane l and lane l ^ 32.
__device__ __forceinline__ float xhalf(float x) { return __shfl_xor(x, 32, 64); }

template <bool BF16>
__global__ __launch_bounds__(NTHREADS) void attn_fwd_kernel(const AttnArgs a)
{
    using E = Elem<BF16>;
    __shared__ __attribute__((aligned(16))) uint16_t sK[2][BN * PITCH];
    __shared__ __attribute__((aligned(16))) uint16_t sVt[2][HD * PITCH];
    __shared__ __attribute__((aligned(16))) uint32_t sM[BM * MPITCH];

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

    // ---- Q^T as MFMA B operands: lane holds query row l32, d = 16*s + 8*hh .. +7 ----
    const int qrow = qt * BM + wave * 32 + l32;
    u32x4 qf[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        u32x4 t = {0u, 0u, 0u, 0u};
        if (qrow < N) t = *reinterpret_cast<const u32x4 *>(qb + (size_t)qrow * HD + 16 * s + 8 * hh);
        qf[s] = t ^ a.qsign;
    }

    // ---- global -> register prefetch of one K/V tile, and register -> LDS store ----
    u32x4 kreg[2];
    u32x2 vreg[4];
    const int v_dg = tid & 15, v_kg = tid >> 4;       // 4 d-columns x 4 keys per thread
    auto load_kv = [&](int t) {
        const int key0 = t * BN;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int off = (j * NTHREADS + tid) * 8;           // element offset inside the tile
            const int row = off >> 6, col = off & 63;
            u32x4 x = {0u, 0u, 0u, 0u};
            if (key0 + row < N) x = *reinterpret_cast<const u32x4 *>(kb + (size_t)(key0 + row) * HD + col);
            kreg[j] = x;
        }
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            const int row = 4 * v_kg + kk;
            u32x2 x = {0u, 0u};
            if (key0 + row < N) x = *reinterpret_cast<const u32x2 *>(vb + (size_t)(key0 + row) * HD + 4 * v_dg);
            vreg[kk] = x;
        }
    };
    auto store_kv = [&](int stage) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int off = (j * NTHREADS + tid) * 8;
            const int row = off >> 6, col = off & 63;
            *reinterpret_cast<u32x4 *>(&sK[stage][row * PITCH + col]) = kreg[j];
        }
        // 4x4 transpose of 16-bit elements: vreg[kk] = {d0 d1 | d2 d3} of key kk.
        // V^T is stored with the 4-key groups of each 16 keys in the order (0,2,1,3), i.e. key
        // bits 2 and 3 swapped, so that the 8 keys one lane feeds to one PV MFMA are contiguous.
        const int pg = (v_kg & 0xC) | ((v_kg & 1) << 1) | ((v_kg >> 1) & 1);
        uint16_t *dst = &sVt[stage][(4 * v_dg) * PITCH + 4 * pg];
        u32x2 o;
        o.x = (vreg[0].x & 0xffffu) | (vreg[1].x << 16);
        o.y = (vreg[2].x & 0xffffu) | (vreg[3].x << 16);
        *reinterpret_cast<u32x2 *>(dst) = o;
        o.x = (vreg[0].x >> 16) | (vreg[1].x & 0xffff0000u);
        o.y = (vreg[2].x >> 16) | (vreg[3].x & 0xffff0000u);
        *reinterpret_cast<u32x2 *>(dst + PITCH) = o;
        o.x = (vreg[0].y & 0xffffu) | (vreg[1].y << 16);
        o.y = (vreg[2].y & 0xffffu) | (vreg[3].y << 16);
        *reinterpret_cast<u32x2 *>(dst + 2 * PITCH) = o;
        o.x = (vreg[0].y >> 16) | (vreg[1].y & 0xffff0000u);
        o.y = (vreg[2].y >> 16) | (vreg[3].y & 0xffff0000u);
        *reinterpret_cast<u32x2 *>(dst + 3 * PITCH) = o;
    };
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
            sM[row * MPITCH + wi] = w;
        }
    };

    // ---- running state: one query row per lane (both lane halves hold the same max) ----
    f32x16 oacc[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) { oacc[0][i] = 0.f; oacc[1][i] = 0.f; }
    float m_run = -__builtin_inff();   // running max of the raw (unscaled) kept scores
    float l_run = 0.f;                 // this lane's share of the running denominator
    const float c = a.c;

    const int T = (N + BN - 1) / BN;
    load_kv(0);
    stage_mask(0);
    store_kv(0);
    __syncthreads();

    for (int t = 0; t < T; ++t) {
        const int stage = t & 1;
        const bool has_next = (t + 1 < T);
        if (has_next) load_kv(t + 1);

        const u32x2 w2 = *reinterpret_cast<const u32x2 *>(&sM[(wave * 32 + l32) * MPITCH + 2 * (t & 7)]);
        if (__builtin_amdgcn_ballot_w64((w2.x | w2.y) != 0u) != 0ull) {
            // ---- S^T = K * Q^T : sacc[blk][4g+j] = score(key 32blk + 8g + 4hh + j, query l32) ----
            f32x16 sacc[2];
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
#pragma unroll
                for (int i = 0; i < 16; ++i) sacc[blk][i] = 0.f;
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const u32x4 ka = *reinterpret_cast<const u32x4 *>(
                        &sK[stage][(32 * blk + l32) * PITCH + 16 * s + 8 * hh]);
                    sacc[blk] = E::mfma(ka, qf[s], sacc[blk]);
                }
            }
            // ---- mask, row max ----
            float mx = -__builtin_inff();
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
                const uint32_t wsh = (blk == 0 ? w2.x : w2.y) >> (4 * hh);
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const bool keep = ((wsh >> (8 * g + j)) & 1u) != 0u;
                        const float sv = keep ? sacc[blk][4 * g + j] : -__builtin_inff();
                        sacc[blk][4 * g + j] = sv;
                        mx = __builtin_fmaxf(mx, sv);
                    }
            }
            mx = __builtin_fmaxf(mx, xhalf(mx));
            const float m_new = __builtin_fmaxf(m_run, mx);
            const float m_use = (m_new == -__builtin_inff()) ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);   // m_run = -inf -> 0
            const float mc = m_use * c;
            m_run = m_new;
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
            l_run = l_run * alpha + lsum;
#pragma unroll
            for (int i = 0; i < 16; ++i) { oacc[0][i] *= alpha; oacc[1][i] *= alpha; }
            // ---- O^T += V^T * P^T : oacc[dblk][4g+j] = out(query l32, d = 32dblk + 8g + 4hh + j) ----
#pragma unroll
            for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
                for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        const u32x4 va = *reinterpret_cast<const u32x4 *>(
                            &sVt[stage][(32 * dblk + l32) * PITCH + 32 * blk + 16 * u + 8 * hh]);
                        const u32x4 pv = {pb[blk][u][0], pb[blk][u][1], pb[blk][u][2], pb[blk][u][3]};
                        oacc[dblk] = E::mfma(va, pv, oacc[dblk]);
                    }
        }

        if (has_next) {
            if (((t + 1) & 7) == 0) {        // next tile starts a new 512-key mask chunk
                __syncthreads();             // every wave has read its words of the old chunk
                stage_mask((t + 1) >> 3);
            }
            store_kv(stage ^ 1);
        }
        __syncthreads();
    }

    // ---- epilogue ----
    const float l_tot = l_run + xhalf(l_run);
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
            a.lse[(size_t)bh * N + qrow] =
                (l_tot > 0.f) ? m_run * a.scale_abs + __builtin_logf(l_tot) : -__builtin_inff();
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
