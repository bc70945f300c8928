// Shared device-side helpers of the attention kernels (gfx950): vector types, the fp16 / bf16
// element traits, cross-half lane exchanges, LDS reads (plain and transposing) and the asynchronous
// global -> LDS copies.  Included by attn_fwd.hip and attn_bwd.hip; everything has internal linkage.
#pragma once
#include "sma_internal.h"

namespace sma {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define LDS_PTR(T) __attribute__((address_space(3))) T *

// First element of the (b, h) slab of a strided tensor / of the packed mask.
__device__ __forceinline__ uint16_t *slab(const Rows &r, int b, int h) {
    return r.p + ((size_t)b * r.sb8 + (size_t)h * r.sh8) * 8;
}
__device__ __forceinline__ const uint32_t *slab(const PackedMask &m, int b, int h) { return m.p + b * m.sb + h * m.sh; }

template <bool BF16> struct Elem;

template <> struct Elem<false> {
    static constexpr uint32_t ONES = 0x3c003c00u;           // two fp16 1.0
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    // Two probabilities -> one packed register with the cheapest conversion the format has (fp16:
    // v_cvt_pkrtz, round toward zero); the row sum is taken over the SAME rounded values, so
    // numerator and denominator stay consistent whatever the rounding.
    static __device__ __forceinline__ uint32_t pack2_prob(float a, float b) {
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
    }
    static __device__ __forceinline__ uint32_t pack2_rne(float a, float b) {     // round to nearest even
        const f16x2 h = {(_Float16)a, (_Float16)b};
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ float add2(uint32_t p, float acc) {
        const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, p), ones, acc, false);
    }
    static __device__ __forceinline__ uint16_t cvt1(float a) {          // round to nearest even
        return __builtin_bit_cast(uint16_t, (_Float16)a);
    }
    static __device__ __forceinline__ float up1(uint16_t h) {
        return (float)__builtin_bit_cast(_Float16, h);
    }
    static constexpr float TERM_MAX = 60000.0f;             // keep split terms finite in fp16
};

template <> struct Elem<true> {
    static constexpr uint32_t ONES = 0x3f803f80u;           // two bf16 1.0
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2_prob(float a, float b) {
        // one v_cvt_pk_bf16_f32 (round to nearest even)
        const bf16x2 h = {(__bf16)a, (__bf16)b};
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ uint32_t pack2_rne(float a, float b) {
        const bf16x2 h = {(__bf16)a, (__bf16)b};
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ float add2(uint32_t p, float acc) {
        const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, p), ones, acc, false);
    }
    static __device__ __forceinline__ uint16_t cvt1(float a) {
        return __builtin_bit_cast(uint16_t, (__bf16)a);
    }
    static __device__ __forceinline__ float up1(uint16_t h) {
        return __builtin_bit_cast(float, (uint32_t)h << 16);
    }
    static constexpr float TERM_MAX = 3.0e38f;
};

// Bit reversal of a 3-bit value: the chunk swizzle of tiles that are read both by rows and transposed.
__device__ __forceinline__ int bitrev3(int f) { return ((f & 1) << 2) | (f & 2) | (f >> 2); }

// XCD-aware renumbering of the work-groups.  They are handed to the 8 XCDs round-robin by linear
// id; the number returned gives each XCD (own L2) a contiguous range of (b,h) pairs, with the
// tiles of one (b,h) dispatched next to each other: the matrices of a head are then fetched into
// one L2 only.
__device__ __forceinline__ int renumber_block()
{
    const int total = gridDim.x, bid = blockIdx.x;
    const int xcd = bid & 7, j = bid >> 3;
    const int base = total >> 3, rem = total & 7;
    return xcd * base + (xcd < rem ? xcd : rem) + j;
}

// max / sum of a value with its partner in the other lane half (lane l <-> lane l ^ 32).
// v_permlane32_swap(a, b) leaves {own a | partner's b, partner's a | own b} in lanes < 32 | >= 32.
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
__device__ __forceinline__ u32x2 lds_read_b64(uint32_t addr) {
    return *(LDS_PTR(const u32x2))(uintptr_t)addr;
}
// Transposing LDS read: within each group of 16 lanes, lane i receives element (i % 4) of the
// 8-byte rows addressed by lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4 of the group.
__device__ __forceinline__ u32x2 lds_read_tr16_b64(uint32_t addr) {
    const i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(i16x4))(uintptr_t)addr);
    return __builtin_bit_cast(u32x2, v);
}

// Asynchronous global -> LDS copies.  Lane i's 16 (4) bytes land at lds_base + 16 (4) * i; the
// global address is base + voff (bytes).  They are issued from inline assembly so that the
// compiler's own wait-count bookkeeping does not serialise them against unrelated LDS reads; the
// kernel waits for them explicitly with s_waitcnt vmcnt(n) (completion is in issue order).
__device__ __forceinline__ void async_copy_b128(uint32_t lds_base, const void *base, uint32_t voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_base), "v"(voff), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void async_copy_b32(uint32_t lds_base, const void *base, uint32_t voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(lds_base), "v"(voff), "s"(base) : "memory", "m0");
}
// The same with the LDS address given as a scalar base plus a compile-time offset: a loop that
// copies to many fixed places then keeps one base in a scalar register instead of one per place.
template <int OFF>
__device__ __forceinline__ void async_copy_b128_at(uint32_t lds_base, const void *base, uint32_t voff) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_base), "v"(voff), "s"(base), "n"(OFF) : "memory", "scc", "m0");
}
template <int OFF>
__device__ __forceinline__ void async_copy_b32_at(uint32_t lds_base, const void *base, uint32_t voff) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(lds_base), "v"(voff), "s"(base), "n"(OFF) : "memory", "scc", "m0");
}
#define WAIT_VMCNT(n) asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory")


// Transposed store of a 32 x COLS accumulator block (COLS = 64: acc[dblk][4g+j] = value(row l32,
// column 32dblk + 8g + 4hh + j) with acc = {acc0, acc1}; COLS = 32: acc0 only) times `mult`, through
// 4 KiB of wave-private LDS, as whole 2*COLS-byte pieces of rows (dst_row0: first row, first of the
// COLS columns; sn: row stride in elements).  Non-temporal stores: what is written is not read
// again by the kernel and should not displace its inputs from the caches.
template <bool BF16, int COLS = 64>
__device__ __forceinline__ void store_block(const f32x16 &acc0, const f32x16 &acc1, float mult, uint32_t lds_wave,
                                            uint16_t *dst_row0, int sn, int row0, int N, int lane)
{
    const f32x16 acc[2] = {acc0, acc1};
    using E = Elem<BF16>;
    const int l32 = lane & 31, hh = lane >> 5;
    const uint32_t wrow = lds_wave + l32 * 128 + hh * 8;
    const int fo = (l32 >> 1) & 7;
#pragma unroll
    for (int dblk = 0; dblk < COLS / 32; ++dblk)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const u32x2 o = {E::pack2_rne(acc[dblk][4 * g + 0] * mult, acc[dblk][4 * g + 1] * mult),
                             E::pack2_rne(acc[dblk][4 * g + 2] * mult, acc[dblk][4 * g + 3] * mult)};
            *(LDS_PTR(u32x2))(uintptr_t)(wrow + (((4 * dblk + g) ^ fo) << 4)) = o;
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    constexpr int LPR = COLS / 8;                 // lanes (16-byte chunks) per row
#pragma unroll
    for (int j = 0; j < LPR / 2; ++j) {
        const int row = (64 / LPR) * j + lane / LPR, pos = lane % LPR;
        const u32x4 v = lds_read_b128(lds_wave + row * 128 + ((pos ^ ((row >> 1) & 7)) << 4));
        if (row0 + row < N) __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(dst_row0 + (size_t)row * sn + pos * 8));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

}  // namespace
}  // namespace sma
