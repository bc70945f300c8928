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
                 :: "s"(lds_base), "v"(voff), "s"(base) : "memory");
}
__device__ __forceinline__ void async_copy_b32(uint32_t lds_base, const void *base, uint32_t voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(lds_base), "v"(voff), "s"(base) : "memory");
}
// The same with the LDS address given as a scalar base plus a compile-time offset: a loop that
// copies to many fixed places then keeps one base in a scalar register instead of one per place.
template <int OFF>
__device__ __forceinline__ void async_copy_b128_at(uint32_t lds_base, const void *base, uint32_t voff) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_base), "v"(voff), "s"(base), "n"(OFF) : "memory", "scc");
}
template <int OFF>
__device__ __forceinline__ void async_copy_b32_at(uint32_t lds_base, const void *base, uint32_t voff) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(lds_base), "v"(voff), "s"(base), "n"(OFF) : "memory", "scc");
}
#define WAIT_VMCNT(n) asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory")

}  // namespace
}  // namespace sma
