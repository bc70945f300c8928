// Internal C++ interface between the C-ABI layer (capi.hip) and the kernel launchers.
// Not installed; the public interface is include/sma.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sma {

// A [B, H, N, D] tensor of 16-bit elements (fp16 or bf16 bit patterns).  The D elements of a row
// are contiguous; the other extents have strides that are multiples of 8 elements (rows stay
// 16-byte aligned).  Byte offsets inside one (b, h) slab fit 31 bits (checked by the C-ABI layer).
// Kept small: kernel arguments are fetched by every work-group before it can request any data.
struct Rows {
    uint16_t *p;
    uint32_t sb8, sh8;              // batch and head strides in units of 8 elements (16 bytes)
    uint32_t sn;                    // row stride in elements
};

// The packed mask [Bm, Hm, N, nw] with Bm in {1, B}, Hm in {1, H}: rows are contiguous, a stride of
// 0 (in words) repeats the same mask for every batch entry / head.
struct PackedMask {
    const uint32_t *p;
    long long sb, sh;
};

// Division of a work-group number by a launch constant without the (long, VALU) division sequence:
// n / d == (n * mul) >> shift in 64-bit arithmetic for every 0 <= n < 2^31, with
// shift = 31 + ceil(log2 d) and mul = ceil(2^shift / d) < 2^32 (round-up method: mul * d exceeds
// 2^shift by at most 2^(shift - 31), which cannot carry into the quotient while n < 2^31).
struct FastDiv {
    uint32_t mul, shift;
};
inline FastDiv make_fastdiv(uint32_t d)
{
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    const uint64_t p = 1ull << (31 + l);
    return FastDiv{(uint32_t)((p + d - 1) / d), 31 + l};
}
__host__ __device__ inline uint32_t fastdiv(uint32_t n, FastDiv f)
{
    return (uint32_t)(((uint64_t)n * f.mul) >> f.shift);
}

// Arguments of the fused forward kernel, already validated by the C-ABI layer.
struct AttnArgs {
    Rows q, k, v;                   // inputs (never written)
    PackedMask mask;                // byte_mask != 0: p names boolean bytes [Bm, Hm, N, N], strides in bytes
    Rows out;
    float *lse;                     // [BH, N] contiguous, or nullptr
    int BH, H, N;
    int D;                          // head dim: 32, 64 or 128
    int byte_mask;                  // the mask is the caller's boolean tensor, not packed words
    uint32_t *mask_out;             // byte_mask only: nullptr, or where to leave the packed words [Bm, Hm, N, nw]
    uint32_t *map_out;              // byte_mask only: nullptr, or where to leave the tile map (layout as tile_map below)
    // packed mask only: nullptr, or the tile map [Bm, Hm, T, 2, ceil(T/32)] (T = ceil(N/64)): per block
    // of 64 query rows one bit per 64-key tile "some mask bit set", then one bit per key tile "all
    // mask bits set"; strides between batch entries / heads in words, 0 = shared
    const uint32_t *tile_map;
    long long map_sb, map_sh;
    int qtiles;                     // ceil(N / 128): query tiles (work-groups) per (b,h)
    FastDiv div_qtiles, div_H;      // filled in by the launcher
    // exp(scale * s) is evaluated as exp2(post_mul * (q_scale * q) . k): q is multiplied by
    // q_scale (sign of scale included, |q_scale| <= 1) when it is loaded, post_mul is a power of
    // two that is 1 unless |scale| * log2(e) > 1.
    float q_scale;
    float post_mul;
    uint32_t last_mask0, last_mask1;   // valid-bit masks of the two mask words of the last key tile
    // Work-groups with a linear id >= tail_start lower their waves' priority as they advance, so
    // that the (up to three) work-groups of a CU finish together instead of oldest first.  The
    // launcher sets 0 when the whole grid is resident at once, else the grid size (nobody yields).
    int tail_start;
};

// Arguments of the two backward kernels (dQ, then dK and dV), already validated.
struct AttnBwdArgs {
    Rows dout, q, k, v, out;                   // inputs (never written)
    const float *lse;                          // [BH, N] natural-log-sum-exp saved by the forward
    PackedMask mask;
    Rows dq, dk, dv;
    float *delta;                              // [BH, N] workspace: sum_d dout * out per query row
    const uint32_t *tile_map;                  // nullptr, or the tile map of the mask (as in AttnArgs)
    long long map_sb, map_sh;
    int BH, H, N;
    int D;                                     // head dim: 32, 64 or 128
    int qtiles;                                // ceil(N / 128)
    FastDiv div_qtiles, div_H;                 // filled in by the launcher
    float scale;                               // as given by the caller
    float q_scale, post_mul;                   // as in AttnArgs
    uint32_t last_mask0, last_mask1;
};

hipError_t launch_attn_fwd(const AttnArgs &a, bool bf16, hipStream_t stream);
hipError_t launch_attn_bwd(const AttnBwdArgs &a, bool bf16, hipStream_t stream);
hipError_t launch_pack_mask(const uint8_t *mask, uint32_t *packed, long long rows, int N,
                            hipStream_t stream);
// Whether the current device serves 8- and 16-byte loads from unaligned addresses (the row packers
// and the forward that reads the boolean mask depend on it): 1 yes, 0 no, -1 not known (the
// one-time check could not run because `stream` is being captured into a graph, or failed).  The
// first call per device launches a one-wavefront check on `stream` and waits for it.
int unaligned_access_state(hipStream_t stream);
// tile map [slabs, ceil(N/64), 2, ceil(ceil(N/64)/32)] of packed words [slabs, N, ceil(N/32)]
hipError_t launch_tile_map(const uint32_t *packed, uint32_t *map, long long slabs, int N, hipStream_t stream);

}  // namespace sma
