// Internal C++ interface between the C-ABI layer (capi.hip) and the kernel launchers.
// Not installed; the public interface is include/sma.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sma {

// Arguments of the fused forward kernel, already validated by the C-ABI layer.
struct AttnArgs {
    const uint16_t *q, *k, *v;      // [BH, N, 64] 16-bit elements (fp16 or bf16 bit patterns)
    const uint32_t *mask_packed;    // [BH, N, nw]
    uint16_t *out;                  // [BH, N, 64]
    float *lse;                     // [BH, N] or nullptr
    int BH, N, nw;
    int qtiles;                     // ceil(N / 128): query tiles (work-groups) per (b,h)
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
    const uint16_t *dout, *q, *k, *v, *out;   // [BH, N, 64]
    const float *lse;                          // [BH, N] natural-log-sum-exp saved by the forward
    const uint32_t *mask_packed;               // [BH, N, nw]
    uint16_t *dq, *dk, *dv;                    // [BH, N, 64]
    float *delta;                              // [BH, N] workspace: sum_d dout * out per query row
    int BH, N, nw;
    int qtiles;                                // ceil(N / 128)
    float scale;                               // as given by the caller
    float q_scale, post_mul;                   // as in AttnArgs
    uint32_t last_mask0, last_mask1;
};

hipError_t launch_attn_fwd(const AttnArgs &a, bool bf16, hipStream_t stream);
hipError_t launch_attn_bwd(const AttnBwdArgs &a, bool bf16, hipStream_t stream);
hipError_t launch_pack_mask(const uint8_t *mask, uint32_t *packed, long long rows, int N,
                            hipStream_t stream);

}  // namespace sma
