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
    float c;                        // |scale| * log2(e), > 0
    float scale_abs;                // |scale|
    uint32_t qsign;                 // 0x80008000 when scale < 0 (q is negated on load), else 0
    uint32_t tail_mask;             // valid-bit mask of the last word of a mask row
};

hipError_t launch_attn_fwd(const AttnArgs &a, bool bf16, hipStream_t stream);
hipError_t launch_pack_mask(const uint8_t *mask, uint32_t *packed, long long rows, int N,
                            hipStream_t stream);

}  // namespace sma
