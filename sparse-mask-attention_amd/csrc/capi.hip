// extern "C" layer of libsma_hip.so: argument validation and dispatch.  See include/sma.h.
#include <math.h>

#include "sma.h"
#include "sma_internal.h"

namespace {

inline bool misaligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }

}  // namespace

extern "C" {

int sma_version(void) { return 100; }   // 0.1.0

const char *sma_strerror(int code)
{
    switch (code) {
    case SMA_OK:               return "ok";
    case SMA_ERR_NULL_POINTER: return "a required pointer is NULL";
    case SMA_ERR_BAD_SHAPE:    return "bad shape: negative extent or index range exceeded";
    case SMA_ERR_HEAD_DIM:     return "unsupported head_dim (only 64)";
    case SMA_ERR_DTYPE:        return "unsupported dtype (need fp16 or bf16)";
    case SMA_ERR_SCALE:        return "scale must be finite";
    case SMA_ERR_LAUNCH:       return "HIP kernel launch failed";
    case SMA_ERR_ALIGNMENT:    return "misaligned pointer";
    default:                   return "unknown error code";
    }
}

int sma_pack_mask(const uint8_t *mask, uint32_t *packed, int B, int H, int N, void *stream)
{
    if (B < 0 || H < 0 || N < 0) return SMA_ERR_BAD_SHAPE;
    const long long rows = (long long)B * H * N;
    if (rows == 0) return SMA_OK;
    if (mask == nullptr || packed == nullptr) return SMA_ERR_NULL_POINTER;
    const long long nw = (N + 31) / 32;
    if (rows * nw >= (1ll << 31) || rows >= (1ll << 31)) return SMA_ERR_BAD_SHAPE;
    if (misaligned(packed, 4)) return SMA_ERR_ALIGNMENT;
    const hipError_t e = sma::launch_pack_mask(mask, packed, rows, N, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? SMA_OK : SMA_ERR_LAUNCH;
}

int sma_attn_fwd(const void *q, const void *k, const void *v, const uint32_t *mask_packed,
                 void *out, float *lse, int B, int H, int N, int D, float scale, int dtype,
                 void *stream)
{
    if (B < 0 || H < 0 || N < 0 || D < 0) return SMA_ERR_BAD_SHAPE;
    if (D != 64) return SMA_ERR_HEAD_DIM;
    if (dtype != SMA_DTYPE_F16 && dtype != SMA_DTYPE_BF16) return SMA_ERR_DTYPE;
    if (!isfinite(scale)) return SMA_ERR_SCALE;
    const long long BH = (long long)B * H;
    if (BH == 0 || N == 0) return SMA_OK;
    if (!q || !k || !v || !mask_packed || !out) return SMA_ERR_NULL_POINTER;
    const long long qtiles = (N + 127) / 128;
    if (BH * qtiles >= (1ll << 31) || BH * N >= (1ll << 31)) return SMA_ERR_BAD_SHAPE;
    if (misaligned(q, 16) || misaligned(k, 16) || misaligned(v, 16) || misaligned(out, 16) ||
        misaligned(mask_packed, 4) || (lse && misaligned(lse, 4)))
        return SMA_ERR_ALIGNMENT;

    sma::AttnArgs a;
    a.q = static_cast<const uint16_t *>(q);
    a.k = static_cast<const uint16_t *>(k);
    a.v = static_cast<const uint16_t *>(v);
    a.mask_packed = mask_packed;
    a.out = static_cast<uint16_t *>(out);
    a.lse = lse;
    a.BH = (int)BH;
    a.N = N;
    a.nw = (N + 31) / 32;
    a.qtiles = (int)qtiles;
    // exp(scale*s - max) is evaluated as exp2(c*s' - c*max') with c = |scale|*log2(e) > 0 and
    // s' = s for scale > 0, s' = -s (q negated on load, exact) for scale < 0.  scale == 0 uses a
    // denormal-free tiny c: kept scores all map to exp2(~0) = 1, dropped ones stay at -inf.
    const float LOG2E = 1.4426950408889634f;
    float c = fabsf(scale) * LOG2E;
    if (!(c > 0.0f)) c = 1e-30f;
    a.c = c;
    a.scale_abs = fabsf(scale);
    a.qsign = (scale < 0.0f) ? 0x80008000u : 0u;
    const int tail = N & 31;
    a.tail_mask = tail ? ((1u << tail) - 1u) : 0xffffffffu;

    const hipError_t e = sma::launch_attn_fwd(a, dtype == SMA_DTYPE_BF16, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? SMA_OK : SMA_ERR_LAUNCH;
}

}  // extern "C"
