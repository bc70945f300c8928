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

// exp(scale*s) = exp2(post_mul * (q_scale*q).k) with q_scale*post_mul = scale*log2(e), post_mul a
// power of two >= 1 chosen so that |q_scale| <= 1: scaling q cannot overflow its 16-bit format.
static void split_scale(float scale, float *q_scale, float *post_mul)
{
    const float LOG2E = 1.4426950408889634f;
    const float c = fabsf(scale) * LOG2E;
    float pm = 1.0f;
    if (c > 1.0f) {
        int e = 0;
        (void)frexpf(c, &e);                    // c = f * 2^e, f in [0.5, 1)
        pm = ldexpf(1.0f, e);
    }
    *q_scale = (scale < 0.0f ? -c : c) / pm;
    *post_mul = pm;
}

// valid-bit masks of the two mask words of the last 64-key tile
static void last_tile_masks(int N, uint32_t *m0, uint32_t *m1)
{
    const int T = (N + 63) / 64;
    const int rem = N - 64 * (T - 1);           // keys in the last tile, 1..64
    const int v0 = rem < 32 ? rem : 32, v1 = rem > 32 ? rem - 32 : 0;
    *m0 = v0 >= 32 ? 0xffffffffu : ((1u << v0) - 1u);
    *m1 = v1 >= 32 ? 0xffffffffu : ((1u << v1) - 1u);
}

int sma_attn_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out,
                 const float *lse, const uint32_t *mask_packed, void *dq, void *dk, void *dv,
                 float *delta_ws, int B, int H, int N, int D, float scale, int dtype, void *stream)
{
    if (B < 0 || H < 0 || N < 0 || D < 0) return SMA_ERR_BAD_SHAPE;
    if (D != 64) return SMA_ERR_HEAD_DIM;
    if (dtype != SMA_DTYPE_F16 && dtype != SMA_DTYPE_BF16) return SMA_ERR_DTYPE;
    if (!isfinite(scale)) return SMA_ERR_SCALE;
    const long long BH = (long long)B * H;
    if (BH == 0 || N == 0) return SMA_OK;
    if (!dout || !q || !k || !v || !out || !lse || !mask_packed || !dq || !dk || !dv || !delta_ws)
        return SMA_ERR_NULL_POINTER;
    const long long qtiles = (N + 127) / 128;
    if (BH * qtiles >= (1ll << 31) || BH * N >= (1ll << 31)) return SMA_ERR_BAD_SHAPE;
    if (misaligned(dout, 16) || misaligned(q, 16) || misaligned(k, 16) || misaligned(v, 16) ||
        misaligned(out, 16) || misaligned(dq, 16) || misaligned(dk, 16) || misaligned(dv, 16) ||
        misaligned(mask_packed, 4) || misaligned(lse, 4) || misaligned(delta_ws, 4))
        return SMA_ERR_ALIGNMENT;

    sma::AttnBwdArgs a;
    a.dout = static_cast<const uint16_t *>(dout);
    a.q = static_cast<const uint16_t *>(q);
    a.k = static_cast<const uint16_t *>(k);
    a.v = static_cast<const uint16_t *>(v);
    a.out = static_cast<const uint16_t *>(out);
    a.lse = lse;
    a.mask_packed = mask_packed;
    a.dq = static_cast<uint16_t *>(dq);
    a.dk = static_cast<uint16_t *>(dk);
    a.dv = static_cast<uint16_t *>(dv);
    a.delta = delta_ws;
    a.BH = (int)BH;
    a.N = N;
    a.nw = (N + 31) / 32;
    a.qtiles = (int)qtiles;
    a.scale = scale;
    split_scale(scale, &a.q_scale, &a.post_mul);
    last_tile_masks(N, &a.last_mask0, &a.last_mask1);
    const hipError_t e = sma::launch_attn_bwd(a, dtype == SMA_DTYPE_BF16, static_cast<hipStream_t>(stream));
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
    split_scale(scale, &a.q_scale, &a.post_mul);
    last_tile_masks(N, &a.last_mask0, &a.last_mask1);

    const hipError_t e = sma::launch_attn_fwd(a, dtype == SMA_DTYPE_BF16, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? SMA_OK : SMA_ERR_LAUNCH;
}

}  // extern "C"
