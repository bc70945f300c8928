// extern "C" layer of libsma_hip.so: argument validation and dispatch.  See include/sma.h.
#include <math.h>

#include <atomic>

#include "sma.h"
#include "sma_internal.h"

namespace {

inline bool misaligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }

// a * b < 2^31 for non-negative a, b, without forming a product that could overflow 64 bits
// (B * H alone may reach 2^62)
inline bool below_2_31(long long a, long long b)
{
    const long long lim = 1ll << 31;
    return a == 0 || b == 0 || (a < lim && b < lim && a * b < lim);
}

inline sma_tensor dense(const void *p, int H, int N, int D)
{
    return sma_tensor{const_cast<void *>(p), (int64_t)H * N * D, (int64_t)N * D, (int64_t)D};
}

// Checks one strided [B,H,N,D] tensor and converts it; SMA_OK or an error code.  An output
// (`written`) must not fold several rows onto one address: a row stride below D or a zero stride
// over an extent above 1 would make rows or work-groups overwrite each other.
int to_rows(const sma_tensor *t, int B, int H, int N, int D, bool written, sma::Rows *r)
{
    if (t == nullptr || t->data == nullptr) return SMA_ERR_NULL_POINTER;
    if (misaligned(t->data, 16)) return SMA_ERR_ALIGNMENT;
    if (t->stride_b < 0 || t->stride_h < 0 || t->stride_n < 0) return SMA_ERR_STRIDE;
    if ((t->stride_b | t->stride_h | t->stride_n) & 7) return SMA_ERR_STRIDE;
    if ((long long)(N - 1) * t->stride_n * 2 + 2 * D >= (1ll << 31)) return SMA_ERR_STRIDE;
    if (t->stride_b >= (1ll << 35) || t->stride_h >= (1ll << 35) || t->stride_n >= (1ll << 23)) return SMA_ERR_STRIDE;
    if (written && ((N > 1 && t->stride_n < D) || (H > 1 && t->stride_h == 0) || (B > 1 && t->stride_b == 0)))
        return SMA_ERR_STRIDE;
    r->p = static_cast<uint16_t *>(t->data);
    r->sb8 = (uint32_t)(t->stride_b >> 3);
    r->sh8 = (uint32_t)(t->stride_h >> 3);
    r->sn = (uint32_t)t->stride_n;
    return SMA_OK;
}

// Workspace of sma_attn_bwd_static_ws: the per-row sums the two backward kernels exchange, held in
// the library's own device image instead of a caller's buffer.  Every GPU the library runs on has
// its own copy at its own address; the name below is only a host-side handle for
// hipGetSymbolAddress and is never passed to a kernel.
constexpr long long STATIC_WS_ROWS = 1ll << 20;          // B*H*N the entry point accepts (4 MiB)
static __device__ __align__(256) float scratch[STATIC_WS_ROWS];

// Device address of `scratch` on the current device, looked up once per device ordinal.
float *static_workspace()
{
    static std::atomic<float *> cached[64];     // nullptr = not asked yet; racing threads store the same address
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    float *p = cached[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        void *sym = nullptr;
        if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || sym == nullptr) return nullptr;
        p = static_cast<float *>(sym);
        cached[dev].store(p, std::memory_order_release);
    }
    return p;
}

}  // namespace

extern "C" {

int sma_version(void) { return 100; }   // 0.1.0

const char *sma_strerror(int code)
{
    switch (code) {
    case SMA_OK:               return "ok";
    case SMA_ERR_NULL_POINTER: return "a required pointer is NULL";
    case SMA_ERR_BAD_SHAPE:    return "bad shape: negative extent or index range exceeded";
    case SMA_ERR_HEAD_DIM:     return "unsupported head_dim (32, 64 or 128)";
    case SMA_ERR_DTYPE:        return "unsupported dtype (need fp16 or bf16)";
    case SMA_ERR_SCALE:        return "scale must be finite";
    case SMA_ERR_LAUNCH:       return "HIP kernel launch failed";
    case SMA_ERR_ALIGNMENT:    return "misaligned pointer";
    case SMA_ERR_STRIDE:       return "bad stride: negative, not a multiple of 8 elements, or too large";
    case SMA_ERR_WORKSPACE:    return "problem too large for the library's static workspace";
    case SMA_ERR_DEVICE:       return "the device does not serve loads from unaligned addresses";
    default:                   return "unknown error code";
    }
}

long long sma_tile_map_words(int N)
{
    if (N <= 0) return 0;
    const long long blocks = (N + 63) / 64, tw = (blocks + 31) / 32;
    return blocks * 2 * tw;
}

int sma_tile_map(const uint32_t *mask_packed, uint32_t *tile_map, int B, int H, int N, void *stream)
{
    if (B < 0 || H < 0 || N < 0) return SMA_ERR_BAD_SHAPE;
    const long long slabs = (long long)B * H;
    if (slabs == 0 || N == 0) return SMA_OK;
    if (mask_packed == nullptr || tile_map == nullptr) return SMA_ERR_NULL_POINTER;
    if (misaligned(mask_packed, 4) || misaligned(tile_map, 4)) return SMA_ERR_ALIGNMENT;
    if (N > 131072 || !below_2_31(slabs, (N + 63) / 64)) return SMA_ERR_BAD_SHAPE;
    const hipError_t e = sma::launch_tile_map(mask_packed, tile_map, slabs, N, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? SMA_OK : SMA_ERR_LAUNCH;
}

int sma_device_check(void *stream)
{
    return sma::unaligned_access_state(static_cast<hipStream_t>(stream)) == 0 ? SMA_ERR_DEVICE : SMA_OK;
}

int sma_pack_mask_map(const uint8_t *mask, uint32_t *packed, uint32_t *tile_map, int B, int H, int N,
                      void *stream)
{
    // what sma_tile_map would refuse is refused before anything is written
    if (tile_map != nullptr && B >= 0 && H >= 0 &&
        (N > 131072 || !below_2_31((long long)B * H, (N + 63) / 64) || misaligned(tile_map, 4)))
        return misaligned(tile_map, 4) ? SMA_ERR_ALIGNMENT : SMA_ERR_BAD_SHAPE;
    const int st = sma_pack_mask(mask, packed, B, H, N, stream);
    if (st != SMA_OK || tile_map == nullptr) return st;
    return sma_tile_map(packed, tile_map, B, H, N, stream);
}

int sma_pack_mask(const uint8_t *mask, uint32_t *packed, int B, int H, int N, void *stream)
{
    if (B < 0 || H < 0 || N < 0) return SMA_ERR_BAD_SHAPE;
    if (B == 0 || H == 0 || N == 0) return SMA_OK;
    if (mask == nullptr || packed == nullptr) return SMA_ERR_NULL_POINTER;
    const long long nw = (N + 31) / 32;
    if (!below_2_31((long long)B * H, N) || !below_2_31((long long)B * H * N, nw)) return SMA_ERR_BAD_SHAPE;
    const long long rows = (long long)B * H * N;
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

int sma_attn_bwd_map_strided(const sma_tensor *dout, const sma_tensor *q, const sma_tensor *k,
                             const sma_tensor *v, const sma_tensor *out, const float *lse,
                             const uint32_t *mask_packed, int64_t mask_stride_b, int64_t mask_stride_h,
                             const uint32_t *tile_map, const sma_tensor *dq, const sma_tensor *dk,
                             const sma_tensor *dv, float *delta_ws, int B, int H, int N, int D, float scale,
                             int dtype, void *stream)
{
    if (B < 0 || H < 0 || N < 0 || D < 0) return SMA_ERR_BAD_SHAPE;
    if (D != 32 && D != 64 && D != 128) return SMA_ERR_HEAD_DIM;
    if (dtype != SMA_DTYPE_F16 && dtype != SMA_DTYPE_BF16) return SMA_ERR_DTYPE;
    if (!isfinite(scale)) return SMA_ERR_SCALE;
    const long long BH = (long long)B * H;
    if (BH == 0 || N == 0) return SMA_OK;
    if (!lse || !mask_packed || !delta_ws) return SMA_ERR_NULL_POINTER;
    const long long qtiles = (N + 127) / 128;
    if (!below_2_31(BH, qtiles) || !below_2_31(BH, N)) return SMA_ERR_BAD_SHAPE;
    // a lane's byte offset into the packed mask of one (b,h) is a 32-bit register
    if ((long long)N * ((N + 31) / 32) * 4 >= (1ll << 32)) return SMA_ERR_BAD_SHAPE;
    if (misaligned(mask_packed, 4) || misaligned(lse, 4) || misaligned(delta_ws, 4) || (tile_map && misaligned(tile_map, 4)))
        return SMA_ERR_ALIGNMENT;
    if (tile_map && N > 131072) return SMA_ERR_BAD_SHAPE;
    if (mask_stride_b < 0 || mask_stride_h < 0) return SMA_ERR_STRIDE;

    sma::AttnBwdArgs a;
    const sma_tensor *in[8] = {dout, q, k, v, out, dq, dk, dv};
    sma::Rows *to[8] = {&a.dout, &a.q, &a.k, &a.v, &a.out, &a.dq, &a.dk, &a.dv};
    for (int i = 0; i < 8; ++i) {
        const int st = to_rows(in[i], B, H, N, D, i >= 5, to[i]);
        if (st != SMA_OK) return st;
    }
    a.lse = lse;
    a.mask = sma::PackedMask{mask_packed, mask_stride_b, mask_stride_h};
    a.delta = delta_ws;
    a.tile_map = tile_map;
    const long long map_words = sma_tile_map_words(N);
    a.map_sh = (H > 1 && mask_stride_h != 0) ? map_words : 0;
    a.map_sb = (B > 1 && mask_stride_b != 0) ? ((H > 1 && mask_stride_h != 0) ? (long long)H : 1ll) * map_words : 0;
    a.BH = (int)BH;
    a.H = H;
    a.N = N;
    a.D = D;
    a.qtiles = (int)qtiles;
    a.scale = scale;
    split_scale(scale, &a.q_scale, &a.post_mul);
    last_tile_masks(N, &a.last_mask0, &a.last_mask1);
    const hipError_t e = sma::launch_attn_bwd(a, dtype == SMA_DTYPE_BF16, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? SMA_OK : SMA_ERR_LAUNCH;
}

int sma_attn_bwd_strided(const sma_tensor *dout, const sma_tensor *q, const sma_tensor *k,
                         const sma_tensor *v, const sma_tensor *out, const float *lse,
                         const uint32_t *mask_packed, int64_t mask_stride_b, int64_t mask_stride_h,
                         const sma_tensor *dq, const sma_tensor *dk, const sma_tensor *dv,
                         float *delta_ws, int B, int H, int N, int D, float scale, int dtype,
                         void *stream)
{
    return sma_attn_bwd_map_strided(dout, q, k, v, out, lse, mask_packed, mask_stride_b, mask_stride_h, nullptr, dq,
                                    dk, dv, delta_ws, B, H, N, D, scale, dtype, stream);
}

int sma_attn_bwd_map(const void *dout, const void *q, const void *k, const void *v, const void *out,
                     const float *lse, const uint32_t *mask_packed, const uint32_t *tile_map, void *dq,
                     void *dk, void *dv, float *delta_ws, int B, int H, int N, int D, float scale, int dtype,
                     void *stream)
{
    const sma_tensor t[8] = {dense(dout, H, N, D), dense(q, H, N, D), dense(k, H, N, D), dense(v, H, N, D),
                             dense(out, H, N, D), dense(dq, H, N, D), dense(dk, H, N, D), dense(dv, H, N, D)};
    const int64_t msh = (int64_t)N * ((N + 31) / 32);
    return sma_attn_bwd_map_strided(&t[0], &t[1], &t[2], &t[3], &t[4], lse, mask_packed, msh * H, msh, tile_map,
                                    &t[5], &t[6], &t[7], delta_ws, B, H, N, D, scale, dtype, stream);
}

int sma_attn_fwd_map_strided(const sma_tensor *q, const sma_tensor *k, const sma_tensor *v,
                             const uint32_t *mask_packed, int64_t mask_stride_b, int64_t mask_stride_h,
                             const uint32_t *tile_map, const sma_tensor *out, float *lse, int B, int H,
                             int N, int D, float scale, int dtype, void *stream)
{
    if (B < 0 || H < 0 || N < 0 || D < 0) return SMA_ERR_BAD_SHAPE;
    if (D != 32 && D != 64 && D != 128) return SMA_ERR_HEAD_DIM;
    if (dtype != SMA_DTYPE_F16 && dtype != SMA_DTYPE_BF16) return SMA_ERR_DTYPE;
    if (!isfinite(scale)) return SMA_ERR_SCALE;
    const long long BH = (long long)B * H;
    if (BH == 0 || N == 0) return SMA_OK;
    if (!mask_packed) return SMA_ERR_NULL_POINTER;
    const long long qtiles = (N + 127) / 128;
    if (!below_2_31(BH, qtiles) || !below_2_31(BH, N)) return SMA_ERR_BAD_SHAPE;
    // a lane's byte offset into the packed mask of one (b,h) is a 32-bit register
    if ((long long)N * ((N + 31) / 32) * 4 >= (1ll << 32)) return SMA_ERR_BAD_SHAPE;
    if (misaligned(mask_packed, 4) || (lse && misaligned(lse, 4)) || (tile_map && misaligned(tile_map, 4)))
        return SMA_ERR_ALIGNMENT;
    if (tile_map && N > 131072) return SMA_ERR_BAD_SHAPE;      // the limit of sma_tile_map, which makes the maps
    if (mask_stride_b < 0 || mask_stride_h < 0) return SMA_ERR_STRIDE;

    sma::AttnArgs a;
    const sma_tensor *in[4] = {q, k, v, out};
    sma::Rows *to[4] = {&a.q, &a.k, &a.v, &a.out};
    for (int i = 0; i < 4; ++i) {
        const int st = to_rows(in[i], B, H, N, D, i == 3, to[i]);
        if (st != SMA_OK) return st;
    }
    a.mask = sma::PackedMask{mask_packed, mask_stride_b, mask_stride_h};
    a.lse = lse;
    a.BH = (int)BH;
    a.H = H;
    a.N = N;
    a.D = D;
    a.byte_mask = 0;
    a.mask_out = nullptr;
    a.map_out = nullptr;
    // the map is contiguous [Bm, Hm, ...] with the mask's own Bm, Hm (1 where the mask is shared)
    a.tile_map = tile_map;
    const long long map_words = sma_tile_map_words(N);
    a.map_sh = (H > 1 && mask_stride_h != 0) ? map_words : 0;
    a.map_sb = (B > 1 && mask_stride_b != 0) ? ((H > 1 && mask_stride_h != 0) ? (long long)H : 1ll) * map_words : 0;
    a.qtiles = (int)qtiles;
    split_scale(scale, &a.q_scale, &a.post_mul);
    last_tile_masks(N, &a.last_mask0, &a.last_mask1);

    const hipError_t e = sma::launch_attn_fwd(a, dtype == SMA_DTYPE_BF16, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? SMA_OK : SMA_ERR_LAUNCH;
}

int sma_attn_fwd_strided(const sma_tensor *q, const sma_tensor *k, const sma_tensor *v,
                         const uint32_t *mask_packed, int64_t mask_stride_b, int64_t mask_stride_h,
                         const sma_tensor *out, float *lse, int B, int H, int N, int D, float scale,
                         int dtype, void *stream)
{
    return sma_attn_fwd_map_strided(q, k, v, mask_packed, mask_stride_b, mask_stride_h, nullptr, out, lse, B, H, N,
                                    D, scale, dtype, stream);
}

int sma_attn_fwd_map(const void *q, const void *k, const void *v, const uint32_t *mask_packed,
                     const uint32_t *tile_map, void *out, float *lse, int B, int H, int N, int D,
                     float scale, int dtype, void *stream)
{
    const sma_tensor t[4] = {dense(q, H, N, D), dense(k, H, N, D), dense(v, H, N, D), dense(out, H, N, D)};
    const int64_t msh = (int64_t)N * ((N + 31) / 32);
    return sma_attn_fwd_map_strided(&t[0], &t[1], &t[2], mask_packed, msh * H, msh, tile_map, &t[3], lse, B, H, N, D,
                                    scale, dtype, stream);
}

int sma_attn_fwd_bool_mask(const void *q, const void *k, const void *v, const uint8_t *mask,
                           int64_t mask_stride_b, int64_t mask_stride_h, void *out, float *lse,
                           uint32_t *packed_out, int B, int H, int N, int D, float scale, int dtype,
                           void *stream)
{
    return sma_attn_fwd_bool_mask_map(q, k, v, mask, mask_stride_b, mask_stride_h, out, lse, packed_out, nullptr, B,
                                      H, N, D, scale, dtype, stream);
}

int sma_attn_fwd_bool_mask_map(const void *q, const void *k, const void *v, const uint8_t *mask,
                               int64_t mask_stride_b, int64_t mask_stride_h, void *out, float *lse,
                               uint32_t *packed_out, uint32_t *map_out, int B, int H, int N, int D,
                               float scale, int dtype, void *stream)
{
    const sma_tensor t[4] = {dense(q, H, N, D), dense(k, H, N, D), dense(v, H, N, D), dense(out, H, N, D)};
    return sma_attn_fwd_bool_mask_strided(&t[0], &t[1], &t[2], mask, mask_stride_b, mask_stride_h, &t[3], lse,
                                          packed_out, map_out, B, H, N, D, scale, dtype, stream);
}

int sma_attn_fwd_bool_mask_strided(const sma_tensor *q, const sma_tensor *k, const sma_tensor *v,
                                   const uint8_t *mask, int64_t mask_stride_b, int64_t mask_stride_h,
                                   const sma_tensor *out, float *lse, uint32_t *packed_out, uint32_t *map_out,
                                   int B, int H, int N, int D, float scale, int dtype, void *stream)
{
    if (B < 0 || H < 0 || N < 0 || D < 0) return SMA_ERR_BAD_SHAPE;
    if (D != 32 && D != 64 && D != 128) return SMA_ERR_HEAD_DIM;
    if (dtype != SMA_DTYPE_F16 && dtype != SMA_DTYPE_BF16) return SMA_ERR_DTYPE;
    if (!isfinite(scale)) return SMA_ERR_SCALE;
    const long long BH = (long long)B * H;
    if (BH == 0 || N == 0) return SMA_OK;
    if (!mask) return SMA_ERR_NULL_POINTER;
    if (N < 16) return SMA_ERR_BAD_SHAPE;               // a row holds at least one 16-byte copy
    const long long qtiles = (N + 127) / 128;
    if (!below_2_31(BH, qtiles) || !below_2_31(BH, N)) return SMA_ERR_BAD_SHAPE;
    // a lane's byte offset into the mask of one (b,h) is a 32-bit register
    if ((long long)N * N >= (1ll << 31)) return SMA_ERR_BAD_SHAPE;
    if ((lse && misaligned(lse, 4)) || (packed_out && misaligned(packed_out, 4)) || (map_out && misaligned(map_out, 4)))
        return SMA_ERR_ALIGNMENT;
    // the kernel collects the map in 32 words of 32 key tiles per wavefront (N <= 65536; the limit on
    // N * N above is the tighter one)
    if (map_out && (N + 63) / 64 > 32 * 32) return SMA_ERR_BAD_SHAPE;
    if (mask_stride_b < 0 || mask_stride_h < 0) return SMA_ERR_STRIDE;

    sma::AttnArgs a;
    const sma_tensor *in[4] = {q, k, v, out};
    sma::Rows *to[4] = {&a.q, &a.k, &a.v, &a.out};
    for (int i = 0; i < 4; ++i) {
        const int st = to_rows(in[i], B, H, N, D, i == 3, to[i]);
        if (st != SMA_OK) return st;
    }
    // mask rows start at any byte address: the kernel's 16-byte copies rely on the device serving them
    if (sma::unaligned_access_state(static_cast<hipStream_t>(stream)) == 0) return SMA_ERR_DEVICE;
    a.mask = sma::PackedMask{reinterpret_cast<const uint32_t *>(mask), mask_stride_b, mask_stride_h};
    a.lse = lse;
    a.BH = (int)BH;
    a.H = H;
    a.N = N;
    a.D = D;
    a.byte_mask = 1;
    a.mask_out = packed_out;
    a.map_out = map_out;
    a.tile_map = nullptr;
    a.map_sb = a.map_sh = 0;
    a.qtiles = (int)qtiles;
    split_scale(scale, &a.q_scale, &a.post_mul);
    last_tile_masks(N, &a.last_mask0, &a.last_mask1);

    const hipError_t e = sma::launch_attn_fwd(a, dtype == SMA_DTYPE_BF16, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? SMA_OK : SMA_ERR_LAUNCH;
}

int sma_attn_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out,
                 const float *lse, const uint32_t *mask_packed, void *dq, void *dk, void *dv,
                 float *delta_ws, int B, int H, int N, int D, float scale, int dtype, void *stream)
{
    const sma_tensor t[8] = {dense(dout, H, N, D), dense(q, H, N, D), dense(k, H, N, D), dense(v, H, N, D),
                             dense(out, H, N, D), dense(dq, H, N, D), dense(dk, H, N, D), dense(dv, H, N, D)};
    const int64_t msh = (int64_t)N * ((N + 31) / 32);
    return sma_attn_bwd_strided(&t[0], &t[1], &t[2], &t[3], &t[4], lse, mask_packed, msh * H, msh,
                                &t[5], &t[6], &t[7], delta_ws, B, H, N, D, scale, dtype, stream);
}

int sma_attn_bwd_static_ws(const void *dout, const void *q, const void *k, const void *v, const void *out,
                           const float *lse, const uint32_t *mask_packed, void *dq, void *dk, void *dv,
                           int B, int H, int N, int D, float scale, int dtype, void *stream)
{
    // the cheap argument checks of sma_attn_bwd first, so that a bad call reports what is wrong with
    // it and neither an empty nor an invalid call touches the workspace
    if (B < 0 || H < 0 || N < 0 || D < 0) return SMA_ERR_BAD_SHAPE;
    if (D != 32 && D != 64 && D != 128) return SMA_ERR_HEAD_DIM;
    if (dtype != SMA_DTYPE_F16 && dtype != SMA_DTYPE_BF16) return SMA_ERR_DTYPE;
    if (!isfinite(scale)) return SMA_ERR_SCALE;
    if (B == 0 || H == 0 || N == 0) return SMA_OK;
    if ((long long)B * H > STATIC_WS_ROWS || (long long)B * H * N > STATIC_WS_ROWS) return SMA_ERR_WORKSPACE;
    float *ws = static_workspace();
    if (ws == nullptr) return SMA_ERR_LAUNCH;
    // Both kernels run on `stream`, the first writes every entry the second reads: nothing has to
    // be cleared between calls, and what a previous (larger) call left behind is never read.
    return sma_attn_bwd(dout, q, k, v, out, lse, mask_packed, dq, dk, dv, ws, B, H, N, D, scale, dtype, stream);
}

int sma_attn_fwd(const void *q, const void *k, const void *v, const uint32_t *mask_packed,
                 void *out, float *lse, int B, int H, int N, int D, float scale, int dtype,
                 void *stream)
{
    const sma_tensor t[4] = {dense(q, H, N, D), dense(k, H, N, D), dense(v, H, N, D), dense(out, H, N, D)};
    const int64_t msh = (int64_t)N * ((N + 31) / 32);
    return sma_attn_fwd_strided(&t[0], &t[1], &t[2], mask_packed, msh * H, msh, &t[3], lse, B, H, N, D,
                                scale, dtype, stream);
}

}  // extern "C"
