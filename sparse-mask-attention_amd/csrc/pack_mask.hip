// Mask bit-packer for gfx950: bool bytes [rows, N] -> uint32 words [rows, ceil(N/32)].
//
// Stands in for pack_mask_kernel (csrc/sparse_attention.cu:549-568 of the reference): bit j of
// word w of a row is column 32*w+j, bits for columns >= N are zero.  The op is pure HBM streaming
// (1 byte in per mask entry, 1 bit out), so the kernels are organised around memory coalescing:
//
//   pack_flat_kernel   N % 32 == 0.  Rows then hold whole words and the tensor is one flat stream:
//                      lane l of a wavefront loads the 16 bytes at 16*l of a contiguous 1 KiB span
//                      (one global_load_dwordx4, fully coalesced), turns them into 16 bits, pairs up
//                      with its neighbour lane, and even lanes store one word (coalesced 128 B per
//                      wavefront).  Two independent spans per thread keep loads in flight.
//   pack_row8_kernel   N % 8 == 0 (rows 8-byte aligned, e.g. N = 1000).  One wavefront per mask row:
//                      lane l loads the 8 bytes at 8*l of a 512-byte segment (coalesced), makes 8
//                      bits, the four lanes of a quad combine theirs with two DPP-style exchanges and
//                      lane 4k stores word k of the segment; the last word of a row is short.
//   pack_rows_kernel   any N.  One lane per output word, 4-byte loads when N % 4 == 0, byte loads
//                      otherwise; the last word of a row is filled only up to column N-1.
//
// A mask byte counts as "attend" when it is non-zero (torch.bool storage holds 0/1).
//
// The loads are ordinary (temporal) ones.  Non-temporal loads make the packer alone 15 % faster in
// a loop over the same mask, but the sequence pack -> attention, which is what a caller runs,
// 8 % slower (measured on MI355X: 32.5 vs 29.7 us for B=16, H=12, N=512).
#include "sma_internal.h"

namespace sma {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int PACK_THREADS = 256;
constexpr int PACK_UNROLL = 2;

// Four mask bytes -> four bytes that are 1 where the input byte is non-zero.
__device__ __forceinline__ uint32_t nonzero_bytes(uint32_t x)
{
    const uint32_t t = (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;
    return t >> 7;
}

// Sixteen mask bytes -> 16 bits (byte i -> bit i).  udot4 multiplies the four 0/1 bytes by the
// weights 1,2,4,8 (or 16..128) and adds the previous partial value: two dot products per 8 bytes.
__device__ __forceinline__ uint32_t bits16(u32x4 d)
{
    uint32_t lo = __builtin_amdgcn_udot4(nonzero_bytes(d.x), 0x08040201u, 0u, false);
    lo = __builtin_amdgcn_udot4(nonzero_bytes(d.y), 0x80402010u, lo, false);
    uint32_t hi = __builtin_amdgcn_udot4(nonzero_bytes(d.z), 0x08040201u, 0u, false);
    hi = __builtin_amdgcn_udot4(nonzero_bytes(d.w), 0x80402010u, hi, false);
    return lo | (hi << 8);
}

__global__ __launch_bounds__(PACK_THREADS) void pack_flat_kernel(const u32x4 *__restrict__ mask,
                                                                 uint32_t *__restrict__ packed,
                                                                 long long n_chunks)   // 16-byte chunks, even
{
    const long long base = (long long)blockIdx.x * (PACK_THREADS * PACK_UNROLL) + threadIdx.x;
    u32x4 d[PACK_UNROLL];
#pragma unroll
    for (int u = 0; u < PACK_UNROLL; ++u) {
        const long long ci = base + (long long)u * PACK_THREADS;
        u32x4 x = {0u, 0u, 0u, 0u};
        if (ci < n_chunks) x = mask[ci];
        d[u] = x;
    }
#pragma unroll
    for (int u = 0; u < PACK_UNROLL; ++u) {
        const long long ci = base + (long long)u * PACK_THREADS;
        const uint32_t h = bits16(d[u]);
        const uint32_t other = __shfl_down(h, 1, 64);      // neighbour lane holds the upper half-word
        if ((threadIdx.x & 1) == 0 && ci < n_chunks) packed[ci >> 1] = h | (other << 16);
    }
}

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__global__ __launch_bounds__(PACK_THREADS) void pack_row8_kernel(const uint8_t *__restrict__ mask,
                                                                 uint32_t *__restrict__ packed,
                                                                 long long rows, int N, int nw)
{
    const int lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * (PACK_THREADS / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;                       // whole wavefront leaves together
    const uint8_t *src = mask + row * (long long)N;
    uint32_t *dst = packed + row * (long long)nw;
    for (int seg0 = 0; seg0 * 512 < N; seg0 += 4) {          // four 512-byte segments in flight
        u32x2 d[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int col = (seg0 + u) * 512 + lane * 8;    // first column of this lane's 8 bytes
            u32x2 x = {0u, 0u};
            if (col < N) x = *reinterpret_cast<const u32x2 *>(src + col);
            d[u] = x;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            uint32_t b = __builtin_amdgcn_udot4(nonzero_bytes(d[u].x), 0x08040201u, 0u, false);
            b = __builtin_amdgcn_udot4(nonzero_bytes(d[u].y), 0x80402010u, b, false);
            b <<= 8 * (lane & 3);                          // position inside the word of this quad
            b |= __shfl_xor(b, 1, 64);
            b |= __shfl_xor(b, 2, 64);
            const int w = (seg0 + u) * 16 + (lane >> 2);
            if ((lane & 3) == 0 && w < nw) dst[w] = b;
        }
    }
}

template <bool ALIGNED4>
__global__ __launch_bounds__(PACK_THREADS) void pack_rows_kernel(const uint8_t *__restrict__ mask,
                                                                 uint32_t *__restrict__ packed,
                                                                 uint32_t total_words, int N, int nw)
{
    const uint32_t idx = blockIdx.x * (uint32_t)PACK_THREADS + threadIdx.x;
    if (idx >= total_words) return;
    const uint32_t row = idx / (uint32_t)nw;
    const int w = (int)(idx - row * (uint32_t)nw);
    const uint8_t *src = mask + (size_t)row * N + 32 * w;
    const int valid = min(32, N - 32 * w);          // columns of this word that exist (>= 1)
    uint32_t acc = 0u;
    if (ALIGNED4) {
        // N % 4 == 0: the row start and every 4-column group are 4-byte aligned and a group is
        // either wholly inside the row or wholly outside.
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            uint32_t x = 0u;
            if (4 * g < valid) x = *reinterpret_cast<const uint32_t *>(src + 4 * g);
            acc |= __builtin_amdgcn_udot4(nonzero_bytes(x), 0x08040201u, 0u, false) << (4 * g);
        }
    } else {
        for (int j = 0; j < valid; ++j) acc |= (uint32_t)(src[j] != 0) << j;
    }
    packed[idx] = acc;
}

}  // namespace

hipError_t launch_pack_mask(const uint8_t *mask, uint32_t *packed, long long rows, int N,
                            hipStream_t stream)
{
    if (rows == 0 || N == 0) return hipSuccess;
    const int nw = (N + 31) / 32;
    const bool flat = (N % 32 == 0) && ((reinterpret_cast<uintptr_t>(mask) & 15u) == 0);
    if (flat) {
        const long long n_chunks = rows * (long long)N / 16;
        const long long per_block = (long long)PACK_THREADS * PACK_UNROLL;
        const unsigned grid = (unsigned)((n_chunks + per_block - 1) / per_block);
        hipLaunchKernelGGL(pack_flat_kernel, dim3(grid), dim3(PACK_THREADS), 0, stream,
                           reinterpret_cast<const u32x4 *>(mask), packed, n_chunks);
    } else if ((N % 8 == 0) && ((reinterpret_cast<uintptr_t>(mask) & 7u) == 0)) {
        const unsigned grid = (unsigned)((rows + PACK_THREADS / 64 - 1) / (PACK_THREADS / 64));
        hipLaunchKernelGGL(pack_row8_kernel, dim3(grid), dim3(PACK_THREADS), 0, stream, mask, packed, rows, N, nw);
    } else {
        const uint32_t total = (uint32_t)(rows * nw);
        const unsigned grid = (total + PACK_THREADS - 1) / PACK_THREADS;
        const bool aligned4 = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(mask) & 3u) == 0);
        if (aligned4)
            hipLaunchKernelGGL(pack_rows_kernel<true>, dim3(grid), dim3(PACK_THREADS), 0, stream,
                               mask, packed, total, N, nw);
        else
            hipLaunchKernelGGL(pack_rows_kernel<false>, dim3(grid), dim3(PACK_THREADS), 0, stream,
                               mask, packed, total, N, nw);
    }
    return hipGetLastError();
}

}  // namespace sma
