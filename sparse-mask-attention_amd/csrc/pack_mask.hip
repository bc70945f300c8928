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
//   pack_row_kernel    any other N >= 8 (e.g. N = 1000) or mask address.  One wavefront per mask row:
//                      lane l loads the 8 bytes at 8*l of a 512-byte segment (coalesced, at whatever
//                      alignment the row has), makes 8 bits, the four lanes of a quad combine theirs
//                      with two DPP-style exchanges and lane 4k stores word k of the segment.  The
//                      lane that holds the row's end loads the row's last 8 bytes and shifts.
//   pack_few_lanes_per_row_kernel   the same for rows of 8 to 256 bytes with 4, 8, 16 or 32 lanes per
//                      row: a wavefront packs 16 to 2 rows at once.
//   pack_short_rows_kernel   N < 8: one lane per row, byte loads.
//
// A mask byte counts as "attend" when it is non-zero (torch.bool storage holds 0/1).
//
// The loads are ordinary (temporal) ones.  Non-temporal loads make the packer alone 15 % faster in
// a loop over the same mask, but the sequence pack -> attention, which is what a caller runs,
// 8 % slower (measured on MI355X: 32.5 vs 29.7 us for B=16, H=12, N=512).
#include <stdlib.h>

#include <atomic>

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

// U times eight bytes from any byte addresses, one global_load_dwordx2 each (gfx950 under ROCm
// serves vector loads of any alignment; the compiler itself would split a load it cannot prove
// aligned into bytes).  Issue and wait sit in one statement, so no use can come before the data.
__device__ __forceinline__ void load8_any(u32x2 (&d)[1], const uint8_t *const (&p)[1])
{
    asm volatile("global_load_dwordx2 %0, %1, off\n\t"
                 "s_waitcnt vmcnt(0)"
                 : "=&v"(d[0]) : "v"(p[0]) : "memory");
}
__device__ __forceinline__ void load8_any(u32x2 (&d)[2], const uint8_t *const (&p)[2])
{
    asm volatile("global_load_dwordx2 %0, %2, off\n\t"
                 "global_load_dwordx2 %1, %3, off\n\t"
                 "s_waitcnt vmcnt(0)"
                 : "=&v"(d[0]), "=&v"(d[1]) : "v"(p[0]), "v"(p[1]) : "memory");
}
__device__ __forceinline__ void load8_any(u32x2 (&d)[4], const uint8_t *const (&p)[4])
{
    asm volatile("global_load_dwordx2 %0, %4, off\n\t"
                 "global_load_dwordx2 %1, %5, off\n\t"
                 "global_load_dwordx2 %2, %6, off\n\t"
                 "global_load_dwordx2 %3, %7, off\n\t"
                 "s_waitcnt vmcnt(0)"
                 : "=&v"(d[0]), "=&v"(d[1]), "=&v"(d[2]), "=&v"(d[3])
                 : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3])
                 : "memory");
}

// U: 512-byte segments in flight per wavefront (the host picks 1, 2 or 4 by the row length, so that
// short rows do not issue loads that fetch nothing new)
template <int U>
__global__ __launch_bounds__(PACK_THREADS) void pack_row_kernel(const uint8_t *__restrict__ mask,
                                                                uint32_t *__restrict__ packed,
                                                                long long rows, int N, int nw)   // N >= 8
{
    const int lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * (PACK_THREADS / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;                       // whole wavefront leaves together
    const uint8_t *src = mask + row * (long long)N;
    uint32_t *dst = packed + row * (long long)nw;
    for (int seg0 = 0; seg0 * 512 < N; seg0 += U) {
        u32x2 d[U];
        const uint8_t *p[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int col = (seg0 + u) * 512 + lane * 8;    // first column of this lane's 8 bytes
            // bytes that would lie beyond the row are not touched: the row's last 8 bytes instead
            p[u] = src + (col + 8 <= N ? col : N - 8);
        }
        load8_any(d, p);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int col = (seg0 + u) * 512 + lane * 8;
            uint64_t v = ((uint64_t)d[u].y << 32) | d[u].x;
            if (col + 8 > N) v = col < N ? v >> (8 * (col + 8 - N)) : 0ull;      // the row's last columns, moved down
            uint32_t b = __builtin_amdgcn_udot4(nonzero_bytes((uint32_t)v), 0x08040201u, 0u, false);
            b = __builtin_amdgcn_udot4(nonzero_bytes((uint32_t)(v >> 32)), 0x80402010u, b, false);
            b <<= 8 * (lane & 3);                          // position inside the word of this quad
            b |= __shfl_xor(b, 1, 64);
            b |= __shfl_xor(b, 2, 64);
            const int w = (seg0 + u) * 16 + (lane >> 2);
            if ((lane & 3) == 0 && w < nw) dst[w] = b;
        }
    }
}

// Rows of 8 to 256 bytes: 2^lpr_shift = 4, 8, 16 or 32 lanes per row, so a wavefront packs 16 to 2
// rows at once instead of leaving most of its lanes idle.
__global__ __launch_bounds__(PACK_THREADS) void pack_few_lanes_per_row_kernel(const uint8_t *__restrict__ mask,
                                                                              uint32_t *__restrict__ packed,
                                                                              long long rows, int N, int nw,
                                                                              int lpr_shift)
{
    const int lane = threadIdx.x & 63;
    const long long wave = (long long)blockIdx.x * (PACK_THREADS / 64) + (threadIdx.x >> 6);
    const long long row = (wave << (6 - lpr_shift)) + (lane >> lpr_shift);
    if ((wave << (6 - lpr_shift)) >= rows) return;            // whole wavefront leaves together
    const bool live = row < rows;
    const long long r = live ? row : rows - 1;
    const int l = lane & ((1 << lpr_shift) - 1);
    const int col = l * 8;
    u32x2 d[1];
    const uint8_t *const p[1] = {mask + r * (long long)N + (col + 8 <= N ? col : N - 8)};
    load8_any(d, p);
    uint64_t v = ((uint64_t)d[0].y << 32) | d[0].x;
    if (col + 8 > N) v = col < N ? v >> (8 * (col + 8 - N)) : 0ull;
    uint32_t b = __builtin_amdgcn_udot4(nonzero_bytes((uint32_t)v), 0x08040201u, 0u, false);
    b = __builtin_amdgcn_udot4(nonzero_bytes((uint32_t)(v >> 32)), 0x80402010u, b, false);
    b <<= 8 * (lane & 3);
    b |= __shfl_xor(b, 1, 64);
    b |= __shfl_xor(b, 2, 64);
    if (live && (lane & 3) == 0 && (l >> 2) < nw) packed[r * (long long)nw + (l >> 2)] = b;
}

__global__ __launch_bounds__(PACK_THREADS) void pack_short_rows_kernel(const uint8_t *__restrict__ mask,
                                                                       uint32_t *__restrict__ packed,
                                                                       uint32_t rows, int N)            // N < 8
{
    const uint32_t row = blockIdx.x * (uint32_t)PACK_THREADS + threadIdx.x;
    if (row >= rows) return;
    const uint8_t *src = mask + (size_t)row * N;
    uint32_t acc = 0u;
    for (int j = 0; j < N; ++j) acc |= (uint32_t)(src[j] != 0) << j;
    packed[row] = acc;
}

// Any N, byte loads only, one lane per output word: the packer for a device that does not serve
// 8-byte loads from unaligned addresses (see unaligned_access_state below); several times slower
// than the kernels above and never used where they work.
__global__ __launch_bounds__(PACK_THREADS) void pack_bytewise_kernel(const uint8_t *__restrict__ mask,
                                                                     uint32_t *__restrict__ packed,
                                                                     long long words, int N, int nw)
{
    const long long idx = (long long)blockIdx.x * PACK_THREADS + threadIdx.x;
    if (idx >= words) return;
    const long long row = idx / nw;
    const int w = (int)(idx - row * nw);
    const uint8_t *src = mask + row * N + 32 * w;
    const int n = N - 32 * w < 32 ? N - 32 * w : 32;
    uint32_t acc = 0u;
    for (int j = 0; j < n; ++j) acc |= (uint32_t)(src[j] != 0) << j;
    packed[idx] = acc;
}

// ---- one-time check of the device: are 8- and 16-byte loads from unaligned addresses served? ----
// The row packers above and the forward that reads the boolean mask load 8 bytes (into registers)
// and 16 bytes (into LDS) from whatever address a mask row starts at.  ROCm runs compute queues in
// the memory pipeline's unaligned-access mode, in which that is served; with the mode off the
// hardware drops the low address bits and the results would be silently wrong.  One wavefront
// writes a byte pattern, loads it back both ways from odd addresses and compares.
constexpr int PROBE_BYTES = 1024 + 64;
__device__ __align__(16) unsigned char unaligned_probe_src[PROBE_BYTES];
__device__ int unaligned_probe_verdict;

__device__ __forceinline__ uint32_t probe_byte(uint32_t i) { return (i * 37u + 11u) & 0xffu; }

__global__ __launch_bounds__(64) void unaligned_probe_kernel(unsigned char *src, int *verdict)
{
    __shared__ __attribute__((aligned(16))) unsigned char landing[1024];
    const uint32_t lane = threadIdx.x;
    for (uint32_t i = lane * 17u; i < lane * 17u + 17u; ++i) src[i] = (unsigned char)probe_byte(i);
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "agent");
    __builtin_amdgcn_s_barrier();
    bool ok = true;
    // 8 bytes into registers from an address that is 3 mod 8
    {
        uint64_t v;
        const unsigned char *p = src + 3 + 8 * lane;
        asm volatile("global_load_dwordx2 %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
        for (uint32_t b = 0; b < 8; ++b) ok &= ((v >> (8 * b)) & 0xffu) == probe_byte(3 + 8 * lane + b);
    }
    // 16 bytes into LDS from an address that is 5 mod 16 (lane i's bytes land at 16 * i)
    {
        const uint32_t lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)landing;
        const uint32_t voff = 5u + 16u * lane;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_waitcnt vmcnt(0)"
                     :: "s"(lds), "v"(voff), "s"(src) : "memory", "m0");
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
        __builtin_amdgcn_s_barrier();
        for (uint32_t b = 0; b < 16; ++b) ok &= landing[16 * lane + b] == probe_byte(5 + 16 * lane + b);
    }
    const bool all_ok = __builtin_amdgcn_ballot_w64(!ok) == 0ull;
    if (lane == 0) *verdict = all_ok ? 1 : 2;
}

// Tile map of a packed mask: for every (slab, block of 64 query rows) one bit per 64-key tile that
// says "some mask bit of this 64 x 64 block is set" (word group 0) and one that says "every bit of
// the block is set" (word group 1; only rows and columns below N count).  Layout
// [slab][row block][2][tw], tw = ceil(T / 32) words, T = ceil(N / 64); bits of tiles >= T are zero.
// One work-group per (slab, row block): it streams the block's 64 x nw words (coalesced), every
// thread ORs what its words say into per-key-tile flags in LDS, and the first tw threads write the
// words.  No atomics on global memory, nothing to clear beforehand, deterministic.
constexpr int MAP_MAX_TW = 64;      // key tiles per query tile <= 2048, i.e. N <= 131072
__global__ __launch_bounds__(PACK_THREADS) void tile_map_kernel(const uint32_t *__restrict__ packed,
                                                                uint32_t *__restrict__ map,
                                                                int N, int nw, int qblocks, int tw)
{
    __shared__ uint32_t some[MAP_MAX_TW], hole[MAP_MAX_TW];       // hole: a valid bit of the tile is clear
    const int slab = blockIdx.x / qblocks, qt = blockIdx.x - slab * qblocks;
    if ((int)threadIdx.x < tw) { some[threadIdx.x] = 0u; hole[threadIdx.x] = 0u; }
    __syncthreads();
    const int row0 = qt * 64;
    const int rows = N - row0 < 64 ? N - row0 : 64;
    const uint32_t *src = packed + ((size_t)slab * N + row0) * nw;
    const int words = rows * nw;
    const uint32_t tail = (N & 31) ? ((1u << (N & 31)) - 1u) : 0xffffffffu;     // valid bits of a row's last word
    for (int i = threadIdx.x; i < words; i += PACK_THREADS) {
        const int w = i % nw;
        const uint32_t valid = w == nw - 1 ? tail : 0xffffffffu;
        const uint32_t x = src[i] & valid;
        const int kt = w >> 1;
        const uint32_t bit = 1u << (kt & 31);
        // most blocks are mixed: look before the (serialising) LDS atomic
        if (x != 0u && (some[kt >> 5] & bit) == 0u) atomicOr(&some[kt >> 5], bit);
        if (x != valid && (hole[kt >> 5] & bit) == 0u) atomicOr(&hole[kt >> 5], bit);
    }
    __syncthreads();
    if ((int)threadIdx.x < tw) {
        const int T = (N + 63) / 64;
        const int w = threadIdx.x;
        const uint32_t in_range = (w == tw - 1 && (T & 31)) ? ((1u << (T & 31)) - 1u) : 0xffffffffu;
        uint32_t *dst = map + ((size_t)slab * qblocks + qt) * 2 * tw;
        dst[w] = some[w] & in_range;
        dst[tw + w] = ~hole[w] & in_range;
    }
}

}  // namespace

hipError_t launch_tile_map(const uint32_t *packed, uint32_t *map, long long slabs, int N, hipStream_t stream)
{
    if (slabs == 0 || N == 0) return hipSuccess;
    const int nw = (N + 31) / 32, qblocks = (N + 63) / 64, tw = (qblocks + 31) / 32;
    if (tw > MAP_MAX_TW) return hipErrorInvalidValue;
    hipLaunchKernelGGL(tile_map_kernel, dim3((unsigned)(slabs * qblocks)), dim3(PACK_THREADS), 0, stream, packed, map,
                       N, nw, qblocks, tw);
    return hipGetLastError();
}

int unaligned_access_state(hipStream_t stream)
{
    static std::atomic<int> cached[64];      // 0 = not checked yet, 1 = served, 2 = not served
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -1;
    const int known = cached[dev].load(std::memory_order_acquire);
    if (known != 0) return known == 1 ? 1 : 0;
    // not under graph capture: the check reads its verdict back and waits for it
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return -1;
    }
    int verdict = 0;
    const char *forced = getenv("SMA_ASSUME_NO_UNALIGNED_ACCESS");      // for tests of the fallbacks
    if (forced != nullptr && forced[0] == '1') {
        verdict = 2;
    } else {
        void *src = nullptr, *res = nullptr;
        if (hipGetSymbolAddress(&src, HIP_SYMBOL(unaligned_probe_src)) != hipSuccess ||
            hipGetSymbolAddress(&res, HIP_SYMBOL(unaligned_probe_verdict)) != hipSuccess)
            return -1;
        hipLaunchKernelGGL(unaligned_probe_kernel, dim3(1), dim3(64), 0, stream, static_cast<unsigned char *>(src),
                           static_cast<int *>(res));
        if (hipGetLastError() != hipSuccess) return -1;
        if (hipMemcpyAsync(&verdict, res, sizeof(int), hipMemcpyDeviceToHost, stream) != hipSuccess) return -1;
        if (hipStreamSynchronize(stream) != hipSuccess) return -1;
        if (verdict != 1 && verdict != 2) return -1;
    }
    cached[dev].store(verdict, std::memory_order_release);
    return verdict == 1 ? 1 : 0;
}

hipError_t launch_pack_mask(const uint8_t *mask, uint32_t *packed, long long rows, int N,
                            hipStream_t stream)
{
    if (rows == 0 || N == 0) return hipSuccess;
    const int nw = (N + 31) / 32;
    const bool flat = (N % 32 == 0) && ((reinterpret_cast<uintptr_t>(mask) & 15u) == 0);
    if (!flat && N >= 8 && unaligned_access_state(stream) == 0) {
        const long long words = rows * nw;
        const unsigned grid = (unsigned)((words + PACK_THREADS - 1) / PACK_THREADS);
        hipLaunchKernelGGL(pack_bytewise_kernel, dim3(grid), dim3(PACK_THREADS), 0, stream, mask, packed, words, N, nw);
        return hipGetLastError();
    }
    if (flat) {
        const long long n_chunks = rows * (long long)N / 16;
        const long long per_block = (long long)PACK_THREADS * PACK_UNROLL;
        const unsigned grid = (unsigned)((n_chunks + per_block - 1) / per_block);
        hipLaunchKernelGGL(pack_flat_kernel, dim3(grid), dim3(PACK_THREADS), 0, stream,
                           reinterpret_cast<const u32x4 *>(mask), packed, n_chunks);
    } else if (N >= 8 && N <= 256) {
        int lpr_shift = 2;                                     // lanes per row: 8 bytes each, at least a quad
        while ((8 << lpr_shift) < N) ++lpr_shift;
        const long long waves = (rows + (64 >> lpr_shift) - 1) >> (6 - lpr_shift);
        const unsigned grid = (unsigned)((waves + PACK_THREADS / 64 - 1) / (PACK_THREADS / 64));
        hipLaunchKernelGGL(pack_few_lanes_per_row_kernel, dim3(grid), dim3(PACK_THREADS), 0, stream, mask, packed,
                           rows, N, nw, lpr_shift);
    } else if (N >= 8) {
        const unsigned grid = (unsigned)((rows + PACK_THREADS / 64 - 1) / (PACK_THREADS / 64));
        const int segments = (N + 511) / 512;
        auto kernel = segments >= 4 ? pack_row_kernel<4> : segments >= 2 ? pack_row_kernel<2> : pack_row_kernel<1>;
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(PACK_THREADS), 0, stream, mask, packed, rows, N, nw);
    } else {
        const unsigned grid = (unsigned)((rows + PACK_THREADS - 1) / PACK_THREADS);
        hipLaunchKernelGGL(pack_short_rows_kernel, dim3(grid), dim3(PACK_THREADS), 0, stream, mask, packed,
                           (uint32_t)rows, N);
    }
    return hipGetLastError();
}

}  // namespace sma
