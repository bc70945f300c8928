// Yardstick for the MFMA roofline: what one MI355X sustains on a pure stream of the MFMA the
// attention kernels are made of (v_mfma_f32_32x32x16_f16), with operands that are all zero or
// random fp16 numbers, and the shader clock it gets while doing so.  The dense FP16 peak of the
// data sheet (256 CUs x 4096 FLOP/clk x 2.4 GHz) assumes the top clock; the part lowers its clock
// under a stream of MFMAs on real data, and this probe measures by how much on the GPU at hand.
// No counterpart in the reference.  Benchmark infrastructure: built into libsma_probe.so, which only
// bench.py and one test load; libsma_hip.so, the product, does not contain it.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mfma_probe.h"

namespace sma {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t mix(uint32_t x)
{
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}
// two fp16 numbers of magnitude 0.5 .. 2 with random signs and mantissas
__device__ __forceinline__ uint32_t random_pair(uint32_t seed)
{
    const uint32_t h = mix(seed);
    const uint32_t lo = 0x3800u | (h & 0x87ffu) | ((h >> 3) & 0x0400u);
    const uint32_t hi = 0x3800u | ((h >> 16) & 0x87ffu) | ((h >> 19) & 0x0400u);
    return lo | (hi << 16);
}

// Every wavefront issues 8 * iters MFMAs (two accumulator chains of four, restarted from zero each
// round so that nothing overflows).  Thread 0 of each work-group leaves the shader-clock ticks
// (s_memtime) and the 100 MHz ticks (s_memrealtime) that the loop took.
__global__ __launch_bounds__(768) void mfma_stream_kernel(int random_operands, int iters, long long *stamps, float *sink)
{
    const uint32_t t = threadIdx.x;
    u32x4 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a[i][j] = random_operands ? random_pair(t * 64 + i * 4 + j + blockIdx.x * 977) : 0u;
            b[i][j] = random_operands ? random_pair(t * 64 + 32 + i * 4 + j + blockIdx.x * 131) : 0u;
        }
    f32x16 acc0 = {0}, acc1 = {0};
    const long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
        const f32x16 zero = {0};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[i]), __builtin_bit_cast(f16x8, b[i]),
                                                          i == 0 ? zero : acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[(i + 1) & 3]),
                                                          __builtin_bit_cast(f16x8, b[i]), i == 0 ? zero : acc1, 0, 0, 0);
        }
        asm volatile("" : "+v"(acc0), "+v"(acc1));
    }
    const long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
    if (t == 0) {
        stamps[2 * blockIdx.x] = c1 - c0;
        stamps[2 * blockIdx.x + 1] = r1 - r0;
    }
    if (iters < 0) sink[t] = acc0[0] + acc1[0];       // never taken: keeps the chains alive
}

}  // namespace
}  // namespace sma

extern "C" int sma_probe_mfma_stream(int random_operands, int iters, int work_groups, long long *stamps, void *stream)
{
    // a wavefront's loop is iters * 8 MFMAs of 32 cycles: the cap keeps a mistyped count from
    // turning into a kernel that runs for minutes
    if (iters < 0 || iters > SMA_PROBE_MAX_ITERS || work_groups < 0 || work_groups > 65536) return SMA_PROBE_ERR_RANGE;
    if (work_groups == 0) return SMA_PROBE_OK;
    if (stamps == nullptr) return SMA_PROBE_ERR_NULL;
    // the kernel's last argument is a sink that is never written (see the kernel); any device address does
    hipLaunchKernelGGL(sma::mfma_stream_kernel, dim3((unsigned)work_groups), dim3(768), 0, static_cast<hipStream_t>(stream),
                       random_operands, iters, stamps, reinterpret_cast<float *>(stamps));
    return hipGetLastError() == hipSuccess ? SMA_PROBE_OK : SMA_PROBE_ERR_LAUNCH;
}
