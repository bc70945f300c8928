/* mfma_probe.h - C ABI of libsma_probe.so, a yardstick for the MFMA roofline used by bench.py.
 *
 * Not part of the attention path and not part of libsma_hip.so: a diagnostic that measures what one
 * GPU sustains on a pure stream of the MFMA the attention kernels are made of.  No counterpart in
 * the reference.
 */
#ifndef SMA_MFMA_PROBE_H_
#define SMA_MFMA_PROBE_H_

#ifdef __cplusplus
extern "C" {
#endif

#define SMA_PROBE_OK           0
#define SMA_PROBE_ERR_NULL    -1   /* stamps is NULL */
#define SMA_PROBE_ERR_RANGE   -2   /* iters or work_groups negative or above the caps below */
#define SMA_PROBE_ERR_LAUNCH  -6   /* the HIP runtime refused the launch */

#define SMA_PROBE_MAX_ITERS (1 << 22)

/* Launches `work_groups` (<= 65536) work-groups of 12 wavefronts that each issue 8 * iters MFMAs
 * (v_mfma_f32_32x32x16_f16; iters <= SMA_PROBE_MAX_ITERS) on operands that are all zero
 * (random_operands == 0) or random fp16 numbers.  Thread 0 of work-group g leaves in stamps[2g] the
 * shader-clock ticks and in stamps[2g+1] the 100 MHz ticks that its loop took (stamps: device
 * memory, 2 * work_groups int64).  Time the launch to get the sustained MFMA rate; the quotient of
 * the two stamps is the shader clock in units of 100 MHz.  Asynchronous on `stream` (a hipStream_t,
 * NULL = the default stream).
 */
int sma_probe_mfma_stream(int random_operands, int iters, int work_groups, long long *stamps, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SMA_MFMA_PROBE_H_ */
