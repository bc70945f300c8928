/* sma.h - C ABI of libsma_hip.so: sparse-mask attention for AMD MI355X (gfx950).
 *
 * Plain C, plain pointers and sizes.  Every pointer is a DEVICE pointer in the address space of
 * the GPU that is current on the calling thread; `stream` is a hipStream_t passed as void*
 * (NULL = the default stream).  Tensors are dense row-major ("contiguous") except in the *_strided
 * entry points, which take explicit strides.  Launches are asynchronous on `stream`; the functions
 * never synchronise and never allocate.  The only state the library keeps is per device and is set
 * on first use: the address of the fixed workspace of sma_attn_bwd_static_ws, and the verdict of a
 * one-time check that the device serves copies from unaligned addresses (see sma_attn_fwd_bool_mask).
 * Return value: SMA_OK (0) or a negative SMA_ERR_* code; sma_strerror() names it.
 *
 * Each entry point cites the interface of the reference implementation that it stands in for
 * (paths relative to the reference tree).
 */
#ifndef SMA_H_
#define SMA_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SMA_OK                 0
#define SMA_ERR_NULL_POINTER  -1   /* a required pointer is NULL */
#define SMA_ERR_BAD_SHAPE     -2   /* a negative extent, or an extent beyond the 32-bit index range */
#define SMA_ERR_HEAD_DIM      -3   /* head_dim other than 32, 64 or 128 */
#define SMA_ERR_DTYPE         -4   /* dtype other than SMA_DTYPE_F16 / SMA_DTYPE_BF16 */
#define SMA_ERR_SCALE         -5   /* scale is NaN or infinite */
#define SMA_ERR_LAUNCH        -6   /* the HIP runtime refused the launch (hipGetLastError) */
#define SMA_ERR_ALIGNMENT     -7   /* q/k/v/out not 16-byte aligned, or mask_packed/lse not 4-byte aligned */
#define SMA_ERR_STRIDE        -8   /* a stride is negative, not a multiple of 8 elements, or too large */
#define SMA_ERR_WORKSPACE     -9   /* B*H*N exceeds SMA_STATIC_WS_ROWS (sma_attn_bwd_static_ws only) */
#define SMA_ERR_DEVICE       -10   /* the device does not serve loads from unaligned addresses (sma_device_check) */

#define SMA_DTYPE_F16   0
#define SMA_DTYPE_BF16  1

/* Library version, major*10000 + minor*100 + patch. */
int sma_version(void);

/* Static, never-NULL description of a return code. */
const char *sma_strerror(int code);

/* One-time check of the current device: are 8- and 16-byte loads from unaligned addresses served?
 *
 * The packers for rows that do not start 16-byte aligned and sma_attn_fwd_bool_mask read mask rows
 * at whatever byte address they start.  ROCm runs compute queues in the unaligned-access mode of the
 * memory pipeline, in which such loads are served; on a device where they are not, the results
 * would be wrong without any fault.  The library therefore checks once per device, in the first
 * call that depends on it (or in this one): a one-wavefront kernel on `stream`, whose verdict the
 * call waits for - the one place where the library synchronises.  It cannot run while `stream` is
 * being captured into a graph (the dependent calls then proceed unchecked): make the first call on
 * a device outside capture.  Returns SMA_OK, or SMA_ERR_DEVICE when such loads are not served;
 * sma_pack_mask then packs with byte loads (slower, same words) and sma_attn_fwd_bool_mask
 * returns SMA_ERR_DEVICE (use sma_pack_mask + sma_attn_fwd).
 *
 * No counterpart in the reference.
 */
int sma_device_check(void *stream);

/* Bit-pack a boolean attend-mask.
 *
 *   mask    uint8 [B,H,N,N], one byte per entry, non-zero = attend (torch.bool storage)
 *   packed  uint32 [B,H,N,ceil(N/32)]; bit j of word w of row i is column 32*w+j of that row;
 *           bits that stand for columns >= N are written as 0.  Every word is written, so the
 *           output needs no pre-clearing.
 *
 * Replaces: void pack_mask_bits(const bool*, uint32_t*, int B, int H, int N, cudaStream_t)
 *           csrc/sparse_attention.h:67-72, defined csrc/sparse_attention.cu:603-610
 *           (kernel pack_mask_kernel, csrc/sparse_attention.cu:549-568).
 */
int sma_pack_mask(const uint8_t *mask, uint32_t *packed, int B, int H, int N, void *stream);

/* Tile map of a packed mask: which 64-key tiles matter to which block of 64 query rows.
 *
 *   tile_map  uint32 [B,H,T,2,TW], T = ceil(N/64) blocks of 64 query rows (and as many key tiles of
 *             64 keys), TW = ceil(T/32) words: for row block r, word group 0 holds one bit per key
 *             tile t (bit t%32 of word t/32) that is set when some mask bit of the 64 x 64 block
 *             (r, t) is set; word group 1 one bit that is set when every bit of the block is set
 *             (rows and columns below N).  sma_tile_map_words(N) = T*2*TW words per (batch entry,
 *             head).  Every word is written.
 *
 * sma_attn_fwd_map visits only the key tiles whose first bit is set: for the others nothing is
 * copied and nothing computed, which is what a block-structured mask (sliding window, block-sparse,
 * causal) needs; the reference's own skip (csrc/sparse_attention.cu:238-252) still loads the tile
 * (:211) and is taken per 64 query rows.  A map costs one pass over the packed words; make it once
 * for a mask that is used many times.  N <= 131072 (sma_tile_map, sma_pack_mask_map with a map and
 * every entry point that takes a map return SMA_ERR_BAD_SHAPE beyond it, before anything is written).
 *
 * Word group 1 ("every bit set") is written for callers; the kernels of this library read word
 * group 0 only.
 *
 * sma_pack_mask_map = sma_pack_mask followed by sma_tile_map on its output (tile_map may be NULL:
 * then it is sma_pack_mask).
 *
 * No counterpart in the reference beyond the block skip cited above.
 */
long long sma_tile_map_words(int N);
int sma_tile_map(const uint32_t *mask_packed, uint32_t *tile_map, int B, int H, int N, void *stream);
int sma_pack_mask_map(const uint8_t *mask, uint32_t *packed, uint32_t *tile_map, int B, int H, int N,
                      void *stream);

/* Fused masked attention forward:  out = softmax_row(mask ? (q k^T) * scale : -inf) v.
 *
 *   q, k, v      [B,H,N,D] fp16 or bf16 (dtype), D = 64 (the reference's only head dim), 32 or 128
 *   mask_packed  uint32 [B,H,N,ceil(N/32)] in the sma_pack_mask format (pad bits are ignored)
 *   out          [B,H,N,D], same dtype; every element is written
 *   lse          NULL, or float [B,H,N]: natural-log-sum-exp of the kept scaled scores of each
 *                query row, -inf for a row that keeps no key
 *   scale        any finite float (the reference passes 1/sqrt(D))
 *
 * A query row whose mask keeps no key yields zeros.  Accumulation is fp32.
 *
 * Replaces: void sparse_attention_fwd_fp16(const SparseAttentionParams&, cudaStream_t) and
 *           void sparse_attention_fwd_bf16(const SparseAttentionParams&, cudaStream_t),
 *           csrc/sparse_attention.h:45-54, defined csrc/sparse_attention.cu:574-601; the
 *           arguments are the live fields of SparseAttentionParams, csrc/sparse_attention.h:12-38
 *           (lse == NULL plays the part of is_training == false, csrc/binding.cpp:30).
 */
int sma_attn_fwd(const void *q, const void *k, const void *v, const uint32_t *mask_packed,
                 void *out, float *lse, int B, int H, int N, int D, float scale, int dtype,
                 void *stream);

/* sma_attn_fwd with a tile map (see sma_tile_map) of the same packed mask; tile_map == NULL is
 * sma_attn_fwd.  The results are those of sma_attn_fwd bit for bit; only the tiles visited differ.
 * A map that does not belong to the mask gives wrong results (tiles it calls empty are not read).
 */
int sma_attn_fwd_map(const void *q, const void *k, const void *v, const uint32_t *mask_packed,
                     const uint32_t *tile_map, void *out, float *lse, int B, int H, int N, int D,
                     float scale, int dtype, void *stream);

/* Masked attention backward:  given dout = dLoss/dout, the gradients with respect to q, k and v.
 *
 *   dout, q, k, v, out  [B,H,N,D] fp16 or bf16 (dtype), D = 32, 64 or 128; out and lse are the results
 *                       of sma_attn_fwd on the same q, k, v, mask_packed and scale
 *   lse                 float [B,H,N] as written by sma_attn_fwd (-inf for rows that keep no key)
 *   mask_packed         uint32 [B,H,N,ceil(N/32)]
 *   dq, dk, dv          [B,H,N,D], same dtype; every element is written (rows that keep no key
 *                       get dq = 0; keys that no row keeps get dk = dv = 0)
 *   delta_ws            float [B,H,N] workspace owned by the caller; holds sum_d dout*out per query
 *                       row on return (the library never allocates)
 *
 * Two launches on `stream` (dq, then dk and dv; three for D = 128: dq, dk, dv); no atomics, results are
 * bit-reproducible.
 *
 * Replaces: void sparse_attention_bwd_bf16(const SparseAttentionParams&, const void* dout,
 *           void* dq, void* dk, void* dv, cudaStream_t), declared csrc/sparse_attention.h:57-64 and
 *           never defined; its caller is python/sparse_attention.py:91-94 and the mathematics is
 *           the PyTorch fallback at python/sparse_attention.py:97-111.
 */
int sma_attn_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out,
                 const float *lse, const uint32_t *mask_packed, void *dq, void *dk, void *dv,
                 float *delta_ws, int B, int H, int N, int D, float scale, int dtype, void *stream);

/* sma_attn_bwd with a tile map (see sma_tile_map) of the same packed mask: both kernels visit only
 * the 64 x 64 blocks in which the mask keeps something.  tile_map == NULL is sma_attn_bwd; the
 * gradients are the same bit for bit.  sma_attn_bwd_map_strided is the strided form (map
 * contiguous [Bm,Hm,T,2,TW] with the mask's own Bm, Hm).
 */
int sma_attn_bwd_map(const void *dout, const void *q, const void *k, const void *v, const void *out,
                     const float *lse, const uint32_t *mask_packed, const uint32_t *tile_map, void *dq,
                     void *dk, void *dv, float *delta_ws, int B, int H, int N, int D, float scale, int dtype,
                     void *stream);


/* sma_attn_bwd without the workspace argument, for callers that cannot allocate device memory at
 * all (code running under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): the per-row sums that the two kernels exchange live in a fixed array inside the
 * library's device image (SMA_STATIC_WS_ROWS floats = 4 MiB, held by every GPU the library has
 * been called on until the process ends).  Arguments and results are exactly those of
 * sma_attn_bwd.  The call allocates nothing; B*H*N > SMA_STATIC_WS_ROWS returns SMA_ERR_WORKSPACE
 * and launches nothing.  All calls on one GPU share the array: calls that may overlap in time (on
 * different streams of the same GPU) race and must use sma_attn_bwd with workspaces of their own.
 * The first call on a device looks the array's address up (hipGetSymbolAddress); make that call
 * outside graph capture.
 *
 * No counterpart in the reference: this entry point exists only for callers that cannot allocate.
 */
#define SMA_STATIC_WS_ROWS (1 << 20)
int sma_attn_bwd_static_ws(const void *dout, const void *q, const void *k, const void *v, const void *out,
                           const float *lse, const uint32_t *mask_packed, void *dq, void *dk, void *dv,
                           int B, int H, int N, int D, float scale, int dtype, void *stream);

/* A [B,H,N,D] tensor of 16-bit elements with explicit strides, in ELEMENTS.  The D elements of a
 * row are contiguous (stride 1, not stored).  Every stride must be >= 0 and a multiple of 8 (rows
 * stay 16-byte aligned); stride_n < 2^23, (N-1)*stride_n*2 + 2*D < 2^31 (bytes inside one (b,h)
 * slab) and stride_b, stride_h < 2^35.  A stride of 0 on
 * an input repeats the same data; the rows of an output must not overlap (an output with a row
 * stride below D, or with a zero stride over an extent above 1, is refused with SMA_ERR_STRIDE).
 *
 * Replaces: the twelve stride fields of SparseAttentionParams (stride_qb .. stride_on,
 *           csrc/sparse_attention.h:30-33), which the reference declares and never reads.
 */
typedef struct sma_tensor {
    void *data;                 /* element (0,0,0,0) */
    int64_t stride_b, stride_h, stride_n;
} sma_tensor;

/* sma_attn_fwd for strided q, k, v, out and for a mask shared between batch entries and/or heads.
 *
 *   mask_packed     uint32 [Bm,Hm,N,ceil(N/32)] with Bm in {1,B} and Hm in {1,H}; its rows are
 *                   contiguous; mask_stride_b / mask_stride_h are in 32-bit WORDS, >= 0, and 0 means
 *                   that every batch entry / head reads the same mask (a [1,1,N,N] or [B,1,N,N]
 *                   attend-mask is then packed once, not B*H times)
 *   lse             NULL or float [B,H,N], contiguous
 *
 * Everything else is as for sma_attn_fwd, which is this function with contiguous strides.
 */
int sma_attn_fwd_strided(const sma_tensor *q, const sma_tensor *k, const sma_tensor *v,
                         const uint32_t *mask_packed, int64_t mask_stride_b, int64_t mask_stride_h,
                         const sma_tensor *out, float *lse, int B, int H, int N, int D, float scale,
                         int dtype, void *stream);

/* sma_attn_fwd_strided with a tile map: contiguous [Bm,Hm,T,2,TW] with the mask's own Bm, Hm (1
 * where the mask stride is 0), or NULL.
 */
int sma_attn_fwd_map_strided(const sma_tensor *q, const sma_tensor *k, const sma_tensor *v,
                             const uint32_t *mask_packed, int64_t mask_stride_b, int64_t mask_stride_h,
                             const uint32_t *tile_map, const sma_tensor *out, float *lse, int B, int H,
                             int N, int D, float scale, int dtype, void *stream);

/* sma_pack_mask and sma_attn_fwd in one launch, for a mask that is used once: the kernel reads the
 * boolean bytes themselves and forms the packed words of each 64-key tile on the fly, so the packing
 * pass, its launch and the round trip of the words through memory disappear.
 *
 *   q, k, v, out    contiguous [B,H,N,D] (sma_attn_fwd_bool_mask_strided takes strided ones), D = 32, 64
 *                   or 128; 16 <= N <= 46340
 *   mask            uint8 [Bm,Hm,N,N] with Bm in {1,B}, Hm in {1,H}, rows contiguous, at any byte
 *                   address; a byte counts as "attend" when it is non-zero, as in sma_pack_mask;
 *                   mask_stride_b / mask_stride_h in BYTES, 0 = shared between batch entries /
 *                   heads.  No byte outside the mask is read.
 *   lse             NULL or float [B,H,N]
 *   packed_out      NULL, or uint32 [Bm,Hm,N,ceil(N/32)] (contiguous): receives exactly what
 *                   sma_pack_mask would write for this mask, as a by-product, for callers who
 *                   need the packed words afterwards (sma_attn_bwd)
 *
 * Anything outside these limits returns an error code and is served by sma_pack_mask followed by
 * sma_attn_fwd (or its strided form), which give the same results.
 *
 * Replaces: the pair of launches the reference's forward makes for every call,
 *           python/sparse_attention.py:146 + :171 (pack_mask, then forward), run.py:151-154.
 */
int sma_attn_fwd_bool_mask(const void *q, const void *k, const void *v, const uint8_t *mask,
                           int64_t mask_stride_b, int64_t mask_stride_h, void *out, float *lse,
                           uint32_t *packed_out, int B, int H, int N, int D, float scale, int dtype,
                           void *stream);

/* sma_attn_fwd_bool_mask that also leaves the mask's tile map behind.
 *
 *   map_out         NULL, or uint32 [Bm,Hm,T,2,TW] (contiguous; sma_tile_map_words(N) words per
 *                   (batch entry, head) of the mask): receives exactly what sma_tile_map would
 *                   write for packed_out, as a by-product of the same launch, for callers who go
 *                   on to sma_attn_bwd_map (or to sma_attn_fwd_map with the same mask)
 *
 * Everything else as in sma_attn_fwd_bool_mask, which is this call with map_out = NULL.
 *
 * Replaces: as sma_attn_fwd_bool_mask; the map itself has no counterpart in the reference (its
 *           kernel tests each 16 x 64 block after loading it, csrc/sparse_attention.cu:238-252).
 */
int sma_attn_fwd_bool_mask_map(const void *q, const void *k, const void *v, const uint8_t *mask,
                               int64_t mask_stride_b, int64_t mask_stride_h, void *out, float *lse,
                               uint32_t *packed_out, uint32_t *map_out, int B, int H, int N, int D,
                               float scale, int dtype, void *stream);

/* sma_attn_fwd_bool_mask_map for strided q, k, v, out (see sma_attn_fwd_strided for what a layout
 * may be): a [B,N,H,D] buffer viewed as [B,H,N,D] or the slices of a fused qkv projection go through
 * the one launch as they are.  The mask, lse, packed_out and map_out are as in
 * sma_attn_fwd_bool_mask_map, which is this function with contiguous strides.
 *
 * Replaces: as sma_attn_fwd_bool_mask; the strides are those of SparseAttentionParams
 *           (csrc/sparse_attention.h:30-33), which the reference declares and never reads.
 */
int sma_attn_fwd_bool_mask_strided(const sma_tensor *q, const sma_tensor *k, const sma_tensor *v,
                                   const uint8_t *mask, int64_t mask_stride_b, int64_t mask_stride_h,
                                   const sma_tensor *out, float *lse, uint32_t *packed_out, uint32_t *map_out,
                                   int B, int H, int N, int D, float scale, int dtype, void *stream);

/* sma_attn_bwd for strided dout, q, k, v, out, dq, dk, dv and a shared mask (see
 * sma_attn_fwd_strided); lse and delta_ws are contiguous float [B,H,N].
 */
int sma_attn_bwd_strided(const sma_tensor *dout, const sma_tensor *q, const sma_tensor *k,
                         const sma_tensor *v, const sma_tensor *out, const float *lse,
                         const uint32_t *mask_packed, int64_t mask_stride_b, int64_t mask_stride_h,
                         const sma_tensor *dq, const sma_tensor *dk, const sma_tensor *dv,
                         float *delta_ws, int B, int H, int N, int D, float scale, int dtype,
                         void *stream);

/* sma_attn_bwd_map for strided tensors and a shared mask (see sma_attn_bwd_map). */
int sma_attn_bwd_map_strided(const sma_tensor *dout, const sma_tensor *q, const sma_tensor *k,
                             const sma_tensor *v, const sma_tensor *out, const float *lse,
                             const uint32_t *mask_packed, int64_t mask_stride_b, int64_t mask_stride_h,
                             const uint32_t *tile_map, const sma_tensor *dq, const sma_tensor *dk,
                             const sma_tensor *dv, float *delta_ws, int B, int H, int N, int D, float scale,
                             int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SMA_H_ */
