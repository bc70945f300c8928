// Fused masked-attention forward for gfx950 (MI355X), head_dim 32, 64 or 128, fp16 / bf16, fp32 accumulate.
//
// Stands in for sparse_attn_wmma_full_fp16 (csrc/sparse_attention.cu:82-412 of the reference) and
// for its scalar bf16 kernel (csrc/sparse_attention.cu:418-543); the design below is specific to
// CDNA4 and shares nothing with either beyond the function computed.
//
// Work decomposition
//   work-group  = 4 wavefronts = 128 query rows of one (b,h); it walks the keys in tiles of 64.
//                 Three work-groups fit a CU (<= 168 VGPRs, ~34 KB LDS each): one wavefront of
//                 each per SIMD, so that the softmax VALU work of one overlaps the MFMAs of another.
//   wavefront   = 32 query rows.  It computes S^T = K_tile (64x64) * Q^T (64x32) with
//                 v_mfma_f32_32x32x16, so every lane owns ONE query row (lane % 32) and 32 of the
//                 tile's 64 keys: the online softmax is a per-lane register loop plus a single
//                 exchange between lane l and lane l+32 (v_permlane32_swap).  P^T is already in
//                 the B-operand layout of O^T += V^T * P^T: probabilities never leave registers.
//   K/V tiles   = copied global -> LDS by global_load_lds_dwordx4 (no VGPR staging) into a ring of
//                 two stages, one tile ahead of the one being computed.  Rows are 128 B; the
//                 16-byte chunks of a row are XOR-swizzled (the permutation is applied to the
//                 global address of each lane; the LDS side of such a load is always linear) so
//                 that K's ds_read_b128 (32 consecutive rows, same column) and V's
//                 ds_read_b64_tr_b16 (transposing read, 8 consecutive rows x 64 B) are free of
//                 bank conflicts on the 64-bank LDS.
//   mask        = each wavefront copies the two packed words per query row of a tile into LDS with
//                 one global_load_lds_dword, one tile ahead.  A lane reads the two words of its
//                 row; each nibble selects one of 16 rows of a small LDS table of four floats that
//                 are 0 (keep) or -inf (drop); one ds_read_b128 of that row initialises four
//                 accumulator registers of the QK^T MFMA chain.  Masking costs no VALU work per score.
//   exponent    = q is multiplied by scale*log2(e) when it is loaded, and the reference point of
//                 the softmax (a per-row value r, see below) is subtracted INSIDE the MFMA chain by
//                 one extra MFMA whose B operand holds -r split into four 16-bit terms and whose
//                 A operand is all ones.  The accumulator then holds log2 of the unnormalised
//                 probability: the per-score VALU work is exp2, pack, row-sum and row-max only.
//   reference r = the online softmax does not track the running maximum.  r moves (and O, l are
//                 rescaled) only when a row's scores leave the window [r-8, r+8] upwards, or when its
//                 first kept score lies below the window.  The row maximum of a tile is not even
//                 computed unless a row meets its first kept key there or the sum of the tile's
//                 weights shows, afterwards, that a score has run away (then they are redone).
//   skipping    = with a tile map (one "some bit set" bit per 64 x 64 block of the mask, made by
//                 the packer) the work-group visits only the key tiles that hold a set bit for its
//                 rows: no copies, no barrier for the others.  Without a map every tile is
//                 copied.  Either way a wavefront whose own 32 x 64 block of mask bits is empty
//                 skips its GEMMs and its softmax for that tile.
//   head dim    = the description above is for 64.  128 runs the same code on two column halves of
//                 64 (see Cfg below): twice the MFMAs per tile for the same softmax work, a ring of
//                 two stages and two work-groups per CU.  32 uses half of every tile row.
#include <atomic>
#include <type_traits>

#include "attn_common.h"

namespace sma {
namespace {

constexpr int HD = 64;             // columns of one LDS tile: the head dim, or one half of a head dim of 128
constexpr int BM = 128;            // query rows per work-group
constexpr int BN = 64;             // keys per tile
constexpr int NTHREADS = 256;
constexpr int TILE_BYTES = BN * HD * 2;          // 8 KiB, rows of 128 B
constexpr float WINDOW_LOG2 = 8.0f;
constexpr float SUM_LIMIT = 16384.0f;     // a lane's 32 weights of a tile sum to more: some score is far above the window

// Head dims (HDIM) other than 64 reuse the 64-column LDS tile with its 128-byte rows, swizzles and
// read patterns:
//   128  two column halves (NH = 2): K and V tiles are kept in LDS as two 64-column tiles each, the
//        QK^T chain runs over both halves of K and q, and P multiplies each half of V into its own
//        pair of accumulators.  A stage is twice as large (32 KiB) and the kernel needs about 224
//        registers, so two work-groups share a CU.
//   32   half a tile: the copies fill the upper half of every LDS row with a second copy of the
//        lower half (global chunk index & 3), which is never read; the QK^T chain has two steps
//        instead of four and P multiplies one 32-column block of V.
//
// BYTEMASK: the mask arrives as the caller's boolean bytes (one per score, 0 or 1) instead of packed
// words.  Each wavefront copies the 32 x 64 bytes of a tile for its rows into LDS and turns them
// into the two words per row itself (eight dot products with the weights 1, 2, 4 .. 128 per lane
// and one exchange between the lane halves): the separate packing pass, its launch and the
// round trip of the words through memory disappear for a mask that is used once.
template <int NH, bool BYTEMASK> struct Cfg {
    static constexpr int NSTAGE = 2;                                // ring of two stages: copies run one tile ahead
    static constexpr int MASK_COPIES = BYTEMASK ? 2 : 1;
    static constexpr int COPIES = MASK_COPIES + 4 * NH;             // async copies per wave and tile
    // LDS map (bytes)
    static constexpr int STAGE_BYTES = 2 * NH * TILE_BYTES;         // K halves, then V halves
    static constexpr int OFF_V = NH * TILE_BYTES;                   // V inside a stage
    // mask: packed words in NSTAGE slots of 4 waves x 64 words; bytes in slots of 4 waves x 2 KiB,
    // two of them for head dims up to 64 and, for want of LDS, ONE for 128: a wave has turned its
    // bytes into words before it requests the next tile's (see the main loop), so one slot is
    // enough, at the price of waiting for those reads before the requests (3 % on the headline
    // workload, which is why two are used where they fit)
    static constexpr int OFF_MASK = NSTAGE * STAGE_BYTES;
    static constexpr int BYTE_SLOTS = NH == 1 ? 2 : 1;
    static constexpr int MASK_SLOT = BYTEMASK ? (BYTE_SLOTS - 1) * 8192 : 1024;     // distance between the slots
    static constexpr int OFF_LUT = OFF_MASK + (BYTEMASK ? BYTE_SLOTS * 8192 : NSTAGE * 1024);   // 16 x 16 B
    // byte mask only: the tile-map bits the wavefronts collect, [4 waves][MAP_WORDS][some, hole],
    // and one arrival counter per pair of wavefronts (block of 64 rows)
    static constexpr int MAP_WORDS = 32;                            // 32 x 32 key tiles: N <= 65536
    static constexpr int OFF_MAP = OFF_LUT + 256;
    static constexpr int OFF_MAP_ARRIVED = OFF_MAP + 4 * MAP_WORDS * 8;
    static constexpr int LDS_BYTES = BYTEMASK ? OFF_MAP_ARRIVED + 16 : OFF_MAP;
};

template <int N> __device__ __forceinline__ void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }

// PACKED_ROWS: the rows of q, k, v and out follow each other without gaps (row stride 64), as in
// contiguous tensors; the strides between heads and batch entries stay free.  A row stride known
// at compile time measured 0.25 us less fixed cost per launch than the same value read at run time.
// BYPRODUCTS (with BYTEMASK): the caller wants the packed words and / or the tile map of the mask
// left behind; a separate instantiation, so that the kernel of a caller who wants neither carries
// none of that code (it measured 1.5 % on the headline workload even when switched off at run time).
// PAIRS (with BYTEMASK, head dims up to 64, N a multiple of 128): the mask bytes of
// TWO key tiles are requested at once, every second visit: 128 bytes per row, i.e. whole cache lines
// where one tile's 64 bytes are half of one.  The forward from the boolean mask measured 1 to 5 %
// faster this way on random masks of every length tried (128 to 2048) and 7 % on the
// block-structured workload -- except where the whole grid is one round of work-groups that run in
// step (the even-progress case of the launcher, e.g. the headline shape): there the first visit,
// which waits for twice the bytes, is not hidden behind other work-groups' work, it measured 1 to 4 %
// slower, and the launcher leaves it off.
template <bool BF16, bool POSTMUL, bool PACKED_ROWS, int HDIM, bool BYTEMASK = false, bool BYPRODUCTS = false,
          bool PAIRS = false>
__global__ __launch_bounds__(NTHREADS, HDIM == 128 ? 2 : 3) void attn_fwd_kernel(const AttnArgs a)
{
    static_assert(!PAIRS || (BYTEMASK && HDIM <= 64), "PAIRS: byte mask, two byte slots");
    using E = Elem<BF16>;
    constexpr int NH = HDIM == 128 ? 2 : 1;       // 64-column tiles per matrix
    constexpr int KS = HDIM / 16;                 // MFMA steps of the QK^T chain
    constexpr int OB = HDIM / 32;                 // 32-column accumulator blocks of O
    constexpr int CHM = HDIM == 32 ? 3 : 7;       // 16-byte chunks per global row, minus one
    using C = Cfg<NH, BYTEMASK>;
    constexpr int NSTAGE = C::NSTAGE, STAGE_BYTES = C::STAGE_BYTES, OFF_MASK = C::OFF_MASK, OFF_LUT = C::OFF_LUT;
    constexpr int MASK_SLOT = C::MASK_SLOT;
    constexpr int D = HDIM;
    __shared__ __attribute__((aligned(1024))) unsigned char smem[C::LDS_BYTES];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(LDS_PTR(unsigned char))smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, hh = lane >> 5;

    const int nid = renumber_block();
    const int bh = (int)fastdiv((uint32_t)nid, a.div_qtiles);
    const int qt = nid - bh * a.qtiles;
    const int N = a.N, nw = (N + 31) >> 5;
    const int T = (N + BN - 1) / BN;
    const bool ragged = (N & (BN - 1)) != 0;
    const float pm = POSTMUL ? a.post_mul : 1.0f;

    const int bi = (int)fastdiv((uint32_t)bh, a.div_H), hi = bh - bi * a.H;
    // ---- tile map: which key tiles hold a set mask bit for this work-group's rows ("live"; the map
    // also says which hold nothing else, which this kernel does not use).  The map has one row of
    // bits (one per key tile, 32 per word) for every block of 64 query rows: this work-group ORs
    // the rows of its two blocks.  The first words are requested here with scalar loads and awaited
    // just before the first copies are issued; the address arithmetic in between covers the latency.
    const int TW = (T + 31) >> 5;
    const uint32_t *mapw = nullptr, *mapw2 = nullptr;       // the two 64-row blocks (the same one if the second does not exist)
    if constexpr (!BYTEMASK) {
        if (a.tile_map != nullptr) {
            mapw = a.tile_map + bi * a.map_sb + hi * a.map_sh + (size_t)(2 * qt) * 2 * TW;
            mapw2 = (2 * qt + 1 < T) ? mapw + 2 * TW : mapw;
        }
    }
    // The first map words are read here, with ordinary (scalar) loads, long before they are needed:
    // the address arithmetic below covers their latency.
    // (Without a map they read the first word of q, which exists, and the result is dropped: no
    // branch, so the loads stay where they are written.  The words are combined only where the walk
    // starts; the compiler puts its wait there.)
    const bool has_map = mapw != nullptr;
    const uint32_t *mapa = has_map ? mapw : reinterpret_cast<const uint32_t *>(a.q.p);
    const uint32_t *mapb = has_map ? mapw2 : reinterpret_cast<const uint32_t *>(a.q.p);
    const uint32_t first_w = mapa[0], first_w2 = mapb[0];
    const uint16_t *qb = slab(a.q, bi, hi);
    const uint16_t *kb = slab(a.k, bi, hi);
    const uint16_t *vb = slab(a.v, bi, hi);
    // packed: words, strides in words; BYTEMASK: bytes, strides in bytes
    const uint32_t *mb = BYTEMASK ? reinterpret_cast<const uint32_t *>(reinterpret_cast<const uint8_t *>(a.mask.p) +
                                                                       bi * a.mask.sb + hi * a.mask.sh)
                                  : slab(a.mask, bi, hi);
    const uint32_t q_sn = PACKED_ROWS ? D : a.q.sn, k_sn = PACKED_ROWS ? D : a.k.sn;       // row strides, elements
    const uint32_t v_sn = PACKED_ROWS ? D : a.v.sn, o_sn = PACKED_ROWS ? D : a.out.sn;
    const uint32_t q_rb = 2u * q_sn, k_rb = 2u * k_sn, v_rb = 2u * v_sn;                   // row pitch, bytes

    // ---- mask words: wave-private async copies, slot = tile % NSTAGE, lane i -> (row i/2, word i%2) ----
    // BYTEMASK (N >= 16): the wave's 32 x 64 bytes of a tile as two copies of 16 rows; lane i
    // fills (row 16j + i/4, position i%4) with the global 16-byte chunk position ^ ((row >> 2) & 3),
    // which makes the reads below (lane = row, two chunks each) free of bank conflicts.  The copies
    // take any byte address (rows of N bytes start anywhere; ROCm runs the memory pipeline in its
    // unaligned access mode, in which a 16-byte copy may start at any byte).  In a last tile of fewer than 64 keys
    // every chunk that would reach beyond the row's end is read from the 16 bytes before that end
    // instead, so that nothing after the mask's last byte is touched; the bits of the chunk that
    // holds the end are shifted to their places below, those of later chunks cleared as pad bits.
    const int mrow = BYTEMASK ? 0 : qt * BM + wave * 32 + (lane >> 1);
    const uint32_t m_voff = BYTEMASK ? 0u : (uint32_t)(((size_t)(mrow < N ? mrow : N - 1) * nw + (lane & 1)) * 4);
    uint32_t mb_voff[2] = {0u, 0u}, mb_chunk[2] = {0u, 0u};
    if constexpr (BYTEMASK) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int row = 16 * j + (lane >> 2);
            const int grow = qt * BM + wave * 32 + row;
            mb_chunk[j] = (uint32_t)(((lane & 3) ^ ((row >> 2) & 3)) << 4);
            mb_voff[j] = (uint32_t)(grow < N ? grow : N - 1) * (uint32_t)N + mb_chunk[j];
        }
    }
    const uint32_t mask_dst = lds0 + wave * (BYTEMASK ? 2048 : 256);
    auto issue_mask = [&](int x, auto slot_c) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        if constexpr (BYTEMASK) {
            const uint8_t *src = reinterpret_cast<const uint8_t *>(mb) + (size_t)x * BN;
            // a single slot is refilled: this wave's reads of the previous tile's bytes must be over
            if constexpr (C::BYTE_SLOTS == 1) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            uint32_t vo[2] = {mb_voff[0], mb_voff[1]};
            if (ragged && x == T - 1) {
                const uint32_t row_end = (uint32_t)(N - x * BN);       // bytes of the row left in this tile
                // the lane offsets are unsigned: what is taken from them below is first taken from the
                // base (a tile that is not the first has 64 bytes of the row before it; in the first,
                // row_end = N >= 16 and nothing goes below zero)
                const uint32_t back = x > 0 ? 16u : 0u;
                src -= back;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    vo[j] += back;
                    if (mb_chunk[j] + 16 > row_end) vo[j] -= mb_chunk[j] + 16 - row_end;
                }
            }
            async_copy_b128_at<OFF_MASK + SLOT * MASK_SLOT>(mask_dst, src, vo[0]);
            async_copy_b128_at<OFF_MASK + SLOT * MASK_SLOT + 1024>(mask_dst, src, vo[1]);
        } else {
            uint32_t voff = m_voff;
            if (2 * x + 1 >= nw) voff -= (lane & 1) * 4;           // odd word count: re-read the last word
            async_copy_b32_at<OFF_MASK + SLOT * MASK_SLOT>(mask_dst, mb + 2 * x, voff);
        }
    };
    // PAIRS: four copies per wave and pair of tiles; lane i of copy j fills (row 8j + i/8, position i%8)
    // from the row's chunk (i%8) ^ ((row >> 1) & 7).  (row >> 1) & 7 is (i/8 >> 1) for j = 0, 2 and that
    // plus 4 for j = 1, 3: one lane offset and the same with chunk bit 2 flipped (N is a multiple of
    // 128, so the low seven bits of the offset are the chunk alone).
    uint32_t pair_voff = 0u;
    if constexpr (PAIRS) {
        const int row = lane >> 3;
        pair_voff = (uint32_t)(qt * BM + wave * 32 + row) * (uint32_t)N + (uint32_t)(((lane & 7) ^ (row >> 1)) << 4);
    }
    auto issue_mask_pair = [&](int p) __attribute__((always_inline)) {      // bytes of tiles 2p and 2p + 1
        const uint8_t *src = reinterpret_cast<const uint8_t *>(mb) + (size_t)p * (2 * BN);
        const uint32_t dst = lds0 + wave * 4096;
        async_copy_b128_at<OFF_MASK>(dst, src, pair_voff);
        async_copy_b128_at<OFF_MASK + 1024>(dst, src + (size_t)8 * N, pair_voff ^ 64u);
        async_copy_b128_at<OFF_MASK + 2048>(dst, src + (size_t)16 * N, pair_voff);
        async_copy_b128_at<OFF_MASK + 3072>(dst, src + (size_t)24 * N, pair_voff ^ 64u);
    };
    // BYTEMASK: where this lane's row of packed words goes, if the caller wants them ([Bm, Hm, N, nw]
    // like the mask; a mask shared between batch entries / heads is written by the first of them)
    const int qrow = qt * BM + wave * 32 + l32;
    uint32_t *words_out = nullptr;
    // ... and where the tile map of this work-group's two blocks of 64 rows goes ([Bm, Hm, T, 2, TW]).
    // Each wavefront notes per key tile whether its 32 rows hold a set bit and whether they hold a
    // clear one, 32 tiles to a pair of registers that goes to LDS when it is full.  After
    // its last tile a wavefront counts itself in; the second of a block's two to do so combines
    // both and writes the block's words, which then travel while the output is being stored.
    // (Per-lane bits ORed into LDS by all lanes at once, instead of the two ballots per tile,
    // measured 4 us slower on the headline workload: 64 atomics on one address.)
    uint32_t *map_dst = nullptr;
    uint32_t some_acc = 0u, hole_acc = 0u;
    u32x4 pend = {0u, 0u, 0u, 0u};        // packed words waiting to be stored, see mask_words
    if constexpr (BYPRODUCTS) {
        const bool writer = (a.mask.sb != 0 || bi == 0) && (a.mask.sh != 0 || hi == 0);
        const int Hm = a.mask.sh != 0 ? a.H : 1;
        const size_t slab_m = (size_t)((a.mask.sb != 0 ? bi : 0) * Hm + (a.mask.sh != 0 ? hi : 0));
        if (a.mask_out != nullptr && writer) words_out = a.mask_out + (slab_m * N + (qrow < N ? qrow : 0)) * nw;
        if (a.map_out != nullptr && writer) map_dst = a.map_out + (slab_m * T + 2 * qt) * 2 * TW;
    }
    const uint32_t map_lds = lds0 + C::OFF_MAP + wave * (C::MAP_WORDS * 8);
    if constexpr (BYPRODUCTS) {     // ordered before any arrival by the barriers of the main loop (T >= 1)
        if (tid < 2) *(LDS_PTR(uint32_t))(uintptr_t)(lds0 + C::OFF_MAP_ARRIVED + 4 * tid) = 0u;
    }
    const uint32_t maddr = BYTEMASK ? lds0 + OFF_MASK + wave * 2048 + l32 * 64 : lds0 + OFF_MASK + wave * 256 + l32 * 8;
    const int msw = (l32 >> 2) & 3;
    // PAIRS: a wave's bytes of a pair of tiles are 32 rows of 128 bytes in the 4 KiB that its two byte
    // slots occupy otherwise; the 16-byte chunks of a row are swizzled like K's (position ^ ((row >> 1)
    // & 7), applied on the global side), which keeps the reads below free of bank conflicts.
    // `pair_half` (0 or 1) says which tile of the pair; -1: the ordinary slots.
    const uint32_t pair_base = lds0 + OFF_MASK + wave * 4096 + l32 * 128;
    const int psw = (l32 >> 1) & 7;
    auto mask_words = [&](int x, int slot, int pair_half = -1) __attribute__((always_inline)) -> u32x2 {
        u32x2 w;
        if constexpr (BYTEMASK) {
            // this lane: the 32 bytes of row l32 for keys 32hh .. 32hh+31 -> one word
            const uint32_t a0 = !PAIRS || pair_half < 0 ? maddr + slot * MASK_SLOT + (((2 * hh) ^ msw) << 4)
                                                        : pair_base + (((4 * pair_half + 2 * hh) ^ psw) << 4);
            const uint32_t a1 = !PAIRS || pair_half < 0 ? maddr + slot * MASK_SLOT + (((2 * hh + 1) ^ msw) << 4)
                                                        : pair_base + (((4 * pair_half + 2 * hh + 1) ^ psw) << 4);
            const u32x4 d0 = lds_read_b128(a0);
            const u32x4 d1 = lds_read_b128(a1);
            // a byte counts as "attend" when it is non-zero, as in the packer: nz() leaves 0x80 in
            // every non-zero byte, the dot products weigh those with 1, 2, 4 .. 128 (times 128)
            auto nz = [](uint32_t x) -> uint32_t { return (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u; };
            // ... which costs three instructions per four bytes.  Bytes that are all 0 or 1 (every
            // mask PyTorch itself made) need none of it: one look at the wavefront's 2 KiB decides.
            const uint32_t other = (d0.x | d0.y | d0.z | d0.w | d1.x | d1.y | d1.z | d1.w) & 0xfefefefeu;
            uint32_t mine;
            if (__builtin_amdgcn_ballot_w64(other != 0u) == 0ull) {
                uint32_t b0 = __builtin_amdgcn_udot4(d0.x, 0x08040201u, 0u, false);
                uint32_t b1 = __builtin_amdgcn_udot4(d0.z, 0x08040201u, 0u, false);
                uint32_t b2 = __builtin_amdgcn_udot4(d1.x, 0x08040201u, 0u, false);
                uint32_t b3 = __builtin_amdgcn_udot4(d1.z, 0x08040201u, 0u, false);
                b0 = __builtin_amdgcn_udot4(d0.y, 0x80402010u, b0, false);
                b1 = __builtin_amdgcn_udot4(d0.w, 0x80402010u, b1, false);
                b2 = __builtin_amdgcn_udot4(d1.y, 0x80402010u, b2, false);
                b3 = __builtin_amdgcn_udot4(d1.w, 0x80402010u, b3, false);
                mine = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
            } else {
                uint32_t b0 = __builtin_amdgcn_udot4(nz(d0.x), 0x08040201u, 0u, false);
                uint32_t b1 = __builtin_amdgcn_udot4(nz(d0.z), 0x08040201u, 0u, false);
                uint32_t b2 = __builtin_amdgcn_udot4(nz(d1.x), 0x08040201u, 0u, false);
                uint32_t b3 = __builtin_amdgcn_udot4(nz(d1.z), 0x08040201u, 0u, false);
                b0 = __builtin_amdgcn_udot4(nz(d0.y), 0x80402010u, b0, false);
                b1 = __builtin_amdgcn_udot4(nz(d0.w), 0x80402010u, b1, false);
                b2 = __builtin_amdgcn_udot4(nz(d1.y), 0x80402010u, b2, false);
                b3 = __builtin_amdgcn_udot4(nz(d1.w), 0x80402010u, b3, false);
                // each partial value is 128 x (8 bits): bits 7..14
                mine = (b0 >> 7) | (b1 << 1) | (b2 << 9) | (b3 << 17);
            }
            if (x == T - 1) {
                // the chunk that holds the row's end was copied from 16 bytes before that end: its
                // bits move down to their places (zeros follow them)
                const int row_end = N - x * BN, part = row_end >> 4, shift = (16 - (row_end & 15)) & 15;
                const uint32_t lo = (mine & 0xffffu) >> (part == 2 * hh ? shift : 0);
                const uint32_t hi = (mine >> 16) >> (part == 2 * hh + 1 ? shift : 0);
                mine = (lo | (hi << 16)) & (hh ? a.last_mask1 : a.last_mask0);       // bits of keys >= N
            }
            if (BYPRODUCTS && map_dst != nullptr) {
                // rows beyond N repeat row N - 1 and change nothing; key bits beyond N are not valid
                const uint32_t valid = x == T - 1 ? (hh ? a.last_mask1 : a.last_mask0) : 0xffffffffu;
                const uint32_t some = __builtin_amdgcn_ballot_w64(mine != 0u) != 0ull ? 1u : 0u;
                const uint32_t hole = __builtin_amdgcn_ballot_w64(mine != valid) != 0ull ? 1u : 0u;
                some_acc |= some << (x & 31);
                hole_acc |= hole << (x & 31);
                if ((x & 31) == 31 || x == T - 1) {
                    if (lane == 0) *(LDS_PTR(u32x2))(uintptr_t)(map_lds + (uint32_t)(x >> 5) * 8) = u32x2{some_acc, hole_acc};
                    some_acc = hole_acc = 0u;
                }
            }
            // lanes < 32 hold the word of keys 0..31, lanes >= 32 that of keys 32..63: both to both
            const auto r = __builtin_amdgcn_permlane32_swap(mine, mine, false, false);
            w.x = (uint32_t)r[0];
            w.y = (uint32_t)r[1];
            // A caller who will need the packed words (for the backward) gets them as a by-product.
            // Stored tile by tile they would leave as 4-byte pieces of 64 different rows; instead
            // the lower lane half keeps the words of tiles 4g and 4g + 1, the upper half those of
            // tiles 4g + 2 and 4g + 3, and after every fourth tile each lane stores 16 bytes: 32
            // consecutive bytes of each row per store instruction.
            if (BYPRODUCTS && words_out != nullptr) {
                const int j = x & 3;
                const bool turn = hh == (j >> 1);
                if ((j & 1) == 0) {
                    pend.x = turn ? w.x : pend.x;
                    pend.y = turn ? w.y : pend.y;
                } else {
                    pend.z = turn ? w.x : pend.z;
                    pend.w = turn ? w.y : pend.w;
                }
                if (j == 3 || x == T - 1) {
                    // words of tiles beyond the last one have indices >= nw and stay unwritten
                    const int wb = 8 * (x >> 2) + 4 * hh;
                    if (qrow < N) {
                        typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
                        if (wb + 3 < nw) {
                            __builtin_nontemporal_store((u32x4_a4)pend, reinterpret_cast<u32x4_a4 *>(words_out + wb));
                        } else {
                            if (wb < nw) words_out[wb] = pend.x;
                            if (wb + 1 < nw) words_out[wb + 1] = pend.y;
                            if (wb + 2 < nw) words_out[wb + 2] = pend.z;
                        }
                    }
                }
            }
        } else {
            w = lds_read_b64(maddr + slot * MASK_SLOT);
            const bool last = (x == T - 1);
            w.x &= last ? a.last_mask0 : 0xffffffffu;
            w.y &= last ? a.last_mask1 : 0xffffffffu;
        }
        return w;
    };
    // ---- K/V tiles: async copies --------------------------------------------------------------
    // One global_load_lds_dwordx4 fills 1 KiB = 8 tile rows.  Wave w copies row blocks 2w, 2w+1 of
    // K and of V.  Lane i fills LDS chunk (row = 8*blk + i/8, position i%8) with the global chunk
    // position ^ swz(row):   K: swz(row) = (row >> 1) & 7      V: swz(row) = bitrev3((row >> 1) & 7)
    uint32_t kv_voff[2][2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int row = 8 * (2 * wave + j) + (lane >> 3);
        const int pos = lane & 7;
        const int f = (row >> 1) & 7;
        const int fr = bitrev3(f);
        // row pitches are below 2^24 bytes (checked by the C-ABI layer): full-rate 24-bit multiplies
        kv_voff[0][j] = __umul24(row, k_rb) + (((pos ^ f) & CHM) << 4);
        kv_voff[1][j] = __umul24(row, v_rb) + (((pos ^ fr) & CHM) << 4);
    }
    const uint32_t kv_dst = lds0 + wave * 2048;
    auto issue_kv = [&](int t, auto stage_c) __attribute__((always_inline)) {
        constexpr int SO = decltype(stage_c)::value * STAGE_BYTES;
        const int key0 = t * BN;
        uint32_t ko[2] = {kv_voff[0][0], kv_voff[0][1]}, vo[2] = {kv_voff[1][0], kv_voff[1][1]};
        if (ragged && t == T - 1) {           // rows beyond N: copy row N-1 instead (zeroed later)
            int last0 = key0;
            asm volatile("" : "+s"(last0));   // opaque: keeps this once-only arithmetic out of the loop's registers
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int row = 8 * (2 * wave + j) + (lane >> 3);
                const int over = last0 + row - (N - 1);
                if (over > 0) { ko[j] -= __umul24(over, k_rb); vo[j] -= __umul24(over, v_rb); }
            }
        }
        const uint16_t *ksrc = kb + (size_t)key0 * k_sn, *vsrc = vb + (size_t)key0 * v_sn;
        async_copy_b128_at<SO>(kv_dst, ksrc, ko[0]);
        async_copy_b128_at<SO + 1024>(kv_dst, ksrc, ko[1]);
        if constexpr (NH == 2) {              // second column half: 128 bytes further along each row
            async_copy_b128_at<SO + TILE_BYTES>(kv_dst, ksrc + HD, ko[0]);
            async_copy_b128_at<SO + TILE_BYTES + 1024>(kv_dst, ksrc + HD, ko[1]);
        }
        async_copy_b128_at<SO + C::OFF_V>(kv_dst, vsrc, vo[0]);
        async_copy_b128_at<SO + C::OFF_V + 1024>(kv_dst, vsrc, vo[1]);
        if constexpr (NH == 2) {
            async_copy_b128_at<SO + C::OFF_V + TILE_BYTES>(kv_dst, vsrc + HD, vo[0]);
            async_copy_b128_at<SO + C::OFF_V + TILE_BYTES + 1024>(kv_dst, vsrc + HD, vo[1]);
        }
    };
    auto zero_tail_rows = [&](int t, int stage) __attribute__((always_inline)) {   // after the copies of the last tile have landed
        const int key0 = t * BN;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int row = 8 * (2 * wave + j) + (lane >> 3);
            if (key0 + row >= N) {
                const uint32_t p = lds0 + stage * STAGE_BYTES + wave * 2048 + j * 1024 + lane * 16;
                const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
                for (int part = 0; part < 2 * NH; ++part) *(LDS_PTR(u32x4))(uintptr_t)(p + part * TILE_BYTES) = z;
            }
        }
    };

    // ---- per-lane LDS read addresses (stage 0, first column half); everything else is an immediate offset ----
    // K operand (blk, s): row 32*blk + l32, chunk 2s + hh           -> kaddr[s] + 4096*blk
    // V operand (dblk, blk, u, x), read by ds_read_b64_tr_b16: the lane supplies
    //   row 32blk + 16u + 8x + 4hh + (i >> 2), columns 32dblk + 16G + 4(i & 3) .. +3
    //   with i = lane % 16, G = (lane % 32) / 16                     -> vaddr[dblk][x] + 4096*blk + 2048*u
    uint32_t kaddr[4], vaddr[2][2];
    {
        const int fk = (l32 >> 1) & 7;
#pragma unroll
        for (int s = 0; s < 4; ++s) kaddr[s] = lds0 + l32 * 128 + (((2 * s + hh) ^ fk) << 4);
        const int i16 = lane & 15, G = l32 >> 4;
        const int r3 = 4 * hh + (i16 >> 2);
#pragma unroll
        for (int x = 0; x < 2; ++x) {
            const int row = 8 * x + r3;
            const int f = (row >> 1) & 7;
            const int fr = bitrev3(f);
#pragma unroll
            for (int dblk = 0; dblk < 2; ++dblk) {
                const int chunk = 4 * dblk + 2 * G + ((i16 & 3) >> 1);
                vaddr[dblk][x] = lds0 + C::OFF_V + row * 128 + ((chunk ^ fr) << 4) + ((i16 & 1) << 3);
            }
        }
    }
    const uint32_t lut_addr = lds0 + OFF_LUT;
    const uint32_t nib_shift = 4u - 4u * hh;

    // ================================ prologue: one memory round trip ================================
    // Requested at once, oldest first: q (this wave's 32 rows, staged through the second K/V stage,
    // which the prologue leaves unused, K-swizzled), then K/V and the mask words of tile 0.
    {
        const int qbase = qt * BM + wave * 32 < N ? qt * BM + wave * 32 : N - 1;   // wave-uniform
        const uint16_t *qsrc = qb + (size_t)qbase * q_sn;
        const int last = N - 1 - qbase;                      // rows beyond N re-read row N-1
        const uint32_t dst = lds0 + (NSTAGE - 1) * STAGE_BYTES + wave * 4096;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = 8 * j + (lane >> 3);
            const int pos = lane & 7;
            const int lrow = row < last ? row : last;
            const uint32_t voff = __umul24(lrow, q_rb) + (((pos ^ ((row >> 1) & 7)) & CHM) << 4);
            async_copy_b128(dst + j * 1024, qsrc, voff);
            if constexpr (NH == 2) async_copy_b128(dst + 16384 + j * 1024, qsrc + HD, voff);
        }
    }
    using std::integral_constant;
    uint32_t live_w = has_map ? (first_w | first_w2) : 0xffffffffu;
    if ((T & 31) != 0 && TW == 1) live_w &= (1u << (T & 31)) - 1u;
    const int n_visits = TW == 1 ? __builtin_popcount(live_w) : T;
    // Walk over the set bits of the "live" words: `live_w` holds the bits of word `cur_w` that have
    // not been visited yet.  Words beyond the first (N > 2048) are fetched when the walk gets there.
    int cur_w = 0;
    auto next_tile = [&]() __attribute__((always_inline)) -> int {     // next live tile, T if there is none; wave-uniform
        while (live_w == 0u) {
            if (++cur_w >= TW) return T;
            uint32_t lv = 0xffffffffu, lv2 = 0u;
            if (mapw != nullptr)
                asm volatile("s_load_dword %0, %2, 0x0\n\ts_load_dword %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
                             : "=&s"(lv), "=&s"(lv2) : "s"(mapw + cur_w), "s"(mapw2 + cur_w) : "memory");
            lv |= lv2;
            if (cur_w == TW - 1 && (T & 31) != 0) lv &= (1u << (T & 31)) - 1u;
            live_w = lv;
        }
        const int b = __builtin_ctz(live_w);
        live_w &= live_w - 1u;
        return 32 * cur_w + b;
    };
    const int t_first = next_tile();
    if (t_first < T) {
        if constexpr (PAIRS) {          // the first pair's bytes before K/V: the walk below counts on that order
            issue_mask_pair(0);
            issue_kv(t_first, integral_constant<int, 0>{});
        } else {
            issue_kv(t_first, integral_constant<int, 0>{});
            issue_mask(t_first, integral_constant<int, 0>{});
        }
    }
    // small LDS table for the mask: entry n (16 B) holds four floats, float j = (bit j of n) ? 0 : -inf
    if (tid < 64)
        reinterpret_cast<float *>(smem + OFF_LUT)[tid] = (((tid >> 2) >> (tid & 3)) & 1) ? 0.f : -__builtin_inff();
    const bool even_progress = NH == 1 && (int)blockIdx.x >= a.tail_start;   // three work-groups per CU
    if (even_progress && n_visits >= 4) __builtin_amdgcn_s_setprio(3);
    if (PAIRS) wait_vmcnt<8>();                   // q has landed; 4 mask and 4 K/V copies may still be in flight
    else if (t_first < T) wait_vmcnt<C::COPIES>();     // q has landed; the copies of the first tile may still be in flight
    else wait_vmcnt<0>();
    // ---- Q^T as MFMA B operands, scaled by scale*log2(e)/post_mul:
    //      lane holds query row l32, d = 16*s + 8*hh .. +7
    u32x4 qf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        u32x4 t = lds_read_b128(kaddr[s & 3] + (NSTAGE - 1) * STAGE_BYTES + (s >> 2) * 16384 + wave * 4096);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float lo = E::up1((uint16_t)(t[i] & 0xffffu)) * a.q_scale;
            const float hi = E::up1((uint16_t)(t[i] >> 16)) * a.q_scale;
            t[i] = (uint32_t)E::cvt1(lo) | ((uint32_t)E::cvt1(hi) << 16);
        }
        qf[s] = t;
    }

    // ---- running state: one query row per lane; both lane halves hold the same ref ----
    f32x16 oacc[OB];                    // [2 * half + dblk]: 32 columns each
#pragma unroll
    for (int b = 0; b < OB; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[b][i] = 0.f;
    float ref = 0.f;                    // reference point r, in accumulator units (log2 / pm)
    float rmax = -__builtin_inff();     // largest score seen when the maximum was last taken, minus r; -inf = no kept key yet
    bool all_seen = false;              // wave-uniform: every row of this wavefront has met a kept key
    float l_run = 0.f;                  // this lane's share of sum exp2(pm * (score - r))
    u32x4 refb = {0u, 0u, 0u, 0u};      // -r as four 16-bit terms (lane half 0 only), B operand
    bool ref_used = false;              // false while r == 0 for every row: the extra MFMA is skipped
    u32x4 ones = {E::ONES, E::ONES, E::ONES, E::ONES};
    asm volatile("" : "+v"(ones));      // keep the constant operand resident in registers

    auto set_ref = [&](float r_wanted) __attribute__((always_inline)) -> float {      // returns the value actually represented
        float rest = -r_wanted, sum = 0.f;
        uint16_t term[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float clipped = __builtin_fminf(__builtin_fmaxf(rest, -E::TERM_MAX), E::TERM_MAX);
            term[i] = E::cvt1(clipped);
            const float got = E::up1(term[i]);
            rest -= got;
            sum += got;
        }
        const uint32_t keep = hh == 0 ? 0xffffffffu : 0u;
        refb.x = ((uint32_t)term[0] | ((uint32_t)term[1] << 16)) & keep;
        refb.y = ((uint32_t)term[2] | ((uint32_t)term[3] << 16)) & keep;
        return -sum;
    };

    // One key tile for this wavefront.  `so` (LDS offset of the stage) is a compile-time constant
    // in every call, so all LDS addresses below are a register plus an immediate.
    auto compute_tile = [&](const u32x2 w2, const uint32_t so) __attribute__((always_inline)) {
        if (__builtin_amdgcn_ballot_w64((w2.x | w2.y) != 0u) == 0ull) return;
        // ---- S^T: sacc[blk][4g+j] = log2 weight / pm of (key 32blk + 8g + 4hh + j, query l32) ----
        f32x16 sacc[2];
        // The K fragments of MFMA step s + 1 are requested before the MFMAs of step s are issued, the
        // first pair before the table look-ups below.  The scheduling barriers hold that order: left
        // alone, the compiler requests each pair just before its MFMAs (it saves eight registers)
        // and the wavefront sits out four LDS round trips per tile one after the other.
        u32x4 kf[2][2];
        kf[0][0] = lds_read_b128(kaddr[0] + so);
        kf[0][1] = lds_read_b128(kaddr[0] + so + 4096);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const uint32_t wa = (blk == 0 ? w2.x : w2.y) << nib_shift;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x4 b = lds_read_b128(lut_addr + ((wa >> (8 * g)) & 0xF0u));
#pragma unroll
                for (int j = 0; j < 4; ++j) sacc[blk][4 * g + j] = __builtin_bit_cast(float, (uint32_t)b[j]);
            }
        }
        if (ref_used) {               // wave-uniform: some row of this wavefront has r != 0
            sacc[0] = E::mfma(ones, refb, sacc[0]);
            sacc[1] = E::mfma(ones, refb, sacc[1]);
        }
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            if (s + 1 < KS) {
                const uint32_t ka = kaddr[(s + 1) & 3] + so + ((s + 1) >> 2) * TILE_BYTES;
                kf[(s + 1) & 1][0] = lds_read_b128(ka);
                kf[(s + 1) & 1][1] = lds_read_b128(ka + 4096);
            }
            __builtin_amdgcn_sched_barrier(0);
            sacc[0] = E::mfma(kf[s & 1][0], qf[s], sacc[0]);
            sacc[1] = E::mfma(kf[s & 1][1], qf[s], sacc[1]);
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- the row maximum of the tile is taken only when it can matter ----
        // Moves the reference point when a row's scores leave the window [r-8, r+8] upwards, or when
        // the first kept score of a row lies below it.
        auto recentre = [&]() __attribute__((always_inline)) {
            float mx = -__builtin_inff();
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int i = 0; i < 16; ++i) mx = __builtin_fmaxf(mx, sacc[blk][i]);
            mx = xhalf_max(mx);
            const float mxs = POSTMUL ? mx * pm : mx;
            const bool first = (rmax == -__builtin_inff());
            const bool move = (mxs > WINDOW_LOG2) | (first & (mxs < -WINDOW_LOG2) & (mx > -__builtin_inff()));
            const float top = __builtin_fmaxf(rmax, mx);
            if (__builtin_amdgcn_ballot_w64(move) != 0ull) {
                // every row of the wavefront re-centres on its own largest score so far
                const bool any = top > -__builtin_inff();
                const float new_ref = set_ref(any ? ref + top : ref);
                const float delta = ref - new_ref;                       // ~ -top
                const float alpha = first ? 1.0f : __builtin_amdgcn_exp2f(POSTMUL ? delta * pm : delta);
                ref = new_ref;
                ref_used = true;
                l_run *= alpha;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
#pragma unroll
                    for (int b = 0; b < OB; ++b) oacc[b][i] *= alpha;
                    sacc[0][i] += delta; sacc[1][i] += delta;
                }
                rmax = top + delta;
            } else {
                rmax = top;
            }
        };
        // probabilities, packed as the B operands of the PV product; returns this lane's sum of them
        uint32_t pb[2][2][4];
        auto exponentials = [&]() __attribute__((always_inline)) -> float {
            float lsum = 0.f;
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float s0 = sacc[blk][8 * u + 2 * i], s1 = sacc[blk][8 * u + 2 * i + 1];
                        const float p0 = __builtin_amdgcn_exp2f(POSTMUL ? s0 * pm : s0);
                        const float p1 = __builtin_amdgcn_exp2f(POSTMUL ? s1 * pm : s1);
                        const uint32_t pk = E::pack2_prob(p0, p1);
                        pb[blk][u][i] = pk;
                        lsum = E::add2(pk, lsum);
                    }
            return lsum;
        };
        // A row needs the maximum when it meets its first kept key (to choose its reference point)
        // and when a score runs away above the window.  The first is known beforehand; the second
        // shows afterwards, in the sum of the exponentials (needed anyway): a weight above 2^14, an
        // infinity or a NaN makes a lane's sum of 32 weights exceed SUM_LIMIT, and no weight that
        // the window would have let pass (<= 2^8) can.  Only then are the maximum taken, the
        // reference moved and the exponentials redone.
        bool with_max = false;
        if (!all_seen) with_max = __builtin_amdgcn_ballot_w64((rmax == -__builtin_inff()) & ((w2.x | w2.y) != 0u)) != 0ull;
        if (with_max) {
            recentre();
            all_seen = __builtin_amdgcn_ballot_w64(rmax == -__builtin_inff()) == 0ull;
        }
        float lsum = exponentials();
        if (!with_max && __builtin_amdgcn_ballot_w64(!(lsum <= SUM_LIMIT)) != 0ull) {
            recentre();
            lsum = exponentials();
        }
        l_run += lsum;
        // ---- O^T += V^T * P^T : oacc[b][4g+j] = out(query l32, d = 32b + 8g + 4hh + j) ----
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const u32x4 pv = {pb[blk][u][0], pb[blk][u][1], pb[blk][u][2], pb[blk][u][3]};
                const uint32_t off = so + 4096 * blk + 2048 * u;
#pragma unroll
                for (int b = 0; b < OB; ++b) {
                    const uint32_t voff = off + (b >> 1) * TILE_BYTES;
                    const u32x2 lo = lds_read_tr16_b64(vaddr[b & 1][0] + voff);
                    const u32x2 hi = lds_read_tr16_b64(vaddr[b & 1][1] + voff);
                    const u32x4 va = {lo.x, lo.y, hi.x, hi.y};
                    oacc[b] = E::mfma(va, pv, oacc[b]);
                }
            }
    };

    // ================================ main loop ================================
    // The tiles visited: every tile whose "some bit set" bit is on (all of them without a map), in
    // ascending order; the prologue has requested the first.  The i-th visit uses stage and mask
    // slot i % 2; the loop is unrolled by 2 so that these are constants.
    // In a visit of tile t:
    //   wait for the copies of tile t  ->  barrier  ->  request the copies of the next tile to be
    //   visited (K/V, then the mask words) into the stage the barrier has freed  ->  compute, unless
    //   this wave's 32 x 64 block of mask bits is empty.
    // (A ring of three stages, copies two tiles ahead, measured the same to 2 % slower on every
    // workload and costs 18 KB more LDS.)
    int visits = 0;
    auto visit = [&](const int t, const int t_next, auto slot_c) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        constexpr int SLOT2 = SLOT ^ 1;       // the stage freed by the barrier below
        if (even_progress) {
            // The hardware serves the oldest wave first, so of three co-resident work-groups one
            // finishes early and the last runs alone, at a worse rate than three together.  When
            // no other work-group waits for the slot, a wave therefore yields as it advances.
            if (visits == n_visits / 4) __builtin_amdgcn_s_setprio(2);
            else if (visits == n_visits / 2) __builtin_amdgcn_s_setprio(1);
            else if (visits == (3 * n_visits) / 4) __builtin_amdgcn_s_setprio(0);
        }
        ++visits;
        wait_vmcnt<0>();          // the copies of tile t (the only ones in flight) have landed
        if (ragged && t == T - 1) zero_tail_rows(t, SLOT);
        __syncthreads();          // tile t landed for every wave; the stage of the previous visit is free
        const u32x2 w2 = mask_words(t, SLOT);
        if (t_next < T) {       // K/V first: the MFMA operands are what the next visit needs first (1-2 % with a byte mask)
            issue_kv(t_next, integral_constant<int, SLOT2>{});
            issue_mask(t_next, integral_constant<int, SLOT2>{});
        }
        compute_tile(w2, (uint32_t)(SLOT * STAGE_BYTES));
    };
    if constexpr (PAIRS) {
        // Every tile is visited (there is no tile map with a boolean mask) and their number is even.
        // Copies in flight, oldest first, at the top of an even visit t: the bytes of the pair
        // (t, t + 1), then K/V of t; after its barrier K/V of t + 1 and then the bytes of the next
        // pair are requested, and the odd visit requests K/V of t + 2 after its barrier: the bytes of
        // a pair are always followed by exactly four younger copies when they are needed.  (The stores
        // of the by-products, when asked for, only add to the count: copies complete in the order of
        // their requests, so "at most four outstanding" still means that all older copies are in.)
        auto progress = [&]() __attribute__((always_inline)) {
            if (even_progress) {
                if (visits == n_visits / 4) __builtin_amdgcn_s_setprio(2);
                else if (visits == n_visits / 2) __builtin_amdgcn_s_setprio(1);
                else if (visits == (3 * n_visits) / 4) __builtin_amdgcn_s_setprio(0);
            }
            ++visits;
        };
        for (int t = 0; t < T; t += 2) {
            progress();
            wait_vmcnt<4>();                                  // this wave's bytes of the pair have landed
            const u32x2 w_even = mask_words(t, 0, 0);
            const u32x2 w_odd = mask_words(t + 1, 0, 1);
            wait_vmcnt<0>();                                  // K/V of tile t
            __syncthreads();
            issue_kv(t + 1, integral_constant<int, 1>{});
            if (t + 2 < T) issue_mask_pair((t >> 1) + 1);     // the words above are in registers: the bytes may go
            compute_tile(w_even, 0u);
            progress();
            if (t + 2 < T) wait_vmcnt<4>(); else wait_vmcnt<0>();   // K/V of tile t + 1 (the next pair's bytes may be on their way)
            __syncthreads();
            if (t + 2 < T) issue_kv(t + 2, integral_constant<int, 0>{});
            compute_tile(w_odd, (uint32_t)STAGE_BYTES);
        }
    } else
    for (int t = t_first; t < T;) {
        const int tn = next_tile();
        visit(t, tn, integral_constant<int, 0>{});
        if (tn >= T) break;
        t = next_tile();
        visit(tn, t, integral_constant<int, 1>{});
    }
    wait_vmcnt<0>();              // no copy may outlive the work-group's LDS allocation

    if constexpr (BYPRODUCTS) {
        if (map_dst != nullptr) {
            const int rb = wave >> 1;                          // block of 64 rows
            uint32_t before = 0u;
            if (lane == 0)
                before = __hip_atomic_fetch_add((LDS_PTR(uint32_t))(uintptr_t)(lds0 + C::OFF_MAP_ARRIVED + 4 * rb), 1u,
                                                __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
            before = __builtin_amdgcn_readfirstlane(before);
            if (before == 1u && lane < TW && 2 * qt + rb < T) {
                const int w = lane;                            // word of 32 key tiles
                const uint32_t src = lds0 + C::OFF_MAP + (uint32_t)(2 * rb) * (C::MAP_WORDS * 8) + (uint32_t)w * 8;
                const u32x2 x0 = lds_read_b64(src), x1 = lds_read_b64(src + C::MAP_WORDS * 8);
                const uint32_t in_range = (w == TW - 1 && (T & 31)) ? ((1u << (T & 31)) - 1u) : 0xffffffffu;
                uint32_t *dst = map_dst + (size_t)rb * 2 * TW;
                dst[w] = (x0.x | x1.x) & in_range;
                dst[TW + w] = ~(x0.y | x1.y) & in_range;
            }
        }
    }

    // ---- epilogue ----
    // out = O / l.  The accumulator layout gives a lane 8-byte pieces of one row; written as they
    // are, a store instruction would touch 32 different 128-byte rows.  Each wave therefore
    // transposes its 32 x 64 block (one per column half) through 4 KiB of LDS and stores whole
    // 128-byte pieces of rows, non-temporally: the output is not read again here and should not
    // displace K, V and the mask.  The LDS used is the stage that tile T would have gone to: its
    // last occupant was tile T - 2, which every wave had finished before the barrier of the last
    // iteration, and no copy into it is in flight, so no further barrier is needed and a wave
    // that is done early stores early.
    const float l_tot = xhalf_sum(l_run);
    const float inv = (l_tot > 0.f) ? 1.0f / l_tot : 0.f;
    {
        const int row0 = qt * BM + wave * 32;
        uint16_t *ob = slab(a.out, bi, hi) + (size_t)row0 * o_sn;
        const uint32_t ebase = lds0 + (uint32_t)(visits & 1) * STAGE_BYTES + wave * 4096;
        if constexpr (HDIM == 32) {
            store_block<BF16, 32>(oacc[0], oacc[0], inv, ebase, ob, (int)o_sn, row0, N, lane);
        } else {
#pragma unroll
            for (int half = 0; half < NH; ++half)
                store_block<BF16>(oacc[2 * half], oacc[2 * half + 1], inv, ebase + half * 16384,
                                  ob + half * HD, (int)o_sn, row0, N, lane);
        }
    }
    if (qrow < N) {
        if (a.lse != nullptr && hh == 0) {
            // log2 of the row's sum of exp(scale * score) is pm * r + log2(l)
            a.lse[(size_t)bh * N + qrow] =
                (l_tot > 0.f) ? __builtin_fmaf(pm * ref, 0.6931471805599453f, __builtin_logf(l_tot)) : -__builtin_inff();
            // (an explicit fma: left to the compiler, the sum was contracted in some instantiations of
            // this kernel and not in others, and their lse differed in the last bit)
        }
    }
}

}  // namespace

// Number of compute units of the current device (cached per device ordinal).
static int compute_units()
{
    static std::atomic<int> cached[64];      // 0 = not asked yet; threads may race to store the same value
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0 && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess)
        cached[dev].store(n, std::memory_order_relaxed);
    return n;
}

hipError_t launch_attn_fwd(const AttnArgs &args, bool bf16, hipStream_t stream)
{
    AttnArgs a = args;
    a.div_qtiles = make_fastdiv((uint32_t)a.qtiles);
    a.div_H = make_fastdiv((uint32_t)a.H);
    const long long groups = (long long)a.BH * a.qtiles;
    if (groups == 0) return hipSuccess;
    // Only a grid that is resident all at once with three work-groups on (almost) every CU evens out
    // its progress; with several rounds oldest-first is what frees slots for the waiting ones, and
    // applying it to the last round only measured neutral.
    const long long cus = compute_units();
    a.tail_start = (groups > 2 * cus && groups <= 3 * cus) ? 0 : (int)groups;
    const dim3 grid((unsigned)groups), block(NTHREADS);
    const bool postmul = a.post_mul != 1.0f;
    const int D = a.D;
    const bool packed = (int)a.q.sn == D && (int)a.k.sn == D && (int)a.v.sn == D && (int)a.out.sn == D;
    if (D == 2 * HD) a.tail_start = (int)groups;              // two work-groups per CU: nobody yields
    void (*kernel)(const AttnArgs) = nullptr;
    const int variant = (bf16 ? 4 : 0) | (postmul ? 2 : 0) | (packed ? 1 : 0);
#define SMA_FWD_VARIANTS(HDIM)                                                          \
    switch (variant) {                                                                 \
    case 0: kernel = attn_fwd_kernel<false, false, false, HDIM>; break;                \
    case 1: kernel = attn_fwd_kernel<false, false, true, HDIM>; break;                 \
    case 2: kernel = attn_fwd_kernel<false, true, false, HDIM>; break;                 \
    case 3: kernel = attn_fwd_kernel<false, true, true, HDIM>; break;                  \
    case 4: kernel = attn_fwd_kernel<true, false, false, HDIM>; break;                 \
    case 5: kernel = attn_fwd_kernel<true, false, true, HDIM>; break;                  \
    case 6: kernel = attn_fwd_kernel<true, true, false, HDIM>; break;                  \
    default: kernel = attn_fwd_kernel<true, true, true, HDIM>; break;                  \
    }
#define SMA_FWD_BYTEMASK_VARIANTS(HDIM)                                                 \
    switch (variant | (byproducts ? 8 : 0)) {                                          \
    case 0: kernel = attn_fwd_kernel<false, false, false, HDIM, true>; break;          \
    case 1: kernel = attn_fwd_kernel<false, false, true, HDIM, true>; break;           \
    case 2: kernel = attn_fwd_kernel<false, true, false, HDIM, true>; break;           \
    case 3: kernel = attn_fwd_kernel<false, true, true, HDIM, true>; break;            \
    case 4: kernel = attn_fwd_kernel<true, false, false, HDIM, true>; break;           \
    case 5: kernel = attn_fwd_kernel<true, false, true, HDIM, true>; break;            \
    case 6: kernel = attn_fwd_kernel<true, true, false, HDIM, true>; break;            \
    case 7: kernel = attn_fwd_kernel<true, true, true, HDIM, true>; break;             \
    case 8: kernel = attn_fwd_kernel<false, false, false, HDIM, true, true>; break;    \
    case 9: kernel = attn_fwd_kernel<false, false, true, HDIM, true, true>; break;     \
    case 10: kernel = attn_fwd_kernel<false, true, false, HDIM, true, true>; break;    \
    case 11: kernel = attn_fwd_kernel<false, true, true, HDIM, true, true>; break;     \
    case 12: kernel = attn_fwd_kernel<true, false, false, HDIM, true, true>; break;    \
    case 13: kernel = attn_fwd_kernel<true, false, true, HDIM, true, true>; break;     \
    case 14: kernel = attn_fwd_kernel<true, true, false, HDIM, true, true>; break;     \
    default: kernel = attn_fwd_kernel<true, true, true, HDIM, true, true>; break;      \
    }
#define SMA_FWD_PAIRS_VARIANTS(HDIM)                                                    \
    switch (variant | (byproducts ? 8 : 0)) {                                          \
    case 0: kernel = attn_fwd_kernel<false, false, false, HDIM, true, false, true>; break;   \
    case 1: kernel = attn_fwd_kernel<false, false, true, HDIM, true, false, true>; break;    \
    case 2: kernel = attn_fwd_kernel<false, true, false, HDIM, true, false, true>; break;    \
    case 3: kernel = attn_fwd_kernel<false, true, true, HDIM, true, false, true>; break;     \
    case 4: kernel = attn_fwd_kernel<true, false, false, HDIM, true, false, true>; break;    \
    case 5: kernel = attn_fwd_kernel<true, false, true, HDIM, true, false, true>; break;     \
    case 6: kernel = attn_fwd_kernel<true, true, false, HDIM, true, false, true>; break;     \
    case 7: kernel = attn_fwd_kernel<true, true, true, HDIM, true, false, true>; break;      \
    case 8: kernel = attn_fwd_kernel<false, false, false, HDIM, true, true, true>; break;    \
    case 9: kernel = attn_fwd_kernel<false, false, true, HDIM, true, true, true>; break;     \
    case 10: kernel = attn_fwd_kernel<false, true, false, HDIM, true, true, true>; break;    \
    case 11: kernel = attn_fwd_kernel<false, true, true, HDIM, true, true, true>; break;     \
    case 12: kernel = attn_fwd_kernel<true, false, false, HDIM, true, true, true>; break;    \
    case 13: kernel = attn_fwd_kernel<true, false, true, HDIM, true, true, true>; break;     \
    case 14: kernel = attn_fwd_kernel<true, true, false, HDIM, true, true, true>; break;     \
    default: kernel = attn_fwd_kernel<true, true, true, HDIM, true, true, true>; break;      \
    }
    const bool byproducts = a.mask_out != nullptr || a.map_out != nullptr;
    // two tiles' mask bytes per request (see PAIRS at the kernel), unless the grid is the single round
    // of work-groups in step for which tail_start was set to 0 above
    const bool pairs = a.byte_mask && D <= 64 && a.N % (2 * BN) == 0 && a.tail_start != 0;
    if (pairs) {
        if (D == 32) { SMA_FWD_PAIRS_VARIANTS(32) } else { SMA_FWD_PAIRS_VARIANTS(64) }
    } else if (a.byte_mask) {
        if (a.N < 16) return hipErrorInvalidValue;          // a row holds at least one 16-byte copy (checked by the C-ABI layer)
        if (D == 32) { SMA_FWD_BYTEMASK_VARIANTS(32) } else if (D == 64) { SMA_FWD_BYTEMASK_VARIANTS(64) } else { SMA_FWD_BYTEMASK_VARIANTS(128) }
    } else if (D == 32) { SMA_FWD_VARIANTS(32) } else if (D == 64) { SMA_FWD_VARIANTS(64) } else { SMA_FWD_VARIANTS(128) }
#undef SMA_FWD_VARIANTS
#undef SMA_FWD_BYTEMASK_VARIANTS
#undef SMA_FWD_PAIRS_VARIANTS
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, a);
    return hipGetLastError();
}

}  // namespace sma
