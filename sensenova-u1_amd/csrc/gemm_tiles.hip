// Dequant-GEMM, large-tile variant for Q8_0 (K % 64 == 0) and Q4_K - and for weights already decoded to
// bf16 (second pass of the workspace route) in the launches that the four-wavefront dense kernel of
// gemm_dense4.hip does not take (an odd number of K steps per workgroup): 256 x 256 output tile per
// workgroup, K step 64, eight wavefronts of 64 (rows) x 128 (columns) - 2 x 4 MFMA tiles of 32 x 32,
// 128 accumulator registers each, two wavefronts per SIMD - and two LDS stages.
//
// Per K step and workgroup: the 256 x 64 activation tile (32 KB) is copied global -> LDS,
// directly.  The packed bytes a thread needs for its 32 weights of the step are copied global ->
// a small per-wavefront LDS slab, also directly, as three pieces per row: Q8_0 the 36 bytes that
// hold one block and the scale (12-byte pieces); Q4_K the 16-byte super-block head (d, dmin, packed
// sub-scales) and the 32 quant bytes of the step's 64-element chunk (16-byte pieces).  One step
// later each thread picks up its row (wavefronts 0-3 the first 32 elements of the step, 4-7 the
// second: the second Q8_0 block, or the high nibbles of the Q4_K chunk), decodes it to 32 bf16
// with the rounding chain of the numerics mode and writes it to the other LDS stage while the
// matrix cores work on the current one.  Weight rows are the MFMA A operand, activation rows the
// B operand (v_mfma_f32_32x32x16_bf16), so a lane ends up with runs of four consecutive output
// columns of one activation row.
//
// Tiles are numbered so that the workgroups that land on one XCD (workgroup id modulo 8) work on a
// contiguous range of tiles, and within it on blocks of 4 row tiles x 8 column tiles at a time: the
// 32 workgroups that run together on an XCD then share 4 activation tiles and 8 packed weight
// tiles in that XCD's L2.
#include "gemm_args.hpp"
#include "sngguf_common.hpp"

// One scheduling region per 16-wide K slice: the eight matrix instructions of the slice with the
// decode arithmetic of the next step's weights and the fragment reads of the next slice slotted
// between them, so that the vector ALU and LDS work under the matrix cores instead of after them.
#define SNGGUF_INTERLEAVE()                                                  \
    do {                                                                     \
        _Pragma("unroll") for (int m_ = 0; m_ < 8; m_++) {                   \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);               \
            if (m_ < 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   \
            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);               \
        }                                                                    \
        __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);                   \
        __builtin_amdgcn_sched_barrier(0);                                   \
    } while (0)

namespace sngguf {

namespace {

constexpr int TM = 256;      // activation rows per tile
constexpr int TN = 256;      // weight rows (output columns) per tile
constexpr int TK = 64;       // K step
constexpr int kTileBytes = 256 * 64 * 2;          // one operand tile in LDS (rows of 128 bytes, swizzled)
constexpr int kRawDwords = 64 * 12;               // raw slab of one wavefront: 64 rows x 3 pieces of 16 bytes
constexpr int kLdsBytes = 4 * kTileBytes + 8 * kRawDwords * 4;  // two stages of both tiles + raw slabs
constexpr int kTypeBF16 = 30;                     // ggml's id for plain bf16 rows: weights that need no decode

// Q4_K: (D, DM) = (d * sc, dmin * mn) of sub-block j from the super-block head, as the bit pattern
// the decode uses: NUM 1 the fp16 product copied into both halves of a dword, NUM 0 the fp32 product.
template <int NUM>
__device__ __forceinline__ void q4k_sub_block_scales(uint32_t dd, uint32_t s0, uint32_t s1, uint32_t s2, int j,
                                                     uint32_t& D_bits, uint32_t& DM_bits) {
    typedef Num<NUM> A;
    const int i = j & 3;
    const uint32_t lo_sc = (s0 >> (8 * i)) & 63u, lo_mn = (s1 >> (8 * i)) & 63u;
    const uint32_t b = (s2 >> (8 * i)) & 0xFFu;
    const uint32_t hi_sc = (b & 0x0Fu) | (((s0 >> (8 * i + 6)) & 3u) << 4), hi_mn = (b >> 4) | (((s1 >> (8 * i + 6)) & 3u) << 4);
    const uint32_t sc = j < 4 ? lo_sc : hi_sc, mn = j < 4 ? lo_mn : hi_mn;
    const typename A::T D = A::scale((uint16_t)(dd & 0xFFFF)) * A::integer((int)sc);
    const typename A::T DM = A::scale((uint16_t)(dd >> 16)) * A::integer((int)mn);
    if constexpr (NUM == SNGGUF_NUM_UPSTREAM_FP16) {
        const uint32_t Dh = __builtin_bit_cast(uint16_t, D), Mh = __builtin_bit_cast(uint16_t, DM);
        D_bits = Dh | (Dh << 16);
        DM_bits = Mh | (Mh << 16);
    } else {
        D_bits = __builtin_bit_cast(uint32_t, D);
        DM_bits = __builtin_bit_cast(uint32_t, DM);
    }
}

// Four 4-bit quants (one per byte of v) -> q * D - DM as two packed bf16 pairs; NUM 1 rounds to fp16
// after the product and after the subtraction, NUM 0 works in fp32 (both products exact).
template <int NUM>
__device__ __forceinline__ void q4k_dword_bf16(uint32_t D_bits, uint32_t DM_bits, uint32_t v, uint32_t& p01, uint32_t& p23) {
    // 0x6400 | n is the half 1024 + n
    const half2_t k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
    const half2_t q01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u)) - k1024;
    const half2_t q23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u)) - k1024;
    if constexpr (NUM == SNGGUF_NUM_UPSTREAM_FP16) {
        const half2_t D2 = __builtin_bit_cast(half2_t, D_bits), M2 = __builtin_bit_cast(half2_t, DM_bits);
        const half2_t a = q01 * D2 - M2, b = q23 * D2 - M2;   // two roundings each (no contraction)
        p01 = pack_bf16((float)a[0], (float)a[1]);
        p23 = pack_bf16((float)b[0], (float)b[1]);
    } else {
        const float D = __builtin_bit_cast(float, D_bits), DM = __builtin_bit_cast(float, DM_bits);
        p01 = pack_bf16(D * (float)q01[0] - DM, D * (float)q01[1] - DM);
        p23 = pack_bf16(D * (float)q23[0] - DM, D * (float)q23[1] - DM);
    }
}

// A pointer that is the same in all lanes, pinned to scalar registers: the loop optimiser cannot fold it into
// per-lane 64-bit induction variables, and the request uses the scalar-base + 32-bit-offset address form.
__device__ __forceinline__ const uint8_t* scalar_ptr(const void* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const uint8_t*>(((uint64_t)hi << 32) | lo);
}

template <int QT, int NUM>
__global__ __launch_bounds__(512) void gemm_tile_kernel(GemmArgs a) {
    constexpr bool kQ4K = QT == SNGGUF_TYPE_Q4_K;
    constexpr bool kDense = QT == kTypeBF16;  // weights already bf16 [N][K]: both operand tiles are plain copies
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    // the wavefront index is the same in all lanes: holding it in a scalar register keeps every address derived
    // from it (LDS slabs, tile rows) in scalar arithmetic
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;  // 4 x 2 wavefronts: rows wm * 64, columns wn * 128

    // ---- tile of this workgroup ---------------------------------------------------------------------
    const int64_t n0 = a.n0_dev ? (int64_t)*a.n0_dev : a.n0;
    const int64_t t0 = (a.group_mask & 1) ? (n0 + TM - 1) / TM : 0;            // row tiles of group 0
    const int64_t t1 = (a.group_mask & 2) ? (a.M - n0 + TM - 1) / TM : 0;      // row tiles of group 1
    const int64_t ntn = (a.N + TN - 1) / TN;
    const int S = a.ksplit > 1 ? a.ksplit : 1;                                 // workgroups per output tile (K slices)
    const int64_t total = (t0 + t1) * ntn * S;
    const int64_t pid = blockIdx.x;
    if (pid >= total) return;
    // consecutive tile numbers on one XCD: workgroup ids are dealt round-robin over 8 XCDs
    const int64_t per = total >> 3, rem = total & 7;
    const int64_t xcd = pid & 7, idx = pid >> 3;
    const int64_t tile_slice = xcd * per + (xcd < rem ? xcd : rem) + idx;
    const int64_t tile = tile_slice / S;
    const int slice = (int)(tile_slice - tile * S);
    // The 32 workgroups that run at the same time on one XCD cover a block of 4 row tiles x 8 column
    // tiles when the tile grid divides that way (4 activation tiles + 8 packed weight tiles pass
    // through the XCD's L2 per block instead of 1 + 32), else 32 consecutive column tiles of one row.
    int64_t ty, tn;
    constexpr int BY = 4, BX = 8;
    if ((ntn % BX) == 0 && ((t0 + t1) % BY) == 0) {
        const int64_t blk = tile >> 5, within = tile & 31, bpr = ntn / BX;   // blocks per block row
        ty = (blk / bpr) * BY + (within / BX);
        tn = (blk % bpr) * BX + (within % BX);
    } else {
        ty = tile / ntn;
        tn = tile - ty * ntn;
    }
    int g;
    int64_t row_begin, row_end;
    if (ty < t0) {
        g = 0; row_begin = ty * TM; row_end = n0;
    } else {
        g = 1; row_begin = n0 + (ty - t0) * TM; row_end = a.M;
    }
    if (row_end > row_begin + TM) row_end = row_begin + TM;
    const uint8_t* __restrict__ q = a.q[g];
    const bf16_t* __restrict__ bias = a.bias[g];
    const int64_t nb0 = tn * TN;
    const int64_t row_bytes = kDense ? 2 * a.K : kQ4K ? (a.K >> 8) * 144 : (a.K >> 5) * 34;
    // this workgroup's K steps: [ks0, ks0 + ksteps) of the K / 64 in all (everything when K is not split)
    const int ksteps_all = (int)(a.K / TK);
    const int ks0 = (int)((int64_t)slice * ksteps_all / S);
    const int ksteps = (int)((int64_t)(slice + 1) * ksteps_all / S) - ks0;

    // ---- LDS: two stages of (activation tile, weight tile) + one raw-weight slab per wavefront ------------
    // A tile is 256 rows of 64 bf16 (128 bytes, no padding); the eight 16-byte chunks of a row are
    // stored at chunk ^ ((row / 2) % 8): two consecutive rows cover all 64 banks, so sixteen
    // consecutive rows at one logical chunk fall into sixteen different 16-byte bank groups and both
    // the fragment reads and the row-wise writes run without conflicts (swizzling by row % 8 leaves
    // rows r and r + 8 on the same banks and halves the ds_read_b128 rate).
    bf16_t* xs[2] = {reinterpret_cast<bf16_t*>(lds), reinterpret_cast<bf16_t*>(lds + 2 * kTileBytes)};
    bf16_t* ws[2] = {reinterpret_cast<bf16_t*>(lds + kTileBytes), reinterpret_cast<bf16_t*>(lds + 3 * kTileBytes)};
    uint32_t* raw = reinterpret_cast<uint32_t*>(lds + 4 * kTileBytes) + wave * kRawDwords;

    // ---- per-thread assignments ---------------------------------------------------------------------------
    // activations: 256 rows x 8 pieces of 16 bytes, copied global -> LDS directly
    // (global_load_lds_dwordx4: lane l of a wavefront writes LDS bytes [16 l, +16) after a uniform
    // base, so one instruction fills eight consecutive 128-byte tile rows).  Instruction i of
    // wavefront w covers rows 64 i + 8 w .. + 7; the lane that fills physical chunk p of row r
    // fetches logical chunk p ^ ((r / 2) % 8), i.e. the swizzle is applied on the global side.
    // Rows past the end of the group re-read the group's last row: they only feed output rows
    // that are never stored.
    // Sources are kept as 32-bit byte offsets from a.x (the launcher routes problems with 2 M K >= 2^32 bytes to
    // the 128-tile kernel): with the K-step part of the address in scalar registers a request needs no vector
    // arithmetic.
    uint32_t xoff[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int64_t rr = row_begin + (tid >> 3) + 64 * i;
        if (rr >= row_end) rr = row_end - 1;
        const int64_t gr = a.rowmap ? (int64_t)a.rowmap[rr] : rr;
        xoff[i] = (uint32_t)(2 * (gr * a.K + 8 * ((tid & 7) ^ ((tid >> 4) & 7))));
    }
    const int xrow0 = 8 * wave;  // first tile row this wavefront fills with instruction 0 (+ 64 i)
    // dense weights: the weight tile is filled the same way, from rows nb0 .. nb0 + 255 of q
    uint32_t woff[4] = {0, 0, 0, 0};
    if constexpr (kDense) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int64_t n = (tid >> 3) + 64 * i;                 // row of the tile
            if (nb0 + n >= a.N) n = a.N - 1 - nb0;           // rows past the end re-read the last row
            woff[i] = (uint32_t)(2 * (n * a.K + 8 * ((tid & 7) ^ ((tid >> 4) & 7))));
        }
    }
    // weights: wavefront w decodes elements 32 `wblk` .. + 31 (wblk = w / 4) of the K step for rows
    // 64 (w % 4) .. + 63, one row per lane.  The bytes it needs are fetched as three pieces per row,
    // consecutive lanes walking along a row (3 lanes per row), into the wavefront's raw slab and
    // picked up row-wise one step later.  Q8_0: 12-byte pieces of the 36 bytes that hold the block
    // and its scale.  Q4_K: piece 0 is the super-block head, pieces 1 and 2 the 32 quant bytes of the
    // step's chunk; the head moves every fourth step, the quants every step.
    const int wblk = wave >> 2;
    const int wrow_l = 64 * (wave & 3) + lane;  // row of the tile this lane decodes
    uint32_t goff[3];
    bool head_piece[3];
#pragma unroll
    for (int i = 0; i < 3; i++) {
        const int f = lane + 64 * i, fr = f / 3, fj = f - 3 * fr;  // piece fj of slab row fr
        int64_t n = nb0 + 64 * (wave & 3) + fr;
        if (n >= a.N) n = a.N - 1;
        head_piece[i] = fj == 0;
        goff[i] = kQ4K ? (uint32_t)((n - nb0) * row_bytes + 16 * fj) : (uint32_t)((n - nb0) * row_bytes + 32 * wblk + 12 * fj);
    }
    const uint8_t* __restrict__ wbase = q + nb0 * row_bytes;
    const int wsw = (wrow_l >> 1) & 7;
    // v_perm_b32 selectors (bytes 0-3 = second operand, 4-7 = first operand)
    const uint32_t sel_q = wblk ? 0x07060504u : 0x05040302u;  // quant dword: next dword as is / 2 bytes off
    const uint32_t sel_d = wblk ? 0x03020302u : 0x01000100u;  // block scale copied into both halves
    const int nib_shift = 4 * wblk;                           // Q4_K: low or high nibbles
    bf16_t* wdst[2] = {ws[0] + wrow_l * 64, ws[1] + wrow_l * 64};

    // fragment reads: row (lane % 32) of a 32-row tile, logical chunk 2 ks + lane / 32
    int foff[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) foff[ks] = (lane & 31) * 64 + 8 * ((2 * ks + (lane >> 5)) ^ ((lane >> 1) & 7));

    f32x16_t acc[4][2];  // [column tile i][row tile j]
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    uint32_t rw[12];  // this lane's pieces, read back from the raw slab (Q8_0 uses 9 dwords)

// One global -> LDS copy request written as the instruction itself: uniform 64-bit base in scalar registers + this
// lane's 32-bit byte offset, LDS destination base in M0 (one wait state between the scalar write of M0 and the request
// that reads it).  The builtin gets a 64-bit address per lane and a 64-bit vector add in front of it; the dense form
// is 7 % faster with this one.  The compiler does not count these requests: every use below is followed by an explicit
// s_waitcnt vmcnt(0) before the data is read.
#define SNGGUF_ASM_COPY(INSN, ldsptr_, voff_, sbase_)                                                         \
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t" INSN " %1, %2"                                           \
                 :: "s"((uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)(ldsptr_)), "v"(voff_), "s"(sbase_) : "memory", "m0")
// global -> raw slab, directly: lane l writes its piece into the 16-byte slot l after a uniform base
// (a 12-byte piece leaves the slot's last dword unwritten); three slots make one row of the slab.
// Pieces [I0, I1) of step kb.
#define SNGGUF_FETCH_W(kb, I0, I1)                                                                           \
    do {                                                                                                     \
        if constexpr (kQ4K) {                                                                                \
            const uint8_t* ph_ = scalar_ptr(wbase + (int64_t)(((kb) + ks0) >> 2) * 144);                     \
            const uint8_t* pq_ = ph_ + 32 * (((kb) + ks0) & 3);                                              \
            _Pragma("unroll") for (int i_ = (I0); i_ < (I1); i_++)                                           \
                __builtin_amdgcn_global_load_lds(                                                            \
                    (const __attribute__((address_space(1))) void*)((head_piece[i_] ? ph_ : pq_) + goff[i_]),\
                    (__attribute__((address_space(3))) void*)(raw + 256 * i_), 16, 0, 0);                    \
        } else {                                                                                             \
            const uint8_t* p_ = scalar_ptr(wbase + (int64_t)((kb) + ks0) * 68);                              \
            _Pragma("unroll") for (int i_ = (I0); i_ < (I1); i_++)                                           \
                SNGGUF_ASM_COPY("global_load_lds_dwordx3", raw + 256 * i_, goff[i_], p_);                    \
        }                                                                                                    \
    } while (0)
#define SNGGUF_PICK_W()                                                                                      \
    do {                                                                                                     \
        if constexpr (kQ4K) {                                                                                \
            _Pragma("unroll") for (int i_ = 0; i_ < 12; i_++) rw[i_] = raw[12 * lane + i_];                  \
        } else {                                                                                             \
            _Pragma("unroll") for (int i_ = 0; i_ < 9; i_++) rw[i_] = raw[12 * lane + 4 * (i_ / 3) + i_ % 3]; \
        }                                                                                                    \
    } while (0)
#define SNGGUF_LOAD_X(kb, stage, I0, I1)                                                                     \
    do {                                                                                                     \
        const uint8_t* xb_ = scalar_ptr(a.x + (int64_t)((kb) + ks0) * TK);                                   \
        _Pragma("unroll") for (int i_ = (I0); i_ < (I1); i_++)                                               \
            SNGGUF_ASM_COPY("global_load_lds_dwordx4", xs[stage] + (xrow0 + 64 * i_) * 64, xoff[i_], xb_);   \
    } while (0)
#define SNGGUF_LOAD_WD(kb, stage, I0, I1)                                                                    \
    do {                                                                                                     \
        const uint8_t* wb_ = scalar_ptr(wbase + (int64_t)((kb) + ks0) * (2 * TK));                           \
        _Pragma("unroll") for (int i_ = (I0); i_ < (I1); i_++)                                               \
            SNGGUF_ASM_COPY("global_load_lds_dwordx4", ws[stage] + (xrow0 + 64 * i_) * 64, woff[i_], wb_);   \
    } while (0)
// Scales of the 32 elements this thread decodes out of rw (the pieces of step kbn): Q8_0 the block
// scale copied into both halves of sc_a (first block of a pair: low half of dword 0, second: high
// half); Q4_K (D, DM) of sub-block 2 (kbn % 4) + wblk.
#define SNGGUF_SCALES_W(kbn)                                                                                 \
    do {                                                                                                     \
        if constexpr (kQ4K) q4k_sub_block_scales<NUM>(rw[0], rw[1], rw[2], rw[3], 2 * (((kbn) + ks0) & 3) + wblk, sc_a, sc_b); \
        else sc_a = __builtin_amdgcn_perm(rw[0], rw[0], sel_d);                                              \
    } while (0)
// decode quarter `part` (8 elements) of this thread's 32 into LDS.  Q8_0: quant dwords 2 part,
// 2 part + 1 of the block - for the first block of a pair they start 2 bytes into dword 0, for the
// second at dword 1; one v_perm_b32 per dword with a per-wavefront byte selector covers both cases
// without a branch.  Q4_K: the low (wblk 0) or high (wblk 1) nibbles of quant bytes 8 part .. + 7.
#define SNGGUF_DECODE_W(stage, part)                                                                         \
    do {                                                                                                     \
        uint32_t o0_, o1_, o2_, o3_;                                                                         \
        if constexpr (kQ4K) {                                                                                \
            const uint32_t v0_ = (rw[4 + 2 * (part)] >> nib_shift) & 0x0F0F0F0Fu;                            \
            const uint32_t v1_ = (rw[5 + 2 * (part)] >> nib_shift) & 0x0F0F0F0Fu;                            \
            q4k_dword_bf16<NUM>(sc_a, sc_b, v0_, o0_, o1_);                                                  \
            q4k_dword_bf16<NUM>(sc_a, sc_b, v1_, o2_, o3_);                                                  \
        } else {                                                                                             \
            const uint32_t q0_ = __builtin_amdgcn_perm(rw[1 + 2 * (part)], rw[2 * (part)], sel_q);           \
            const uint32_t q1_ = __builtin_amdgcn_perm(rw[2 + 2 * (part)], rw[1 + 2 * (part)], sel_q);       \
            q8_dword_bf16_d2<NUM>(sc_a, q0_, o0_, o1_);                                                      \
            q8_dword_bf16_d2<NUM>(sc_a, q1_, o2_, o3_);                                                      \
        }                                                                                                    \
        *reinterpret_cast<u32x4_t*>(wdst[stage] + 8 * ((4 * wblk + (part)) ^ wsw)) = u32x4_t{o0_, o1_, o2_, o3_}; \
    } while (0)
// One K step on LDS stage CUR.  On entry the raw slab holds the packed blocks of step kb + 1: they
// are picked up (NEXT) and decoded into the other stage while the MFMAs run; once picked up, the
// slab is refilled with the blocks of step kb + 2 (FETCH), and the other stage's activation tile
// with that of step kb + 1.  Global requests are spread over the MFMA slices instead of being
// issued in one burst: a burst from all eight wavefronts right after the barrier fills the
// address pipeline and holds every wavefront - and with it the matrix cores - at its next request.
#define SNGGUF_K_STEP(kb, CUR, NEXT, FETCH)                                                                  \
    do {                                                                                                     \
        const bf16_t* a_base_ = ws[CUR] + wn * 128 * 64;                                                     \
        const bf16_t* b_base_ = xs[CUR] + wm * 64 * 64;                                                      \
        bf16x8_t af_[2][4], bf_[2][2];  /* fragments of this 16-wide K slice and of the next one */          \
        _Pragma("unroll") for (int i = 0; i < 4; i++)                                                        \
            af_[0][i] = *reinterpret_cast<const bf16x8_t*>(a_base_ + i * 32 * 64 + foff[0]);                 \
        _Pragma("unroll") for (int j = 0; j < 2; j++)                                                        \
            bf_[0][j] = *reinterpret_cast<const bf16x8_t*>(b_base_ + j * 32 * 64 + foff[0]);                 \
        if (NEXT) SNGGUF_PICK_W();                                                                           \
        /* The slab is refilled during this step: its reads must not sink below this point (the  */          \
        /* scheduler is otherwise free to delay the dwords that are decoded last).                */          \
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                   \
        uint32_t sc_a = 0, sc_b = 0;                                                                         \
        if (NEXT) SNGGUF_SCALES_W((kb) + 1);                                                                 \
        _Pragma("unroll") for (int ks = 0; ks < 4; ks++) {                                                   \
            if (ks < 3) {                                                                                    \
                _Pragma("unroll") for (int i = 0; i < 4; i++)                                                \
                    af_[(ks + 1) & 1][i] =                                                                   \
                        *reinterpret_cast<const bf16x8_t*>(a_base_ + i * 32 * 64 + foff[(ks + 1) & 3]);      \
                _Pragma("unroll") for (int j = 0; j < 2; j++)                                                \
                    bf_[(ks + 1) & 1][j] =                                                                   \
                        *reinterpret_cast<const bf16x8_t*>(b_base_ + j * 32 * 64 + foff[(ks + 1) & 3]);      \
            }                                                                                                \
            _Pragma("unroll") for (int i = 0; i < 4; i++)                                                    \
                _Pragma("unroll") for (int j = 0; j < 2; j++)                                                \
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af_[ks & 1][i], bf_[ks & 1][j],      \
                                                                        acc[i][j], 0, 0, 0);                 \
            if (FETCH) {                                                                                     \
                if (ks == 0) SNGGUF_FETCH_W((kb) + 2, 0, 2);                                                 \
                if (ks == 1) SNGGUF_FETCH_W((kb) + 2, 2, 3);                                                 \
            }                                                                                                \
            if (NEXT) {                                                                                      \
                if (ks == 1) SNGGUF_LOAD_X((kb) + 1, (CUR) ^ 1, 0, 1);                                       \
                if (ks == 2) SNGGUF_LOAD_X((kb) + 1, (CUR) ^ 1, 1, 3);                                       \
                if (ks == 3) SNGGUF_LOAD_X((kb) + 1, (CUR) ^ 1, 3, 4);                                       \
            }                                                                                                \
            if (NEXT) SNGGUF_DECODE_W((CUR) ^ 1, ks);                                                        \
            SNGGUF_INTERLEAVE();                                                                             \
        }                                                                                                    \
        /* the next activation tile and the next raw blocks must have landed in LDS */                      \
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                     \
        __syncthreads();                                                                                     \
    } while (0)

// Dense weights (plain bf16 rows): the same tile loop without the decode stage.  The workgroup's one barrier per
// step sits in front of the LAST 16-wide slice: by then every wavefront holds the fragments of that slice in
// registers, so stage CUR is free, and the copies into the other stage - requested a whole step earlier, behind
// the previous barrier - have had a step's worth of matrix work to arrive.  The copies of step kb + 2 go into stage
// CUR behind the barrier, half of them at once, half in the first slice of the next step; the fragments of the next
// step's first slice are read there too (its stage has just been declared complete), so a step starts with its
// operands in registers.
#define SNGGUF_INTERLEAVE_DENSE()                                            \
    do {                                                                     \
        _Pragma("unroll") for (int m_ = 0; m_ < 8; m_++) {                   \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);               \
            if (m_ < 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   \
        }                                                                    \
        __builtin_amdgcn_sched_barrier(0);                                   \
    } while (0)
#define SNGGUF_FRAGS_DENSE(stage, ks_, buf)                                                                  \
    do {                                                                                                     \
        const bf16_t* a_base_ = ws[stage] + wn * 128 * 64;                                                   \
        const bf16_t* b_base_ = xs[stage] + wm * 64 * 64;                                                    \
        _Pragma("unroll") for (int i = 0; i < 4; i++)                                                        \
            daf_[buf][i] = *reinterpret_cast<const bf16x8_t*>(a_base_ + i * 32 * 64 + foff[ks_]);            \
        _Pragma("unroll") for (int j = 0; j < 2; j++)                                                        \
            dbf_[buf][j] = *reinterpret_cast<const bf16x8_t*>(b_base_ + j * 32 * 64 + foff[ks_]);            \
    } while (0)
#define SNGGUF_K_STEP_DENSE(kb, CUR, NEXT, FETCH)                                                            \
    do {                                                                                                     \
        _Pragma("unroll") for (int ks = 0; ks < 4; ks++) {                                                   \
            if (ks < 3) SNGGUF_FRAGS_DENSE(CUR, ks + 1, (ks + 1) & 1);                                       \
            if (ks == 0 && (NEXT)) {                                                                         \
                SNGGUF_LOAD_WD((kb) + 1, (CUR) ^ 1, 2, 4);                                                   \
                SNGGUF_LOAD_X((kb) + 1, (CUR) ^ 1, 2, 4);                                                    \
            }                                                                                                \
            if (ks == 3) {                                                                                   \
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");                                  \
                __syncthreads();                                                                             \
                if (NEXT) SNGGUF_FRAGS_DENSE((CUR) ^ 1, 0, 0);                                               \
                if (FETCH) {                                                                                 \
                    SNGGUF_LOAD_WD((kb) + 2, CUR, 0, 2);                                                     \
                    SNGGUF_LOAD_X((kb) + 2, CUR, 0, 2);                                                      \
                }                                                                                            \
            }                                                                                                \
            _Pragma("unroll") for (int i = 0; i < 4; i++)                                                    \
                _Pragma("unroll") for (int j = 0; j < 2; j++)                                                \
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(daf_[ks & 1][i], dbf_[ks & 1][j],    \
                                                                        acc[i][j], 0, 0, 0);                 \
            SNGGUF_INTERLEAVE_DENSE();                                                                       \
        }                                                                                                    \
    } while (0)

    if constexpr (kDense) {
        bf16x8_t daf_[2][4], dbf_[2][2];
        SNGGUF_LOAD_X(0, 0, 0, 4);
        SNGGUF_LOAD_WD(0, 0, 0, 4);
        if (ksteps > 1) {
            SNGGUF_LOAD_X(1, 1, 0, 2);
            SNGGUF_LOAD_WD(1, 1, 0, 2);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        SNGGUF_FRAGS_DENSE(0, 0, 0);
        int kd = 0;
        for (; kd + 3 < ksteps; kd += 2) {
            SNGGUF_K_STEP_DENSE(kd, 0, true, true);
            SNGGUF_K_STEP_DENSE(kd + 1, 1, true, true);
        }
        for (; kd < ksteps; kd += 2) {
            SNGGUF_K_STEP_DENSE(kd, 0, kd + 1 < ksteps, kd + 2 < ksteps);
            if (kd + 1 < ksteps) SNGGUF_K_STEP_DENSE(kd + 1, 1, kd + 2 < ksteps, kd + 3 < ksteps);
        }
    } else {
    // ---- prologue: stage 0 holds K step 0, the raw slab step 1 ------------------------------------------------
    SNGGUF_LOAD_X(0, 0, 0, 4);
    SNGGUF_FETCH_W(0, 0, 3);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    SNGGUF_PICK_W();
    {
        uint32_t sc_a = 0, sc_b = 0;
        SNGGUF_SCALES_W(0);
#pragma unroll
        for (int part = 0; part < 4; part++) SNGGUF_DECODE_W(0, part);
    }
    if (ksteps > 1) SNGGUF_FETCH_W(1, 0, 3);  // after the pick-up: the slab is free again
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    int kb = 0;
    // steady state: both flags are known, so every K slice is one straight-line region in which
    // the decode arithmetic can be slotted between the matrix instructions
    for (; kb + 3 < ksteps; kb += 2) {
        SNGGUF_K_STEP(kb, 0, true, true);
        SNGGUF_K_STEP(kb + 1, 1, true, true);
    }
    for (; kb < ksteps; kb += 2) {
        {
            const bool next = kb + 1 < ksteps, fetch = kb + 2 < ksteps;
            SNGGUF_K_STEP(kb, 0, next, fetch);
        }
        if (kb + 1 < ksteps) {
            const bool next = kb + 2 < ksteps, fetch = kb + 3 < ksteps;
            SNGGUF_K_STEP(kb + 1, 1, next, fetch);
        }
    }
    }  // quantized weights
#undef SNGGUF_K_STEP
#undef SNGGUF_K_STEP_DENSE
#undef SNGGUF_FRAGS_DENSE
#undef SNGGUF_INTERLEAVE_DENSE
#undef SNGGUF_LOAD_WD
#undef SNGGUF_INTERLEAVE
#undef SNGGUF_DECODE_W
#undef SNGGUF_SCALES_W
#undef SNGGUF_LOAD_X
#undef SNGGUF_PICK_W
#undef SNGGUF_FETCH_W

    // ---- epilogue: D[i][j], i = weight row (n), j = activation row (m) ----------------------------------------
    // lane: j = lane % 32; register v: i = 8 * (v / 4) + 4 * (lane / 32) + v % 4
    if (a.partial) {
        // K split over workgroups: this slice's sums go out as fp32, to be added up by splitk_reduce_kernel
        float* part = a.partial + (int64_t)slice * a.M * a.N;
        const bool vec = (a.N & 3) == 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int vg = 0; vg < 4; vg++) {
                const int64_t n = nb0 + wn * 128 + i * 32 + 8 * vg + 4 * (lane >> 5);
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const int64_t rr = row_begin + wm * 64 + j * 32 + (lane & 31);
                    if (rr >= row_end || n >= a.N) continue;
                    const int64_t gr = a.rowmap ? (int64_t)a.rowmap[rr] : rr;
                    float* pp = part + gr * a.N + n;
                    if (vec) {
                        *reinterpret_cast<f32x4_t*>(pp) = f32x4_t{acc[i][j][4 * vg], acc[i][j][4 * vg + 1], acc[i][j][4 * vg + 2], acc[i][j][4 * vg + 3]};
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (n + e < a.N) pp[e] = acc[i][j][4 * vg + e];
                    }
                }
            }
        }
        return;
    }
    if ((a.N & 7) == 0) {
        // Rows of y are 16-byte aligned: stage the tile in LDS as bf16 [256 m][256 n] (all K-loop
        // buffers are dead after the last barrier) and write it out as 16-byte pieces, 32 lanes
        // along one output row, so that every store instruction fills whole lines.  Storing
        // straight from the accumulator layout would scatter 8-byte pieces over 32 rows.
        constexpr int kYRow = 2 * TN + 16;  // bytes; the padding spreads rows over the banks
        static_assert(TM * kYRow <= kLdsBytes, "output tile must fit the K-loop buffers");
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int vg = 0; vg < 4; vg++) {
                const int nl = wn * 128 + i * 32 + 8 * vg + 4 * (lane >> 5);
                float b[4] = {0.f, 0.f, 0.f, 0.f};
                if (bias && nb0 + nl < a.N) {
#pragma unroll
                    for (int e = 0; e < 4; e++) b[e] = bf16_to_f32(bias[nb0 + nl + e]);
                }
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const int ml = wm * 64 + j * 32 + (lane & 31);
                    *reinterpret_cast<u32x2_t*>(lds + ml * kYRow + 2 * nl) =
                        u32x2_t{pack_bf16(acc[i][j][4 * vg] + b[0], acc[i][j][4 * vg + 1] + b[1]),
                                pack_bf16(acc[i][j][4 * vg + 2] + b[2], acc[i][j][4 * vg + 3] + b[3])};
                }
            }
        }
        __syncthreads();
        const int64_t n = nb0 + 8 * (tid & 31);
        if (n >= a.N) return;
#pragma unroll 4
        for (int p = 0; p < TM / 16; p++) {
            const int ml = (tid >> 5) + 16 * p;
            const int64_t rr = row_begin + ml;
            if (rr >= row_end) break;
            const int64_t gr = a.rowmap ? (int64_t)a.rowmap[rr] : rr;
            u32x4_t o = *reinterpret_cast<const u32x4_t*>(lds + ml * kYRow + 16 * (tid & 31));
            if (a.residual) {
                // the staged values are the rounded projection outputs: add the residual row and round again
                const u32x4_t rs = *reinterpret_cast<const u32x4_t*>(a.residual + gr * a.N + n);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    o[e] = pack_bf16(bf16lo_to_f32(rs[e]) + bf16lo_to_f32(o[e]), bf16hi_to_f32(rs[e]) + bf16hi_to_f32(o[e]));
            }
            __builtin_nontemporal_store(o, reinterpret_cast<u32x4_t*>(a.y + gr * a.N + n));   // (see gemm_dense4.hip)
        }
        return;
    }
    const bool fast = (a.N & 3) == 0;  // rows of y are 8-byte aligned and a run of four columns never straddles N
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int vg = 0; vg < 4; vg++) {
            const int64_t n = nb0 + wn * 128 + i * 32 + 8 * vg + 4 * (lane >> 5);
            float b[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias) {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < a.N) b[e] = bf16_to_f32(bias[n + e]);
            }
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int64_t rr = row_begin + wm * 64 + j * 32 + (lane & 31);
                if (rr >= row_end || n >= a.N) continue;
                const int64_t gr = a.rowmap ? (int64_t)a.rowmap[rr] : rr;
                bf16_t* yp = a.y + gr * a.N + n;
                const int64_t yi = gr * a.N + n;
                const float o0 = add_residual(acc[i][j][4 * vg] + b[0], a.residual, yi);
                const float o1 = n + 1 < a.N ? add_residual(acc[i][j][4 * vg + 1] + b[1], a.residual, yi + 1) : 0.f;
                const float o2 = n + 2 < a.N ? add_residual(acc[i][j][4 * vg + 2] + b[2], a.residual, yi + 2) : 0.f;
                const float o3 = n + 3 < a.N ? add_residual(acc[i][j][4 * vg + 3] + b[3], a.residual, yi + 3) : 0.f;
                if (fast) {
                    *reinterpret_cast<u32x2_t*>(yp) = u32x2_t{pack_bf16(o0, o1), pack_bf16(o2, o3)};
                } else {
                    yp[0] = f32_to_bf16(o0);
                    if (n + 1 < a.N) yp[1] = f32_to_bf16(o1);
                    if (n + 2 < a.N) yp[2] = f32_to_bf16(o2);
                    if (n + 3 < a.N) yp[3] = f32_to_bf16(o3);
                }
            }
        }
    }
}

template <int QT, int NUM>
int launch_tiles(const GemmArgs& a, hipStream_t stream) {
    // 152 KB of dynamic LDS: above the default limit, so it is requested once per kernel
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tile_kernel<QT, NUM>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (attr != hipSuccess) return SNGGUF_E_LAUNCH;
    const int64_t row_tiles = (a.M + TM - 1) / TM + 1;  // a split adds at most one partial tile
    const int64_t ntn = (a.N + TN - 1) / TN;
    const int64_t slices = a.ksplit > 1 ? a.ksplit : 1;
    gemm_tile_kernel<QT, NUM><<<dim3((unsigned)(row_tiles * ntn * slices)), dim3(512), kLdsBytes, stream>>>(a);
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

// y[m][n] = bf16(sum over slices of partial[s][m][n] + bias_g[n]), slices added in ascending order; one thread per
// four consecutive outputs.  Row m belongs to group 1 (bias1) when indicator[m] != 0, or without an indicator when
// m >= n_text.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int slices, int64_t M, int64_t N,
                                                            const uint8_t* __restrict__ indicator, int64_t n_text,
                                                            const bf16_t* __restrict__ bias0, const bf16_t* __restrict__ bias1,
                                                            bf16_t* __restrict__ y) {
    const int64_t total = M * N;
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i0 >= total) return;
    auto bias_of = [&](int64_t m) { return (indicator ? indicator[m] != 0 : m >= n_text) ? bias1 : bias0; };
    if ((N & 3) == 0) {
        f32x4_t s = *reinterpret_cast<const f32x4_t*>(partial + i0);
        for (int k = 1; k < slices; k++) {
            const f32x4_t t = *reinterpret_cast<const f32x4_t*>(partial + (int64_t)k * total + i0);
            s[0] += t[0]; s[1] += t[1]; s[2] += t[2]; s[3] += t[3];
        }
        const int64_t m = i0 / N, n = i0 - m * N;
        const bf16_t* bias = bias_of(m);
        if (bias) {
#pragma unroll
            for (int e = 0; e < 4; e++) s[e] += bf16_to_f32(bias[n + e]);
        }
        *reinterpret_cast<u32x2_t*>(y + i0) = u32x2_t{pack_bf16(s[0], s[1]), pack_bf16(s[2], s[3])};
    } else {
        for (int e = 0; e < 4 && i0 + e < total; e++) {
            float s = partial[i0 + e];
            for (int k = 1; k < slices; k++) s += partial[(int64_t)k * total + i0 + e];
            const int64_t m = (i0 + e) / N;
            const bf16_t* bias = bias_of(m);
            if (bias) s += bf16_to_f32(bias[(i0 + e) - m * N]);
            y[i0 + e] = f32_to_bf16(s);
        }
    }
}

}  // namespace

int launch_gemm_dense4(const GemmArgs& a, hipStream_t stream);

// Q8_0 with K % 64 == 0 (rows are then 4-byte aligned), Q4_K, or type 30 = weights that are already bf16 rows
// (K % 64 == 0; the numerics mode plays no role); both row groups of that type.
int launch_gemm_tiles(const GemmArgs& a, int qtype, int numerics, hipStream_t stream) {
#define SNGGUF_CASE(QT, NUM) if (qtype == QT && numerics == NUM) return launch_tiles<QT, NUM>(a, stream)
    SNGGUF_CASE(SNGGUF_TYPE_Q8_0, SNGGUF_NUM_GGML_FP32);
    SNGGUF_CASE(SNGGUF_TYPE_Q8_0, SNGGUF_NUM_UPSTREAM_FP16);
    SNGGUF_CASE(SNGGUF_TYPE_Q4_K, SNGGUF_NUM_GGML_FP32);
    SNGGUF_CASE(SNGGUF_TYPE_Q4_K, SNGGUF_NUM_UPSTREAM_FP16);
    if (qtype == kTypeBF16) {
        // the four-wavefront form takes every launch whose workgroups get an even number of K steps (its loop has
        // one body for a pair of steps); the dense form of the tile kernel above keeps the rest
        const int64_t S = a.ksplit > 1 ? a.ksplit : 1;
        if ((a.K / TK) % (2 * S) == 0) return launch_gemm_dense4(a, stream);
        return launch_tiles<kTypeBF16, SNGGUF_NUM_GGML_FP32>(a, stream);
    }
#undef SNGGUF_CASE
    return SNGGUF_E_BADTYPE;
}

// The partial sums of a launch with a.ksplit > 1 -> a.y (+ the bias of each row's group: group 1 where indicator[m] != 0,
// or from row n_text on without an indicator).
int launch_splitk_reduce(const GemmArgs& a, const uint8_t* indicator, int64_t n_text, hipStream_t stream) {
    const int64_t quads = (a.M * a.N + 3) / 4;
    splitk_reduce_kernel<<<dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream>>>(a.partial, a.ksplit, a.M, a.N, indicator, n_text,
                                                                                          a.bias[0], a.bias[1], a.y);
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

}  // namespace sngguf
