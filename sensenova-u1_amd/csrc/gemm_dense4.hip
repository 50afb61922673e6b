// Dense bf16 GEMM for weights that are already bf16 rows (the second pass of the workspace routes, and plain BF16
// tensors), four-wavefront form: 256 x 256 output tile per workgroup, K step 64, four wavefronts of 128 (rows) x 128
// (columns) - 8 x 8 MFMA tiles of 16 x 16 (x 32 of K), 256 accumulator registers each, one wavefront per SIMD - and
// two LDS stages of 64 KB.  (The 32 x 32 x 16 instruction, with the same tile, the same copies and bit-equal sums,
// runs the gate shape 7 % slower: it moves half the operand registers per flop but twice the accumulator registers,
// and the device sustains a lower clock under it.)
//
// Against the eight-wavefront form of gemm_tiles.hip (wavefronts of 64 x 128) every wavefront reads a third fewer
// LDS bytes per flop (128 + 128 rows of fragments per 128 x 128 outputs instead of 64 + 128 per 64 x 128).  There the fragment reads and
// the direct copies together keep the LDS port busy for as long as the matrix instructions take, so neither ever
// runs at its own rate; here the port has a quarter of its time to spare.  Tile numbering, operand copies (global ->
// LDS directly, swizzle applied on the global side), barrier placement and epilogues are those of the
// eight-wavefront form.
#include "gemm_args.hpp"
#include "sngguf_common.hpp"

namespace sngguf {

namespace {

constexpr int TM = 256;      // activation rows per tile
constexpr int TN = 256;      // weight rows (output columns) per tile
constexpr int TK = 64;       // K step
constexpr int kTileBytes = 256 * 64 * 2;        // one operand tile in LDS (rows of 128 bytes, swizzled)
constexpr int kYRow = 2 * TN + 16;              // bytes of one staged output row; the padding spreads rows over the banks
constexpr int kLdsBytes = TM * kYRow > 4 * kTileBytes ? TM * kYRow : 4 * kTileBytes;

// A pointer that is the same in all lanes, pinned to scalar registers: the request then uses the scalar-base +
// 32-bit-offset address form and needs no vector arithmetic per K step.
__device__ __forceinline__ const uint8_t* uniform_ptr(const void* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const uint8_t*>(((uint64_t)hi << 32) | lo);
}

// exp(-g) for a g with at most 16 significant bits (here: bf16 values)
__device__ __forceinline__ float exp_neg(float g) {
    const float e = __builtin_amdgcn_exp2f(g * -1.44268798828125f);               // exact product
    const float c = __builtin_fmaf(e, g * -4.8884952e-06f, e);                    // x exp2(-g lo), lo ln 2 = 4.8884952e-6
    return e == 0.f ? 0.f : c;                                                    // (0 x inf at g = +inf)
}

// g / (1 + exp(-g)): hardware reciprocal, then one correction step of the quotient with the exact remainder
__device__ __forceinline__ float silu_f32(float g) {
    const float d = 1.0f + exp_neg(g);
    const float r = __builtin_amdgcn_rcpf(d);
    const float q = g * r;
    const float c = __builtin_fmaf(__builtin_fmaf(-d, q, g), r, q);
    // exp(-g) overflows below g = -88.7: the quotient is -0 as it stands; at g = +inf the remainder inf - inf is a NaN
    // and the quotient +inf is the value
    return (d < __builtin_inff() && __builtin_fabsf(g) < __builtin_inff()) ? c : q;
}

// byte offset of an LDS address within the workgroup's LDS allocation (what M0 and the ds instructions take)
__device__ __forceinline__ uint32_t lds_offset(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}

// EP: which epilogue this instance carries (one per instance, so that the 256 accumulators of a lane are read out of
// their accumulation registers group by group on one path instead of all at once in front of a three-way branch):
// 0 = bf16 tile staged through LDS (N % 8 == 0), 1 = fp32 partial sums of a K slice, 2 = direct stores (any N),
// 3 = gated pair: the tile's first 128 columns are gate sums, its last 128 the up sums of the same outputs.
template <int EP>
__global__ __launch_bounds__(256) void gemm_dense4_kernel(GemmArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;  // 2 x 2 wavefronts: activation rows wm * 128, weight rows wn * 128

    // ---- tile of this workgroup (same numbering as the eight-wavefront form) ------------------------------------
    const int64_t n0 = a.n0_dev ? (int64_t)*a.n0_dev : a.n0;
    const int64_t t0 = (a.group_mask & 1) ? (n0 + TM - 1) / TM : 0;
    const int64_t t1 = (a.group_mask & 2) ? (a.M - n0 + TM - 1) / TM : 0;
    const int64_t ntn = (a.N + TN - 1) / TN;
    const int S = a.ksplit > 1 ? a.ksplit : 1;
    const int64_t total = (t0 + t1) * ntn * S;
    const int64_t pid = blockIdx.x;
    if (pid >= total) return;
    const int64_t per = total >> 3, rem = total & 7;
    const int64_t xcd = pid & 7, idx = pid >> 3;
    const int64_t tile_slice = xcd * per + (xcd < rem ? xcd : rem) + idx;
    const int64_t tile = tile_slice / S;
    const int slice = (int)(tile_slice - tile * S);
    int64_t ty, tn;
    constexpr int BY = 4, BX = 8;
    if ((ntn % BX) == 0 && ((t0 + t1) % BY) == 0) {
        const int64_t blk = tile >> 5, within = tile & 31, bpr = ntn / BX;
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
    const int64_t row_bytes = 2 * a.K;
    const int ksteps_all = (int)(a.K / TK);
    const int ks0 = (int)((int64_t)slice * ksteps_all / S);
    const int ksteps = (int)((int64_t)(slice + 1) * ksteps_all / S) - ks0;

    // ---- LDS: two stages of (activation tile, weight tile); chunk c of row r sits at c ^ ((r / 2) % 8) ------------
    bf16_t* xs[2] = {reinterpret_cast<bf16_t*>(lds), reinterpret_cast<bf16_t*>(lds + 2 * kTileBytes)};
    bf16_t* ws[2] = {reinterpret_cast<bf16_t*>(lds + kTileBytes), reinterpret_cast<bf16_t*>(lds + 3 * kTileBytes)};

    // copies: instruction i of wavefront w fills tile rows 32 i + 8 w .. + 7 (lane l the 16 bytes at 16 l after a
    // uniform base); the lane that fills physical chunk p of row r fetches logical chunk p ^ ((r / 2) % 8).  Rows
    // past the end re-read the last row: they only feed outputs that are never stored.
    uint32_t xoff[8], woff[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        int64_t rr = row_begin + (tid >> 3) + 32 * i;
        if (rr >= row_end) rr = row_end - 1;
        const int64_t gr = a.rowmap ? (int64_t)a.rowmap[rr] : rr;
        xoff[i] = (uint32_t)(2 * (gr * a.K + 8 * ((tid & 7) ^ ((tid >> 4) & 7))));
        int64_t n = (tid >> 3) + 32 * i;
        if (nb0 + n >= a.N) n = a.N - 1 - nb0;
        woff[i] = (uint32_t)(2 * (n * a.K + 8 * ((tid & 7) ^ ((tid >> 4) & 7))));
    }
    const int xrow0 = 8 * wave;
    const uint8_t* __restrict__ wbase = q + nb0 * row_bytes;

    // fragment reads: row (lane % 16) of a 16-row tile, logical chunk 4 ks + lane / 16 (ks: the two 32-element halves
    // of a K step)
    int foff[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) foff[ks] = (lane & 15) * 64 + 8 * ((4 * ks + (lane >> 4)) ^ ((lane >> 1) & 7));

    f32x4_t acc[8][8];  // [weight-row tile i][activation-row tile j]
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

// Base pointers of the copies of K step kb (clamped to the last step: the loop below requests one and two steps
// ahead without asking whether they exist; a repeated last step lands in a stage nobody reads any more).
#define SNGGUF_STEP_BASE(kb, xb_, wb_)                                                                       \
    const int kc_##xb_ = (kb) < ksteps ? (kb) : ksteps - 1;                                                  \
    const uint8_t* xb_ = uniform_ptr(a.x + (int64_t)(kc_##xb_ + ks0) * TK);                                  \
    const uint8_t* wb_ = uniform_ptr(wbase + (int64_t)(kc_##xb_ + ks0) * (2 * TK))
// One copy request, written as the instruction itself: uniform 64-bit base in scalar registers + this lane's 32-bit
// byte offset, LDS destination base in M0.  (Left to the compiler, the request gets a 64-bit address per lane and a
// 64-bit vector add in front of it - twice the address traffic and an extra vector instruction in a stream where
// everything between two matrix instructions has to fit under one of them.)  The compiler does not count these
// requests: the loop waits for them itself (s_waitcnt vmcnt(0) in front of every barrier).  The s_nop is the wait
// state the hardware wants between a scalar write of M0 and a request that reads it.
#define SNGGUF_COPY1(base_, off_, tile_, i_)                                                                 \
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"                             \
                 :: "s"(lds_offset((tile_) + (xrow0 + 32 * (i_)) * 64)), "v"((off_)[i_]), "s"(base_) : "memory", "m0")
// fragment f (0..7 weight tiles, 8..15 activation tiles) of half ks_ of a stage
#define SNGGUF_FRAG1(stage, ks_, buf, f)                                                                     \
    do {                                                                                                     \
        if ((f) < 8) af_[buf][(f) & 7] = *reinterpret_cast<const bf16x8_t*>(ws[stage] + wn * 128 * 64 + ((f) & 7) * 16 * 64 + foff[ks_]); \
        else bf_[buf][(f) & 7] = *reinterpret_cast<const bf16x8_t*>(xs[stage] + wm * 128 * 64 + ((f) & 7) * 16 * 64 + foff[ks_]);         \
    } while (0)
// One K step on stage CUR: 128 matrix instructions (two halves of 32 elements of K, 8 x 8 tiles each), written out
// instruction group by instruction group with a scheduling fence after each - a lone wavefront per SIMD issues in
// order, so what sits between two matrix instructions decides whether the matrix pipe runs dry.  Every half reads
// the 16 fragments of the next half under its first 32 matrix instructions (one read per two).  The workgroup's one
// barrier per step sits behind the first 32: by then every wavefront holds the fragments of both halves in
// registers, so stage CUR is free, and the copies into the other stage have been on their way since the previous
// step's barrier.  The 16 copies of step kb + 2 go into stage CUR behind the barrier, one per six matrix
// instructions, which spreads them over the rest of the step: requests closer together fill the memory pipeline's
// queue and hold up the matrix instructions behind them (gate shape, one copy per 2 / 4 / 6 matrix instructions:
// 360 / 343 / 336 us in one run; copies behind a barrier between the halves, one per 4: 344 us).
constexpr int kBarrierAt = 32, kCopyEvery = 6, kFragEvery = 2;
static_assert(kBarrierAt > 15 * kFragEvery && kBarrierAt <= 64 && kBarrierAt + 16 * kCopyEvery <= 128, "placement");
#define SNGGUF_K_STEP4(kb, CUR)                                                                                      \
    do {                                                                                                             \
        SNGGUF_STEP_BASE((kb) + 2, xb2_, wb2_);                                                                      \
        _Pragma("unroll") for (int q = 0; q < 128; q++) {                                                            \
            const int ks = q >> 6, m = q & 63;                                                                       \
            if (q == kBarrierAt) {                                                                                   \
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");                                          \
                __syncthreads();                                                                                     \
            }                                                                                                        \
            acc[m >> 3][m & 7] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af_[ks][m >> 3], bf_[ks][m & 7],            \
                                                                         acc[m >> 3][m & 7], 0, 0, 0);               \
            if (m < 16 * kFragEvery && (m % kFragEvery) == 0) {                                                      \
                /* activation fragments first: the next half's first eight matrix instructions need all */           \
                const int f = m / kFragEvery < 8 ? 8 + m / kFragEvery : m / kFragEvery - 8;                          \
                if (ks == 0) SNGGUF_FRAG1(CUR, 1, 1, f);                                                             \
                else SNGGUF_FRAG1((CUR) ^ 1, 0, 0, f);                                                               \
            }                                                                                                        \
            if (q >= kBarrierAt && ((q - kBarrierAt) % kCopyEvery) == kCopyEvery - 1 && (q - kBarrierAt) / kCopyEvery < 16) { \
                const int c = (q - kBarrierAt) / kCopyEvery;                                                         \
                if (c < 8) SNGGUF_COPY1(wb2_, woff, ws[CUR], c & 7);                                                 \
                else SNGGUF_COPY1(xb2_, xoff, xs[CUR], c & 7);                                                       \
            }                                                                                                        \
            __builtin_amdgcn_sched_barrier(0);                                                                       \
        }                                                                                                            \
    } while (0)

    {
        // the launcher sends only even numbers of K steps here: the loop has one body and the accumulators one home
        bf16x8_t af_[2][8], bf_[2][8];
        {
            SNGGUF_STEP_BASE(0, xb0_, wb0_);
            SNGGUF_STEP_BASE(1, xb1_, wb1_);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                SNGGUF_COPY1(xb0_, xoff, xs[0], i);
                SNGGUF_COPY1(wb0_, woff, ws[0], i);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                SNGGUF_COPY1(xb1_, xoff, xs[1], i);
                SNGGUF_COPY1(wb1_, woff, ws[1], i);
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
#pragma unroll
        for (int f = 0; f < 16; f++) SNGGUF_FRAG1(0, 0, 0, f);
        for (int kd = 0; kd < ksteps; kd += 2) {
            SNGGUF_K_STEP4(kd, 0);
            SNGGUF_K_STEP4(kd + 1, 1);
        }
        // the last steps' look-ahead copies may still be in flight, and the epilogue reuses the buffers
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
#undef SNGGUF_K_STEP4
#undef SNGGUF_FRAG1
#undef SNGGUF_COPY1
#undef SNGGUF_STEP_BASE

    // ---- epilogue: D[i][j], i = weight row (n), j = activation row (m) ----------------------------------------
    // lane: j = lane % 16; register v: i = 4 * (lane / 16) + v
    if constexpr (EP == 1) {
        // K split over workgroups: this slice's sums go out as fp32, to be added up by the split-K reduction
        float* part = a.partial + (int64_t)slice * a.M * a.N;
        const bool vec = (a.N & 3) == 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int64_t n = nb0 + wn * 128 + i * 16 + 4 * (lane >> 4);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int64_t rr = row_begin + wm * 128 + j * 16 + (lane & 15);
                if (rr >= row_end || n >= a.N) continue;
                const int64_t gr = a.rowmap ? (int64_t)a.rowmap[rr] : rr;
                float* pp = part + gr * a.N + n;
                if (vec) {
                    *reinterpret_cast<f32x4_t*>(pp) = acc[i][j];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < a.N) pp[e] = acc[i][j][e];
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // one group of accumulators at a time: they live in accumulation registers
        }
        return;
    }
    if constexpr (EP == 0) {
        // Rows of y are 16-byte aligned: stage the tile in LDS as bf16 [256 m][256 n] (the K-loop buffers are dead:
        // nothing reads them after the last barrier) and write it out as 16-byte pieces, 32 lanes along one output row.
#pragma unroll
        for (int i = 0; i < 8; i++) {
            // (an empty statement that wants this row of tiles in accumulation registers: without it the compiler moves
            // all 256 accumulators into vector registers at the loop's exit and runs out of them)
#pragma unroll
            for (int j = 0; j < 8; j++) asm volatile("" : "+a"(acc[i][j]));
            const int nl = wn * 128 + i * 16 + 4 * (lane >> 4);
            float b[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias && nb0 + nl < a.N) {
#pragma unroll
                for (int e = 0; e < 4; e++) b[e] = bf16_to_f32(bias[nb0 + nl + e]);
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int ml = wm * 128 + j * 16 + (lane & 15);
                *reinterpret_cast<u32x2_t*>(lds + ml * kYRow + 2 * nl) =
                    u32x2_t{pack_bf16(acc[i][j][0] + b[0], acc[i][j][1] + b[1]), pack_bf16(acc[i][j][2] + b[2], acc[i][j][3] + b[3])};
                if (j & 1) __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
        const int64_t n = nb0 + 8 * (tid & 31);
        if (n >= a.N) return;
#pragma unroll 4
        for (int p = 0; p < TM / 8; p++) {
            const int ml = (tid >> 5) + 8 * p;
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
            // written once, read by a later launch at the earliest: stored with the non-temporal hint, so that a round's
            // 32 MB of output does not displace the operand tiles the next round's workgroups share in L2 (gate shape -3 %)
            __builtin_nontemporal_store(o, reinterpret_cast<u32x4_t*>(a.y + gr * a.N + n));
        }
        return;
    }
    if constexpr (EP == 3) {
        // Stage the tile as bf16 [256 m][128 gate | 128 up] - the projections' outputs as two separate launches would
        // round them - then every thread combines eight gate values with their eight up values: silu in fp32 rounded to
        // bf16, product rounded to bf16 (what bf16 tensors give `act(gate) * up`; the decode kernels' gated pair rounds
        // the same way).
#pragma unroll
        for (int i = 0; i < 8; i++) {
#pragma unroll
            for (int j = 0; j < 8; j++) asm volatile("" : "+a"(acc[i][j]));  // as above: one row of tiles at a time
            const int nl = wn * 128 + i * 16 + 4 * (lane >> 4);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int ml = wm * 128 + j * 16 + (lane & 15);
                *reinterpret_cast<u32x2_t*>(lds + ml * kYRow + 2 * nl) =
                    u32x2_t{pack_bf16(acc[i][j][0], acc[i][j][1]), pack_bf16(acc[i][j][2], acc[i][j][3])};
                if (j & 1) __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
        const int64_t n = tn * 128 + 8 * (tid & 15);   // output column
        if (n >= a.gated_cols) return;
#pragma unroll 4
        for (int p = 0; p < TM / 16; p++) {
            const int ml = (tid >> 4) + 16 * p;
            const int64_t rr = row_begin + ml;
            if (rr >= row_end) break;
            const int64_t gr = a.rowmap ? (int64_t)a.rowmap[rr] : rr;
            const u32x4_t gt = *reinterpret_cast<const u32x4_t*>(lds + ml * kYRow + 16 * (tid & 15));
            const u32x4_t ut = *reinterpret_cast<const u32x4_t*>(lds + ml * kYRow + 256 + 16 * (tid & 15));
            u32x4_t o;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                // silu on the hardware's exp2 and reciprocal (the library exp and an IEEE division here cost 8 us per
                // tile, 7 % of the launch, against 2 - 3).  exp(-g) = exp2(-g log2(e)): the product with the upper 16 bits
                // of log2(e) is exact for a bf16 g, the rest of log2(e) enters as a first-order correction, and the
                // quotient gets one correction step, so the result is good to about one unit in the last place of fp32
                // before it is rounded to bf16.
                const float g0 = bf16lo_to_f32(gt[e]), g1 = bf16hi_to_f32(gt[e]);
                const float s0 = bf16_to_f32(f32_to_bf16(silu_f32(g0)));
                const float s1 = bf16_to_f32(f32_to_bf16(silu_f32(g1)));
                o[e] = pack_bf16(s0 * bf16lo_to_f32(ut[e]), s1 * bf16hi_to_f32(ut[e]));
            }
            __builtin_nontemporal_store(o, reinterpret_cast<u32x4_t*>(a.y + gr * a.gated_cols + n));
        }
        return;
    }
    const bool fast = (a.N & 3) == 0;  // rows of y are 8-byte aligned and a run of four columns never straddles N
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
        for (int j = 0; j < 8; j++) asm volatile("" : "+a"(acc[i][j]));  // as above: one row of tiles at a time
        const int64_t n = nb0 + wn * 128 + i * 16 + 4 * (lane >> 4);
        float b[4] = {0.f, 0.f, 0.f, 0.f};
        if (bias) {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (n + e < a.N) b[e] = bf16_to_f32(bias[n + e]);
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int64_t rr = row_begin + wm * 128 + j * 16 + (lane & 15);
            if (rr >= row_end || n >= a.N) continue;
            const int64_t gr = a.rowmap ? (int64_t)a.rowmap[rr] : rr;
            bf16_t* yp = a.y + gr * a.N + n;
            const int64_t yi = gr * a.N + n;
            const float o0 = add_residual(acc[i][j][0] + b[0], a.residual, yi);
            const float o1 = n + 1 < a.N ? add_residual(acc[i][j][1] + b[1], a.residual, yi + 1) : 0.f;
            const float o2 = n + 2 < a.N ? add_residual(acc[i][j][2] + b[2], a.residual, yi + 2) : 0.f;
            const float o3 = n + 3 < a.N ? add_residual(acc[i][j][3] + b[3], a.residual, yi + 3) : 0.f;
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

}  // namespace

// Weights that are already bf16 rows, K % 64 == 0, both row groups; same contract as the dense form of the
// eight-wavefront tile kernel (split-K partial sums included).
int launch_gemm_dense4(const GemmArgs& a, hipStream_t stream) {
    const int64_t row_tiles = (a.M + TM - 1) / TM + 1;  // a split adds at most one partial tile
    const int64_t ntn = (a.N + TN - 1) / TN;
    const int64_t slices = a.ksplit > 1 ? a.ksplit : 1;
    const dim3 grid((unsigned)(row_tiles * ntn * slices));
#define SNGGUF_GO(EP)                                                                                                  \
    do {                                                                                                               \
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_dense4_kernel<EP>),     \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);     \
        if (attr != hipSuccess) return SNGGUF_E_LAUNCH;                                                                \
        gemm_dense4_kernel<EP><<<grid, dim3(256), kLdsBytes, stream>>>(a);                                             \
    } while (0)
    if (a.gated_cols > 0) {
        // the pair's layout: whole blocks of 128 + 128 rows, output rows of whole 16-byte pieces
        if (a.partial || a.bias[0] || a.bias[1] || a.residual || (a.N & 255) != 0 || (a.gated_cols & 7) != 0 ||
            a.gated_cols > a.N / 2 || a.gated_cols <= a.N / 2 - 128)
            return SNGGUF_E_BADSHAPE;
        SNGGUF_GO(3);
    } else if (a.partial) SNGGUF_GO(1);
    else if ((a.N & 7) == 0) SNGGUF_GO(0);
    else SNGGUF_GO(2);
#undef SNGGUF_GO
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

}  // namespace sngguf
