// Q8_0 decode GEMV on the matrix cores (1 <= M <= 16, K % 256 == 0).
//
// A workgroup owns 16 weight rows (for the SiLU-gated pair: the same 16 rows of the gate and of
// the up matrix, on separate wavefronts); its wavefronts split K between them and add their
// partial sums through LDS at the end.  Per wavefront and step of CB blocks (CB * 34 packed
// bytes per row, CB = 16 when K allows it):
//   * the 16-row slab is fetched with coalesced 16-byte loads (consecutive lanes walk along a
//     row) into registers one step ahead, then dropped into the wavefront's private LDS slab, so
//     HBM sees long contiguous runs although blocks are 34 bytes long and every 128-byte line
//     is requested by one wavefront (or by two neighbours of one workgroup at the same time);
//   * lane (r = lane % 16, g = lane / 16) picks quants 8g..8g+7 and the scale of each block of
//     row r out of LDS with 4-byte aligned reads (blocks at even positions sit 2 bytes off a
//     dword boundary and are realigned with v_alignbit), decodes them to eight bf16 (rounding
//     chain by numerics mode) and feeds them as the A operand of v_mfma_f32_16x16x32_bf16; the
//     B operand is x[m = lane % 16][32 b + 8 g ..].  One MFMA contracts one 32-element block
//     for 16 weight rows and up to 16 activation rows, so the cost per packed byte does not
//     depend on M and the cross-lane reduction happens inside the matrix core.
// Nothing dequantized is written to memory.

#include <stddef.h>

#include "sngguf_common.hpp"

namespace sngguf {

// CB: blocks per step.  GATED: wavefronts [0, W) work on qa (gate), [W, 2W) on qb (up).
// XS: where the B operand comes from.  0: fragments fetched from global memory one step ahead.  1: RMSNorm(x) with
// weight `gamma` is what gets contracted - each wavefront stages the K range it works on (all M rows) in LDS behind
// the slabs, the workgroup adds up the sums of squares, and every wavefront then normalizes its own share in place;
// the B fragments come from there.  2: the same wavefront-private staging without a norm, read with agent-scope loads:
// x was written by other workgroups of the SAME launch (the one-launch MLP below).
template <int CB>
struct CbGeom {
    static constexpr int kRowStep = CB * 34;             // bytes of one row per step (272 or 544)
    static constexpr int kRowPieces = kRowStep / 16;     // 16-byte pieces per row and step (17 or 34)
    static constexpr int kPieces = 16 * kRowPieces;      // per slab
    static constexpr int kLoads = (kPieces + 63) / 64;   // per lane (5 or 9; the last one is partial)
    static constexpr int kSlab = 16 * kRowStep;          // LDS bytes per wavefront (4352 or 8704)
};

// The body of the block-aligned kernel for workgroup `bid` of `nblocks`, all `blockDim.x / 64` wavefronts taking part.
// `pre` holds the first step's slab pieces if `have_pre` (requested by the caller with cb_first_fetch, so that the
// request can be made long before the activations exist); otherwise the body requests them itself.
template <int NUM, int CB, bool GATED, int WMAX, int XS>
__device__ __forceinline__ void gemv_q8_cb_body(uint8_t* lds, const bf16_t* __restrict__ x, int M, const uint8_t* __restrict__ qa,
                                                const uint8_t* __restrict__ qb, int64_t N, int64_t K, const bf16_t* __restrict__ bias,
                                                const bf16_t* residual, bf16_t* __restrict__ y, const bf16_t* __restrict__ gamma, float eps,
                                                uint64_t* __restrict__ amax, const int bid, const int nblocks,
                                                u32x4_t (&pre)[CbGeom<CB>::kLoads], const bool have_pre) {
    constexpr bool XN = XS != 0;
    constexpr int kRowStep = CbGeom<CB>::kRowStep;
    constexpr int kRowPieces = CbGeom<CB>::kRowPieces;
    constexpr int kPieces = CbGeom<CB>::kPieces;
    constexpr int kLoads = CbGeom<CB>::kLoads;
    constexpr int kSlab = CbGeom<CB>::kSlab;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int W = GATED ? waves >> 1 : waves;     // wavefronts that share one row group's K
    const int kw = GATED ? (wave >= W ? wave - W : wave) : wave;
    const uint8_t* __restrict__ q = (GATED && wave >= W) ? qb : qa;
    const int r = lane & 15, g = lane >> 4;
    const int64_t row_bytes = (K >> 5) * 34;
    const int64_t n0 = (int64_t)bid * 16;

    // this wavefront's share of the K steps
    const int steps = (int)(K / (32 * CB));
    const int s0 = (int)((int64_t)kw * steps / W), s1 = (int)((int64_t)(kw + 1) * steps / W);

    // per-lane slab pieces: piece f = lane + 64 i is bytes [16 (f % P), +16) of slab row f / P
    uint32_t off[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; i++) {
        const int f = lane + 64 * i;
        const bool ok = f < kPieces;
        const int fr = ok ? f / kRowPieces : 0, fp = ok ? f % kRowPieces : 0;
        int64_t n = n0 + fr;
        if (n >= N) n = N - 1;  // rows past the end are decoded from the last row and never stored
        off[i] = (uint32_t)((n - n0) * row_bytes + 16 * fp);
    }
    const uint8_t* __restrict__ base = q + n0 * row_bytes;
    const bool tail_lane = lane + 64 * (kLoads - 1) < kPieces;  // does the last, partial load cover this lane
    uint8_t* slab = lds + wave * kSlab;

    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    auto fetch = [&](int s) {
        const uint8_t* p = base + (int64_t)s * kRowStep;
#pragma unroll
        for (int i = 0; i < kLoads - 1; i++) pre[i] = *reinterpret_cast<const u32x4_t*>(p + off[i]);
        if (tail_lane) pre[kLoads - 1] = *reinterpret_cast<const u32x4_t*>(p + off[kLoads - 1]);
    };
    // Lane (r, g) supplies B-operand column r.  Columns >= M are never stored, so those lanes
    // re-read the last activation row instead of being masked.
    const bool has_x = r < M;
    const bf16_t* xrow = x + (int64_t)(has_x ? r : M - 1) * K + 8 * g;
    const uint8_t* lrow = slab + r * kRowStep + 8 * g;
    // XN: this wavefront's normalized activations, [M][xrow_b bytes]; fragment (step s, block b) of row m at
    // byte ((s - s0) CB + b) * 64 + 16 g of row m
    const int xrow_b = XN ? ((steps + W - 1) / W) * CB * 64 + 16 : 0;
    uint8_t* xw = lds + waves * kSlab + wave * (M * xrow_b);
    const uint8_t* xwrow = xw + (has_x ? r : M - 1) * xrow_b + 16 * g;

    // One step: slab of step s is in `pre`, its activations in `xc`.  The next step's activations
    // (into `xn`) and slab (into `pre`) are requested before this step's MFMAs, so a full step of
    // decode work covers their latency.
    auto step = [&](int s, u32x4_t (&xc)[CB], u32x4_t (&xn)[CB]) {
#pragma unroll
        for (int i = 0; i < kLoads - 1; i++) *reinterpret_cast<u32x4_t*>(slab + 16 * (lane + 64 * i)) = pre[i];
        if (tail_lane) *reinterpret_cast<u32x4_t*>(slab + 16 * (lane + 64 * (kLoads - 1))) = pre[kLoads - 1];
        if (s + 1 < s1) {
            if constexpr (!XN) {
#pragma unroll
                for (int b = 0; b < CB; b++) xn[b] = *reinterpret_cast<const u32x4_t*>(xrow + ((int64_t)(s + 1) * CB + b) * 32);
            }
            fetch(s + 1);
        }
#pragma unroll
        for (int b = 0; b < CB; b++) {
            // block b of row r starts at byte 34 b: scale, then quants; this lane wants quants 8g..8g+7
            const uint16_t d = *reinterpret_cast<const uint16_t*>(slab + r * kRowStep + 34 * b);
            uint32_t q0, q1;
            if ((b & 1) == 0) {
                // 34 b is a multiple of 4: the quants start 2 bytes into a dword
                const uint32_t* w = reinterpret_cast<const uint32_t*>(lrow + 34 * b);
                const uint32_t w0 = w[0], w1 = w[1], w2 = w[2];
                q0 = __builtin_amdgcn_alignbit(w1, w0, 16);
                q1 = __builtin_amdgcn_alignbit(w2, w1, 16);
            } else {
                const uint32_t* w = reinterpret_cast<const uint32_t*>(lrow + 34 * b + 2);
                q0 = w[0];
                q1 = w[1];
            }
            uint32_t a0, a1, a2, a3;
            q8_dword_bf16<NUM>(d, q0, a0, a1);
            q8_dword_bf16<NUM>(d, q1, a2, a3);
            const u32x4_t a = {a0, a1, a2, a3};
            u32x4_t xfrag;
            if constexpr (XN) xfrag = *reinterpret_cast<const u32x4_t*>(xwrow + ((s - s0) * CB + b) * 64);
            else xfrag = xc[b];
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                          __builtin_bit_cast(bf16x8_t, xfrag), acc, 0, 0, 0);
        }
    };
    u32x4_t xa[CB], xb[CB];
    if (s0 < s1) {
        if constexpr (!XN) {
#pragma unroll
            for (int b = 0; b < CB; b++) xa[b] = *reinterpret_cast<const u32x4_t*>(xrow + ((int64_t)s0 * CB + b) * 32);
        }
        if (!have_pre) fetch(s0);
    }
    if constexpr (XS == 2) {
        // this wavefront's share of the activations, written earlier in this launch by other workgroups: 8-byte
        // agent-scope loads (they bypass whatever this compute unit's caches hold), into the wavefront's own LDS rows
        const int pieces8 = (s1 - s0) * CB * 8;            // 8-byte pieces per row in this wavefront's K range
        const int64_t k0 = (int64_t)s0 * CB * 32;
        for (int m = 0; m < M; m++)
            for (int c = lane; c < pieces8; c += 64) {
                const uint64_t v = __hip_atomic_load(reinterpret_cast<const uint64_t*>(x + (int64_t)m * K + k0 + 4 * c), __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT);
                *reinterpret_cast<uint64_t*>(xw + m * xrow_b + 8 * c) = v;
            }
    }
    if constexpr (XS == 1) {
        // the first slab is on its way; stage and normalize this wavefront's activations underneath
        float* ssum = reinterpret_cast<float*>(lds + waves * kSlab + waves * (M * xrow_b));  // [M][waves]
        const int pieces = (s1 - s0) * CB * 4;             // 16-byte pieces per row in this wavefront's K range
        const int64_t k0 = (int64_t)s0 * CB * 32;
        for (int m = 0; m < M; m++) {
            float ss = 0.f;
            for (int c = lane; c < pieces; c += 64) {
                const u32x4_t v = *reinterpret_cast<const u32x4_t*>(x + (int64_t)m * K + k0 + 8 * c);
                *reinterpret_cast<u32x4_t*>(xw + m * xrow_b + 16 * c) = v;
                ss += sumsq_piece(v);
            }
            ss = wave_sum(ss);
            if (lane == 0) ssum[m * waves + wave] = ss;
        }
        __syncthreads();
        for (int m = 0; m < M; m++) {
            float tot = 0.f;
            for (int w = 0; w < W; w++) tot += ssum[m * waves + w];   // wavefronts [0, W) cover K once
            const float rstd = rms_rstd(tot, K, eps);
            for (int c = lane; c < pieces; c += 64) {
                u32x4_t* cell = reinterpret_cast<u32x4_t*>(xw + m * xrow_b + 16 * c);
                const u32x4_t gv = *reinterpret_cast<const u32x4_t*>(gamma + k0 + 8 * c);
                *cell = rmsnorm_piece(*cell, gv, rstd);
            }
        }
    }
    for (int s = s0; s < s1; s += 2) {
        step(s, xa, xb);
        if (s + 1 < s1) step(s + 1, xb, xa);
    }

    // ---- add the wavefronts' partial sums (the slabs are dead: reuse them) -------------------------
    __syncthreads();
    f32x4_t* red = reinterpret_cast<f32x4_t*>(lds);  // [waves][64]
    red[wave * 64 + lane] = acc;
    __syncthreads();
    if (wave != 0 || !has_x) return;
    // D[i][j]: j = lane % 16 is the activation row, register v holds weight row 4 * (lane / 16) + v
    f32x4_t sum = red[lane];
    for (int w = 1; w < W; w++) {
        const f32x4_t t = red[w * 64 + lane];
        sum[0] += t[0]; sum[1] += t[1]; sum[2] += t[2]; sum[3] += t[3];
    }
    const int m = r;
    const int64_t n = n0 + 4 * g;
    float o[4];
    if constexpr (GATED) {
        f32x4_t up = red[W * 64 + lane];
        for (int w = 1; w < W; w++) {
            const f32x4_t t = red[(W + w) * 64 + lane];
            up[0] += t[0]; up[1] += t[1]; up[2] += t[2]; up[3] += t[3];
        }
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const float gt = bf16_to_f32(f32_to_bf16(sum[v]));
            const float ut = bf16_to_f32(f32_to_bf16(up[v]));
            const float sl = bf16_to_f32(f32_to_bf16(gt / (1.0f + expf(-gt))));
            o[v] = sl * ut;
        }
    } else {
#pragma unroll
        for (int v = 0; v < 4; v++) o[v] = n + v < N ? add_residual(sum[v] + (bias ? bf16_to_f32(bias[n + v]) : 0.f), residual, (int64_t)m * N + n + v) : 0.f;
        if (amax) {
            // arg-max form: this row group's best (value, column) per activation row instead of the outputs
            uint64_t key = 0;
#pragma unroll
            for (int v = 0; v < 4; v++)
                if (n + v < N) key = u64_max(key, argmax_key(o[v], n + v));
            argmax_store(key, g, amax, m, bid, nblocks);
            return;
        }
    }
    bf16_t* yr = y + (int64_t)m * N + n;
    if (n + 3 < N && (N & 3) == 0) {
        *reinterpret_cast<u32x2_t*>(yr) = u32x2_t{pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3])};
    } else {
#pragma unroll
        for (int v = 0; v < 4; v++)
            if (n + v < N) yr[v] = f32_to_bf16(o[v]);
    }
}

// The first step's slab pieces of wavefront `wave` of `waves` (not gated), as gemv_q8_cb_body wants them in `pre`.
template <int CB>
__device__ __forceinline__ void cb_first_fetch(const uint8_t* __restrict__ q, int64_t N, int64_t K, int bid, int wave, int waves, int lane,
                                               u32x4_t (&pre)[CbGeom<CB>::kLoads]) {
    constexpr int kRowStep = CbGeom<CB>::kRowStep, kRowPieces = CbGeom<CB>::kRowPieces, kPieces = CbGeom<CB>::kPieces,
                  kLoads = CbGeom<CB>::kLoads;
    const int64_t row_bytes = (K >> 5) * 34;
    const int64_t n0 = (int64_t)bid * 16;
    const int steps = (int)(K / (32 * CB));
    const int s0 = (int)((int64_t)wave * steps / waves);
    const uint8_t* p = q + n0 * row_bytes + (int64_t)s0 * kRowStep;
#pragma unroll
    for (int i = 0; i < kLoads; i++) {
        const int f = lane + 64 * i;
        const bool ok = f < kPieces;
        const int fr = ok ? f / kRowPieces : 0, fp = ok ? f % kRowPieces : 0;
        int64_t n = n0 + fr;
        if (n >= N) n = N - 1;
        if (ok) pre[i] = *reinterpret_cast<const u32x4_t*>(p + (n - n0) * row_bytes + 16 * fp);
    }
}

template <int NUM, int CB, bool GATED, int WMAX, bool XN = false>
__global__ __launch_bounds__(64 * WMAX) void gemv_q8_mfma_kernel(const bf16_t* __restrict__ x, int M,
                                                            const uint8_t* __restrict__ qa,
                                                            const uint8_t* __restrict__ qb, int64_t N, int64_t K,
                                                            const bf16_t* __restrict__ bias, const bf16_t* residual, bf16_t* __restrict__ y,
                                                            const bf16_t* __restrict__ gamma, float eps, uint64_t* __restrict__ amax) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    u32x4_t pre[CbGeom<CB>::kLoads];
    gemv_q8_cb_body<NUM, CB, GATED, WMAX, XN ? 1 : 0>(lds, x, M, qa, qb, N, K, bias, residual, y, gamma, eps, amax, (int)blockIdx.x,
                                                      (int)gridDim.x, pre, false);
}


// ---- line-aligned variant (K % 2048 == 0) ----------------------------------------------------------
// 2048 elements of a Q8_0 row are 64 blocks = 2176 bytes = exactly 17 cache lines of 128 bytes, so
// when K is a multiple of 2048 every row starts on a line boundary and a wavefront can work on
// whole "spans" of 17 lines.  HBM delivers markedly more when every wavefront load covers whole
// lines, so this variant fetches lines (two per row and step, eight full lines per wavefront
// load) instead of block-aligned runs, and keeps them in a four-line ring per row in LDS:
// line L of the span sits at ring bytes [128 (L % 4), +128).  A step still decodes 8 blocks
// (272 bytes, 2.125 lines); the fetch schedule - lines 0..3 before step 0, two more lines per
// step, line 16 for the last step - always has the lines a step needs in the ring and only
// overwrites lines whose blocks are done.  A block that runs over the end of the ring is read
// with wrapped addresses.
// Rows from which the gated pair runs in the paired mode of the span kernel: measured 12288 x 4096 gate/up,
// unpaired / paired us: M=2 26.8 / 30.7, M=4 27.4 / 30.8, M=8 28.2 / 29.7, M=16 34.5 / 30.2.
constexpr int kPairedMinM = 12;
constexpr int kRing = 512;        // ring bytes per row
constexpr int kRingRow = 528;     // LDS bytes per row: 132 dwords, rows fall on distinct banks
constexpr int kSpanBytes = 2176;  // 64 blocks = 17 lines

// PAIRED (gated only): one wavefront works on the gate AND the up matrix of its K range, so that each activation
// fragment is fetched once for both - with several activation rows those fetches, not the weights, fill the
// vector memory path (16 rows x 64 bytes per matrix instruction against 544 bytes of weights).
// The body of the line-aligned kernel for workgroup `bid`.  `after_loop(stores)` is called by every wavefront when it
// has left its K loop, before the workgroup adds up the partial sums (with AGENT_STORES: when the wavefront has left its
// own sums in LDS and counted itself in); `stores` tells whether this wavefront will write outputs.  AGENT_STORES: for consumers inside the same launch, and the wavefronts of a workgroup leave the body one by
// one instead of together (`red_lds` must then be room for the partial sums plus 64 bytes that nothing else uses).
// y is then an array of 8-byte words, word (m N + n) / 2 = { outputs n, n + 1 of row m as two bf16, tag }, each written
// with one agent-scope store (it reaches memory that every compute unit of the device reads): a reader that finds
// `tag` in a word has that word's data, whatever else has or has not arrived.
template <int NUM, bool GATED, int WMAX, bool XLDS, bool PAIRED, bool AGENT_STORES, typename AfterLoop>
__device__ __forceinline__ void gemv_q8_span_body(uint8_t* lds, const bf16_t* __restrict__ x, int M, const uint8_t* __restrict__ qa,
                                                  const uint8_t* __restrict__ qb, int64_t N, int64_t K, const bf16_t* __restrict__ bias,
                                                  const bf16_t* residual, bf16_t* __restrict__ y, const bf16_t* __restrict__ gamma, float eps,
                                                  uint64_t* __restrict__ amax, int gpw, int skew, const int bid, AfterLoop&& after_loop,
                                                  const uint32_t tag = 0, const int ring_stride = 0, uint8_t* red_lds = nullptr) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    static_assert(!PAIRED || GATED, "a pair is the gate and the up matrix");
    constexpr int NQ = PAIRED ? 2 : 1;   // matrices per wavefront
    // A workgroup holds gpw row groups (all wavefronts of a compute unit in one workgroup start together and share
    // one staged copy of the activations); wavefronts [grp * wpg, (grp + 1) * wpg) work on row group grp of it.
    const int waves = blockDim.x >> 6;
    const int wpg = waves / gpw;
    // skew > 0 (twelve wavefronts per workgroup, two K halves of 8 steps per row group and matrix): the three
    // wavefronts that share a SIMD are served oldest first, so the first-placed ones run ahead of the last-placed ones
    // for the whole kernel.  Each K range is therefore shared by a first-placed wavefront (wave 0..3), which takes
    // 8 + skew steps, and a last-placed one (wave 8..11), which takes 8 - skew; the middle four pair up 8 + 8.
    // The first-placed wavefront takes its extra steps - the first `skew` steps of the other one's span - BEFORE its
    // own span, so that the lines the two share are requested by both at the start of the kernel and come from
    // memory once.  lwave is the wavefront's place in the [group][matrix][K half] order the reduction below uses.
    int lwave = wave, skew_lo = 0;
    if (skew > 0) {
        const int slot = wave >> 2, i = wave & 3;
        const int pair = slot == 1 ? 4 + (i >> 1) : i;
        const int khalf = slot == 1 ? (i & 1) : (slot >> 1);
        lwave = 2 * pair + khalf;
        skew_lo = slot == 1 ? 0 : skew;
    }
    const int grp = lwave / wpg, lw = lwave - grp * wpg, wbase = grp * wpg;
    const int W = (GATED && !PAIRED) ? wpg >> 1 : wpg;
    const int kw = (GATED && !PAIRED) ? (lw >= W ? lw - W : lw) : lw;
    const uint8_t* __restrict__ q = (GATED && !PAIRED && lw >= W) ? qb : qa;
    const int r = lane & 15, g = lane >> 4;
    const int64_t row_bytes = (K >> 5) * 34;
    const int64_t n0 = ((int64_t)bid * gpw + grp) * 16;
    const bool live = n0 < N;            // the last workgroup's row groups may lie past the end: those wavefronts idle
    const int spans = (int)(K >> 11);
    const int t0 = live ? (int)((int64_t)kw * spans / W) : 0, t1 = live ? (int)((int64_t)(kw + 1) * spans / W) : 0;
    // this wavefront's steps: an optional pre-segment, steps [0, npre) of span tpre, then steps [gs0, gs1) of the row's
    // 8 * spans (whole spans unless skewed)
    int gs0 = 8 * t0, gs1 = 8 * t1, npre = 0;
    const int tpre = t1;
    if (skew_lo > 0 && live) {
        if (kw == 0) npre = skew_lo;
        else gs0 += skew_lo;
    }
    const int tf = gs0 >> 3, s_first = gs0 & 7;   // a range that starts inside a span starts at one of its steps 1..6

    // Two-line fetch: piece lane + 64 i is bytes [16 c, +16) of the 256-byte window of row
    // (lane / 16) + 4 i, c = lane % 16.  One-line fetch: row (lane / 8) + 8 i, piece lane % 8.
    uint32_t goff2[4], goff1[2];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int64_t n = n0 + (lane >> 4) + 4 * i;
        if (n >= N) n = N - 1;  // rows past the end are decoded from the last row and never stored
        goff2[i] = (uint32_t)((n - n0) * row_bytes + 16 * (lane & 15));
    }
#pragma unroll
    for (int i = 0; i < 2; i++) {
        int64_t n = n0 + (lane >> 3) + 8 * i;
        if (n >= N) n = N - 1;
        goff1[i] = (uint32_t)((n - n0) * row_bytes + 2048 + 16 * (lane & 7));
    }
    const uint8_t* __restrict__ base = q + n0 * row_bytes;
    const uint8_t* __restrict__ base2 = qb + n0 * row_bytes;           // PAIRED: the second matrix
    constexpr int kSlab = 16 * kRingRow;
    // (ring_stride: bytes between the rings of consecutive wavefronts when the caller wants them further apart than
    // they are long; red_lds: where the partial sums are added up when the caller wants the rings left alone)
    const int wave_lds = ring_stride > 0 ? ring_stride : NQ * kSlab;
    uint8_t* slab = lds + wave * wave_lds;                             // PAIRED: two rings per wavefront
    uint8_t* lw2 = slab + (lane >> 4) * kRingRow + 16 * (lane & 15);  // + 4 i rows, + 256 for odd groups
    uint8_t* lw1 = slab + (lane >> 3) * kRingRow + 16 * (lane & 7);   // + 8 i rows (line 16 -> ring slot 0)
    const uint8_t* lr = slab + r * kRingRow;                           // this lane's weight row

    // Lane (r, g) supplies B-operand column r = activation row r.  Columns >= M are never stored,
    // so those lanes re-read the last activation row instead of being masked.
    const bool has_x = r < M;
    const bf16_t* xrow = x + (int64_t)(has_x ? r : M - 1) * K + 8 * g;
    // XLDS: the activations (M * K bf16, a few KB at decode) are copied into LDS once per
    // workgroup and the B fragments come from there; otherwise they are fetched from global
    // memory one step ahead.
    const int64_t xs_stride = 2 * K + 64;   // bytes per activation row in LDS (+64: rows on different banks)
    uint8_t* xs = lds + waves * wave_lds;
    const uint8_t* xsrow = xs + (has_x ? r : M - 1) * xs_stride + 16 * g;

    f32x4_t acc[NQ];
#pragma unroll
    for (int h = 0; h < NQ; h++) acc[h] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    u32x4_t pa[NQ][4], pb[NQ][4];   // fetched lines on their way to the ring(s)
    u32x4_t xa[8], xb[8];           // activation fragments of the current / next step (global path)

    auto fetch2 = [&](int t, int grp, u32x4_t (&dst)[NQ][4]) {
#pragma unroll
        for (int h = 0; h < NQ; h++) {
            const uint8_t* p = (h ? base2 : base) + (int64_t)t * kSpanBytes + 256 * grp;
#pragma unroll
            // whole 128-byte lines, each read once by one wavefront: requested with the non-temporal hint, so that the
            // stream does not displace what the caches hold (2 - 4 % on the gated pair; the block-aligned and K-quant
            // kernels, which touch a line in two consecutive steps, lose 4 - 6 % with the same hint and do not use it)
            for (int i = 0; i < 4; i++) dst[h][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p + goff2[i]));
        }
    };
    auto store2 = [&](int grp, const u32x4_t (&src)[NQ][4]) {
#pragma unroll
        for (int h = 0; h < NQ; h++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                *reinterpret_cast<u32x4_t*>(lw2 + h * kSlab + 4 * i * kRingRow + ((grp & 1) << 8)) = src[h][i];
    };
    auto fetch_x = [&](int t, int s, u32x4_t (&dst)[8]) {
        if constexpr (!XLDS) {
#pragma unroll
            for (int b = 0; b < 8; b++)
                dst[b] = *reinterpret_cast<const u32x4_t*>(xrow + ((int64_t)t * 64 + s * 8 + b) * 32);
        }
    };

    if constexpr (AGENT_STORES) {
        static_assert(XLDS && !PAIRED, "the barrier of the activation staging orders the counters' reset");
        if (tid < 16) (reinterpret_cast<uint32_t*>(reinterpret_cast<f32x4_t*>(red_lds ? red_lds : lds) + waves * 64))[tid] = 0;
    }
    if constexpr (XLDS) {
        // weights of the first step are requested before the activations are staged
        if (npre > 0) {
            fetch2(tpre, 0, pa);
            fetch2(tpre, 1, pb);
        } else if (gs0 < gs1) {
            fetch2(tf, s_first, pa);
            fetch2(tf, s_first + 1, pb);
        }
        const int pieces_per_row = (int)(K >> 3);  // 16-byte pieces
        if (gamma == nullptr) {
            for (int f = tid; f < M * pieces_per_row; f += blockDim.x) {
                const int m = f / pieces_per_row, c = f - m * pieces_per_row;
                *reinterpret_cast<u32x4_t*>(xs + m * xs_stride + 16 * c) = *reinterpret_cast<const u32x4_t*>(x + (int64_t)m * K + 8 * c);
            }
        } else {
            // RMSNorm(x) is what gets contracted: stage the rows, add up their squares over the workgroup, then
            // every thread normalizes the pieces it staged
            float* ssum = reinterpret_cast<float*>(xs + M * xs_stride);   // [M][waves]
            for (int m = 0; m < M; m++) {
                float ss = 0.f;
                for (int c = tid; c < pieces_per_row; c += blockDim.x) {
                    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(x + (int64_t)m * K + 8 * c);
                    *reinterpret_cast<u32x4_t*>(xs + m * xs_stride + 16 * c) = v;
                    ss += sumsq_piece(v);
                }
                ss = wave_sum(ss);
                if (lane == 0) ssum[m * waves + wave] = ss;
            }
            __syncthreads();
            for (int m = 0; m < M; m++) {
                float tot = 0.f;
                for (int w = 0; w < waves; w++) tot += ssum[m * waves + w];
                const float rstd = rms_rstd(tot, K, eps);
                for (int c = tid; c < pieces_per_row; c += blockDim.x) {
                    u32x4_t* cell = reinterpret_cast<u32x4_t*>(xs + m * xs_stride + 16 * c);
                    const u32x4_t gv = *reinterpret_cast<const u32x4_t*>(gamma + 8 * c);
                    *cell = rmsnorm_piece(*cell, gv, rstd);
                }
            }
        }
        __syncthreads();
    } else if (gs0 < gs1) {
        fetch_x(tf, 0, xa);      // (ranges of whole spans only: see the launcher)
        fetch2(tf, 0, pa);
        fetch2(tf, 1, pb);
    }
    const int nit = (npre > 0 ? 1 : 0) + (gs0 < gs1 ? ((gs1 - 1) >> 3) - tf + 1 : 0);
    for (int it = 0; it < nit; it++) {
        const bool in_pre = npre > 0 && it == 0;
        const int t = in_pre ? tpre : tf + it - (npre > 0 ? 1 : 0);
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const int gs = 8 * t + s;
            if (in_pre ? s >= npre : (gs < gs0 || gs >= gs1)) continue;
            // the step after this one: in the same span, in the next segment (which starts at a span's step 0), or none
            const bool more_here = in_pre ? s + 1 < npre : (s < 7 && gs + 1 < gs1);
            const bool more = more_here || (in_pre ? gs0 < gs1 : gs + 1 < gs1);
            const int tn = in_pre ? tf : t + 1;
            u32x4_t (&xc)[8] = (s & 1) ? xb : xa;
            u32x4_t (&xn)[8] = (s & 1) ? xa : xb;
            // -- lines fetched during the previous step go into the ring (a segment's first step: both line pairs)
            if (s == 0 || (s < 7 && !in_pre && gs == gs0)) {
                store2(s, pa);
                store2(s + 1, pb);
            } else if (s < 7) {
                store2(s + 1, pa);
            } else {
#pragma unroll
                for (int h = 0; h < NQ; h++)
#pragma unroll
                    for (int i = 0; i < 2; i++) *reinterpret_cast<u32x4_t*>(lw1 + h * kSlab + 8 * i * kRingRow) = pa[h][i];
            }
            // -- requests for the next step: activations first, so that waiting for them does not
            //    also wait for the weight lines
            if (!more) {
            } else if (more_here) {
                fetch_x(t, s + 1, xn);
                if (s < 6) {
                    fetch2(t, s + 2, pa);
                } else {
#pragma unroll
                    for (int h = 0; h < NQ; h++)
#pragma unroll
                        for (int i = 0; i < 2; i++)
                            pa[h][i] = *reinterpret_cast<const u32x4_t*>((h ? base2 : base) + (int64_t)t * kSpanBytes + goff1[i]);
                }
            } else {
                fetch_x(tn, 0, xn);
                fetch2(tn, 0, pa);
                fetch2(tn, 1, pb);
            }
            // -- decode and contract the 8 blocks of this step
#pragma unroll
            for (int bb = 0; bb < 8; bb++) {
                const int b = 8 * s + bb;                 // block within the span
                const int ro = (34 * b) & (kRing - 1);    // ring offset of the block (compile-time)
                const int qo = (b & 1) ? ro + 2 : ro;     // first 4-byte aligned dword this lane reads, before + 8 g
                const int nd = (b & 1) ? 2 : 3;           // dwords read
                u32x4_t xfrag;
                if constexpr (XLDS) xfrag = *reinterpret_cast<const u32x4_t*>(xsrow + ((int64_t)t * 64 + b) * 64);
                else xfrag = xc[bb];
#pragma unroll
                for (int h = 0; h < NQ; h++) {
                    const uint8_t* lrh = lr + h * kSlab;
                    const uint16_t d = *reinterpret_cast<const uint16_t*>(lrh + ro);
                    uint32_t w[3];
                    if (qo + 24 + 4 * nd <= kRing) {
                        const uint32_t* src = reinterpret_cast<const uint32_t*>(lrh + qo + 8 * g);
#pragma unroll
                        for (int k = 0; k < 3; k++)
                            if (k < nd) w[k] = src[k];
                    } else {  // the block runs over the end of the ring
#pragma unroll
                        for (int k = 0; k < 3; k++)
                            if (k < nd) w[k] = *reinterpret_cast<const uint32_t*>(lrh + ((qo + 8 * g + 4 * k) & (kRing - 1)));
                    }
                    uint32_t q0, q1;
                    if (b & 1) {
                        q0 = w[0];
                        q1 = w[1];
                    } else {  // quants start 2 bytes into the first dword
                        q0 = __builtin_amdgcn_alignbit(w[1], w[0], 16);
                        q1 = __builtin_amdgcn_alignbit(w[2], w[1], 16);
                    }
                    uint32_t a0, a1, a2, a3;
                    q8_dword_bf16<NUM>(d, q0, a0, a1);
                    q8_dword_bf16<NUM>(d, q1, a2, a3);
                    const u32x4_t a = {a0, a1, a2, a3};
                    acc[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                                     __builtin_bit_cast(bf16x8_t, xfrag), acc[h], 0, 0, 0);
                }
            }
        }
    }

    if constexpr (!AGENT_STORES) after_loop(lw == 0 && live);
    // ---- add the wavefronts' partial sums (the rings are dead: reuse them) ---------------------------
    // per row group: [gate partial sums of the W K ranges | up partial sums][64]; the paired mode keeps the up sums of
    // all wavefronts behind the gate sums of all wavefronts
    f32x4_t* red = reinterpret_cast<f32x4_t*>(red_lds ? red_lds : lds);
    if constexpr (AGENT_STORES) {
        // no workgroup barrier: a wavefront leaves its partial sums, counts itself in for its row group and is free; the
        // group's storing wavefront waits for the group's count only (its partners are running and wait for nothing)
        uint32_t* cnt = reinterpret_cast<uint32_t*>(red + waves * 64) + grp;
        red[lwave * 64 + lane] = acc[0];
        if (lane == 0) __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        after_loop(lw == 0 && live);   // (behind the partial sums: what it requests must not hold them up)
        if (lw != 0 || !live) return;
        while (__hip_atomic_load(cnt, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < (uint32_t)wpg) __builtin_amdgcn_s_sleep(1);
    } else {
        __syncthreads();
        red[lwave * 64 + lane] = acc[0];
        if constexpr (PAIRED) red[(waves + lwave) * 64 + lane] = acc[NQ - 1];
        __syncthreads();
    }
    if (lw != 0 || !has_x || !live) return;
    f32x4_t sum = red[wbase * 64 + lane];
    for (int w = 1; w < W; w++) {
        const f32x4_t v = red[(wbase + w) * 64 + lane];
        sum[0] += v[0]; sum[1] += v[1]; sum[2] += v[2]; sum[3] += v[3];
    }
    const int m = r;
    const int64_t n = n0 + 4 * g;
    float o[4];
    if constexpr (GATED) {
        const int ubase = PAIRED ? waves + wbase : wbase + W;
        f32x4_t up = red[ubase * 64 + lane];
        for (int w = 1; w < W; w++) {
            const f32x4_t v = red[(ubase + w) * 64 + lane];
            up[0] += v[0]; up[1] += v[1]; up[2] += v[2]; up[3] += v[3];
        }
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const float gt = bf16_to_f32(f32_to_bf16(sum[v]));
            const float ut = bf16_to_f32(f32_to_bf16(up[v]));
            const float sl = bf16_to_f32(f32_to_bf16(gt / (1.0f + expf(-gt))));
            o[v] = sl * ut;
        }
    } else {
#pragma unroll
        for (int v = 0; v < 4; v++) o[v] = n + v < N ? add_residual(sum[v] + (bias ? bf16_to_f32(bias[n + v]) : 0.f), residual, (int64_t)m * N + n + v) : 0.f;
        if (amax) {
            // arg-max form: this row group's best (value, column) per activation row instead of the outputs
            uint64_t key = 0;
#pragma unroll
            for (int v = 0; v < 4; v++)
                if (n + v < N) key = u64_max(key, argmax_key(o[v], n + v));
            argmax_store(key, g, amax, m, (int64_t)bid * gpw + grp, (N + 15) >> 4);
            return;
        }
    }
    bf16_t* yr = y + (int64_t)m * N + n;
    if (n + 3 < N && (N & 3) == 0) {
        if constexpr (AGENT_STORES) {
            uint64_t* yt = reinterpret_cast<uint64_t*>(y) + (((int64_t)m * N + n) >> 1);
            __hip_atomic_store(yt, (uint64_t)pack_bf16(o[0], o[1]) | ((uint64_t)tag << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(yt + 1, (uint64_t)pack_bf16(o[2], o[3]) | ((uint64_t)tag << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            *reinterpret_cast<u32x2_t*>(yr) = u32x2_t{pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3])};
        }
    } else {
        // (a ragged N: plain stores; the one caller with AGENT_STORES has N % 4 == 0)
#pragma unroll
        for (int v = 0; v < 4; v++)
            if (n + v < N) yr[v] = f32_to_bf16(o[v]);
    }
}

template <int NUM, bool GATED, int WMAX, bool XLDS, bool PAIRED = false>
__global__ __launch_bounds__(64 * WMAX) void gemv_q8_span_kernel(const bf16_t* __restrict__ x, int M,
                                                                 const uint8_t* __restrict__ qa,
                                                                 const uint8_t* __restrict__ qb, int64_t N, int64_t K,
                                                                 const bf16_t* __restrict__ bias, const bf16_t* residual, bf16_t* __restrict__ y,
                                                                 const bf16_t* __restrict__ gamma, float eps, uint64_t* __restrict__ amax,
                                                                 int gpw, int skew) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    gemv_q8_span_body<NUM, GATED, WMAX, XLDS, PAIRED, false>(lds, x, M, qa, qb, N, K, bias, residual, y, gamma, eps, amax, gpw, skew,
                                                             (int)blockIdx.x, [](bool) {});
}

// ---- the SiLU-gated MLP of a decoder layer at decode sizes in ONE launch --------------------------------------
// down(silu(gate(x)) * up(x)) (Qwen3MLP.forward, modeling_qwen3.py:214-216), optionally with the RMSNorm in front
// (post_attention_layernorm, :938) and the residual add behind it (:941).  Workgroup b first works as workgroup b of
// the line-aligned gated pair (three 16-row groups of the gate / up matrices, twelve wavefronts) and writes its 48 gated
// activations; then it contracts 16 rows of the down matrix with ALL gated activations, K split over its twelve
// wavefronts, four steps of 8 blocks each.  The down-projection weights do not depend on the activations:
//   * a wavefront requests its first two steps into registers the moment it leaves the first loop, hands in its
//     partial sums, moves the two steps into LDS and decodes them to matrix-core operands;
//   * once the whole workgroup has left the first phase (one barrier) every wavefront requests steps 3 and 4 and
//     decodes them too - all of it while the slowest compute units still deliver activations;
//   * when the activations of its K range are there, 32 matrix instructions and the reduction over the twelve
//     wavefronts are all that is left.
// So the memory system and the vector ALU stay busy through what would be the tail of one kernel, the launch gap
// and the start of the next (35.9 us against 38.8 us for the two launches at M = 1, same process).
//
// Hand-over between workgroups of one launch: the activations travel as 8-byte words { two bf16, generation tag },
// each written with one agent-scope store, so a word that shows this launch's tag carries this launch's data whatever
// order the stores arrive in.  Behind its 16 outputs a row group also stores the tag into its flag.  A consumer
// wavefront polls the 64 flags of the row groups its K range needs (one 4-byte agent-scope load per lane and poll, at
// most `spin_limit` polls), then reads the words and checks every tag (a flag may overtake data; then it reads again).
// The generation comes from MlpCtl at the start of the workspace (zero before its first use); the last workgroup to
// finish the kernel (a trailing counter that nobody waits for) advances it, so replays of a captured launch need no
// clearing in between.  All workgroups must be resident together (one per compute unit: the launcher checks the
// device's unit count and the kernel's occupancy); if the poll limit is hit - another launch holding compute units for
// that long - the wavefront sets `status`, goes on with whatever the words hold and the kernel still ends normally.
// Inside a workgroup the first phase uses no barrier either: a wavefront leaves its partial sums in LDS and counts
// itself in for its row group, and only that group's storing wavefront waits for the count.
#ifdef SNGGUF_MLP_TRACE
__device__ uint64_t g_mlp_trace[256 * 12 * 8];
#define MLP_TRACE(slot) do { if (lane == 0) g_mlp_trace[((int)blockIdx.x * 12 + wave) * 8 + (slot)] = wall_clock64(); } while (0)
#else
#define MLP_TRACE(slot) do { } while (0)
#endif

constexpr int kMlpWaveLds = 16 * kRingRow;   // per wavefront: its ring of the first phase; in the second phase one slab
                                             // (4352 bytes) and the staged activations of rows 0 and 1 (2 x 2048 bytes)

template <int NUM>
__global__ __launch_bounds__(768) void mlp_q8_decode_kernel(const bf16_t* __restrict__ x, int M, const uint8_t* __restrict__ q_gate,
                                                            const uint8_t* __restrict__ q_up, const uint8_t* __restrict__ q_down,
                                                            int64_t hidden, int64_t inter, const bf16_t* __restrict__ gamma, float eps,
                                                            const bf16_t* residual, bf16_t* __restrict__ y, MlpCtl* ctl,
                                                            uint64_t* ht, int spin_limit) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int CB = 8, kWaves = 12;
    constexpr int kRowStep = CbGeom<CB>::kRowStep, kLoads = CbGeom<CB>::kLoads, kSlab = CbGeom<CB>::kSlab;
    static_assert(kMlpWaveLds == kSlab + 2 * 2048, "a slab and two staged activation rows take the place of a wavefront's ring");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bid = (int)blockIdx.x, nb = (int)gridDim.x;
    const int r = lane & 15, g = lane >> 4;
    MLP_TRACE(0);
    // this launch's tag: nobody advances the generation before every workgroup, this one included, has finished
    const uint32_t gen = __hip_atomic_load(&ctl->gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t tag = gen + 1u;

    // LDS: [12 x (ring of the first phase | slab and staged activation rows of the second)] [x staged for the first
    // phase (M rows)] [partial sums and counters of the first phase]
    uint8_t* const after_rings = lds + kWaves * kMlpWaveLds;
    uint8_t* const red_a = after_rings + (((size_t)M * (2 * hidden + 64) + (gamma ? 4 * M * kWaves : 0) + 255) & ~(size_t)255);

    // ---- down projection, geometry: rows [16 bid, +16), this wavefront's steps [s0, s0 + nst) of 8 blocks ----
    constexpr int kSteps = 4;   // steps per wavefront: inter = 12 wavefronts x 4 steps x 256 elements (the launcher checks)
    const int s0 = wave * kSteps;
    const int64_t drow_bytes = (inter >> 5) * 34;
    const uint8_t* __restrict__ dbase = q_down + (int64_t)bid * 16 * drow_bytes;
    u32x4_t pre[kLoads], pre2[kLoads];
    auto dfetch = [&](int s, u32x4_t (&dst)[kLoads]) {
        const uint8_t* p = dbase + (int64_t)s * kRowStep;
#pragma unroll
        for (int i = 0; i < kLoads; i++) {
            const int f = lane + 64 * i;
            const bool ok = f < CbGeom<CB>::kPieces;
            const int fr = ok ? f / CbGeom<CB>::kRowPieces : 0, fp = ok ? f % CbGeom<CB>::kRowPieces : 0;
            if (ok) dst[i] = *reinterpret_cast<const u32x4_t*>(p + fr * drow_bytes + 16 * fp);
        }
    };
    uint8_t* const slab0 = lds + wave * kMlpWaveLds;
    auto to_slab = [&](const u32x4_t (&src)[kLoads]) {
#pragma unroll
        for (int i = 0; i < kLoads; i++)
            if (lane + 64 * i < CbGeom<CB>::kPieces) *reinterpret_cast<u32x4_t*>(slab0 + 16 * (lane + 64 * i)) = src[i];
    };

    // ---- decode the four steps into matrix-core operands while the activations are still on their way ----
    // (this wavefront's ring is its own again; the vector ALU has room while other wavefronts wait for memory, and once
    // the activations are there only the 32 matrix instructions are left)
    u32x4_t afrag[kSteps * CB];
    const half4_t ident = identity_row(lane);
    auto decode = [&](int i) {
        const uint8_t* sl = slab0;
        const uint8_t* lrow = sl + r * kRowStep + 8 * g;
#pragma unroll
        for (int b = 0; b < CB; b++) {
            const uint16_t d = *reinterpret_cast<const uint16_t*>(sl + r * kRowStep + 34 * b);
            uint32_t q0, q1;
            if ((b & 1) == 0) {
                const uint32_t* w = reinterpret_cast<const uint32_t*>(lrow + 34 * b);
                const uint32_t w0v = w[0], w1v = w[1], w2v = w[2];
                q0 = __builtin_amdgcn_alignbit(w1v, w0v, 16);
                q1 = __builtin_amdgcn_alignbit(w2v, w1v, 16);
            } else {
                const uint32_t* w = reinterpret_cast<const uint32_t*>(lrow + 34 * b + 2);
                q0 = w[0];
                q1 = w[1];
            }
            uint32_t a0, a1, a2, a3;
            // the fp16 -> fp32 step of the decode on the matrix cores: this phase is bound by the vector ALU (36.3 ->
            // 35.1 us for the launch; in the first phase, which waits for memory, and in the separate launches it gains
            // nothing or loses)
            const uint32_t d2 = (uint32_t)d | ((uint32_t)d << 16);
            q8_dword_bf16_widened<NUM>(ident, d2, q0, a0, a1);
            q8_dword_bf16_widened<NUM>(ident, d2, q1, a2, a3);
            // (pinned here: left alone, the compiler moves the roundings down to the matrix instructions behind the wait
            // and keeps the widened values, twice the registers, across it)
            asm volatile("" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));
            afrag[i * CB + b] = u32x4_t{a0, a1, a2, a3};
        }
    };
    // ---- gate / up / SiLU: activations [48 bid, +48) of every row, as tagged words ----
    // Measured on 12288 x 4096 at M = 1 against the two separate launches in one process (37.3 ... 39.5 us, by device):
    // every wavefront fetching and decoding all four steps as soon as it is free, no barrier, 40.4 us (56 us when only
    // the first few to arrive do so); a workgroup barrier before steps 2 and 3 are requested and all decoding behind it
    // 36.6 ... 37.1 us; steps 0 and 1 decoded in front of that barrier by every wavefront 35.5 us (by the first six or
    // eight to arrive only: 36.4 us).  The last wavefronts to leave the loop requesting all four steps at once: no gain.
    // (a counter of the first phase's area that no row group uses: the body zeroes sixteen of them in front of its first barrier)
    uint32_t* const left_a = reinterpret_cast<uint32_t*>(reinterpret_cast<f32x4_t*>(red_a) + kWaves * 64) + 8;
    __builtin_amdgcn_s_setprio(2);   // the first phase is what every other workgroup waits for
    gemv_q8_span_body<NUM, true, 12, true, false, true>(
        lds, x, M, q_gate, q_up, inter, hidden, nullptr, nullptr, reinterpret_cast<bf16_t*>(ht), gamma, eps, nullptr, 3, 1, bid,
        [&](bool stores) {
            MLP_TRACE(1);
            // the first two down-projection steps, requested the moment this wavefront leaves the loop
            dfetch(s0, pre);
            dfetch(s0 + 1, pre2);
            // counted as having left the loop: the other two steps are requested when that count is full
            if (lane == 0) __hip_atomic_fetch_add(left_a, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        },
        tag, kMlpWaveLds, red_a);
    // a wavefront that wrote a row group's activations also raises that group's flag (behind the data, unordered)
    {
        // the body's storing wavefronts are those with lw == 0 in its [group][matrix][K half] order: recomputed here
        const int slot = wave >> 2, i4 = wave & 3;
        const int pair = slot == 1 ? 4 + (i4 >> 1) : i4;
        const int khalf = slot == 1 ? (i4 & 1) : (slot >> 1);
        const int lwave = 2 * pair + khalf;
        if ((lwave & 3) == 0 && lane == 0)
            __hip_atomic_store(&ctl->flags[3 * bid + (lwave >> 2)], tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_s_setprio(0);
    MLP_TRACE(2);
    // steps 0 and 1 move into LDS and are decoded at once, at the lowest priority (this wavefront's partial sums are
    // counted in: nobody waits for it); steps 2 and 3 are requested only when every wavefront of the workgroup has left
    // the first phase's loop - requested earlier, their traffic slows the first phase's last wavefronts, which every
    // workgroup waits for.  (A count that a wavefront joins when it leaves the loop, not a barrier behind the two decode
    // steps: with the barrier the workgroup's last wavefront held the others' requests back by its own two steps,
    // 35.0 against 33.5 us for the launch.  The requests at the loop's end behind the storing wavefront's whole epilogue
    // (partners awaited, activations and flag stored first): 34.1 us.  Each register set refilled the moment it is free, which moves the last two
    // requests in front of the first two decode steps: 35.1 us; only one step requested at the loop's end: 34.7 us.)
    to_slab(pre);
    decode(0);
    to_slab(pre2);
    decode(1);
    while (__hip_atomic_load(left_a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < (uint32_t)kWaves) __builtin_amdgcn_s_sleep(1);
    dfetch(s0 + 2, pre);
    dfetch(s0 + 3, pre2);
    to_slab(pre);
    decode(2);
    to_slab(pre2);
    decode(3);
    MLP_TRACE(6);
    MLP_TRACE(3);

    // ---- wait for this wavefront's K range of the activations ----
    // staged (tags stripped), 2048 bytes per row, behind this wavefront's slab (at most two rows: the launcher checks);
    // fragment (step i, block b) of a row at ((i CB + b) 64 + 16 g)
    // (Requesting the words in front of the last decode step, on the expectation that they are there, and polling only
    // if a tag says otherwise, gained nothing: the last activations become visible about when the last weights arrive.)
    constexpr int xrow_b = kSteps * CB * 64;
    auto xw_row = [&](int m) -> uint8_t* { return slab0 + kSlab + m * xrow_b; };
    {
        const int pairs = kSteps * CB * 8;            // 16-byte pairs of words per row in this wavefront's K range (256)
        const int64_t w0 = (int64_t)s0 * CB * 16;     // first word of the range within a row
        const int64_t row_words = inter >> 1;
        // the row groups whose outputs are this range: 16 outputs each
        const int g0 = (s0 * CB * 32) >> 4, ng = (kSteps * CB * 32) >> 4;
        int polls = 0;
        bool gave_up = false;
        for (;;) {
            bool all = true;
            for (int j = lane; j < ng; j += 64) all = all && __hip_atomic_load(&ctl->flags[g0 + j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == tag;
            if (__builtin_amdgcn_ballot_w64(!all) == 0) break;
            if (++polls > spin_limit) { gave_up = true; break; }
            __builtin_amdgcn_s_sleep(2);
        }
        for (;;) {
            bool all = true;
            for (int m = 0; m < M; m++)
                for (int c = lane; c < pairs; c += 64) {
                    const uint64_t* src = ht + (int64_t)m * row_words + w0 + 2 * c;
                    const uint64_t a = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const uint64_t b = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    all = all && (uint32_t)(a >> 32) == tag && (uint32_t)(b >> 32) == tag;
                    *reinterpret_cast<uint64_t*>(xw_row(m) + 8 * c) = (uint64_t)(uint32_t)a | (b << 32);
                }
            if (gave_up || __builtin_amdgcn_ballot_w64(!all) == 0) break;
            if (++polls > spin_limit) { gave_up = true; break; }
        }
        if (gave_up && lane == 0) __hip_atomic_store(&ctl->status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    MLP_TRACE(4);

    // ---- contract ----
    __builtin_amdgcn_s_setprio(3);
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    const bool has_x = r < M;
    const uint8_t* xwrow = xw_row(has_x ? r : M - 1) + 16 * g;
#pragma unroll
    for (int i = 0; i < kSteps * CB; i++) {
        const u32x4_t xfrag = *reinterpret_cast<const u32x4_t*>(xwrow + i * 64);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, afrag[i]), __builtin_bit_cast(bf16x8_t, xfrag), acc, 0, 0, 0);
    }

    // ---- add the wavefronts' partial sums, residual, store ----
    __syncthreads();
    f32x4_t* red = reinterpret_cast<f32x4_t*>(lds);  // [waves][64]
    red[wave * 64 + lane] = acc;
    __syncthreads();
    if (wave == 0 && has_x) {
        f32x4_t sum = red[lane];
        for (int w = 1; w < kWaves; w++) {
            const f32x4_t t = red[w * 64 + lane];
            sum[0] += t[0]; sum[1] += t[1]; sum[2] += t[2]; sum[3] += t[3];
        }
        const int64_t n = (int64_t)bid * 16 + 4 * g;
        float o[4];
#pragma unroll
        for (int v = 0; v < 4; v++) o[v] = add_residual(sum[v], residual, (int64_t)r * hidden + n + v);
        *reinterpret_cast<u32x2_t*>(y + (int64_t)r * hidden + n) = u32x2_t{pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3])};
    }
    MLP_TRACE(5);
    if (tid == 0) {
        const uint32_t old = __hip_atomic_fetch_add(&ctl->done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old == (uint32_t)nb - 1u) {
            __hip_atomic_store(&ctl->done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&ctl->gen, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

#ifdef SNGGUF_MLP_TRACE
extern "C" int sngguf_debug_mlp_trace(void* host_out) {
    return (int)hipMemcpyFromSymbol(host_out, HIP_SYMBOL(g_mlp_trace), sizeof(g_mlp_trace));
}
#endif

int64_t mlp_q8_decode_workspace_bytes(int64_t M, int64_t inter) { return kMlpCtlBytes + ((4 * M * inter + 255) & ~(int64_t)255); }
int64_t mlp_q8_decode_ctl_bytes() { return kMlpCtlBytes; }
int64_t mlp_q8_decode_status_offset() { return (int64_t)offsetof(MlpCtl, status); }

// Shapes the one-launch form takes: Q8_0 everywhere; hidden = 4096 (two spans per row: the twelve-wavefront form of
// the gated pair); inter = 3 hidden (as many 48-row slices of gate / up as 16-row groups of down: one of each per
// workgroup) and 12 wavefronts x 4 steps x 256 elements of it per row of the down projection; one or two rows (their staged
// copies fit behind a wavefront's slab; three and four rows, staged and contracted two at a time, came out level with
// the separate launches, 38.7 - 39.9 against 39.1 - 40.7 us: every workgroup reads every row's tagged words, 12.5 MB of
// coherent reads per row over the device behind the last weights); as many compute units as workgroups and the kernel
// resident on each.
bool mlp_q8_decode_fits(int64_t M, int64_t hidden, int64_t inter) {
    if (M < 1 || M > 2 || hidden != 4096 || inter != 3 * hidden || inter != 12 * 4 * 256) return false;
    static const int ok = [] {
        int dev = 0, cus = 0, per_cu = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        for (const void* k : {reinterpret_cast<const void*>(&mlp_q8_decode_kernel<0>), reinterpret_cast<const void*>(&mlp_q8_decode_kernel<1>)}) {
            if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) return 0;
        }
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, mlp_q8_decode_kernel<1>, 768, 160 * 1024) != hipSuccess) return 0;
        return per_cu >= 1 ? cus : 0;
    }();
    return ok >= inter / 48;
}

// x [M][hidden], y [M][hidden], residual (may be null) [M][hidden] bf16; gamma (may be null) [hidden]; workspace as
// mlp_q8_decode_workspace_bytes says, its first kMlpCtlBytes zero before the first use and left alone between calls.
int launch_mlp_q8_decode(const void* x, int64_t M, const void* gamma, float eps, const void* q_gate, const void* q_up, const void* q_down,
                         int64_t hidden, int64_t inter, const void* residual, void* y, void* workspace, int numerics, int spin_limit,
                         hipStream_t stream) {
    if (!mlp_q8_decode_fits(M, hidden, inter)) return SNGGUF_E_BADSHAPE;
    // [12 x ring] + x staged + sums of squares + partial sums and counters of the first phase
    const size_t lds_bytes = (size_t)12 * kMlpWaveLds + (((size_t)M * (2 * hidden + 64) + (gamma ? (size_t)4 * M * 12 : 0) + 255) & ~(size_t)255) +
                             (size_t)12 * 64 * 16 + 64;
    if (lds_bytes > 160 * 1024) return SNGGUF_E_BADSHAPE;
    MlpCtl* ctl = static_cast<MlpCtl*>(workspace);
    uint64_t* h = reinterpret_cast<uint64_t*>(static_cast<uint8_t*>(workspace) + kMlpCtlBytes);
    const dim3 grid((unsigned)(inter / 48)), block(768);
    const int limit = spin_limit == 0 ? 1 << 20 : spin_limit < 0 ? 0 : spin_limit;
#define SNGGUF_MLP(NUMV) \
    mlp_q8_decode_kernel<NUMV><<<grid, block, lds_bytes, stream>>>(static_cast<const bf16_t*>(x), (int)M, static_cast<const uint8_t*>(q_gate), \
        static_cast<const uint8_t*>(q_up), static_cast<const uint8_t*>(q_down), hidden, inter, static_cast<const bf16_t*>(gamma), eps, \
        static_cast<const bf16_t*>(residual), static_cast<bf16_t*>(y), ctl, h, limit)
    if (numerics == SNGGUF_NUM_GGML_FP32) SNGGUF_MLP(0);
    else SNGGUF_MLP(1);
#undef SNGGUF_MLP
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

template <int NUM>
static int launch_span(const bf16_t* x, int M, const uint8_t* qa, const uint8_t* qb, int64_t N, int64_t K,
                       const bf16_t* bias, const bf16_t* residual, bf16_t* y, bool gated, const bf16_t* gamma, float eps,
                       hipStream_t stream, uint64_t* amax) {
    const int64_t groups = (N + 15) / 16;
    const int spans = (int)(K >> 11);
    int w = spans < 8 ? spans : 8;                 // one wavefront per span, at most 8 per row group
    if (gated && w > 4) w = 4;
    // (no cap for many row groups: a 151936-row projection runs 3 - 5 % faster with two wavefronts per group than with one)
    // stage the activations in LDS when they are small enough to leave room for a compute unit's worth of rings
    const size_t x_bytes = (size_t)M * (2 * K + 64);
    const size_t x_budget = groups >= 512 ? 48 * 1024 : 96 * 1024;   // (5 rows at K = 4096: M = 4 gate/up 24.6 against 25.1 us fetched per wavefront)
    const bool xlds = x_bytes <= x_budget;
    // activations fetched from global memory for a gated pair: one wavefront takes both matrices of its K range
    const bool paired = gated && !xlds && M >= kPairedMinM;
    const int wpg = (gated && !paired) ? 2 * w : w;                       // wavefronts per row group
    const size_t ring_per_wave = (size_t)(paired ? 2 : 1) * 16 * kRingRow;
    if (gamma && !xlds) return SNGGUF_E_BADSHAPE;   // the norm is applied to activations staged in LDS
    // Row groups per workgroup: all (about 12) wavefronts of a compute unit in ONE workgroup.  Workgroups that arrive
    // on a compute unit one after the other keep the order of their first requests for the whole kernel - the last
    // one finishes microseconds after the first - while the wavefronts of one workgroup start together and share
    // one staged copy of the activations.
    auto lds_for = [&](int g) {
        const size_t wv = (size_t)g * wpg;
        return wv * ring_per_wave + (xlds ? x_bytes : 0) + (gamma ? (((size_t)4 * M * wv + 15) & ~(size_t)15) : 0);
    };
    int gpw = xlds ? 12 / wpg : 1;   // (without a staged copy to share, small workgroups did better: M = 16 gate/up 29.2 against 30.5 us)
    if (gpw < 1) gpw = 1;
    while (gpw > 1 && (lds_for(gpw) > 160 * 1024 || groups < (int64_t)256 * gpw)) gpw--;
    const int waves = gpw * wpg;
    const size_t lds_bytes = lds_for(gpw);
    if (lds_bytes > 160 * 1024) return SNGGUF_E_BADSHAPE;
    const dim3 grid((unsigned)((groups + gpw - 1) / gpw)), block((unsigned)(64 * waves));
    // one extra step for the first-placed wavefront of each K range, one less for the last-placed (12288 x 4096 gate/up at
    // M = 1, extra steps 0 / 1 / 2 / 3: 24.5 / 23.9 / 24.3 / 24.4 us; per-wavefront loop ends by placement 16.8 / 17.7 / 19.6 us
    // unskewed, 18.4 / 18.4 / 19.6 us with one step moved)
    constexpr int kSkewSteps = 1;
    const int skew = (xlds && waves == 12 && spans == 2 && w == 2) ? kSkewSteps : 0;
    // the rings of a dozen wavefronts plus staged activations exceed the default dynamic-LDS limit: raise it once per
    // kernel instance
#define SNGGUF_LAUNCH_ONE(G, WM, XL, PR) \
    do { \
        static const hipError_t attr = hipFuncSetAttribute( \
            reinterpret_cast<const void*>(&gemv_q8_span_kernel<NUM, G, WM, XL, PR>), \
            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
        if (attr != hipSuccess) return SNGGUF_E_LAUNCH; \
        gemv_q8_span_kernel<NUM, G, WM, XL, PR><<<grid, block, lds_bytes, stream>>>(x, M, qa, qb, N, K, bias, residual, y, gamma, eps, amax, gpw, skew); \
    } while (0)
#define SNGGUF_LAUNCH(G, XL, PR) \
    do { \
        if (waves <= 4) SNGGUF_LAUNCH_ONE(G, 4, XL, PR); \
        else if (waves <= 8) SNGGUF_LAUNCH_ONE(G, 8, XL, PR); \
        else SNGGUF_LAUNCH_ONE(G, 12, XL, PR); \
    } while (0)
    if (paired) SNGGUF_LAUNCH(true, false, true);
    else if (gated && xlds) SNGGUF_LAUNCH(true, true, false);
    else if (gated) SNGGUF_LAUNCH(true, false, false);
    else if (xlds) SNGGUF_LAUNCH(false, true, false);
    else SNGGUF_LAUNCH(false, false, false);
#undef SNGGUF_LAUNCH
#undef SNGGUF_LAUNCH_ONE
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

// How many wavefronts share the K range of one 16-row group: enough that the launch fills the
// chip (about 12 wavefronts on each of the 256 compute units), at least one step each.
static int pick_k_split(int64_t groups, int steps, bool gated) {
    const int64_t per_group = gated ? 2 : 1;
    int64_t w = (256 * 12 + groups * per_group - 1) / (groups * per_group);
    if (w < 1) w = 1;
    if (w > steps) w = steps;
    // at most 8 wavefronts per workgroup, 12 where that leaves a wavefront one or two steps (K up to 4096: everything
    // is requested at once and the launch is as long as its slowest wavefront - 4096 x 4096 at M = 1 7.1 against 7.5 us,
    // 1024 x 4096 5.9 against 6.1; with four steps each, 4096 x 12288, twelve lose 2 % to eight)
    const int64_t cap = gated ? 4 : (steps <= 16 ? 12 : 8);
    if (w > cap) w = cap;
    return (int)w;
}

template <int NUM, int CB>
static int launch_cb(const bf16_t* x, int M, const uint8_t* qa, const uint8_t* qb, int64_t N, int64_t K,
                     const bf16_t* bias, const bf16_t* residual, bf16_t* y, bool gated, const bf16_t* gamma, float eps,
                     hipStream_t stream, uint64_t* amax) {
    const int64_t groups = (N + 15) / 16;
    const int steps = (int)(K / (32 * CB));
    const int w = pick_k_split(groups, steps, gated);
    const int waves = gated ? 2 * w : w;
    const dim3 grid((unsigned)groups), block((unsigned)(64 * waves));
    if (gamma) {
        // slabs, then every wavefront's share of the activations ([M][xrow_b]), then [M][waves] sums of squares.
        // The caller keeps M (2 K + 64) within 36 KB; a gated pair stages the rows twice (gate and up wavefronts),
        // so with the slabs this can pass the default dynamic-LDS limit: raise it once per kernel instance
        const size_t xrow_b = (size_t)((steps + w - 1) / w) * CB * 64 + 16;
        const size_t lds_norm = (size_t)waves * 16 * CB * 34 + (size_t)waves * M * xrow_b + (((size_t)4 * M * waves + 15) & ~(size_t)15);
        if (lds_norm > 160 * 1024) return SNGGUF_E_BADSHAPE;
#define SNGGUF_LAUNCH_XN(G, WM)                                                                                         \
    do {                                                                                                                \
        static const hipError_t attr = hipFuncSetAttribute(                                                             \
            reinterpret_cast<const void*>(&gemv_q8_mfma_kernel<NUM, CB, G, WM, true>),                                   \
            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);                                                     \
        if (attr != hipSuccess) return SNGGUF_E_LAUNCH;                                                                  \
        gemv_q8_mfma_kernel<NUM, CB, G, WM, true><<<grid, block, lds_norm, stream>>>(x, M, qa, qb, N, K, bias, residual, \
                                                                                     y, gamma, eps, amax);              \
    } while (0)
        if (gated) {
            if (waves <= 4) SNGGUF_LAUNCH_XN(true, 4);
            else SNGGUF_LAUNCH_XN(true, 8);
        } else {
            if (waves <= 4) SNGGUF_LAUNCH_XN(false, 4);
            else if (waves <= 8) SNGGUF_LAUNCH_XN(false, 8);
            else SNGGUF_LAUNCH_XN(false, 12);
        }
#undef SNGGUF_LAUNCH_XN
        return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
    }
    const size_t lds_bytes = (size_t)waves * 16 * CB * 34;
    // WMAX only sets the register budget the compiler may assume for the workgroup size
#define SNGGUF_LAUNCH(G, WM) gemv_q8_mfma_kernel<NUM, CB, G, WM><<<grid, block, lds_bytes, stream>>>(x, M, qa, qb, N, K, bias, residual, y, nullptr, 0.f, amax)
    if (gated) {
        if (waves <= 4) SNGGUF_LAUNCH(true, 4);
        else SNGGUF_LAUNCH(true, 8);
    } else {
        if (waves <= 4) SNGGUF_LAUNCH(false, 4);
        else if (waves <= 8) SNGGUF_LAUNCH(false, 8);
        else SNGGUF_LAUNCH(false, 12);
    }
#undef SNGGUF_LAUNCH
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

template <int NUM>
static int launch_q8(const bf16_t* x, int M, const uint8_t* qa, const uint8_t* qb, int64_t N, int64_t K,
                     const bf16_t* bias, const bf16_t* residual, bf16_t* y, bool gated, const bf16_t* gamma, float eps,
                     hipStream_t stream, uint64_t* amax) {
    // The line-aligned variant needs whole 2048-element spans per wavefront; with few row groups
    // that leaves the chip short of wavefronts, and the block-aligned variant (which can cut K
    // every 256 elements) is the better fit.
    // (12288 -> 4096, 1536 such wavefronts, block-aligned / line-aligned us: M=1 15.0 / 17.4, M=4 15.9 / 16.3,
    // M=16 21.6 / 19.3 - with a dozen rows the fewer, longer wavefronts of the line-aligned variant fetch fewer
    // activation fragments per weight byte in flight, so the bar is lower there; 4096 -> 4096 loses at every M)
    const int64_t span_waves = ((N + 15) / 16) * (K >> 11) * (gated ? 2 : 1);
    if (K % 2048 == 0 && span_waves >= (M >= 12 ? 1536 : 2048))
        return launch_span<NUM>(x, M, qa, qb, N, K, bias, residual, y, gated, gamma, eps, stream, amax);
    return launch_cb<NUM, 8>(x, M, qa, qb, N, K, bias, residual, y, gated, gamma, eps, stream, amax);
}

// Q8_0, 1 <= M <= 16, K % 256 == 0, 16-byte aligned rows (checked by the caller).  `gamma` (K bf16, 16-byte
// aligned) switches the fused RMSNorm on; the caller keeps M (2 K + 64) <= 36 KB then.  `amax` (plain projections
// only): instead of y, every workgroup writes its best (value, column) key per activation row to
// amax[m * ceil(N / 16) + workgroup].
int launch_gemv_q8_mfma(const void* x, int64_t M, const void* qa, const void* qb, int64_t N, int64_t K, const void* bias,
                        const void* residual, void* y, int numerics, bool gated, hipStream_t stream, const void* gamma,
                        float eps, uint64_t* amax) {
    if (amax && gated) return SNGGUF_E_BADSHAPE;
    const bf16_t* xp = static_cast<const bf16_t*>(x);
    const uint8_t* a = static_cast<const uint8_t*>(qa);
    const uint8_t* b = static_cast<const uint8_t*>(qb);
    const bf16_t* bp = static_cast<const bf16_t*>(bias);
    const bf16_t* rp = static_cast<const bf16_t*>(residual);
    bf16_t* yp = static_cast<bf16_t*>(y);
    const bf16_t* gp = static_cast<const bf16_t*>(gamma);
    if (numerics == SNGGUF_NUM_GGML_FP32) return launch_q8<SNGGUF_NUM_GGML_FP32>(xp, (int)M, a, b, N, K, bp, rp, yp, gated, gp, eps, stream, amax);
    if (numerics == SNGGUF_NUM_UPSTREAM_FP16) return launch_q8<SNGGUF_NUM_UPSTREAM_FP16>(xp, (int)M, a, b, N, K, bp, rp, yp, gated, gp, eps, stream, amax);
    return SNGGUF_E_BADTYPE;
}

}  // namespace sngguf
