// Q8_0 decode GEMV (1 <= M <= 16, K % 256 == 0) on the operand-order ("tiled") weight layout, an opt-in copy of
// the weights made once at load time for models that stay resident on the device.
//
// Layout of one tiled matrix (N rows padded to G = ceil(N / 16) row groups, B = K / 32 blocks per row):
//   quants   [G][B / 2][64 lanes][16 bytes]   lane 16 g + r holds bytes 8 g .. 8 g + 7 of block 2 p of row 16 rg + r,
//                                             then the same eight bytes of block 2 p + 1
//   scales   [G][B / 8][16 rows][8 halves]    the block scales of a run of eight blocks, row after row
// (quants first, scales behind them at byte offset 16 G K; rows >= N are zero).  It holds exactly the bits of the
// GGUF rows - 34 bytes per block - in the order the matrix instruction consumes them: lane (r, g) of
// v_mfma_f32_16x16x32_bf16 supplies elements 8 g .. 8 g + 7 of weight row r.  Every wavefront load is one
// contiguous 1 KB (quants) or 256 bytes (scales) and lands in operand order, so the weights need no LDS round
// trip and no realignment of 34-byte blocks; decode, rounding chain and contraction are those of the kernels
// for the GGUF-native layout.
#include "sngguf_common.hpp"

namespace sngguf {

namespace {

// ---- GGUF-native rows -> tiled ----------------------------------------------------------------------------
// One thread per (row group, block, lane): eight quant bytes; lanes 0..15 of every block also move the scale.
__global__ __launch_bounds__(256) void q8_0_tile_kernel(const uint8_t* __restrict__ q, int64_t N, int64_t K,
                                                        uint8_t* __restrict__ tq, uint16_t* __restrict__ ts) {
    const int64_t B = K >> 5, G = (N + 15) >> 4;
    const int64_t total = G * B * 64;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int lane = (int)(t & 63);
        const int64_t gb = t >> 6, rg = gb / B, b = gb - rg * B;
        const int r = lane & 15, g = lane >> 4;
        const int64_t n = rg * 16 + r;
        uint32_t w0 = 0, w1 = 0;
        uint16_t d = 0;
        if (n < N) {
            const uint8_t* blk = q + (n * B + b) * 34;   // 2-byte aligned
            const uint16_t* h = reinterpret_cast<const uint16_t*>(blk + 2 + 8 * g);
            w0 = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
            w1 = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
            d = *reinterpret_cast<const uint16_t*>(blk);
        }
        uint32_t* dst = reinterpret_cast<uint32_t*>(tq + ((rg * (B >> 1) + (b >> 1)) * 64 + lane) * 16 + 8 * (b & 1));
        dst[0] = w0;
        dst[1] = w1;
        if (g == 0) ts[((rg * (B >> 3) + (b >> 3)) * 16 + r) * 8 + (b & 7)] = d;
    }
}

// ---- the GEMV --------------------------------------------------------------------------------------------------
// grid: row groups; block: W wavefronts that split the K range (GATED: 2 W, the second half on the up matrix).
// XLDS: the activations (M K bf16) are copied into LDS once per workgroup; otherwise each lane fetches its fragments
// from global memory one run ahead.
// PAIRED (gated): one wavefront works on the gate AND the up matrix of its K range, so that each activation fragment is
// fetched once for both - with several activation rows those fetches, not the weights, fill the vector memory path.
template <int NUM, bool GATED, int WMAX, bool XLDS, bool PAIRED = false>
__global__ __launch_bounds__(64 * WMAX) void gemv_q8_tiled_kernel(const bf16_t* __restrict__ x, int M,
                                                                  const uint8_t* __restrict__ ta, const uint8_t* __restrict__ tb,
                                                                  int64_t N, int64_t K, const bf16_t* __restrict__ bias,
                                                                  const bf16_t* residual, bf16_t* __restrict__ y,
                                                                  const bf16_t* __restrict__ gamma, float eps) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    static_assert(!PAIRED || GATED, "a pair is the gate and the up matrix");
    constexpr int NQ = PAIRED ? 2 : 1;   // matrices per wavefront
    const int waves = blockDim.x >> 6;
    const int W = (GATED && !PAIRED) ? waves >> 1 : waves;
    const int kw = (GATED && !PAIRED) ? (wave >= W ? wave - W : wave) : wave;
    const uint8_t* __restrict__ t = (GATED && !PAIRED && wave >= W) ? tb : ta;
    const int r = lane & 15, g = lane >> 4;
    const int64_t rg = blockIdx.x, G = (N + 15) >> 4;
    const int runs = (int)(K >> 8);                       // runs of eight blocks
    const int r0 = kw * runs / W, r1 = (kw + 1) * runs / W;
    // Bases in 64 bits once, everything inside the loop as 32-bit offsets (a group's quants are 16 K bytes, K < 2^27 is
    // checked by the launcher): with 64-bit index arithmetic per request the kernel measured 14.6 instead of 12.6 us.
    const uint8_t* __restrict__ qp = t + rg * (K >> 5) * 512 + 16 * lane;                  // + run * 4096 + pair * 1024
    const uint8_t* __restrict__ sp = t + 16 * G * K + rg * runs * 256 + 16 * r;            // + run * 256
    const int64_t pair_delta = PAIRED ? tb - ta : 0;                                       // the up matrix, same offsets

    const bool has_x = r < M;
    const int xr = has_x ? r : M - 1;   // columns >= M are never stored: those lanes re-read the last activation row
    const bf16_t* xrow = x + (int64_t)xr * K + 8 * g;
    const int xs_stride = 2 * (int)K + 64;                // bytes per activation row in LDS (+64: rows on different banks)
    const uint8_t* xsrow = lds + xr * xs_stride + 16 * g;

    u32x4_t wq[2][NQ][4], ws[2][NQ], xf[2][8];
    auto fetch = [&](int run, int buf) {
#pragma unroll
        for (int h = 0; h < NQ; h++) {
            const uint8_t* qh = qp + h * pair_delta;
            const uint8_t* sh = sp + h * pair_delta;
#pragma unroll
            // whole lines, each read once: non-temporal hint (gate/up at M = 1 22.5 -> 21.5 us, down 13.6 -> 13.0 us)
            for (int p = 0; p < 4; p++) wq[buf][h][p] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(qh + (uint32_t)(run * 4096 + p * 1024)));
            ws[buf][h] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(sh + (uint32_t)(run * 256)));
        }
        if constexpr (!XLDS) {
#pragma unroll
            for (int b = 0; b < 8; b++) xf[buf][b] = *reinterpret_cast<const u32x4_t*>(xrow + (uint32_t)((run * 8 + b) * 32));
        }
    };
    if (r0 < r1) fetch(r0, 0);   // the weights are requested before the activations are staged
    if constexpr (XLDS) {
        const int pieces_per_row = (int)(K >> 3);
        if (gamma == nullptr) {
            for (int m = 0; m < M; m++)
                for (int c = tid; c < pieces_per_row; c += (int)blockDim.x)
                    *reinterpret_cast<u32x4_t*>(lds + m * xs_stride + 16 * c) = *reinterpret_cast<const u32x4_t*>(x + (uint32_t)(m * (int)K + 8 * c));
        } else {
            // RMSNorm(x) with weight gamma is what gets contracted (see rmsnorm_piece): stage the rows, add up their
            // squares over the workgroup, then every thread normalizes the pieces it staged
            float* ssum = reinterpret_cast<float*>(lds + M * xs_stride);   // [M][waves]
            for (int m = 0; m < M; m++) {
                float ss = 0.f;
                for (int c = tid; c < pieces_per_row; c += (int)blockDim.x) {
                    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(x + (uint32_t)(m * (int)K + 8 * c));
                    *reinterpret_cast<u32x4_t*>(lds + m * xs_stride + 16 * c) = v;
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
                for (int c = tid; c < pieces_per_row; c += (int)blockDim.x) {
                    u32x4_t* cell = reinterpret_cast<u32x4_t*>(lds + m * xs_stride + 16 * c);
                    const u32x4_t gv = *reinterpret_cast<const u32x4_t*>(gamma + 8 * c);
                    *cell = rmsnorm_piece(*cell, gv, rstd);
                }
            }
        }
        __syncthreads();
    }

    f32x4_t acc[NQ];
#pragma unroll
    for (int q = 0; q < NQ; q++) acc[q] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    auto step = [&](int run, int buf) {
        if (run + 1 < r1) fetch(run + 1, buf ^ 1);
#pragma unroll
        for (int p = 0; p < 4; p++) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int b = 2 * p + h;
                u32x4_t xb;
                if constexpr (XLDS) xb = *reinterpret_cast<const u32x4_t*>(xsrow + (run * 8 + b) * 64);
                else xb = xf[buf][b];
#pragma unroll
                for (int q = 0; q < NQ; q++) {
                    const uint32_t sdw = ws[buf][q][b >> 1];
                    const uint16_t d = (uint16_t)((b & 1) ? (sdw >> 16) : (sdw & 0xFFFFu));
                    uint32_t a0, a1, a2, a3;
                    q8_dword_bf16<NUM>(d, wq[buf][q][p][2 * h], a0, a1);
                    q8_dword_bf16<NUM>(d, wq[buf][q][p][2 * h + 1], a2, a3);
                    const u32x4_t a = {a0, a1, a2, a3};
                    acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                                     __builtin_bit_cast(bf16x8_t, xb), acc[q], 0, 0, 0);
                }
            }
        }
    };
    int run = r0;
    for (; run + 1 < r1; run += 2) {
        step(run, 0);
        step(run + 1, 1);
    }
    if (run < r1) step(run, 0);

    // ---- add the wavefronts' partial sums (the staged activations are dead: reuse the space) -------------------
    __syncthreads();
    f32x4_t* red = reinterpret_cast<f32x4_t*>(lds);  // [gate partial sums of the W K ranges | up partial sums][64]
    red[wave * 64 + lane] = acc[0];
    if constexpr (PAIRED) red[(W + wave) * 64 + lane] = acc[1];
    __syncthreads();
    if (wave != 0 || !has_x) return;
    // D[i][j]: j = lane % 16 is the activation row, register v holds weight row 4 * (lane / 16) + v
    f32x4_t sum = red[lane];
    for (int w = 1; w < W; w++) {
        const f32x4_t v = red[w * 64 + lane];
        sum[0] += v[0]; sum[1] += v[1]; sum[2] += v[2]; sum[3] += v[3];
    }
    const int m = r;
    const int64_t n = rg * 16 + 4 * g;
    float o[4];
    if constexpr (GATED) {
        f32x4_t up = red[W * 64 + lane];
        for (int w = 1; w < W; w++) {
            const f32x4_t v = red[(W + w) * 64 + lane];
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
        for (int v = 0; v < 4; v++)
            o[v] = n + v < N ? add_residual(sum[v] + (bias ? bf16_to_f32(bias[n + v]) : 0.f), residual, (int64_t)m * N + n + v) : 0.f;
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

// Rows from which the gated pair runs in the paired mode; measured 12288 x 4096 gate/up, unpaired / paired us:
// M=1 23.0 / 23.7, M=2 25.9 / 23.7, M=4 26.3 / 23.1, M=8 28.4 / 23.3, M=16 35.0 / 25.4 (8 instead of 4 wavefronts per
// workgroup in the paired mode: 27.6 - 31.3).
constexpr int kTiledPairedMinM = 2;

template <int NUM>
int launch_tiled(const bf16_t* x, int M, const uint8_t* ta, const uint8_t* tb, int64_t N, int64_t K, const bf16_t* bias,
                 const bf16_t* residual, bf16_t* y, bool gated, const bf16_t* gamma, float eps, hipStream_t stream) {
    const int64_t groups = (N + 15) / 16;
    const int runs = (int)(K >> 8);
    const size_t x_bytes = (size_t)M * (2 * K + 64);
    const bool xlds = x_bytes <= 16 * 1024 || (gamma != nullptr && x_bytes <= 36 * 1024);   // (the fused norm needs the staged copy)
    // wavefronts per matrix and row group: measured best at 8 (4 for the gated pair, which doubles them), never more
    // than there are runs.  With the activations fetched from global memory, fewer when the row groups alone fill the
    // chip several times over (a 151936-row projection at M = 4: 128 us with one wavefront per group, 159 us with eight);
    // with them staged in LDS the full count also there (the same projection at M = 1: 109 against 127 us).
    int w = gated ? 4 : 8;
    if (!xlds)
        while (w > 1 && groups * w * (gated ? 2 : 1) > 256 * 24) w >>= 1;
    // a dozen rows or more on a long K (12288 -> 4096 at M = 16: 17.4 us with four wavefronts per group, 18.5 with eight,
    // 22.5 with two): fewer wavefronts fetch the activation fragments of fewer K ranges at a time
    if (!gated && !xlds && M >= 12 && runs >= 32 && w > 4) w = 4;
    if (w > runs) w = runs;
    // a gated pair with two activation rows or more: one wavefront takes both matrices
    const bool paired = gated && M >= kTiledPairedMinM;
    const int waves = (gated && !paired) ? 2 * w : w;
    const size_t red_bytes = (size_t)(gated ? 2 * w : w) * 1024;
    if (gamma && !xlds) return SNGGUF_E_BADSHAPE;   // the norm is applied to activations staged in LDS
    const size_t stage_bytes = x_bytes + (gamma ? (((size_t)4 * M * waves + 15) & ~(size_t)15) : 0);
    const size_t lds_bytes = xlds && stage_bytes > red_bytes ? stage_bytes : red_bytes;
    const dim3 grid((unsigned)groups), block((unsigned)(64 * waves));
#define SNGGUF_LAUNCH(G, XL) gemv_q8_tiled_kernel<NUM, G, 8, XL><<<grid, block, lds_bytes, stream>>>(x, M, ta, tb, N, K, bias, residual, y, gamma, eps)
    if (paired) {
        if (xlds) gemv_q8_tiled_kernel<NUM, true, 4, true, true><<<grid, block, lds_bytes, stream>>>(x, M, ta, tb, N, K, bias, residual, y, gamma, eps);
        else gemv_q8_tiled_kernel<NUM, true, 4, false, true><<<grid, block, lds_bytes, stream>>>(x, M, ta, tb, N, K, bias, residual, y, gamma, eps);
    } else if (gated) {
        if (xlds) SNGGUF_LAUNCH(true, true);
        else SNGGUF_LAUNCH(true, false);
    } else {
        if (xlds) SNGGUF_LAUNCH(false, true);
        else SNGGUF_LAUNCH(false, false);
    }
#undef SNGGUF_LAUNCH
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

}  // namespace

int64_t q8_0_tiled_bytes(int64_t N, int64_t K) {
    const int64_t G = (N + 15) / 16;
    return 16 * G * K + 16 * G * (K >> 5) * 2;   // quants + scales of the padded rows
}

int launch_q8_0_tile(const void* q, int64_t N, int64_t K, void* tiled, hipStream_t stream) {
    const int64_t G = (N + 15) / 16, total = G * (K >> 5) * 64;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    uint8_t* tq = static_cast<uint8_t*>(tiled);
    q8_0_tile_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(static_cast<const uint8_t*>(q), N, K, tq,
                                                                        reinterpret_cast<uint16_t*>(tq + 16 * G * K));
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

// 1 <= M <= 16, K % 256 == 0, 16-byte aligned pointers (checked by the caller).
// `gamma` (K bf16, 16-byte aligned) switches the fused RMSNorm on; the caller keeps M (2 K + 64) <= 36 KB then.
int launch_gemv_q8_tiled(const void* x, int64_t M, const void* ta, const void* tb, int64_t N, int64_t K, const void* bias,
                         const void* residual, void* y, int numerics, bool gated, hipStream_t stream, const void* gamma,
                         float eps) {
    const bf16_t* xp = static_cast<const bf16_t*>(x);
    const uint8_t* a = static_cast<const uint8_t*>(ta);
    const uint8_t* b = static_cast<const uint8_t*>(tb);
    const bf16_t* bp = static_cast<const bf16_t*>(bias);
    const bf16_t* rp = static_cast<const bf16_t*>(residual);
    bf16_t* yp = static_cast<bf16_t*>(y);
    const bf16_t* gp = static_cast<const bf16_t*>(gamma);
    if (numerics == SNGGUF_NUM_GGML_FP32) return launch_tiled<SNGGUF_NUM_GGML_FP32>(xp, (int)M, a, b, N, K, bp, rp, yp, gated, gp, eps, stream);
    if (numerics == SNGGUF_NUM_UPSTREAM_FP16) return launch_tiled<SNGGUF_NUM_UPSTREAM_FP16>(xp, (int)M, a, b, N, K, bp, rp, yp, gated, gp, eps, stream);
    return SNGGUF_E_BADTYPE;
}

}  // namespace sngguf
