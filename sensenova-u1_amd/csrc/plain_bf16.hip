// GGUF tensors of type BF16 (ggml type 30): rows of plain bfloat16, "blocks" of one element and two bytes.
// Upstream decodes them like any other GGUF type (dequantize_blocks_BF16: the bit pattern shifted into the
// upper half of an fp32 word), so a Linear whose weight is stored as BF16 is a quantized-linear module too.
// Nothing is rounded on the way: both numerics modes give the same values.
//
//   * bf16_widen_kernel: the standalone dequantize (bf16 -> fp32 exact, -> fp16 one rounding, -> bf16 a copy);
//   * gemv_bf16_kernel: decode-sized projections (M <= 16): one wavefront per weight row, 16-byte loads along
//     the row, fp32 accumulation, DPP reduction; the SiLU-gated pair in one launch.
// Larger row counts go to the dense form of the tile kernel (no decode stage) when K is a multiple of 64.

#include "sngguf_common.hpp"

namespace sngguf {

template <int OUT>
__global__ __launch_bounds__(256) void bf16_widen_kernel(const bf16_t* __restrict__ q, int64_t total, void* __restrict__ out) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const bf16_t b = q[i];
        if constexpr (OUT == SNGGUF_OUT_F32) reinterpret_cast<float*>(out)[i] = bf16_to_f32(b);
        else if constexpr (OUT == SNGGUF_OUT_F16) reinterpret_cast<uint16_t*>(out)[i] = f32_to_f16(bf16_to_f32(b));
        else reinterpret_cast<bf16_t*>(out)[i] = b;
    }
}

int launch_dequantize_bf16(const void* q, int64_t rows, int64_t cols, void* out, int out_dtype, hipStream_t stream) {
    const int64_t total = rows * cols;
    if (total == 0) return SNGGUF_OK;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    const dim3 grid((unsigned)blocks), block(256);
    const bf16_t* p = static_cast<const bf16_t*>(q);
    switch (out_dtype) {
    case SNGGUF_OUT_F32: bf16_widen_kernel<SNGGUF_OUT_F32><<<grid, block, 0, stream>>>(p, total, out); break;
    case SNGGUF_OUT_F16: bf16_widen_kernel<SNGGUF_OUT_F16><<<grid, block, 0, stream>>>(p, total, out); break;
    case SNGGUF_OUT_BF16: bf16_widen_kernel<SNGGUF_OUT_BF16><<<grid, block, 0, stream>>>(p, total, out); break;
    default: return SNGGUF_E_BADTYPE;
    }
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

// One wavefront per output column n (GATED: column n of the gate and of the up matrix).  VEC: K % 8 == 0, so
// every row of w and x starts 16-byte aligned and a lane takes 8 elements per step; otherwise 1 element.
template <bool GATED, bool VEC>
__global__ __launch_bounds__(256) void gemv_bf16_kernel(const bf16_t* __restrict__ x, int M, const bf16_t* __restrict__ wa,
                                                        const bf16_t* __restrict__ wb, int64_t N, int64_t K,
                                                        const bf16_t* __restrict__ bias, const bf16_t* residual,
                                                        bf16_t* __restrict__ y) {
    constexpr int NW = GATED ? 2 : 1;
    const int lane = threadIdx.x & 63;
    const int64_t n = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    const bf16_t* rows[2] = {wa + n * K, GATED ? wb + n * K : nullptr};
    float acc[NW][16];
#pragma unroll
    for (int t = 0; t < NW; t++)
#pragma unroll
        for (int m = 0; m < 16; m++) acc[t][m] = 0.f;
    if constexpr (VEC) {
        for (int64_t e0 = (int64_t)lane * 8; e0 < K; e0 += 64 * 8) {
            u32x4_t w[NW];
#pragma unroll
            // weight rows are read once, in whole lines: non-temporal hint (12288 x 4096 gated pair at M = 1 39.0 -> 36.5 us,
            // 4096 x 12288 at M = 4 49.6 -> 40.3 us)
            for (int t = 0; t < NW; t++) w[t] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(rows[t] + e0));
#pragma unroll
            for (int m = 0; m < 16; m++) {
                if (m < M) {
                    const u32x4_t xv = *reinterpret_cast<const u32x4_t*>(x + (int64_t)m * K + e0);
#pragma unroll
                    for (int t = 0; t < NW; t++) {
                        float s = 0.f;
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            s = fmaf(bf16lo_to_f32(w[t][i]), bf16lo_to_f32(xv[i]), s);
                            s = fmaf(bf16hi_to_f32(w[t][i]), bf16hi_to_f32(xv[i]), s);
                        }
                        acc[t][m] += s;
                    }
                }
            }
        }
    } else {
        for (int64_t e = lane; e < K; e += 64) {
#pragma unroll
            for (int m = 0; m < 16; m++) {
                if (m < M) {
                    const float xv = bf16_to_f32(x[(int64_t)m * K + e]);
#pragma unroll
                    for (int t = 0; t < NW; t++) acc[t][m] = fmaf(bf16_to_f32(rows[t][e]), xv, acc[t][m]);
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < 16; m++) {
        if (m < M) {
            float v[NW];
#pragma unroll
            for (int t = 0; t < NW; t++) v[t] = wave_sum(acc[t][m]);
            if (lane == 0) {
                if constexpr (GATED) {
                    const float g = bf16_to_f32(f32_to_bf16(v[0]));
                    const float up = bf16_to_f32(f32_to_bf16(v[NW - 1]));
                    const float sg = bf16_to_f32(f32_to_bf16(g / (1.0f + expf(-g))));
                    y[(int64_t)m * N + n] = f32_to_bf16(sg * up);
                } else {
                    y[(int64_t)m * N + n] = f32_to_bf16(add_residual(v[0] + (bias ? bf16_to_f32(bias[n]) : 0.f), residual, (int64_t)m * N + n));
                }
            }
        }
    }
}

// 1 <= M <= 16; w rows of K bf16 without padding (the base 16-byte aligned, checked by the caller).
int launch_gemv_bf16(const void* x, int64_t M, const void* wa, const void* wb, int64_t N, int64_t K, const void* bias,
                     const void* residual, void* y, bool gated, hipStream_t stream) {
    const bf16_t* xp = static_cast<const bf16_t*>(x);
    const bf16_t* a = static_cast<const bf16_t*>(wa);
    const bf16_t* b = static_cast<const bf16_t*>(wb);
    const bf16_t* bp = static_cast<const bf16_t*>(bias);
    const bf16_t* rp = static_cast<const bf16_t*>(residual);
    bf16_t* yp = static_cast<bf16_t*>(y);
    if (M < 1 || M > 16) return SNGGUF_E_BADSHAPE;
    const dim3 grid((unsigned)((N + 3) / 4)), block(256);
    const bool vec = K % 8 == 0;
    if (gated) {
        if (vec) gemv_bf16_kernel<true, true><<<grid, block, 0, stream>>>(xp, (int)M, a, b, N, K, bp, rp, yp);
        else gemv_bf16_kernel<true, false><<<grid, block, 0, stream>>>(xp, (int)M, a, b, N, K, bp, rp, yp);
    } else {
        if (vec) gemv_bf16_kernel<false, true><<<grid, block, 0, stream>>>(xp, (int)M, a, b, N, K, bp, rp, yp);
        else gemv_bf16_kernel<false, false><<<grid, block, 0, stream>>>(xp, (int)M, a, b, N, K, bp, rp, yp);
    }
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

}  // namespace sngguf
