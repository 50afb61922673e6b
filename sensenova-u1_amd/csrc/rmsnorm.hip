// RMSNorm of the decoder layers as one launch (Qwen3RMSNorm.forward, modeling_qwen3.py:192-197):
//     v = bf16(x * rsqrt(mean(x^2) + eps))   (fp32 arithmetic, one rounding);   y = bf16(gamma * v)
// One workgroup per row: the row is read once into registers (16-byte pieces), the sum of squares goes through a
// wavefront reduction and a small LDS table, and the same registers are normalized and written.  It is what the
// module helpers run in front of a projection when the norm cannot ride inside the projection kernel (more rows
// than its LDS staging takes): one launch where the same arithmetic as tensor operations is five.
#include "sngguf_common.hpp"

namespace sngguf {

namespace {
constexpr int kThreads = 256;
constexpr int kPiecesPerThread = 8;   // up to 256 * 8 * 8 = 16384 elements per row in registers
}  // namespace

__global__ __launch_bounds__(kThreads) void rmsnorm_rows_kernel(const bf16_t* x, int64_t K, const bf16_t* __restrict__ gamma,
                                                                float eps, bf16_t* y) {
    __shared__ float part[kThreads / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bf16_t* xr = x + (int64_t)blockIdx.x * K;
    bf16_t* yr = y + (int64_t)blockIdx.x * K;
    const int64_t pieces = K >> 3;
    u32x4_t v[kPiecesPerThread];
    float ss = 0.f;
    if (pieces <= (int64_t)kThreads * kPiecesPerThread) {
#pragma unroll
        for (int i = 0; i < kPiecesPerThread; i++) {
            const int64_t c = tid + (int64_t)kThreads * i;
            if (c < pieces) {
                v[i] = *reinterpret_cast<const u32x4_t*>(xr + 8 * c);
                ss += sumsq_piece(v[i]);
            }
        }
    } else {
        for (int64_t c = tid; c < pieces; c += kThreads) ss += sumsq_piece(*reinterpret_cast<const u32x4_t*>(xr + 8 * c));
    }
    ss = wave_sum(ss);
    if (lane == 0) part[wave] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < kThreads / 64; w++) tot += part[w];
    const float rstd = rms_rstd(tot, K, eps);
    if (pieces <= (int64_t)kThreads * kPiecesPerThread) {
#pragma unroll
        for (int i = 0; i < kPiecesPerThread; i++) {
            const int64_t c = tid + (int64_t)kThreads * i;
            if (c < pieces)
                *reinterpret_cast<u32x4_t*>(yr + 8 * c) = rmsnorm_piece(v[i], *reinterpret_cast<const u32x4_t*>(gamma + 8 * c), rstd);
        }
    } else {
        for (int64_t c = tid; c < pieces; c += kThreads)
            *reinterpret_cast<u32x4_t*>(yr + 8 * c) = rmsnorm_piece(*reinterpret_cast<const u32x4_t*>(xr + 8 * c),
                                                                    *reinterpret_cast<const u32x4_t*>(gamma + 8 * c), rstd);
    }
}

// x, y [M][K] bf16, gamma [K] bf16, all 16-byte aligned, K % 8 == 0 (checked by the caller); y may be x (neither is
// declared restrict: every thread reads a 16-byte piece of the row before it writes that same piece and no other).
int launch_rmsnorm(const void* x, int64_t M, int64_t K, const void* gamma, float eps, void* y, hipStream_t stream) {
    rmsnorm_rows_kernel<<<dim3((unsigned)M), dim3(kThreads), 0, stream>>>(static_cast<const bf16_t*>(x), K, static_cast<const bf16_t*>(gamma),
                                                                          eps, static_cast<bf16_t*>(y));
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

}  // namespace sngguf
