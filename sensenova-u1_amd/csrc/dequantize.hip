// Standalone block dequantize: packed GGUF rows -> fp32 / fp16 / bf16 rows.
// One thread decodes eight consecutive elements, so a wavefront reads one contiguous run of
// packed bytes and writes one contiguous run of 512 outputs; the kernel is bound by the
// output stream (4 bytes out per ~1 byte in for fp32).
#include "sngguf_common.hpp"

namespace sngguf {

template <int OUT>
__device__ __forceinline__ void store8(void* __restrict__ out, int64_t idx, const float (&w)[8]) {
    if constexpr (OUT == SNGGUF_OUT_F32) {
        f32x4_t* o = reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(out) + idx);
        o[0] = f32x4_t{w[0], w[1], w[2], w[3]};
        o[1] = f32x4_t{w[4], w[5], w[6], w[7]};
    } else if constexpr (OUT == SNGGUF_OUT_F16) {
        u32x4_t v;
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = (uint32_t)f32_to_f16(w[2 * i]) | ((uint32_t)f32_to_f16(w[2 * i + 1]) << 16);
        *reinterpret_cast<u32x4_t*>(reinterpret_cast<uint16_t*>(out) + idx) = v;
    } else {
        u32x4_t v;
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = pack_bf16(w[2 * i], w[2 * i + 1]);
        *reinterpret_cast<u32x4_t*>(reinterpret_cast<uint16_t*>(out) + idx) = v;
    }
}

template <int QT, int NUM, int OUT>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t* __restrict__ q, int64_t rows, int64_t cols,
                                                         int64_t row_bytes, void* __restrict__ out) {
    const int64_t groups_per_row = cols >> 3;
    const int64_t total = rows * groups_per_row;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = g / groups_per_row;
        const int64_t e0 = (g - r * groups_per_row) << 3;
        float w[8];
        decode8<QT, NUM>(q + r * row_bytes, e0, w);
        store8<OUT>(out, r * cols + e0, w);
    }
}

template <int QT, int NUM>
static int launch_out(const uint8_t* q, int64_t rows, int64_t cols, void* out, int out_dtype, hipStream_t stream) {
    const int64_t row_bytes = cols / Fmt<QT>::bs * Fmt<QT>::ts;
    const int64_t total = rows * (cols >> 3);
    if (total == 0) return SNGGUF_OK;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;  // grid-stride beyond 64 blocks per CU
    dim3 grid((unsigned)blocks), block(256);
    switch (out_dtype) {
    case SNGGUF_OUT_F32: dequantize_kernel<QT, NUM, SNGGUF_OUT_F32><<<grid, block, 0, stream>>>(q, rows, cols, row_bytes, out); break;
    case SNGGUF_OUT_F16: dequantize_kernel<QT, NUM, SNGGUF_OUT_F16><<<grid, block, 0, stream>>>(q, rows, cols, row_bytes, out); break;
    case SNGGUF_OUT_BF16: dequantize_kernel<QT, NUM, SNGGUF_OUT_BF16><<<grid, block, 0, stream>>>(q, rows, cols, row_bytes, out); break;
    default: return SNGGUF_E_BADTYPE;
    }
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

template <int QT>
static int launch_num(const uint8_t* q, int64_t rows, int64_t cols, void* out, int out_dtype, int numerics, hipStream_t stream) {
    if (numerics == SNGGUF_NUM_GGML_FP32) return launch_out<QT, SNGGUF_NUM_GGML_FP32>(q, rows, cols, out, out_dtype, stream);
    if (numerics == SNGGUF_NUM_UPSTREAM_FP16) return launch_out<QT, SNGGUF_NUM_UPSTREAM_FP16>(q, rows, cols, out, out_dtype, stream);
    return SNGGUF_E_BADTYPE;
}

int launch_dequantize(const void* q, int qtype, int64_t rows, int64_t cols, void* out, int out_dtype, int numerics,
                      hipStream_t stream) {
    const uint8_t* p = static_cast<const uint8_t*>(q);
#define SNGGUF_CALL(QT) launch_num<QT>(p, rows, cols, out, out_dtype, numerics, stream)
    SNGGUF_DISPATCH_TYPE(qtype, SNGGUF_CALL)
#undef SNGGUF_CALL
}

}  // namespace sngguf
