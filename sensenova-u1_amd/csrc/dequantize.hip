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

// Packed-half decode of eight consecutive elements for the fp16 rounding chain: the chain's last fp16 value IS the
// fp16 output (and what bf16 is rounded from), so nothing is widened to fp32 on the way.  Returns the eight halves in
// four dwords.  Q4_K: R(R(D q) - DM) with D = R(d sc), DM = R(dmin m); Q6_K: R(D q) with D = R(d scale).
template <int QT>
__device__ __forceinline__ u32x4_t decode8_half_chain(const uint8_t* __restrict__ row, int64_t e0) {
    static_assert(QT == SNGGUF_TYPE_Q4_K || QT == SNGGUF_TYPE_Q6_K, "packed decode exists for Q4_K and Q6_K");
    typedef Num<SNGGUF_NUM_UPSTREAM_FP16> A;
    u32x4_t o;
    if constexpr (QT == SNGGUF_TYPE_Q4_K) {
        const uint8_t* blk = row + (e0 >> 8) * 144;
        const int r = (int)(e0 & 255), c = r >> 6, hi = (r >> 5) & 1, l0 = r & 31;
        const uint32_t dd = ld_u32(blk);
        uint32_t sc, mn;
        q4k_scale_min(ld_u32(blk + 4), ld_u32(blk + 8), ld_u32(blk + 12), 2 * c + hi, sc, mn);
        const _Float16 D = A::scale((uint16_t)(dd & 0xFFFF)) * A::integer((int)sc);
        const _Float16 DM = A::scale((uint16_t)(dd >> 16)) * A::integer((int)mn);
        const half2_t D2 = {D, D}, M2 = {DM, DM};
        const half2_t k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
        const uint8_t* qs = blk + 16 + 32 * c + l0;
        const int sh = 4 * hi;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint32_t v = (ld_u32(qs + 4 * i) >> sh) & 0x0F0F0F0Fu;
            // 0x6400 | n is the half 1024 + n
            const half2_t q01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u)) - k1024;
            const half2_t q23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u)) - k1024;
            o[2 * i] = __builtin_bit_cast(uint32_t, q01 * D2 - M2);       // two roundings each (no contraction)
            o[2 * i + 1] = __builtin_bit_cast(uint32_t, q23 * D2 - M2);
        }
    } else {
        const uint8_t* blk = row + (e0 >> 8) * 210;
        const int r = (int)(e0 & 255), h = r >> 7, quad = (r >> 5) & 3, l0 = r & 31;
        const uint8_t* ql = blk + 64 * h + 32 * (quad & 1) + l0;
        const uint8_t* qh = blk + 128 + 32 * h + l0;
        const int sh_l = 4 * (quad >> 1), sh_h = 2 * quad;
        const _Float16 D = A::scale(ld_u16(blk + 208)) * A::integer((int8_t)blk[192 + (r >> 4)]);
        const half2_t D2 = {D, D};
        const half2_t k1056 = {(_Float16)1056.0f, (_Float16)1056.0f};   // 1024 + the quant's offset of 32
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint32_t lo = (ld_u32_a2(ql + 4 * i) >> sh_l) & 0x0F0F0F0Fu;
            const uint32_t hb = ((ld_u32_a2(qh + 4 * i) >> sh_h) & 0x03030303u) << 4;
            const uint32_t v = lo | hb;                                  // 0 .. 63 per byte
            const half2_t q01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u)) - k1056;
            const half2_t q23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u)) - k1056;
            o[2 * i] = __builtin_bit_cast(uint32_t, q01 * D2);
            o[2 * i + 1] = __builtin_bit_cast(uint32_t, q23 * D2);
        }
    }
    return o;
}

template <int QT, int NUM, int OUT>
__device__ __forceinline__ void dequantize8(const uint8_t* __restrict__ row, int64_t e0, void* __restrict__ out, int64_t idx) {
    constexpr bool kHalfChain = NUM == SNGGUF_NUM_UPSTREAM_FP16 && OUT != SNGGUF_OUT_F32 &&
                                (QT == SNGGUF_TYPE_Q4_K || QT == SNGGUF_TYPE_Q6_K);
    if constexpr (kHalfChain) {
        u32x4_t v = decode8_half_chain<QT>(row, e0);
        if constexpr (OUT == SNGGUF_OUT_BF16) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t bits = v[i];   // (a bit cast applied to the element expression itself reads element 0)
                const half2_t h = __builtin_bit_cast(half2_t, bits);
                v[i] = pack_bf16((float)h[0], (float)h[1]);
            }
        }
        *reinterpret_cast<u32x4_t*>(reinterpret_cast<uint16_t*>(out) + idx) = v;
    } else {
        float w[8];
        decode8<QT, NUM>(row, e0, w);
        store8<OUT>(out, idx, w);
    }
}

// WIDE: the number of 8-element groups does not fit 32 bits (the index arithmetic then needs 64-bit divisions).
// Row r of the input is written to output row r + ((r >> spread) << spread) + first: with spread = 63 and first = 0
// that is row r; with spread = 7 the rows go out in blocks of 128 that leave 128 rows free behind each block (first = 0)
// or fill those (first = 128) - two matrices interleaved in blocks of 128 rows.
template <int QT, int NUM, int OUT, bool WIDE>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t* __restrict__ q, int64_t rows, int64_t cols,
                                                         int64_t row_bytes, void* __restrict__ out, int spread, int64_t first) {
    const int64_t groups_per_row = cols >> 3;
    const int64_t total = rows * groups_per_row;
    if constexpr (WIDE) {
        for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += (int64_t)gridDim.x * blockDim.x) {
            const int64_t r = g / groups_per_row;
            const int64_t e0 = (g - r * groups_per_row) << 3;
            dequantize8<QT, NUM, OUT>(q + r * row_bytes, e0, out, (r + ((r >> spread) << spread) + first) * cols + e0);
        }
    } else {
        const uint32_t gpr = (uint32_t)groups_per_row, tot = (uint32_t)total, stride = gridDim.x * blockDim.x;
        for (uint32_t g = blockIdx.x * blockDim.x + threadIdx.x; g < tot; g += stride) {
            const uint32_t r = g / gpr;
            const int64_t e0 = (int64_t)(g - r * gpr) << 3;
            const int64_t ro = (int64_t)r + (((int64_t)r >> spread) << spread) + first;
            dequantize8<QT, NUM, OUT>(q + (int64_t)r * row_bytes, e0, out, ro * cols + e0);
            if (g + stride < g) break;   // the next index would wrap
        }
    }
}

template <int QT, int NUM>
static int launch_out(const uint8_t* q, int64_t rows, int64_t cols, void* out, int out_dtype, hipStream_t stream,
                      int spread, int64_t first) {
    const int64_t row_bytes = cols / Fmt<QT>::bs * Fmt<QT>::ts;
    const int64_t total = rows * (cols >> 3);
    if (total == 0) return SNGGUF_OK;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;  // grid-stride beyond 64 blocks per CU
    dim3 grid((unsigned)blocks), block(256);
    const bool wide = total >= ((int64_t)1 << 32);
#define SNGGUF_DEQ(OUT) \
    do { \
        if (wide) dequantize_kernel<QT, NUM, OUT, true><<<grid, block, 0, stream>>>(q, rows, cols, row_bytes, out, spread, first); \
        else dequantize_kernel<QT, NUM, OUT, false><<<grid, block, 0, stream>>>(q, rows, cols, row_bytes, out, spread, first); \
    } while (0)
    switch (out_dtype) {
    case SNGGUF_OUT_F32: SNGGUF_DEQ(SNGGUF_OUT_F32); break;
    case SNGGUF_OUT_F16: SNGGUF_DEQ(SNGGUF_OUT_F16); break;
    case SNGGUF_OUT_BF16: SNGGUF_DEQ(SNGGUF_OUT_BF16); break;
    default: return SNGGUF_E_BADTYPE;
    }
#undef SNGGUF_DEQ
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

template <int QT>
static int launch_num(const uint8_t* q, int64_t rows, int64_t cols, void* out, int out_dtype, int numerics, hipStream_t stream,
                      int spread, int64_t first) {
    if (numerics == SNGGUF_NUM_GGML_FP32) return launch_out<QT, SNGGUF_NUM_GGML_FP32>(q, rows, cols, out, out_dtype, stream, spread, first);
    if (numerics == SNGGUF_NUM_UPSTREAM_FP16) return launch_out<QT, SNGGUF_NUM_UPSTREAM_FP16>(q, rows, cols, out, out_dtype, stream, spread, first);
    return SNGGUF_E_BADTYPE;
}

int launch_dequantize(const void* q, int qtype, int64_t rows, int64_t cols, void* out, int out_dtype, int numerics,
                      hipStream_t stream) {
    const uint8_t* p = static_cast<const uint8_t*>(q);
#define SNGGUF_CALL(QT) launch_num<QT>(p, rows, cols, out, out_dtype, numerics, stream, 63, 0)
    SNGGUF_DISPATCH_TYPE(qtype, SNGGUF_CALL)
#undef SNGGUF_CALL
}

// The bf16 rows of one of two matrices that share an output in blocks of 128 rows: input row r goes to output row
// 256 (r / 128) + r % 128 (+ 128 for the second matrix).  What the gated dense GEMM reads: each of its 256-row weight
// tiles then holds 128 gate rows and the 128 up rows of the same output columns.
int launch_dequantize_interleaved(const void* q, int qtype, int64_t rows, int64_t cols, void* out, int second, int numerics,
                                  hipStream_t stream) {
    const uint8_t* p = static_cast<const uint8_t*>(q);
#define SNGGUF_CALL(QT) launch_num<QT>(p, rows, cols, out, SNGGUF_OUT_BF16, numerics, stream, 7, second ? 128 : 0)
    SNGGUF_DISPATCH_TYPE(qtype, SNGGUF_CALL)
#undef SNGGUF_CALL
}

}  // namespace sngguf
