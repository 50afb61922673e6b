// Fused dequant-GEMV for decode (M <= 16) on the vector ALU: the path for Q8_0 rows that are not a
// whole number of 256-element runs and for the other 32-element formats when K % 256 != 0 (the
// dispatcher at the end of this file sends everything with K % 256 == 0 to the matrix-core
// kernels).
//
// K % 64 == 0: one wavefront owns two weight rows (or, for the SiLU-gated pair, row n of the gate
// matrix and row n of the up matrix); a lane takes 64 weight elements (68 packed bytes) per step,
// so that one step of the wave reads one contiguous 4352-byte span of each row.  The packed bytes
// go from HBM to registers once, are decoded to bf16 pairs there, multiplied with the bf16
// activations (v_dot2_f32_bf16, fp32 accumulate) and reduced across the wavefront with DPP; no
// dequantized weight ever reaches memory.  Other K (odd block counts): a generic kernel built on
// the 8-element decoders, one lane per 8 elements.

#include "sngguf_common.hpp"

namespace sngguf {

// ---- per-lane unit decoders: 64 elements -> 32 packed bf16 pairs -----------------------------
// The pair order matches x_unit_offset(): pair i holds elements run(i / 8) + 2 * (i % 8) + {0, 1}.

// element offset of 16-element run t (0..3) of unit u
template <int QT>
__device__ __forceinline__ int64_t unit_run_offset(int64_t u, int t) {
    return u * 64 + 16 * t;
}

template <int NUM>
__device__ __forceinline__ void decode_unit_q8_0(const uint8_t* __restrict__ row, int64_t u, uint32_t (&wp)[32]) {
    const uint8_t* p = row + u * 68;  // two blocks; 4-byte aligned because K % 64 == 0
    uint32_t L[17];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const u32x4_t v = ld_u128_a4(p + 16 * i);
        L[4 * i] = v[0]; L[4 * i + 1] = v[1]; L[4 * i + 2] = v[2]; L[4 * i + 3] = v[3];
    }
    L[16] = ld_u32(p + 64);
    const uint16_t d0 = (uint16_t)(L[0] & 0xFFFF), d1 = (uint16_t)(L[8] >> 16);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t q0 = __builtin_amdgcn_alignbit(L[i + 1], L[i], 16);  // block 0 quants sit 2 bytes off
        q8_dword_bf16<NUM>(d0, q0, wp[2 * i], wp[2 * i + 1]);
        q8_dword_bf16<NUM>(d1, L[9 + i], wp[16 + 2 * i], wp[16 + 2 * i + 1]);
    }
}

template <int QT, int NUM>
__device__ __forceinline__ void decode_unit(const uint8_t* __restrict__ row, int64_t u, uint32_t (&wp)[32]) {
    static_assert(QT == SNGGUF_TYPE_Q8_0, "the unit kernel is only instantiated for Q8_0");
    decode_unit_q8_0<NUM>(row, u, wp);
}

__device__ __forceinline__ float dot2(uint32_t w, uint32_t x, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w), __builtin_bit_cast(bf16x2_t, x), acc, false);
}

// ---- kernel ------------------------------------------------------------------------------------
// GATED == false: rows (2p, 2p+1) of one matrix, y[m][n] = bf16(acc + bias[n]).
// GATED == true : row p of qa (gate) and of qb (up), y[m][p] = bf16(bf16(silu(bf16 g)) * bf16 u).

template <int QT, int NUM, int MT, bool GATED>
__global__ __launch_bounds__(256) void gemv_kernel(const bf16_t* __restrict__ x, int M, const uint8_t* __restrict__ qa,
                                                   const uint8_t* __restrict__ qb, int64_t N, int64_t K,
                                                   const bf16_t* __restrict__ bias, const bf16_t* residual, bf16_t* __restrict__ y) {
    const int lane = threadIdx.x & 63;
    const int64_t pair = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t n_pairs = GATED ? N : (N + 1) / 2;
    if (pair >= n_pairs) return;
    const int64_t row_bytes = K / Fmt<QT>::bs * Fmt<QT>::ts;
    int64_t na, nb;
    const uint8_t *ra, *rb;
    if constexpr (GATED) {
        na = nb = pair;
        ra = qa + pair * row_bytes;
        rb = qb + pair * row_bytes;
    } else {
        na = 2 * pair;
        nb = na + 1 < N ? na + 1 : na;  // odd N: the last wave decodes its row twice, stores once
        ra = qa + na * row_bytes;
        rb = qa + nb * row_bytes;
    }
    float acc_a[MT], acc_b[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) acc_a[m] = acc_b[m] = 0.f;

    const int64_t units = K >> 6;
    for (int64_t u = lane; u < units; u += 64) {
        uint32_t wa[32], wb[32];
        decode_unit<QT, NUM>(ra, u, wa);
        decode_unit<QT, NUM>(rb, u, wb);
#pragma unroll
        for (int m = 0; m < MT; m++) {
            if (m < M) {
                const bf16_t* xr = x + (int64_t)m * K;
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const u32x4_t* xp = reinterpret_cast<const u32x4_t*>(xr + unit_run_offset<QT>(u, t));
                    const u32x4_t x0 = xp[0], x1 = xp[1];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        acc_a[m] = dot2(wa[8 * t + i], x0[i], acc_a[m]);
                        acc_b[m] = dot2(wb[8 * t + i], x0[i], acc_b[m]);
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        acc_a[m] = dot2(wa[8 * t + 4 + i], x1[i], acc_a[m]);
                        acc_b[m] = dot2(wb[8 * t + 4 + i], x1[i], acc_b[m]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MT; m++) {
        if (m < M) {
            const float sa = wave_sum(acc_a[m]);
            const float sb = wave_sum(acc_b[m]);
            if (lane == 0) {
                if constexpr (GATED) {
                    const float g = bf16_to_f32(f32_to_bf16(sa));
                    const float up = bf16_to_f32(f32_to_bf16(sb));
                    const float s = bf16_to_f32(f32_to_bf16(g / (1.0f + expf(-g))));
                    y[(int64_t)m * N + pair] = f32_to_bf16(s * up);
                } else {
                    const float ba = bias ? bf16_to_f32(bias[na]) : 0.f;
                    y[(int64_t)m * N + na] = f32_to_bf16(add_residual(sa + ba, residual, (int64_t)m * N + na));
                    if (nb != na) {
                        const float bb = bias ? bf16_to_f32(bias[nb]) : 0.f;
                        y[(int64_t)m * N + nb] = f32_to_bf16(add_residual(sb + bb, residual, (int64_t)m * N + nb));
                    }
                }
            }
        }
    }
}

// Every other case - Q8_0 rows whose block count is odd (not a whole number of 64-element units,
// rows only 2-byte aligned) and Q4_0 / Q4_1 / Q5_0 / Q5_1 rows that are not a whole number of
// 256-element runs - takes this plain path: one wavefront per row (GATED: row n of the gate and
// of the up matrix), eight elements per lane and step through the shared 8-element decoder.
template <int QT, int NUM, bool GATED>
__global__ __launch_bounds__(256) void gemv_generic_kernel(const bf16_t* __restrict__ x, int M, const uint8_t* __restrict__ qa,
                                                           const uint8_t* __restrict__ qb, int64_t N, int64_t K,
                                                           const bf16_t* __restrict__ bias, const bf16_t* residual, bf16_t* __restrict__ y) {
    constexpr int NW = GATED ? 2 : 1;
    const int lane = threadIdx.x & 63;
    const int64_t n = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    const int64_t row_bytes = K / Fmt<QT>::bs * Fmt<QT>::ts;
    const uint8_t* rows[2] = {qa + n * row_bytes, GATED ? qb + n * row_bytes : nullptr};
    float acc[NW][16];
#pragma unroll
    for (int t = 0; t < NW; t++)
#pragma unroll
        for (int m = 0; m < 16; m++) acc[t][m] = 0.f;
    for (int64_t e0 = (int64_t)lane * 8; e0 < K; e0 += 64 * 8) {
        float w[NW][8];
#pragma unroll
        for (int t = 0; t < NW; t++) {
            decode8<QT, NUM>(rows[t], e0, w[t]);
#pragma unroll
            for (int i = 0; i < 8; i++) w[t][i] = bf16_to_f32(f32_to_bf16(w[t][i]));
        }
        for (int m = 0; m < M; m++) {
            const u32x4_t xv = *reinterpret_cast<const u32x4_t*>(x + (int64_t)m * K + e0);
            float s[NW];
#pragma unroll
            for (int t = 0; t < NW; t++) {
                s[t] = 0.f;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    s[t] = fmaf(w[t][2 * i], bf16lo_to_f32(xv[i]), s[t]);
                    s[t] = fmaf(w[t][2 * i + 1], bf16hi_to_f32(xv[i]), s[t]);
                }
            }
#pragma unroll
            for (int mm = 0; mm < 16; mm++)
                if (mm == m) {
#pragma unroll
                    for (int t = 0; t < NW; t++) acc[t][mm] += s[t];
                }
        }
    }
    for (int m = 0; m < M; m++) {
        float v[NW];
#pragma unroll
        for (int t = 0; t < NW; t++) {
            v[t] = 0.f;
#pragma unroll
            for (int mm = 0; mm < 16; mm++)
                if (mm == m) v[t] = acc[t][mm];
            v[t] = wave_sum(v[t]);
        }
        if (lane == 0) {
            if constexpr (GATED) {
                const float g = bf16_to_f32(f32_to_bf16(v[0]));
                const float up = bf16_to_f32(f32_to_bf16(v[1]));
                const float sg = bf16_to_f32(f32_to_bf16(g / (1.0f + expf(-g))));
                y[(int64_t)m * N + n] = f32_to_bf16(sg * up);
            } else {
                y[(int64_t)m * N + n] = f32_to_bf16(add_residual(v[0] + (bias ? bf16_to_f32(bias[n]) : 0.f), residual, (int64_t)m * N + n));
            }
        }
    }
}

// ---- host-side dispatch ------------------------------------------------------------------------

template <int QT, int NUM, bool GATED>
static int launch_mt(const bf16_t* x, int M, const uint8_t* qa, const uint8_t* qb, int64_t N, int64_t K,
                     const bf16_t* bias, const bf16_t* residual, bf16_t* y, hipStream_t stream) {
    const int64_t n_pairs = GATED ? N : (N + 1) / 2;
    dim3 grid((unsigned)((n_pairs + 3) / 4)), block(256);
#define SNGGUF_GEMV_CASE(MT) \
    gemv_kernel<QT, NUM, MT, GATED><<<grid, block, 0, stream>>>(x, M, qa, qb, N, K, bias, residual, y)
    if (M == 1) SNGGUF_GEMV_CASE(1);
    else if (M == 2) SNGGUF_GEMV_CASE(2);
    else if (M <= 4) SNGGUF_GEMV_CASE(4);
    else if (M <= 8) SNGGUF_GEMV_CASE(8);
    else SNGGUF_GEMV_CASE(16);
#undef SNGGUF_GEMV_CASE
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

template <int QT, int NUM>
static int launch_gated(const bf16_t* x, int M, const uint8_t* qa, const uint8_t* qb, int64_t N, int64_t K,
                        const bf16_t* bias, const bf16_t* residual, bf16_t* y, bool gated, hipStream_t stream) {
    if (QT != SNGGUF_TYPE_Q8_0 || K % 64 != 0) {
        dim3 grid((unsigned)((N + 3) / 4)), block(256);
        if (gated) gemv_generic_kernel<QT, NUM, true><<<grid, block, 0, stream>>>(x, M, qa, qb, N, K, bias, residual, y);
        else gemv_generic_kernel<QT, NUM, false><<<grid, block, 0, stream>>>(x, M, qa, qb, N, K, bias, residual, y);
        return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
    }
    if constexpr (QT == SNGGUF_TYPE_Q8_0) {
        if (gated) return launch_mt<QT, NUM, true>(x, M, qa, qb, N, K, bias, residual, y, stream);
        return launch_mt<QT, NUM, false>(x, M, qa, qb, N, K, bias, residual, y, stream);
    }
    return SNGGUF_E_BADTYPE;
}

template <int QT>
static int launch_num(const bf16_t* x, int M, const uint8_t* qa, const uint8_t* qb, int64_t N, int64_t K,
                      const bf16_t* bias, const bf16_t* residual, bf16_t* y, int numerics, bool gated, hipStream_t stream) {
    if (numerics == SNGGUF_NUM_GGML_FP32) return launch_gated<QT, SNGGUF_NUM_GGML_FP32>(x, M, qa, qb, N, K, bias, residual, y, gated, stream);
    if (numerics == SNGGUF_NUM_UPSTREAM_FP16) return launch_gated<QT, SNGGUF_NUM_UPSTREAM_FP16>(x, M, qa, qb, N, K, bias, residual, y, gated, stream);
    return SNGGUF_E_BADTYPE;
}

int launch_gemv_q8_mfma(const void* x, int64_t M, const void* qa, const void* qb, int64_t N, int64_t K, const void* bias,
                        const void* residual, void* y, int numerics, bool gated, hipStream_t stream,
                        const void* gamma = nullptr, float eps = 0.f, uint64_t* amax = nullptr);

int launch_gemv_kq_mfma(const void* x, int64_t M, const void* qa, const void* qb, int qtype, int64_t N, int64_t K,
                        const void* bias, const void* residual, void* y, int numerics, bool gated, hipStream_t stream,
                        const void* gamma = nullptr, float eps = 0.f, uint64_t* amax = nullptr);

// Second pass of the arg-max form of the decode kernels: keys[m][slots] -> out_index[m], one workgroup per activation
// row.  (A key orders by value first and by lower column second, see argmax_key.)
__global__ __launch_bounds__(1024) void argmax_reduce_kernel(const uint64_t* __restrict__ keys, int64_t slots, int64_t* __restrict__ out_index) {
    __shared__ uint64_t best[16];
    const uint64_t* row = keys + (int64_t)blockIdx.x * slots;
    // four independent loads per thread and trip: the keys were just written by the projection and sit in L2, so
    // the pass costs a few load latencies, not one per key
    uint64_t k0 = 0, k1 = 0, k2 = 0, k3 = 0;
    for (int64_t i = threadIdx.x; i < slots; i += 4096) {
        const uint64_t a = row[i];
        const uint64_t b = i + 1024 < slots ? row[i + 1024] : 0;
        const uint64_t c = i + 2048 < slots ? row[i + 2048] : 0;
        const uint64_t d = i + 3072 < slots ? row[i + 3072] : 0;
        k0 = u64_max(k0, a); k1 = u64_max(k1, b); k2 = u64_max(k2, c); k3 = u64_max(k3, d);
    }
    uint64_t k = u64_max(u64_max(k0, k1), u64_max(k2, k3));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) k = u64_max(k, shfl_xor_u64(k, off));
    if ((threadIdx.x & 63) == 0) best[threadIdx.x >> 6] = k;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; w++) k = u64_max(k, best[w]);
        out_index[blockIdx.x] = (int64_t)(0xFFFFFFFFu - (uint32_t)k);
    }
}

int launch_argmax_reduce(const uint64_t* keys, int64_t M, int64_t slots, int64_t* out_index, hipStream_t stream) {
    argmax_reduce_kernel<<<dim3((unsigned)M), dim3(1024), 0, stream>>>(keys, slots, out_index);
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

// M in 1..16 (up to 64 when K % 256 == 0 and not gated), N >= 1, K a positive multiple of the block
// size (checked by the caller).
int launch_gemv(const void* x, int64_t M, const void* qa, const void* qb, int qtype, int64_t N, int64_t K,
                const void* bias, const void* residual, void* y, int numerics, bool gated, hipStream_t stream) {
    const bf16_t* xp = static_cast<const bf16_t*>(x);
    const uint8_t* a = static_cast<const uint8_t*>(qa);
    const uint8_t* b = static_cast<const uint8_t*>(qb);
    const bf16_t* bp = static_cast<const bf16_t*>(bias);
    const bf16_t* rp = static_cast<const bf16_t*>(residual);
    bf16_t* yp = static_cast<bf16_t*>(y);
    if (M > 16) {
        if (K % 256 != 0 || M > 64 || gated) return SNGGUF_E_BADSHAPE;
        return launch_gemv_kq_mfma(x, M, qa, qb, qtype, N, K, bias, residual, y, numerics, gated, stream);
    }
    if (qtype == SNGGUF_TYPE_Q8_0 && K % 256 == 0)
        return launch_gemv_q8_mfma(x, M, qa, qb, N, K, bias, residual, y, numerics, gated, stream);
    if (qtype != SNGGUF_TYPE_Q8_0 && K % 256 == 0)
        return launch_gemv_kq_mfma(x, M, qa, qb, qtype, N, K, bias, residual, y, numerics, gated, stream);
    // rows that are not a whole number of 256-element runs
#define SNGGUF_CALL(QT) launch_num<QT>(xp, (int)M, a, b, N, K, bp, rp, yp, numerics, gated, stream)
    SNGGUF_DISPATCH_TYPE(qtype, SNGGUF_CALL)
#undef SNGGUF_CALL
}

}  // namespace sngguf
