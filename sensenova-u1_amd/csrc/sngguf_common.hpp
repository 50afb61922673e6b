// Shared device helpers of the gfx950 GGUF quantized-linear kernels: scalar format
// conversions, the block decoders and wavefront reductions.  Included by every .hip
// file of the library; nothing here touches the host runtime.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/sngguf.h"

namespace sngguf {

typedef uint16_t bf16_t;  // raw bfloat16 bits
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// ---- scalar formats ---------------------------------------------------------------------

__device__ __forceinline__ float f16_to_f32(uint16_t bits) { return (float)__builtin_bit_cast(_Float16, bits); }
// The empty asm keeps the compiler from folding a preceding fp32 multiply into the conversion as
// a mixed-precision fma with a +0 addend, which turns a product of -0 into +0.
__device__ __forceinline__ uint16_t f32_to_f16(float v) {
    asm volatile("" : "+v"(v));
    return __builtin_bit_cast(uint16_t, (_Float16)v);
}
// One fp16 tensor-op rounding (v_cvt_f16_f32 is round-to-nearest-even with subnormals), widened again.
__device__ __forceinline__ float round_f16(float v) { return (float)(_Float16)v; }
__device__ __forceinline__ bf16_t f32_to_bf16(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }
__device__ __forceinline__ float bf16_to_f32(bf16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }
__device__ __forceinline__ float bf16lo_to_f32(uint32_t p) { return __builtin_bit_cast(float, p << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t p) { return __builtin_bit_cast(float, p & 0xFFFF0000u); }
// two floats -> packed bf16 pair (low half = a), one v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    f2 f = {a, b};
    v2 r = __builtin_convertvector(f, v2);
    return __builtin_bit_cast(uint32_t, r);
}

// Value of one output element before its final rounding: v = accumulator + bias; with a residual
// tensor, residual + bf16(v) - the two roundings of `residual + linear(x)` evaluated as two bf16
// tensor operations.  idx = m * N + n; only read when `residual` is given.
__device__ __forceinline__ float add_residual(float v, const bf16_t* residual, int64_t idx) {
    return residual ? bf16_to_f32(residual[idx]) + bf16_to_f32(f32_to_bf16(v)) : v;
}

// Arithmetic of the block decode.  Num<SNGGUF_NUM_GGML_FP32> works in fp32, where every product
// of the three formats is exact.  Num<SNGGUF_NUM_UPSTREAM_FP16> works in native fp16
// (v_mul_f16 / v_sub_f16, round-to-nearest-even, subnormals and signed zeros kept): each
// upstream tensor op is "compute in fp32, round to fp16", and because the operands are fp16
// values or small integers the exact result fits fp32, so the single fp16 rounding of the
// native instruction gives the same bits.  The library is compiled with -ffp-contract=off so
// that no two of these roundings are fused.
template <int NUM> struct Num;
template <> struct Num<SNGGUF_NUM_GGML_FP32> {
    typedef float T;
    static __device__ __forceinline__ T scale(uint16_t f16_bits) { return f16_to_f32(f16_bits); }
    static __device__ __forceinline__ T integer(int q) { return (float)q; }
    static __device__ __forceinline__ float widen(T v) { return v; }
};
template <> struct Num<SNGGUF_NUM_UPSTREAM_FP16> {
    typedef _Float16 T;
    static __device__ __forceinline__ T scale(uint16_t f16_bits) { return __builtin_bit_cast(_Float16, f16_bits); }
    static __device__ __forceinline__ T integer(int q) { return (_Float16)(short)q; }  // |q| <= 2048: exact
    static __device__ __forceinline__ float widen(T v) { return (float)v; }
};

// ---- unaligned loads ----------------------------------------------------------------------
// GGUF blocks are only 2-byte aligned (34- and 210-byte blocks).  memcpy from a pointer of
// declared alignment lets the compiler pick the widest legal access.

__device__ __forceinline__ uint16_t ld_u16(const uint8_t* p) {
    return *reinterpret_cast<const uint16_t*>(p);
}
// 4 / 16 bytes from an address that is only 2-byte aligned (gfx950 runs global and LDS
// accesses in unaligned mode, so these become one dword / dwordx4 access)
__device__ __forceinline__ uint32_t ld_u32_a2(const uint8_t* p) {
    uint32_t v;
    __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 4);
    return v;
}
__device__ __forceinline__ u32x4_t ld_u128_a2(const uint8_t* p) {
    u32x4_t v;
    __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 16);
    return v;
}
__device__ __forceinline__ u32x4_t ld_u128_a4(const uint8_t* p) {
    u32x4_t v;
    __builtin_memcpy(&v, __builtin_assume_aligned(p, 4), 16);
    return v;
}
__device__ __forceinline__ uint32_t ld_u32(const uint8_t* p) { return *reinterpret_cast<const uint32_t*>(p); }

// ---- format constants -----------------------------------------------------------------------

template <int QT> struct Fmt;
template <> struct Fmt<SNGGUF_TYPE_Q4_0> { static constexpr int bs = 32, ts = 18; };
template <> struct Fmt<SNGGUF_TYPE_Q4_1> { static constexpr int bs = 32, ts = 20; };
template <> struct Fmt<SNGGUF_TYPE_Q5_0> { static constexpr int bs = 32, ts = 22; };
template <> struct Fmt<SNGGUF_TYPE_Q5_1> { static constexpr int bs = 32, ts = 24; };
template <> struct Fmt<SNGGUF_TYPE_Q8_0> { static constexpr int bs = 32, ts = 34; };
template <> struct Fmt<SNGGUF_TYPE_Q2_K> { static constexpr int bs = 256, ts = 84; };
template <> struct Fmt<SNGGUF_TYPE_Q3_K> { static constexpr int bs = 256, ts = 110; };
template <> struct Fmt<SNGGUF_TYPE_Q4_K> { static constexpr int bs = 256, ts = 144; };
template <> struct Fmt<SNGGUF_TYPE_Q5_K> { static constexpr int bs = 256, ts = 176; };
template <> struct Fmt<SNGGUF_TYPE_Q6_K> { static constexpr int bs = 256, ts = 210; };

// Q4_K: 6-bit (scale, min) of sub-block j from the 12 packed bytes held as three dwords
// s0 = bytes 0..3, s1 = bytes 4..7, s2 = bytes 8..11.
__device__ __forceinline__ void q4k_scale_min(uint32_t s0, uint32_t s1, uint32_t s2, int j, uint32_t& sc, uint32_t& mn) {
    if (j < 4) {
        sc = (s0 >> (8 * j)) & 63u;
        mn = (s1 >> (8 * j)) & 63u;
    } else {
        const int i = j - 4;
        const uint32_t b = (s2 >> (8 * i)) & 0xFFu;
        sc = (b & 0x0Fu) | (((s0 >> (8 * i + 6)) & 3u) << 4);
        mn = (b >> 4) | (((s1 >> (8 * i + 6)) & 3u) << 4);
    }
}

// Runs CALL(<type constant>) for the run-time quant type (CALL is a macro or a generic lambda-like
// macro that returns); unknown types return SNGGUF_E_BADTYPE.
#define SNGGUF_DISPATCH_TYPE(qtype, CALL)                       \
    switch (qtype) {                                            \
    case SNGGUF_TYPE_Q4_0: return CALL(SNGGUF_TYPE_Q4_0);       \
    case SNGGUF_TYPE_Q4_1: return CALL(SNGGUF_TYPE_Q4_1);       \
    case SNGGUF_TYPE_Q5_0: return CALL(SNGGUF_TYPE_Q5_0);       \
    case SNGGUF_TYPE_Q5_1: return CALL(SNGGUF_TYPE_Q5_1);       \
    case SNGGUF_TYPE_Q8_0: return CALL(SNGGUF_TYPE_Q8_0);       \
    case SNGGUF_TYPE_Q2_K: return CALL(SNGGUF_TYPE_Q2_K);       \
    case SNGGUF_TYPE_Q3_K: return CALL(SNGGUF_TYPE_Q3_K);       \
    case SNGGUF_TYPE_Q4_K: return CALL(SNGGUF_TYPE_Q4_K);       \
    case SNGGUF_TYPE_Q5_K: return CALL(SNGGUF_TYPE_Q5_K);       \
    case SNGGUF_TYPE_Q6_K: return CALL(SNGGUF_TYPE_Q6_K);       \
    default: return SNGGUF_E_BADTYPE;                           \
    }

// ---- 8-element decoders (standalone dequantize, GEMM tile fill) -------------------------------
// decode8<QT,NUM>(row, e0, w): eight consecutive elements e0..e0+7 (e0 % 8 == 0) of a packed
// row, as the fp32 value of the ggml decode (NUM 0) or of the upstream fp16 tensor (NUM 1).

template <int QT, int NUM>
__device__ __forceinline__ void decode8(const uint8_t* __restrict__ row, int64_t e0, float (&w)[8]);

template <int NUM>
__device__ __forceinline__ void decode8_q8_0(const uint8_t* __restrict__ row, int64_t e0, float (&w)[8]) {
    typedef Num<NUM> A;
    const uint8_t* blk = row + (e0 >> 5) * 34;
    const typename A::T d = A::scale(ld_u16(blk));
    const uint8_t* qs = blk + 2 + (e0 & 31);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t h = ld_u16(qs + 2 * i);
        w[2 * i] = A::widen(d * A::integer((int8_t)(h & 0xFF)));
        w[2 * i + 1] = A::widen(d * A::integer((int8_t)(h >> 8)));
    }
}

// The four legacy formats: 32-element blocks, element l in the low nibble of qs[l], element
// l + 16 in the high nibble; Q5_x add bit e of a 32-bit word as fifth bit of element e; the _0
// formats subtract half the range, the _1 formats add a block minimum m.
// HDR = bytes before qh/qs (2: d; 4: d, m); FIVE = has the fifth-bit word.
template <int NUM, int TS, bool HAS_MIN, bool FIVE>
__device__ __forceinline__ void decode8_legacy(const uint8_t* __restrict__ row, int64_t e0, float (&w)[8]) {
    typedef Num<NUM> A;
    const uint8_t* blk = row + (e0 >> 5) * TS;  // only 2-byte aligned in general
    const int r = (int)(e0 & 31);
    const int hi = r >> 4;
    const int l0 = r & 15;
    constexpr int kHdr = HAS_MIN ? 4 : 2;
    const typename A::T d = A::scale(ld_u16(blk));
    const uint32_t hbits = FIVE ? (ld_u32_a2(blk + kHdr) >> r) : 0u;
    const uint8_t* qs = blk + kHdr + (FIVE ? 4 : 0) + l0;
    const uint32_t q0 = ld_u32_a2(qs), q1 = ld_u32_a2(qs + 4);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t byte = ((i < 4 ? q0 : q1) >> (8 * (i & 3))) & 0xFFu;
        int q = (int)(hi ? (byte >> 4) : (byte & 0x0Fu));
        if constexpr (FIVE) q |= (int)(((hbits >> i) & 1u) << 4);
        if constexpr (HAS_MIN) {
            // fp32: d*q exact, one rounding in the sum; fp16: R(R(d*q) + m)
            w[i] = A::widen(d * A::integer(q) + A::scale(ld_u16(blk + 2)));
        } else {
            w[i] = A::widen(d * A::integer(q - (FIVE ? 16 : 8)));
        }
    }
}

// Q2_K: { u8 scales[16]; u8 qs[64]; f16 d; f16 dmin }.  Per 128-element half, bit pair j of
// qs[32 * half + l] is element 32 * j + l; group g = e / 16 has scale scales[g] & 15 and min
// scales[g] >> 4.
template <int NUM>
__device__ __forceinline__ void decode8_q2_k(const uint8_t* __restrict__ row, int64_t e0, float (&w)[8]) {
    typedef Num<NUM> A;
    const uint8_t* blk = row + (e0 >> 8) * 84;
    const int r = (int)(e0 & 255);
    const int half = r >> 7, j = (r >> 5) & 3, l0 = r & 31;
    const uint32_t sm = blk[r >> 4];
    const uint32_t dd = ld_u32_a2(blk + 80);
    const typename A::T DL = A::scale((uint16_t)(dd & 0xFFFF)) * A::integer((int)(sm & 15u));
    const typename A::T ML = A::scale((uint16_t)(dd >> 16)) * A::integer((int)(sm >> 4));
    const uint8_t* qs = blk + 16 + 32 * half + l0;
    const uint32_t q0 = ld_u32_a2(qs) >> (2 * j), q1 = ld_u32_a2(qs + 4) >> (2 * j);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int q = (int)(((i < 4 ? q0 : q1) >> (8 * (i & 3))) & 3u);
        w[i] = A::widen(DL * A::integer(q) - ML);
    }
}

// Q3_K: { u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d }.  Quant = bit pair as in Q2_K, minus 4
// unless bit (4 * half + j) of hmask[l] is set; the 6-bit scale of group g has its low nibble in
// scales[g % 8] (upper nibble for g >= 8), its high two bits in scales[8 + g % 4] at bit
// 2 * (g / 4), and is offset by -32.
template <int NUM>
__device__ __forceinline__ void decode8_q3_k(const uint8_t* __restrict__ row, int64_t e0, float (&w)[8]) {
    typedef Num<NUM> A;
    const uint8_t* blk = row + (e0 >> 8) * 110;  // 2-byte aligned
    const int r = (int)(e0 & 255);
    const int half = r >> 7, j = (r >> 5) & 3, l0 = r & 31;
    const int g = r >> 4;
    const uint32_t lo = g < 8 ? (blk[96 + g] & 15u) : ((uint32_t)blk[96 + g - 8] >> 4);
    const uint32_t hi = ((uint32_t)blk[104 + (g & 3)] >> (2 * (g >> 2))) & 3u;
    const typename A::T DL = A::scale(ld_u16(blk + 108)) * A::integer((int)(lo | (hi << 4)) - 32);
    const uint8_t* qs = blk + 32 + 32 * half + l0;
    const uint32_t q0 = ld_u32_a2(qs) >> (2 * j), q1 = ld_u32_a2(qs + 4) >> (2 * j);
    const int hb = 4 * half + j;
    const uint32_t h0 = ld_u32_a2(blk + l0) >> hb, h1 = ld_u32_a2(blk + l0 + 4) >> hb;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int sh = 8 * (i & 3);
        const int q = (int)(((i < 4 ? q0 : q1) >> sh) & 3u) - ((((i < 4 ? h0 : h1) >> sh) & 1u) ? 0 : 4);
        w[i] = A::widen(DL * A::integer(q));
    }
}

template <int NUM>
__device__ __forceinline__ void decode8_q4_k(const uint8_t* __restrict__ row, int64_t e0, float (&w)[8]) {
    typedef Num<NUM> A;
    const uint8_t* blk = row + (e0 >> 8) * 144;  // 144 = 16 * 9: blocks stay 4-byte aligned when the row is
    const int r = (int)(e0 & 255);
    const int c = r >> 6;          // 64-element chunk
    const int hi = (r >> 5) & 1;   // 0: low nibbles (sub-block 2c), 1: high nibbles (sub-block 2c+1)
    const int l0 = r & 31;
    const uint32_t dd = ld_u32(blk);
    uint32_t sc, mn;
    q4k_scale_min(ld_u32(blk + 4), ld_u32(blk + 8), ld_u32(blk + 12), 2 * c + hi, sc, mn);
    const typename A::T D = A::scale((uint16_t)(dd & 0xFFFF)) * A::integer((int)sc);
    const typename A::T DM = A::scale((uint16_t)(dd >> 16)) * A::integer((int)mn);
    const uint8_t* qs = blk + 16 + 32 * c + l0;
    const uint32_t q0 = ld_u32(qs), q1 = ld_u32(qs + 4);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t byte = ((i < 4 ? q0 : q1) >> (8 * (i & 3))) & 0xFFu;
        const int q = (int)(hi ? (byte >> 4) : (byte & 0x0Fu));
        // fp32: both products exact, one rounding in the subtraction; fp16: R(R(D*q) - DM)
        w[i] = A::widen(D * A::integer(q) - DM);
    }
}

// Q5_K: Q4_K with a fifth quant bit, bit j of qh[l] for element l of sub-block j
template <int NUM>
__device__ __forceinline__ void decode8_q5_k(const uint8_t* __restrict__ row, int64_t e0, float (&w)[8]) {
    typedef Num<NUM> A;
    const uint8_t* blk = row + (e0 >> 8) * 176;  // 176 = 16 * 11: blocks stay 4-byte aligned when the row is
    const int r = (int)(e0 & 255);
    const int c = r >> 6;
    const int hi = (r >> 5) & 1;
    const int l0 = r & 31;
    const int j = 2 * c + hi;
    const uint32_t dd = ld_u32(blk);
    uint32_t sc, mn;
    q4k_scale_min(ld_u32(blk + 4), ld_u32(blk + 8), ld_u32(blk + 12), j, sc, mn);
    const typename A::T D = A::scale((uint16_t)(dd & 0xFFFF)) * A::integer((int)sc);
    const typename A::T DM = A::scale((uint16_t)(dd >> 16)) * A::integer((int)mn);
    const uint8_t* qh = blk + 16 + l0;
    const uint8_t* qs = blk + 48 + 32 * c + l0;
    const uint32_t q0 = ld_u32(qs), q1 = ld_u32(qs + 4), h0 = ld_u32(qh), h1 = ld_u32(qh + 4);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t byte = ((i < 4 ? q0 : q1) >> (8 * (i & 3))) & 0xFFu;
        const uint32_t hbit = (((i < 4 ? h0 : h1) >> (8 * (i & 3))) >> j) & 1u;
        const int q = (int)((hi ? (byte >> 4) : (byte & 0x0Fu)) | (hbit << 4));
        w[i] = A::widen(D * A::integer(q) - DM);
    }
}

template <int NUM>
__device__ __forceinline__ void decode8_q6_k(const uint8_t* __restrict__ row, int64_t e0, float (&w)[8]) {
    typedef Num<NUM> A;
    const uint8_t* blk = row + (e0 >> 8) * 210;
    const int r = (int)(e0 & 255);
    const int h = r >> 7;           // 128-element half
    const int quad = (r >> 5) & 3;  // which of q1..q4
    const int l0 = r & 31;
    const uint8_t* ql = blk + 64 * h + 32 * (quad & 1) + l0;
    const uint8_t* qh = blk + 128 + 32 * h + l0;
    const int sh_l = 4 * (quad >> 1);
    const int sh_h = 2 * quad;
    const typename A::T D = A::scale(ld_u16(blk + 208)) * A::integer((int8_t)blk[192 + (r >> 4)]);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t lo2 = ld_u16(ql + 2 * i), hi2 = ld_u16(qh + 2 * i);
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const uint32_t lb = (lo2 >> (8 * k)) & 0xFFu, hb = (hi2 >> (8 * k)) & 0xFFu;
            const int q = (int)(((lb >> sh_l) & 0x0Fu) | (((hb >> sh_h) & 3u) << 4)) - 32;
            w[2 * i + k] = A::widen(D * A::integer(q));
        }
    }
}

template <int QT, int NUM>
__device__ __forceinline__ void decode8(const uint8_t* __restrict__ row, int64_t e0, float (&w)[8]) {
    if constexpr (QT == SNGGUF_TYPE_Q8_0) decode8_q8_0<NUM>(row, e0, w);
    else if constexpr (QT == SNGGUF_TYPE_Q4_0) decode8_legacy<NUM, 18, false, false>(row, e0, w);
    else if constexpr (QT == SNGGUF_TYPE_Q4_1) decode8_legacy<NUM, 20, true, false>(row, e0, w);
    else if constexpr (QT == SNGGUF_TYPE_Q5_0) decode8_legacy<NUM, 22, false, true>(row, e0, w);
    else if constexpr (QT == SNGGUF_TYPE_Q5_1) decode8_legacy<NUM, 24, true, true>(row, e0, w);
    else if constexpr (QT == SNGGUF_TYPE_Q2_K) decode8_q2_k<NUM>(row, e0, w);
    else if constexpr (QT == SNGGUF_TYPE_Q3_K) decode8_q3_k<NUM>(row, e0, w);
    else if constexpr (QT == SNGGUF_TYPE_Q4_K) decode8_q4_k<NUM>(row, e0, w);
    else if constexpr (QT == SNGGUF_TYPE_Q5_K) decode8_q5_k<NUM>(row, e0, w);
    else {
        static_assert(QT == SNGGUF_TYPE_Q6_K, "no decoder for this quant type");
        decode8_q6_k<NUM>(row, e0, w);
    }
}

// ---- Q8_0: one dword of quants -> four bf16 (shared by the GEMV and GEMM kernels) ---------------

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// Four int8 quants of one dword times the block scale (given in both halves of d2_bits, fp16)
// -> two packed bf16 pairs.
template <int NUM>
__device__ __forceinline__ void q8_dword_bf16_d2(uint32_t d2_bits, uint32_t dw, uint32_t& p01, uint32_t& p23) {
    if constexpr (NUM == SNGGUF_NUM_UPSTREAM_FP16) {
        // bytes -> fp16 without a convert: 0x6400 | u is the half 1024 + u, u = q + 128
        const uint32_t u = dw ^ 0x80808080u;
        const half2_t bias = {(_Float16)1152.0f, (_Float16)1152.0f};
        const half2_t d2 = __builtin_bit_cast(half2_t, d2_bits);
        const half2_t a = (__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - bias) * d2;
        const half2_t b = (__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - bias) * d2;
        p01 = pack_bf16((float)a[0], (float)a[1]);
        p23 = pack_bf16((float)b[0], (float)b[1]);
    } else {
        const float d = f16_to_f32((uint16_t)(d2_bits & 0xFFFF));
        p01 = pack_bf16(d * (float)(int8_t)(dw & 0xFF), d * (float)(int8_t)((dw >> 8) & 0xFF));
        p23 = pack_bf16(d * (float)(int8_t)((dw >> 16) & 0xFF), d * (float)(int8_t)(dw >> 24));
    }
}
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

// fp16 -> fp32 on the matrix core.  With A = the 16 x 16 identity, v_mfma_f32_16x16x16_f16 computes
// D = I . B + C, and because a lane's B elements (column lane % 16, rows 4 (lane / 16) .. + 3) sit
// at the same positions as its D elements, every lane gets back its own four fp16 values as
// exact fp32 (+ c).  The K-quant decode is bound by the vector ALU while the matrix cores are
// nearly idle, so this takes one conversion per element off the busy unit.  fp16 subnormals are
// widened exactly; a signed zero comes back as + 0, and a non-finite element (a scale product
// beyond the fp16 range) turns the other values of its weight row in that instruction into NaN
// (0 . inf) - the row's dot product is non-finite either way.
__device__ __forceinline__ half4_t identity_row(int lane) {
    half4_t a;
#pragma unroll
    for (int e = 0; e < 4; e++) a[e] = (4 * (lane >> 4) + e == (lane & 15)) ? (_Float16)1.0f : (_Float16)0.0f;
    return a;
}
__device__ __forceinline__ f32x4_t widen_f16x4(half4_t ident, half2_t lo, half2_t hi, f32x4_t c) {
    const half4_t b = {lo[0], lo[1], hi[0], hi[1]};
    return __builtin_amdgcn_mfma_f32_16x16x16f16(ident, b, c, 0, 0, 0);
}

// q8_dword_bf16_d2 with the fp16 -> fp32 step on the matrix core (all 64 lanes must call it): two vector instructions
// per weight instead of three.  NUM 0: the widening instruction's accumulator input takes the 1024 + 128 off, so the
// quant arrives as an exact float without a convert either.
template <int NUM>
__device__ __forceinline__ void q8_dword_bf16_widened(half4_t ident, uint32_t d2_bits, uint32_t dw, uint32_t& p01, uint32_t& p23) {
    const uint32_t u = dw ^ 0x80808080u;
    const half2_t h01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u));
    const half2_t h23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u));
    if constexpr (NUM == SNGGUF_NUM_UPSTREAM_FP16) {
        const half2_t bias = {(_Float16)1152.0f, (_Float16)1152.0f};
        const half2_t d2 = __builtin_bit_cast(half2_t, d2_bits);
        const f32x4_t w = widen_f16x4(ident, (h01 - bias) * d2, (h23 - bias) * d2, f32x4_t{0.f, 0.f, 0.f, 0.f});
        p01 = pack_bf16(w[0], w[1]);
        p23 = pack_bf16(w[2], w[3]);
    } else {
        const float d = f16_to_f32((uint16_t)(d2_bits & 0xFFFF));
        const f32x4_t qf = widen_f16x4(ident, h01, h23, f32x4_t{-1152.f, -1152.f, -1152.f, -1152.f});
        p01 = pack_bf16(d * qf[0], d * qf[1]);
        p23 = pack_bf16(d * qf[2], d * qf[3]);
    }
}
// Same with the scale as the 16 bits of the block header.
template <int NUM>
__device__ __forceinline__ void q8_dword_bf16(uint16_t d_bits, uint32_t dw, uint32_t& p01, uint32_t& p23) {
    q8_dword_bf16_d2<NUM>((uint32_t)d_bits | ((uint32_t)d_bits << 16), dw, p01, p23);
}

// ---- wavefront sum ---------------------------------------------------------------------------
// Butterfly over the 64 lanes: four DPP steps inside each row of 16 lanes, then two
// ds_swizzle/bpermute steps across rows.  Every lane ends with the full sum.

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);  // row_half_mirror
    v += dpp_f32<0x140>(v);  // row_mirror
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

// ---- arg-max over output columns (lm_head followed by torch.argmax) ------------------------------------------
// A (value, column) pair packed so that an unsigned 64-bit maximum picks the largest bf16 value and, among equal
// values, the lowest column - what torch.argmax returns (first maximal index); a NaN counts as the largest value,
// as it does there; -0 and +0 compare equal there, so both map to the key of +0.  High word: the bf16 bits mapped to
// an unsigned number that grows with the value; low word: 2^32 - 1 - column.
__device__ __forceinline__ uint64_t argmax_key(float v, int64_t n) {
    uint32_t b = f32_to_bf16(v);
    if ((b & 0x7FFFu) == 0) b = 0;              // a zero of either sign
    uint32_t k = (b & 0x8000u) ? (~b & 0xFFFFu) : (b | 0x8000u);
    if ((b & 0x7FFFu) > 0x7F80u) k = 0xFFFFu;   // NaN of either sign
    return ((uint64_t)k << 32) | (uint64_t)(0xFFFFFFFFu - (uint32_t)n);
}
__device__ __forceinline__ uint64_t u64_max(uint64_t a, uint64_t b) { return a > b ? a : b; }
__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int mask) {
    const uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)v, mask, 64), hi = (uint32_t)__shfl_xor((int)(uint32_t)(v >> 32), mask, 64);
    return ((uint64_t)hi << 32) | lo;
}
// The four lanes (r, g = 0..3) that hold one activation row's outputs of a 16-row group combine their keys; lane
// g = 0 then writes the group's entry.  All four lanes of a row take the same branches, so the exchange is safe
// inside code that rows >= M have left.
__device__ __forceinline__ void argmax_store(uint64_t key, int g, uint64_t* __restrict__ amax, int m, int64_t slot, int64_t slots) {
    key = u64_max(key, shfl_xor_u64(key, 16));
    key = u64_max(key, shfl_xor_u64(key, 32));
    if (g == 0) amax[(int64_t)m * slots + slot] = key;
}

// ---- RMSNorm in front of the contraction -------------------------------------------------------------
// The decoder layers feed q / k / v and gate / up with RMSNorm(hidden) (modeling_qwen3.py:183-197, :919, :938):
//   v = bf16(x * rsqrt(mean(x^2) + eps))   (fp32 arithmetic, one rounding)      out = bf16(gamma * v)
// With `gamma` given, a kernel below applies it to the activations it has staged in LDS, so the norm needs no
// launch and no buffer of its own.  Only offered where the activations are staged once per workgroup (or once
// per wavefront share) - a few rows; applied per fragment it would cost as much vector work as the weight decode.
// 1 / sqrt(mean of squares + eps) with a correctly rounded square root and a correctly rounded division - the two
// roundings of torch.rsqrt on the CPU - instead of the hardware's reciprocal-square-root approximation, which is
// within one unit in the last place of that.  A last-place difference in rstd is invisible except for a row whose
// activations share a mantissa for which x * rstd falls exactly between two bf16 values: dozens of normalized
// activations then round the other way.  (The order in which the squares are added up is the other source of such
// a difference, and that one cannot be matched to a CPU reduction.)
__device__ __forceinline__ float rms_rstd(float sum_of_squares, int64_t K, float eps) {
    return 1.0f / sqrtf(sum_of_squares / (float)K + eps);
}
__device__ __forceinline__ float sumsq_piece(u32x4_t xv) {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t d = xv[i];
        const float a = __builtin_bit_cast(float, d << 16), b = __builtin_bit_cast(float, d & 0xFFFF0000u);
        ss += a * a;
        ss += b * b;
    }
    return ss;
}
__device__ __forceinline__ u32x4_t rmsnorm_piece(u32x4_t xv, u32x4_t gv, float rstd) {
    u32x4_t o;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t xd = xv[i], gd = gv[i];
        const float x0 = __builtin_bit_cast(float, xd << 16), x1 = __builtin_bit_cast(float, xd & 0xFFFF0000u);
        const float g0 = __builtin_bit_cast(float, gd << 16), g1 = __builtin_bit_cast(float, gd & 0xFFFF0000u);
        const float v0 = bf16_to_f32(f32_to_bf16(x0 * rstd)), v1 = bf16_to_f32(f32_to_bf16(x1 * rstd));
        o[i] = pack_bf16(g0 * v0, g1 * v1);
    }
    return o;
}


// ---- hand-over state of the one-launch decode MLP kernels ----------------------------------------------------
// At the start of the caller's workspace, zero before its first use: the generation counter that tags the activation
// words of a launch (advanced by the last workgroup to finish, through the trailing `done` counter), a sticky status word
// (1: some wavefront gave up waiting), and one flag per 16-row group of gate / up.
struct MlpCtl {
    uint32_t gen, done, status, pad[61];
    uint32_t flags[1024];
};
constexpr int64_t kMlpCtlBytes = 8192;   // the tagged activation words [M][inter / 2] follow at this offset

}  // namespace sngguf
