// Q4_K / Q5_K / Q6_K decode GEMV on the matrix cores (1 <= M <= 16, K % 256 == 0).
//
// Same shape as the Q8_0 kernel: a workgroup owns R * 16 weight rows (for the SiLU-gated pair the
// same rows of the gate and of the up matrix, on separate wavefronts), its wavefronts split K by
// super-blocks and add their partial sums through LDS at the end.  Per wavefront and super-block
// (256 elements of each row):
//   * the packed bytes of the R * 16 rows are fetched with 16-byte loads, consecutive lanes walking
//     along a row, one super-block ahead, and dropped into the wavefront's private LDS slab.  Q4_K
//     and Q5_K super-blocks (144 / 176 bytes) are 16-byte aligned; Q6_K super-blocks (210 bytes) are only 2-byte
//     aligned and are fetched as 13 unaligned 16-byte pieces plus the 2-byte scale, which never
//     touches a byte outside the super-block and puts every field at an aligned LDS address;
//   * lane (r = lane % 16, g = lane / 16) decodes, for each 32-element sub-block j, elements
//     8 g .. 8 g + 7 of row r to bf16 (rounding chain by numerics mode) as the A operand of
//     v_mfma_f32_16x16x32_bf16; the B operand is x[m = lane % 16][256 s + 32 j + 8 g ..].  With R = 2
//     one activation fragment feeds two row groups, which halves the activation traffic per
//     packed byte at M = 16.
// Nothing dequantized is written to memory.

#include "sngguf_common.hpp"

namespace sngguf {

namespace {


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

// Four small unsigned integers (one per byte of v, each < 256) -> (v - zero) * D - DM as two packed
// bf16 pairs.  NUM 1: every operation rounds to fp16 (0x6400 | b is the half 1024 + b, so the
// integer is formed without a convert); NUM 0: exact fp32 products, one rounding in the subtraction
// (the - 1024 - zero rides on the accumulator input of the widening instruction).  Must be called
// by all 64 lanes; `ident` is identity_row(lane).
template <int NUM, bool HAS_MIN>
__device__ __forceinline__ void kq_dword_bf16(half4_t ident, uint32_t v, float zero, typename Num<NUM>::T D,
                                              typename Num<NUM>::T DM, uint32_t& p01, uint32_t& p23) {
    const half2_t h01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u));
    const half2_t h23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u));
    if constexpr (NUM == SNGGUF_NUM_UPSTREAM_FP16) {
        const _Float16 off = (_Float16)(1024.0f + zero);
        const half2_t off2 = {off, off};
        const half2_t D2 = {D, D};
        half2_t a = (h01 - off2) * D2, b = (h23 - off2) * D2;
        if constexpr (HAS_MIN) {
            const half2_t M2 = {DM, DM};
            a = a - M2;
            b = b - M2;
        }
        const f32x4_t w = widen_f16x4(ident, a, b, f32x4_t{0.f, 0.f, 0.f, 0.f});
        p01 = pack_bf16(w[0], w[1]);
        p23 = pack_bf16(w[2], w[3]);
    } else {
        const float c = -(1024.0f + zero);
        const f32x4_t qf = widen_f16x4(ident, h01, h23, f32x4_t{c, c, c, c});
        float w[4] = {D * qf[0], D * qf[1], D * qf[2], D * qf[3]};
        if constexpr (HAS_MIN) {
#pragma unroll
            for (int e = 0; e < 4; e++) w[e] = w[e] - DM;
        }
        p01 = pack_bf16(w[0], w[1]);
        p23 = pack_bf16(w[2], w[3]);
    }
}

template <int QT> struct Slab;
// Q4_K: 9 pieces per row and super-block, rows back to back (144 = 9 * 16)
template <> struct Slab<SNGGUF_TYPE_Q4_K> {
    static constexpr int ts = 144, pieces = 9, stride = 144;
};
// Q5_K: 11 pieces per row and super-block (176 = 11 * 16); 44-dword rows fall on distinct bank groups
template <> struct Slab<SNGGUF_TYPE_Q5_K> {
    static constexpr int ts = 176, pieces = 11, stride = 176;
};
// Q6_K: 13 pieces (208 bytes) + the fp16 scale at byte 208; 240-byte rows fall on distinct banks
template <> struct Slab<SNGGUF_TYPE_Q6_K> {
    static constexpr int ts = 210, pieces = 13, stride = 240;
};

// The four A operands of half a super-block (sub-blocks 4 HALF .. 4 HALF + 3) of one row, fed to
// `emit(jj, a)` with jj = 0..3.  `row` points at the row's super-block in the slab; g = lane / 16.
template <int NUM, int HALF, typename Emit>
__device__ __forceinline__ void decode_q4_k(half4_t ident, const uint8_t* row, int g, Emit&& emit) {
    typedef Num<NUM> A;
    const u32x4_t head = *reinterpret_cast<const u32x4_t*>(row);  // d, dmin, 12 scale bytes
    const typename A::T d = A::scale((uint16_t)(head[0] & 0xFFFF)), dmin = A::scale((uint16_t)(head[0] >> 16));
#pragma unroll
    for (int cc = 0; cc < 2; cc++) {
        const int c = 2 * HALF + cc;
        const u32x2_t qs = *reinterpret_cast<const u32x2_t*>(row + 16 + 32 * c + 8 * g);
#pragma unroll
        for (int hi = 0; hi < 2; hi++) {
            const int j = 2 * c + hi;
            uint32_t sc, mn;
            q4k_scale_min(head[1], head[2], head[3], j, sc, mn);
            const typename A::T D = d * A::integer((int)sc), DM = dmin * A::integer((int)mn);
            const uint32_t v0 = (hi ? qs[0] >> 4 : qs[0]) & 0x0F0F0F0Fu, v1 = (hi ? qs[1] >> 4 : qs[1]) & 0x0F0F0F0Fu;
            uint32_t a0, a1, a2, a3;
            kq_dword_bf16<NUM, true>(ident, v0, 0.f, D, DM, a0, a1);
            kq_dword_bf16<NUM, true>(ident, v1, 0.f, D, DM, a2, a3);
            emit(j - 4 * HALF, u32x4_t{a0, a1, a2, a3});
        }
    }
}

// Q5_K: as Q4_K, the fifth bit of element l of sub-block j is bit j of qh[l]
template <int NUM, int HALF, typename Emit>
__device__ __forceinline__ void decode_q5_k(half4_t ident, const uint8_t* row, int g, Emit&& emit) {
    typedef Num<NUM> A;
    const u32x4_t head = *reinterpret_cast<const u32x4_t*>(row);  // d, dmin, 12 scale bytes
    const typename A::T d = A::scale((uint16_t)(head[0] & 0xFFFF)), dmin = A::scale((uint16_t)(head[0] >> 16));
    const u32x2_t qh = *reinterpret_cast<const u32x2_t*>(row + 16 + 8 * g);
#pragma unroll
    for (int cc = 0; cc < 2; cc++) {
        const int c = 2 * HALF + cc;
        const u32x2_t qs = *reinterpret_cast<const u32x2_t*>(row + 48 + 32 * c + 8 * g);
#pragma unroll
        for (int hi = 0; hi < 2; hi++) {
            const int j = 2 * c + hi;
            uint32_t sc, mn;
            q4k_scale_min(head[1], head[2], head[3], j, sc, mn);
            const typename A::T D = d * A::integer((int)sc), DM = dmin * A::integer((int)mn);
            uint32_t a[4];
#pragma unroll
            for (int w = 0; w < 2; w++) {
                const uint32_t lo = (hi ? qs[w] >> 4 : qs[w]) & 0x0F0F0F0Fu;
                const uint32_t hb = ((qh[w] >> j) & 0x01010101u) << 4;
                kq_dword_bf16<NUM, true>(ident, lo | hb, 0.f, D, DM, a[2 * w], a[2 * w + 1]);
            }
            emit(j - 4 * HALF, u32x4_t{a[0], a[1], a[2], a[3]});
        }
    }
}

template <int NUM, int HALF, typename Emit>
__device__ __forceinline__ void decode_q6_k(half4_t ident, const uint8_t* row, int g, Emit&& emit) {
    typedef Num<NUM> A;
    constexpr int h = HALF;  // 128-element half of the super-block = sub-blocks 4 h .. 4 h + 3
    const u32x2_t scales = *reinterpret_cast<const u32x2_t*>(row + 192 + 8 * h);  // int8 sub-scales 8 h .. 8 h + 7
    const typename A::T d = A::scale(*reinterpret_cast<const uint16_t*>(row + 208));
    const u32x2_t qh = *reinterpret_cast<const u32x2_t*>(row + 128 + 32 * h + 8 * g);
#pragma unroll
    for (int half = 0; half < 2; half++) {  // ql bytes 64 h + 32 half + 8 g ..: low nibbles p = half, high nibbles p = half + 2
        const u32x2_t ql = *reinterpret_cast<const u32x2_t*>(row + 64 * h + 32 * half + 8 * g);
#pragma unroll
        for (int top = 0; top < 2; top++) {
            const int p = half + 2 * top;
            // sub-scale of elements 128 h + 32 p + 8 g ..: index 8 h + 2 p + g / 2
            const uint32_t sw = scales[p >> 1];
            const int sc = (int)(int8_t)((sw >> (8 * (2 * (p & 1) + (g >> 1)))) & 0xFF);
            const typename A::T D = d * A::integer(sc);
            uint32_t a[4];
#pragma unroll
            for (int w = 0; w < 2; w++) {
                const uint32_t lo = (top ? ql[w] >> 4 : ql[w]) & 0x0F0F0F0Fu;
                const uint32_t hb = ((qh[w] >> (2 * p)) & 0x03030303u) << 4;
                kq_dword_bf16<NUM, false>(ident, lo | hb, 32.f, D, D, a[2 * w], a[2 * w + 1]);
            }
            emit(p, u32x4_t{a[0], a[1], a[2], a[3]});
        }
    }
}

template <int QT, int NUM, int R, bool GATED, int WMAX>
__global__ __launch_bounds__(64 * WMAX) void gemv_kq_mfma_kernel(const bf16_t* __restrict__ x, int M,
                                                                 const uint8_t* __restrict__ qa,
                                                                 const uint8_t* __restrict__ qb, int64_t N, int64_t K,
                                                                 const bf16_t* __restrict__ bias, bf16_t* __restrict__ y) {
    typedef Slab<QT> S;
    constexpr int kRows = 16 * R;
    constexpr int kPieces = kRows * S::pieces;
    constexpr int kLoads = (kPieces + 63) / 64;
    constexpr int kSlab = kRows * S::stride;
    constexpr bool kQ6 = QT == SNGGUF_TYPE_Q6_K;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int W = GATED ? waves >> 1 : waves;  // wavefronts that share one row group's K
    const int kw = GATED ? (wave >= W ? wave - W : wave) : wave;
    const uint8_t* __restrict__ q = (GATED && wave >= W) ? qb : qa;
    const int r = lane & 15, g = lane >> 4;
    const half4_t ident = identity_row(lane);
    const int64_t nsb = K >> 8;
    const int64_t row_bytes = nsb * S::ts;
    const int64_t n0 = (int64_t)blockIdx.x * kRows;
    const int s0 = (int)((int64_t)kw * nsb / W), s1 = (int)((int64_t)(kw + 1) * nsb / W);

    // piece f = lane + 64 i: 16 bytes at 16 (f % pieces) of row f / pieces
    uint32_t off[kLoads], dst[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; i++) {
        const int f = lane + 64 * i;
        const bool ok = f < kPieces;
        const int fr = ok ? f / S::pieces : 0, fp = ok ? f % S::pieces : 0;
        int64_t n = n0 + fr;
        if (n >= N) n = N - 1;  // rows past the end are decoded from the last row and never stored
        off[i] = (uint32_t)((n - n0) * row_bytes + 16 * fp);
        dst[i] = (uint32_t)(fr * S::stride + 16 * fp);
    }
    const bool tail_lane = lane + 64 * (kLoads - 1) < kPieces;
    // Q6_K: lane l < 16 R also fetches the fp16 scale (bytes 208, 209) of row l
    uint32_t doff = 0;
    if constexpr (kQ6) {
        int64_t n = n0 + (lane < kRows ? lane : 0);
        if (n >= N) n = N - 1;
        doff = (uint32_t)((n - n0) * row_bytes + 208);
    }
    const uint8_t* __restrict__ base = q + n0 * row_bytes;
    uint8_t* slab = lds + wave * kSlab;

    f32x4_t acc[R];
#pragma unroll
    for (int rg = 0; rg < R; rg++) acc[rg] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    u32x4_t pre[kLoads];
    uint16_t pre_d = 0;
    auto fetch = [&](int s) {
        const uint8_t* p = base + (int64_t)s * S::ts;
#pragma unroll
        for (int i = 0; i < kLoads - 1; i++) pre[i] = kQ6 ? ld_u128_a2(p + off[i]) : *reinterpret_cast<const u32x4_t*>(p + off[i]);
        if (tail_lane) pre[kLoads - 1] = kQ6 ? ld_u128_a2(p + off[kLoads - 1]) : *reinterpret_cast<const u32x4_t*>(p + off[kLoads - 1]);
        if constexpr (kQ6) {
            if (lane < kRows) pre_d = ld_u16(p + doff);
        }
    };
    // Lane (r, g) supplies B-operand column r.  Columns >= M are never stored, so those lanes
    // re-read the last activation row instead of being masked.
    const bool has_x = r < M;
    const bf16_t* xrow = x + (int64_t)(has_x ? r : M - 1) * K + 8 * g;

    // Activations are buffered by half super-blocks (four fragments): `xa` holds the first half of
    // the current super-block on entry; the second half is requested into `xb` before the first is
    // used, and the first half of the next super-block into `xa` before the second is used, so each
    // request has half a step of decode work to cover its latency.
    auto load_x = [&](int s, int half, u32x4_t (&dstx)[4]) {
#pragma unroll
        for (int j = 0; j < 4; j++) dstx[j] = *reinterpret_cast<const u32x4_t*>(xrow + ((int64_t)s * 8 + 4 * half + j) * 32);
    };
    u32x4_t xa[4], xb[4];
    auto step = [&](int s) {
#pragma unroll
        for (int i = 0; i < kLoads - 1; i++) *reinterpret_cast<u32x4_t*>(slab + dst[i]) = pre[i];
        if (tail_lane) *reinterpret_cast<u32x4_t*>(slab + dst[kLoads - 1]) = pre[kLoads - 1];
        if constexpr (kQ6) {
            if (lane < kRows) *reinterpret_cast<uint16_t*>(slab + lane * S::stride + 208) = pre_d;
        }
        load_x(s, 1, xb);
        if (s + 1 < s1) fetch(s + 1);
#pragma unroll
        for (int rg = 0; rg < R; rg++) {
            const uint8_t* row = slab + (16 * rg + r) * S::stride;
            auto emit = [&](int jj, const u32x4_t& a) {
                acc[rg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                                  __builtin_bit_cast(bf16x8_t, xa[jj]), acc[rg], 0, 0, 0);
            };
            if constexpr (kQ6) decode_q6_k<NUM, 0>(ident, row, g, emit);
            else if constexpr (QT == SNGGUF_TYPE_Q5_K) decode_q5_k<NUM, 0>(ident, row, g, emit);
            else decode_q4_k<NUM, 0>(ident, row, g, emit);
        }
        if (s + 1 < s1) load_x(s + 1, 0, xa);
#pragma unroll
        for (int rg = 0; rg < R; rg++) {
            const uint8_t* row = slab + (16 * rg + r) * S::stride;
            auto emit = [&](int jj, const u32x4_t& a) {
                acc[rg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                                  __builtin_bit_cast(bf16x8_t, xb[jj]), acc[rg], 0, 0, 0);
            };
            if constexpr (kQ6) decode_q6_k<NUM, 1>(ident, row, g, emit);
            else if constexpr (QT == SNGGUF_TYPE_Q5_K) decode_q5_k<NUM, 1>(ident, row, g, emit);
            else decode_q4_k<NUM, 1>(ident, row, g, emit);
        }
    };
    if (s0 < s1) {
        load_x(s0, 0, xa);
        fetch(s0);
    }
    for (int s = s0; s < s1; s++) step(s);

    // ---- add the wavefronts' partial sums (the slabs are dead: reuse them) -------------------------
    __syncthreads();
    f32x4_t* red = reinterpret_cast<f32x4_t*>(lds);  // [waves][R][64]
#pragma unroll
    for (int rg = 0; rg < R; rg++) red[(wave * R + rg) * 64 + lane] = acc[rg];
    __syncthreads();
    if (wave != 0 || !has_x) return;
    // D[i][j]: j = lane % 16 is the activation row, register v holds weight row 4 * (lane / 16) + v
    const int m = r;
#pragma unroll
    for (int rg = 0; rg < R; rg++) {
        f32x4_t sum = red[rg * 64 + lane];
        for (int w = 1; w < W; w++) {
            const f32x4_t t = red[(w * R + rg) * 64 + lane];
            sum[0] += t[0]; sum[1] += t[1]; sum[2] += t[2]; sum[3] += t[3];
        }
        const int64_t n = n0 + 16 * rg + 4 * g;
        float o[4];
        if constexpr (GATED) {
            f32x4_t up = red[(W * R + rg) * 64 + lane];
            for (int w = 1; w < W; w++) {
                const f32x4_t t = red[((W + w) * R + rg) * 64 + lane];
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
            for (int v = 0; v < 4; v++) o[v] = sum[v] + ((bias && n + v < N) ? bf16_to_f32(bias[n + v]) : 0.f);
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
}

template <int QT, int NUM, int R>
int launch_r(const bf16_t* x, int M, const uint8_t* qa, const uint8_t* qb, int64_t N, int64_t K, const bf16_t* bias,
             bf16_t* y, bool gated, hipStream_t stream) {
    const int64_t groups = (N + 16 * R - 1) / (16 * R);
    const int nsb = (int)(K >> 8);
    // wavefronts per row group: enough that the launch fills the chip (about 12 per compute unit),
    // at least one super-block each, at most 8 per workgroup
    const int64_t per_group = gated ? 2 : 1;
    int64_t w = (256 * 12 + groups * per_group - 1) / (groups * per_group);
    if (w < 1) w = 1;
    if (w > nsb) w = nsb;
    const int64_t cap = gated ? 4 : 8;
    if (w > cap) w = cap;
    const int waves = (int)(gated ? 2 * w : w);
    const size_t slab = (size_t)waves * 16 * R * Slab<QT>::stride;
    const size_t red = (size_t)waves * R * 64 * sizeof(f32x4_t);
    const size_t lds_bytes = slab > red ? slab : red;
    const dim3 grid((unsigned)groups), block((unsigned)(64 * waves));
#define SNGGUF_LAUNCH(G, WM) gemv_kq_mfma_kernel<QT, NUM, R, G, WM><<<grid, block, lds_bytes, stream>>>(x, M, qa, qb, N, K, bias, y)
    if (gated) {
        if (waves <= 4) SNGGUF_LAUNCH(true, 4);
        else SNGGUF_LAUNCH(true, 8);
    } else {
        if (waves <= 4) SNGGUF_LAUNCH(false, 4);
        else SNGGUF_LAUNCH(false, 8);
    }
#undef SNGGUF_LAUNCH
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

template <int QT, int NUM>
int launch_qt(const bf16_t* x, int M, const uint8_t* qa, const uint8_t* qb, int64_t N, int64_t K, const bf16_t* bias,
              bf16_t* y, bool gated, hipStream_t stream) {
    // Two row groups per wavefront only when one per wavefront would already give far more
    // wavefronts than the chip holds (a vocabulary-sized projection): otherwise more, smaller
    // workgroups spread more evenly over the 256 compute units.
    if (N >= 32768) return launch_r<QT, NUM, 2>(x, M, qa, qb, N, K, bias, y, gated, stream);
    return launch_r<QT, NUM, 1>(x, M, qa, qb, N, K, bias, y, gated, stream);
}

}  // namespace

// Q4_K, Q5_K or Q6_K, 1 <= M <= 16, K % 256 == 0, 16-byte aligned x and q (checked by the caller).
int launch_gemv_kq_mfma(const void* x, int64_t M, const void* qa, const void* qb, int qtype, int64_t N, int64_t K,
                        const void* bias, void* y, int numerics, bool gated, hipStream_t stream) {
    const bf16_t* xp = static_cast<const bf16_t*>(x);
    const uint8_t* a = static_cast<const uint8_t*>(qa);
    const uint8_t* b = static_cast<const uint8_t*>(qb);
    const bf16_t* bp = static_cast<const bf16_t*>(bias);
    bf16_t* yp = static_cast<bf16_t*>(y);
#define SNGGUF_CASE(QT, NUM) \
    if (qtype == QT && numerics == NUM) return launch_qt<QT, NUM>(xp, (int)M, a, b, N, K, bp, yp, gated, stream)
    SNGGUF_CASE(SNGGUF_TYPE_Q4_K, SNGGUF_NUM_GGML_FP32);
    SNGGUF_CASE(SNGGUF_TYPE_Q4_K, SNGGUF_NUM_UPSTREAM_FP16);
    SNGGUF_CASE(SNGGUF_TYPE_Q5_K, SNGGUF_NUM_GGML_FP32);
    SNGGUF_CASE(SNGGUF_TYPE_Q5_K, SNGGUF_NUM_UPSTREAM_FP16);
    SNGGUF_CASE(SNGGUF_TYPE_Q6_K, SNGGUF_NUM_GGML_FP32);
    SNGGUF_CASE(SNGGUF_TYPE_Q6_K, SNGGUF_NUM_UPSTREAM_FP16);
#undef SNGGUF_CASE
    return SNGGUF_E_BADTYPE;
}

}  // namespace sngguf
