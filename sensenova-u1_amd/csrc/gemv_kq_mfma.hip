// Decode GEMV on the matrix cores (K % 256 == 0): the K-quants Q2_K .. Q6_K, one 256-element
// super-block per step, and the 32-element formats Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, eight blocks per
// step.  Up to 16 activation rows are one matrix operand; 17 .. 64 rows use MT = 2 .. 4 operands per
// decoded weight fragment, so the weights are still fetched and decoded once.  (Q8_0 with at most
// 16 rows has faster kernels of its own.)
//
// Same shape as the Q8_0 kernel: a workgroup owns R * 16 weight rows (for the SiLU-gated pair the
// same rows of the gate and of the up matrix, on separate wavefronts), its wavefronts split K by
// super-blocks and add their partial sums through LDS at the end.  Per wavefront and super-block
// (256 elements of each row):
//   * the packed bytes of the R * 16 rows are fetched with 16-byte loads, consecutive lanes walking
//     along a row, one super-block ahead, and dropped into the wavefront's private LDS slab.  Q4_K
//     and Q5_K super-blocks (144 / 176 bytes) are 16-byte aligned; Q6_K super-blocks (210 bytes) are only 2-byte
//     aligned and are fetched as 13 unaligned 16-byte pieces plus the 2-byte scale, which never
//     touches a byte outside the super-block and puts every field at an aligned LDS address; Q2_K
//     (84 bytes) and Q3_K (110 bytes) take their last piece from the last 16 bytes of the
//     super-block, so it overlaps the piece before it in memory but not in the slab;
//   * lane (r = lane % 16, g = lane / 16) decodes, for each 32-element sub-block j, elements
//     8 g .. 8 g + 7 of row r to bf16 (rounding chain by numerics mode) as the A operand of
//     v_mfma_f32_16x16x32_bf16; the B operand is x[m = lane % 16][256 s + 32 j + 8 g ..].  With R = 2
//     one activation fragment feeds two row groups, which halves the activation traffic per
//     packed byte at M = 16.
// Nothing dequantized is written to memory.

#include "sngguf_common.hpp"

namespace sngguf {

namespace {


// Four small unsigned integers (one per byte of v, each < 256) -> (v - zero) * D - DM as two packed
// bf16 pairs.  NUM 1: every operation rounds to fp16 (0x6400 | b is the half 1024 + b, so the
// integer is formed without a convert); NUM 0: exact fp32 products, one rounding in the subtraction
// (the - 1024 - zero rides on the accumulator input of the widening instruction).  Must be called
// by all 64 lanes; `ident` is identity_row(lane).
// FUSED (formats with a minimum and zero = 0): the product and the operation next to it as one fused multiply-add
// where that gives the same bits.  NUM 0: D * q is exact in fp32 (at most 11 + 6 + 5 significant bits), so
// fma(D, q, -DM) rounds once exactly where D * q - DM does.  NUM 1: (1024 + q) * D - 1024 * D, exact inside the
// fused operation, rounds once to fp16(q * D); -1024 * D is exact in fp16 unless it overflows, so the caller takes
// this form only where every |D| of the wavefront is below 64 (a scale product that large has not been seen in a
// file; the plain form stays for it).
template <int NUM, bool HAS_MIN, bool FUSED = false>
__device__ __forceinline__ void kq_dword_bf16(half4_t ident, uint32_t v, float zero, typename Num<NUM>::T D,
                                              typename Num<NUM>::T DM, uint32_t& p01, uint32_t& p23) {
    const half2_t h01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04010400u));
    const half2_t h23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, v, 0x04030402u));
    if constexpr (NUM == SNGGUF_NUM_UPSTREAM_FP16) {
        const half2_t D2 = {D, D};
        half2_t a, b;
        if constexpr (FUSED) {
            const _Float16 c = (_Float16)(-1024.0f) * D;
            const half2_t C2 = {c, c};
            a = __builtin_elementwise_fma(h01, D2, C2);
            b = __builtin_elementwise_fma(h23, D2, C2);
        } else {
            const _Float16 off = (_Float16)(1024.0f + zero);
            const half2_t off2 = {off, off};
            a = (h01 - off2) * D2;
            b = (h23 - off2) * D2;
        }
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
        float w[4];
        if constexpr (FUSED && HAS_MIN) {
#pragma unroll
            for (int e = 0; e < 4; e++) w[e] = __builtin_fmaf(D, qf[e], -DM);
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) w[e] = D * qf[e];
            if constexpr (HAS_MIN) {
#pragma unroll
                for (int e = 0; e < 4; e++) w[e] = w[e] - DM;
            }
        }
        p01 = pack_bf16(w[0], w[1]);
        p23 = pack_bf16(w[2], w[3]);
    }
}

// Slab<QT>: how the `ts` bytes that hold 256 elements of one row travel to the wavefront's LDS slab.
// `pieces` 16-byte loads per row; piece p comes from byte 16 p of the run, except that the last one
// comes from byte `last_src` (formats whose run is not a multiple of 16 bytes end with a piece that
// overlaps its predecessor in memory); piece p lands at byte 16 p of the row's `stride`-byte slot.
// `align` is what the format guarantees for the address of a run when the matrix is 16-byte aligned.
// Strides are chosen so that 16 rows start in 16 different groups of four LDS banks.
template <int QT> struct Slab;
template <> struct Slab<SNGGUF_TYPE_Q4_0> {  // 8 blocks of 18 bytes
    static constexpr int ts = 144, pieces = 9, last_src = 128, stride = 144, align = 16;
};
template <> struct Slab<SNGGUF_TYPE_Q4_1> {  // 8 blocks of 20 bytes
    static constexpr int ts = 160, pieces = 10, last_src = 144, stride = 176, align = 16;
};
template <> struct Slab<SNGGUF_TYPE_Q5_0> {  // 8 blocks of 22 bytes
    static constexpr int ts = 176, pieces = 11, last_src = 160, stride = 176, align = 16;
};
template <> struct Slab<SNGGUF_TYPE_Q8_0> {  // 8 blocks of 34 bytes
    static constexpr int ts = 272, pieces = 17, last_src = 256, stride = 272, align = 16;
};
template <> struct Slab<SNGGUF_TYPE_Q5_1> {  // 8 blocks of 24 bytes
    static constexpr int ts = 192, pieces = 12, last_src = 176, stride = 208, align = 16;
};
// Q2_K: bytes 0..79 (scales, quants) as five pieces, bytes 68..83 as the sixth: d, dmin land at slab bytes 92, 94
template <> struct Slab<SNGGUF_TYPE_Q2_K> {
    static constexpr int ts = 84, pieces = 6, last_src = 68, stride = 112, align = 4;
};
// Q3_K: bytes 0..95 (mask, quants) as six pieces, bytes 94..109 as the seventh: the 12 scale bytes land at slab
// bytes 98..109, d at 110
template <> struct Slab<SNGGUF_TYPE_Q3_K> {
    static constexpr int ts = 110, pieces = 7, last_src = 94, stride = 112, align = 2;
};
template <> struct Slab<SNGGUF_TYPE_Q4_K> {
    static constexpr int ts = 144, pieces = 9, last_src = 128, stride = 144, align = 16;
};
template <> struct Slab<SNGGUF_TYPE_Q5_K> {
    static constexpr int ts = 176, pieces = 11, last_src = 160, stride = 176, align = 16;
};
// Q6_K: 13 pieces (208 bytes) + the fp16 scale at byte 208, fetched on its own
template <> struct Slab<SNGGUF_TYPE_Q6_K> {
    static constexpr int ts = 210, pieces = 13, last_src = 192, stride = 240, align = 2;
};

template <int ALIGN>
__device__ __forceinline__ u32x4_t ld_piece(const uint8_t* p) {
    if constexpr (ALIGN >= 16) return *reinterpret_cast<const u32x4_t*>(p);
    else if constexpr (ALIGN >= 4) return ld_u128_a4(p);
    else return ld_u128_a2(p);
}

// Eight bytes from slab address p, which is a multiple of 4 (ALIGNED) or 2 more than one.
template <bool ALIGNED>
__device__ __forceinline__ u32x2_t lds_u64(const uint8_t* p) {
    if constexpr (ALIGNED) {
        const uint32_t* w = reinterpret_cast<const uint32_t*>(p);
        return u32x2_t{w[0], w[1]};
    } else {
        const uint32_t* w = reinterpret_cast<const uint32_t*>(p - 2);
        const uint32_t w0 = w[0], w1 = w[1], w2 = w[2];
        return u32x2_t{__builtin_amdgcn_alignbit(w1, w0, 16), __builtin_amdgcn_alignbit(w2, w1, 16)};
    }
}
template <bool ALIGNED>
__device__ __forceinline__ uint32_t lds_u32(const uint8_t* p) {
    if constexpr (ALIGNED) {
        return *reinterpret_cast<const uint32_t*>(p);
    } else {
        const uint32_t* w = reinterpret_cast<const uint32_t*>(p - 2);
        return __builtin_amdgcn_alignbit(w[1], w[0], 16);
    }
}

// Q4_0 / Q4_1 / Q5_0 / Q5_1: sub-block jj of the half is block 4 HALF + jj of the eight in the slab
// row.  TS block bytes; HAS_MIN: f16 m after d, value d q + m, else d (q - 8 or 16); FIVE: 32-bit
// fifth-bit word before the quants.  Lane group g covers elements 8 g .. 8 g + 7: bytes
// 8 (g % 2) .. of qs, low nibbles for g < 2, high nibbles otherwise; fifth bits = byte g of qh.
template <int NUM, int B, int TS, bool HAS_MIN, bool FIVE>
__device__ __forceinline__ u32x4_t legacy_block(half4_t ident, const uint8_t* row, int g) {
    typedef Num<NUM> A;
    constexpr int kHdr = HAS_MIN ? 4 : 2;
    constexpr int kQs = kHdr + (FIVE ? 4 : 0);
    constexpr float kZero = HAS_MIN ? 0.f : (FIVE ? 16.f : 8.f);
    const uint8_t* blk = row + B * TS;
    const typename A::T d = A::scale(*reinterpret_cast<const uint16_t*>(blk));
    typename A::T DM = d;
    if constexpr (HAS_MIN) DM = -A::scale(*reinterpret_cast<const uint16_t*>(blk + 2));
    const int sh = 4 * (g >> 1);
    const u32x2_t qs = lds_u64<((B * TS + kQs) & 3) == 0>(blk + kQs + 8 * (g & 1));
    uint32_t v0 = (qs[0] >> sh) & 0x0F0F0F0Fu, v1 = (qs[1] >> sh) & 0x0F0F0F0Fu;
    if constexpr (FIVE) {
        const uint32_t bits = lds_u32<((B * TS + kHdr) & 3) == 0>(blk + kHdr) >> (8 * g);
        // bits 0..3 -> bit 4 of bytes 0..3
        v0 |= (((bits & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
        v1 |= ((((bits >> 4) & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
    }
    uint32_t a0, a1, a2, a3;
    kq_dword_bf16<NUM, HAS_MIN>(ident, v0, kZero, d, DM, a0, a1);
    kq_dword_bf16<NUM, HAS_MIN>(ident, v1, kZero, d, DM, a2, a3);
    return u32x4_t{a0, a1, a2, a3};
}
template <int NUM, int HALF, int TS, bool HAS_MIN, bool FIVE, typename Emit>
__device__ __forceinline__ void decode_legacy(half4_t ident, const uint8_t* row, int g, Emit&& emit) {
    emit(0, legacy_block<NUM, 4 * HALF + 0, TS, HAS_MIN, FIVE>(ident, row, g));
    emit(1, legacy_block<NUM, 4 * HALF + 1, TS, HAS_MIN, FIVE>(ident, row, g));
    emit(2, legacy_block<NUM, 4 * HALF + 2, TS, HAS_MIN, FIVE>(ident, row, g));
    emit(3, legacy_block<NUM, 4 * HALF + 3, TS, HAS_MIN, FIVE>(ident, row, g));
}

// Q8_0: block b at byte 34 b of the slab row: f16 d, then 32 int8 quants (2 bytes off a dword for even b)
template <int NUM, int B>
__device__ __forceinline__ u32x4_t q8_0_block(const uint8_t* row, int g) {
    const uint8_t* blk = row + B * 34;
    const uint16_t d = *reinterpret_cast<const uint16_t*>(blk);
    const u32x2_t qs = lds_u64<(B & 1) == 1>(blk + 2 + 8 * g);
    uint32_t a0, a1, a2, a3;
    q8_dword_bf16<NUM>(d, qs[0], a0, a1);
    q8_dword_bf16<NUM>(d, qs[1], a2, a3);
    return u32x4_t{a0, a1, a2, a3};
}
template <int NUM, int HALF, typename Emit>
__device__ __forceinline__ void decode_q8_0(const uint8_t* row, int g, Emit&& emit) {
    emit(0, q8_0_block<NUM, 4 * HALF + 0>(row, g));
    emit(1, q8_0_block<NUM, 4 * HALF + 1>(row, g));
    emit(2, q8_0_block<NUM, 4 * HALF + 2>(row, g));
    emit(3, q8_0_block<NUM, 4 * HALF + 3>(row, g));
}

// Q2_K: element 128 h + 32 j + l is bit pair j of qs[32 h + l]; its 16-element group
// 8 h + 2 j + l / 16 has scale (low nibble) and min (high nibble) in one byte.
template <int NUM, int HALF, typename Emit>
__device__ __forceinline__ void decode_q2_k(half4_t ident, const uint8_t* row, int g, Emit&& emit) {
    typedef Num<NUM> A;
    constexpr int h = HALF;
    const u32x2_t sm = *reinterpret_cast<const u32x2_t*>(row + 8 * h);  // groups 8 h .. 8 h + 7
    const uint32_t dd = *reinterpret_cast<const uint32_t*>(row + 92);
    const typename A::T d = A::scale((uint16_t)(dd & 0xFFFF)), dmin = A::scale((uint16_t)(dd >> 16));
    const u32x2_t qs = *reinterpret_cast<const u32x2_t*>(row + 16 + 32 * h + 8 * g);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t byte = (sm[j >> 1] >> (8 * (2 * (j & 1) + (g >> 1)))) & 0xFFu;
        const typename A::T D = d * A::integer((int)(byte & 15u)), DM = dmin * A::integer((int)(byte >> 4));
        uint32_t a0, a1, a2, a3;
        kq_dword_bf16<NUM, true>(ident, (qs[0] >> (2 * j)) & 0x03030303u, 0.f, D, DM, a0, a1);
        kq_dword_bf16<NUM, true>(ident, (qs[1] >> (2 * j)) & 0x03030303u, 0.f, D, DM, a2, a3);
        emit(j, u32x4_t{a0, a1, a2, a3});
    }
}

// Q3_K: stored quant (0..7) = bit pair as in Q2_K | mask bit (4 h + j of hmask[l]) << 2, value
// stored - 4; 6-bit group scales split over the 12 scale bytes, value stored - 32.
template <int NUM, int HALF, typename Emit>
__device__ __forceinline__ void decode_q3_k(half4_t ident, const uint8_t* row, int g, Emit&& emit) {
    typedef Num<NUM> A;
    constexpr int h = HALF;
    const u32x4_t t = *reinterpret_cast<const u32x4_t*>(row + 96);  // source bytes 94..109
    const uint32_t s0 = __builtin_amdgcn_alignbit(t[1], t[0], 16);  // scale bytes 0..3
    const uint32_t s1 = __builtin_amdgcn_alignbit(t[2], t[1], 16);  // 4..7
    const uint32_t s2 = __builtin_amdgcn_alignbit(t[3], t[2], 16);  // 8..11
    const typename A::T d = A::scale((uint16_t)(t[3] >> 16));
    const u32x2_t hm = *reinterpret_cast<const u32x2_t*>(row + 8 * g);
    const u32x2_t qs = *reinterpret_cast<const u32x2_t*>(row + 32 + 32 * h + 8 * g);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        // group 8 h + tt, tt = 2 j + g / 2: low nibble in byte tt (upper nibble for h = 1), high bits in
        // byte 8 + tt % 4 at bit 2 (2 h + tt / 4)
        const int t3 = (2 * (j & 1) + (g >> 1));  // tt % 4
        const uint32_t lo = (((j < 2 ? s0 : s1) >> (8 * t3)) >> (4 * h)) & 15u;
        const uint32_t hi = (((s2 >> (8 * t3)) & 0xFFu) >> (2 * (2 * h + (j >> 1)))) & 3u;
        const typename A::T D = d * A::integer((int)(lo | (hi << 4)) - 32);
        uint32_t a[4];
#pragma unroll
        for (int w = 0; w < 2; w++) {
            const uint32_t v = ((qs[w] >> (2 * j)) & 0x03030303u) | (((hm[w] >> (4 * h + j)) & 0x01010101u) << 2);
            kq_dword_bf16<NUM, false>(ident, v, 4.f, D, D, a[2 * w], a[2 * w + 1]);
        }
        emit(j, u32x4_t{a[0], a[1], a[2], a[3]});
    }
}


// (d * scale, dmin * min) of sub-blocks 4 HALF .. 4 HALF + 3 of the lane's row (Q4_K and Q5_K).  The four lanes
// (r, g = 0..3) that decode one row all need the same four pairs: lane (r, g) extracts and scales the pair of
// sub-block 4 HALF + g only, and the four exchange their results through the cross-lane network (ds_bpermute, which
// touches no LDS memory).  Same arithmetic on the same operands as computing every pair in every lane, so the
// values are bit-identical; it takes a quarter of the decode's vector instructions away.  Must be called by all
// 64 lanes.
template <int NUM, int HALF>
__device__ __forceinline__ bool q4k_pairs(const u32x4_t& head, int g, typename Num<NUM>::T (&D)[4], typename Num<NUM>::T (&DM)[4]) {
    typedef Num<NUM> A;
    uint32_t sc, mn;
    if constexpr (HALF == 0) {
        sc = (head[1] >> (8 * g)) & 63u;
        mn = (head[2] >> (8 * g)) & 63u;
    } else {
        const uint32_t b = (head[3] >> (8 * g)) & 0xFFu;
        sc = (b & 0x0Fu) | (((head[1] >> (8 * g + 6)) & 3u) << 4);
        mn = (b >> 4) | (((head[2] >> (8 * g + 6)) & 3u) << 4);
    }
    const typename A::T mine_d = A::scale((uint16_t)(head[0] & 0xFFFF)) * A::integer((int)sc);
    const typename A::T mine_m = A::scale((uint16_t)(head[0] >> 16)) * A::integer((int)mn);
    const int self = 4 * (int)(threadIdx.x & 15);  // byte address of lane (r, 0) for ds_bpermute
    if constexpr (NUM == SNGGUF_NUM_UPSTREAM_FP16) {
        const half2_t both = {mine_d, mine_m};
        const int bits = __builtin_bit_cast(int, both);
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const half2_t got = __builtin_bit_cast(half2_t, __builtin_amdgcn_ds_bpermute(self + 64 * jj, bits));
            D[jj] = got[0];
            DM[jj] = got[1];
        }
        // every |d * scale| of the wavefront below 64 (0x5400): the fused form of kq_dword_bf16 is exact
        return __builtin_amdgcn_ballot_w64(((uint32_t)bits & 0x7FFFu) >= 0x5400u) == 0;
    } else {
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            D[jj] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(self + 64 * jj, __builtin_bit_cast(int, mine_d)));
            DM[jj] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(self + 64 * jj, __builtin_bit_cast(int, mine_m)));
        }
        return true;
    }
}

// The four A operands of half a super-block (sub-blocks 4 HALF .. 4 HALF + 3) of one row, fed to
// `emit(jj, a)` with jj = 0..3.  `row` points at the row's super-block in the slab; g = lane / 16.
template <int NUM, int HALF, bool FUSED, typename Emit>
__device__ __forceinline__ void decode_q4_k_body(half4_t ident, const uint8_t* row, int g, const typename Num<NUM>::T (&Ds)[4],
                                                 const typename Num<NUM>::T (&DMs)[4], Emit&& emit) {
#pragma unroll
    for (int cc = 0; cc < 2; cc++) {
        const int c = 2 * HALF + cc;
        const u32x2_t qs = *reinterpret_cast<const u32x2_t*>(row + 16 + 32 * c + 8 * g);
#pragma unroll
        for (int hi = 0; hi < 2; hi++) {
            const int j = 2 * c + hi;
            const typename Num<NUM>::T D = Ds[j - 4 * HALF], DM = DMs[j - 4 * HALF];
            const uint32_t v0 = (hi ? qs[0] >> 4 : qs[0]) & 0x0F0F0F0Fu, v1 = (hi ? qs[1] >> 4 : qs[1]) & 0x0F0F0F0Fu;
            uint32_t a0, a1, a2, a3;
            kq_dword_bf16<NUM, true, FUSED>(ident, v0, 0.f, D, DM, a0, a1);
            kq_dword_bf16<NUM, true, FUSED>(ident, v1, 0.f, D, DM, a2, a3);
            emit(j - 4 * HALF, u32x4_t{a0, a1, a2, a3});
        }
    }
}
template <int NUM, int HALF, typename Emit>
__device__ __forceinline__ void decode_q4_k(half4_t ident, const uint8_t* row, int g, Emit&& emit) {
    typedef Num<NUM> A;
    const u32x4_t head = *reinterpret_cast<const u32x4_t*>(row);  // d, dmin, 12 scale bytes
    typename A::T Ds[4], DMs[4];
    if (q4k_pairs<NUM, HALF>(head, g, Ds, DMs)) decode_q4_k_body<NUM, HALF, true>(ident, row, g, Ds, DMs, emit);
    else decode_q4_k_body<NUM, HALF, false>(ident, row, g, Ds, DMs, emit);
}

// Q5_K: as Q4_K, the fifth bit of element l of sub-block j is bit j of qh[l]
template <int NUM, int HALF, bool FUSED, typename Emit>
__device__ __forceinline__ void decode_q5_k_body(half4_t ident, const uint8_t* row, int g, const typename Num<NUM>::T (&Ds)[4],
                                                 const typename Num<NUM>::T (&DMs)[4], Emit&& emit) {
    const u32x2_t qh = *reinterpret_cast<const u32x2_t*>(row + 16 + 8 * g);
#pragma unroll
    for (int cc = 0; cc < 2; cc++) {
        const int c = 2 * HALF + cc;
        const u32x2_t qs = *reinterpret_cast<const u32x2_t*>(row + 48 + 32 * c + 8 * g);
#pragma unroll
        for (int hi = 0; hi < 2; hi++) {
            const int j = 2 * c + hi;
            const typename Num<NUM>::T D = Ds[j - 4 * HALF], DM = DMs[j - 4 * HALF];
            uint32_t a[4];
#pragma unroll
            for (int w = 0; w < 2; w++) {
                const uint32_t lo = (hi ? qs[w] >> 4 : qs[w]) & 0x0F0F0F0Fu;
                const uint32_t hb = ((qh[w] >> j) & 0x01010101u) << 4;
                kq_dword_bf16<NUM, true, FUSED>(ident, lo | hb, 0.f, D, DM, a[2 * w], a[2 * w + 1]);
            }
            emit(j - 4 * HALF, u32x4_t{a[0], a[1], a[2], a[3]});
        }
    }
}
template <int NUM, int HALF, typename Emit>
__device__ __forceinline__ void decode_q5_k(half4_t ident, const uint8_t* row, int g, Emit&& emit) {
    typedef Num<NUM> A;
    const u32x4_t head = *reinterpret_cast<const u32x4_t*>(row);  // d, dmin, 12 scale bytes
    typename A::T Ds[4], DMs[4];
    if (q4k_pairs<NUM, HALF>(head, g, Ds, DMs)) decode_q5_k_body<NUM, HALF, true>(ident, row, g, Ds, DMs, emit);
    else decode_q5_k_body<NUM, HALF, false>(ident, row, g, Ds, DMs, emit);
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

// One half (sub-blocks 4 HALF .. 4 HALF + 3) of a slab row -> four A operands through `emit(jj, a)`.
template <int QT, int NUM, int HALF, typename Emit>
__device__ __forceinline__ void decode_half(half4_t ident, const uint8_t* row, int g, Emit&& emit) {
    if constexpr (QT == SNGGUF_TYPE_Q4_0) decode_legacy<NUM, HALF, 18, false, false>(ident, row, g, emit);
    else if constexpr (QT == SNGGUF_TYPE_Q4_1) decode_legacy<NUM, HALF, 20, true, false>(ident, row, g, emit);
    else if constexpr (QT == SNGGUF_TYPE_Q5_0) decode_legacy<NUM, HALF, 22, false, true>(ident, row, g, emit);
    else if constexpr (QT == SNGGUF_TYPE_Q5_1) decode_legacy<NUM, HALF, 24, true, true>(ident, row, g, emit);
    else if constexpr (QT == SNGGUF_TYPE_Q8_0) decode_q8_0<NUM, HALF>(row, g, emit);
    else if constexpr (QT == SNGGUF_TYPE_Q2_K) decode_q2_k<NUM, HALF>(ident, row, g, emit);
    else if constexpr (QT == SNGGUF_TYPE_Q3_K) decode_q3_k<NUM, HALF>(ident, row, g, emit);
    else if constexpr (QT == SNGGUF_TYPE_Q4_K) decode_q4_k<NUM, HALF>(ident, row, g, emit);
    else if constexpr (QT == SNGGUF_TYPE_Q5_K) decode_q5_k<NUM, HALF>(ident, row, g, emit);
    else {
        static_assert(QT == SNGGUF_TYPE_Q6_K, "no matrix-core decoder for this quant type");
        decode_q6_k<NUM, HALF>(ident, row, g, emit);
    }
}

// XN (MT = 1 only): the B fragments come from LDS.  Each wavefront stages the K range it works on (all M rows)
// behind the slabs.  With `gamma` set, RMSNorm(x) with weight `gamma` is what gets contracted (see rmsnorm_piece):
// the workgroup adds up the sums of squares and every wavefront normalizes its own share in place.  Without it
// the rows are staged as they are, which takes the eight activation requests per step off the vector memory
// path (worth it for Q6_K, whose unaligned slab pieces already load that path most).
template <int QT, int NUM, int R, bool GATED, int WMAX, int MT, bool XN = false>
__global__ __launch_bounds__(64 * WMAX) void gemv_kq_mfma_kernel(const bf16_t* __restrict__ x, int M,
                                                                 const uint8_t* __restrict__ qa,
                                                                 const uint8_t* __restrict__ qb, int64_t N, int64_t K,
                                                                 const bf16_t* __restrict__ bias, const bf16_t* residual, bf16_t* __restrict__ y,
                                                                 const bf16_t* __restrict__ gamma, float eps, uint64_t* __restrict__ amax) {
    static_assert(!XN || MT == 1, "the fused norm is for at most 16 rows");
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
        off[i] = (uint32_t)((n - n0) * row_bytes + (fp == S::pieces - 1 ? S::last_src : 16 * fp));
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

    f32x4_t acc[R][MT];
#pragma unroll
    for (int rg = 0; rg < R; rg++)
#pragma unroll
        for (int t = 0; t < MT; t++) acc[rg][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    u32x4_t pre[kLoads];
    uint16_t pre_d = 0;
    auto fetch = [&](int s) {
        const uint8_t* p = base + (int64_t)s * S::ts;
#pragma unroll
        for (int i = 0; i < kLoads - 1; i++) pre[i] = ld_piece<S::align>(p + off[i]);
        if (tail_lane) pre[kLoads - 1] = ld_piece<S::align>(p + off[kLoads - 1]);
        if constexpr (kQ6) {
            if (lane < kRows) pre_d = ld_u16(p + doff);
        }
    };
    // Lane (r, g) supplies column r of B operand t, i.e. activation row 16 t + r.  Rows >= M are never
    // stored, so those lanes re-read the last activation row instead of being masked.
    const bf16_t* xrow[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) xrow[t] = x + (int64_t)(16 * t + r < M ? 16 * t + r : M - 1) * K + 8 * g;

    // Activations are buffered by half super-blocks (four fragments): `xa` holds the first half of
    // the current super-block on entry; the second half is requested into `xb` before the first is
    // used, and the first half of the next super-block into `xa` before the second is used, so each
    // request has half a step of decode work to cover its latency.
    // XN: this wavefront's normalized activations, [M][xrow_b bytes]; the fragment of super-block s, half, j of
    // row m sits at byte ((s - s0) * 8 + 4 * half + j) * 64 + 16 g of row m
    const int xrow_b = XN ? (int)((nsb + W - 1) / W) * 512 + 16 : 0;
    uint8_t* xw = lds + waves * kSlab + wave * (M * xrow_b);
    const uint8_t* xwrow = xw + (r < M ? r : M - 1) * xrow_b + 16 * g;
    auto load_x = [&](int s, int half, u32x4_t (&dstx)[MT][4]) {
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if constexpr (XN) dstx[t][j] = *reinterpret_cast<const u32x4_t*>(xwrow + ((s - s0) * 8 + 4 * half + j) * 64);
                else dstx[t][j] = *reinterpret_cast<const u32x4_t*>(xrow[t] + ((int64_t)s * 8 + 4 * half + j) * 32);
            }
    };
    u32x4_t xa[MT][4], xb[MT][4];
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
#pragma unroll
                for (int t = 0; t < MT; t++)
                    acc[rg][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, xa[t][jj]), acc[rg][t], 0, 0, 0);
            };
            decode_half<QT, NUM, 0>(ident, row, g, emit);
        }
        if (s + 1 < s1) load_x(s + 1, 0, xa);
#pragma unroll
        for (int rg = 0; rg < R; rg++) {
            const uint8_t* row = slab + (16 * rg + r) * S::stride;
            auto emit = [&](int jj, const u32x4_t& a) {
#pragma unroll
                for (int t = 0; t < MT; t++)
                    acc[rg][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, xb[t][jj]), acc[rg][t], 0, 0, 0);
            };
            decode_half<QT, NUM, 1>(ident, row, g, emit);
        }
    };
    if constexpr (XN) {
        // the first slab is requested, then the activations are staged and normalized underneath it
        if (s0 < s1) fetch(s0);
        float* ssum = reinterpret_cast<float*>(lds + waves * kSlab + waves * (M * xrow_b));  // [M][waves]
        const int pieces = (s1 - s0) * 32;               // 16-byte pieces per row in this wavefront's K range
        const int64_t k0 = (int64_t)s0 * 256;
        if (!gamma) {
            // plain staging, four requests in flight per lane; a wavefront reads back only what it wrote itself
            for (int m = 0; m < M; m++)
                for (int c0 = lane; c0 < pieces; c0 += 256) {
                    u32x4_t v[4];
#pragma unroll
                    for (int u = 0; u < 4; u++)
                        if (c0 + 64 * u < pieces) v[u] = *reinterpret_cast<const u32x4_t*>(x + (int64_t)m * K + k0 + 8 * (c0 + 64 * u));
#pragma unroll
                    for (int u = 0; u < 4; u++)
                        if (c0 + 64 * u < pieces) *reinterpret_cast<u32x4_t*>(xw + m * xrow_b + 16 * (c0 + 64 * u)) = v[u];
                }
        }
        for (int m = 0; gamma && m < M; m++) {
            float ss = 0.f;
            for (int c = lane; c < pieces; c += 64) {
                const u32x4_t v = *reinterpret_cast<const u32x4_t*>(x + (int64_t)m * K + k0 + 8 * c);
                *reinterpret_cast<u32x4_t*>(xw + m * xrow_b + 16 * c) = v;
                ss += sumsq_piece(v);
            }
            ss = wave_sum(ss);
            if (lane == 0) ssum[m * waves + wave] = ss;
        }
        if (gamma) __syncthreads();   // (uniform over the workgroup)
        for (int m = 0; gamma && m < M; m++) {
            float tot = 0.f;
            for (int w = 0; w < W; w++) tot += ssum[m * waves + w];   // wavefronts [0, W) cover K once
            const float rstd = rms_rstd(tot, K, eps);
            for (int c = lane; c < pieces; c += 64) {
                u32x4_t* cell = reinterpret_cast<u32x4_t*>(xw + m * xrow_b + 16 * c);
                const u32x4_t gv = *reinterpret_cast<const u32x4_t*>(gamma + k0 + 8 * c);
                *cell = rmsnorm_piece(*cell, gv, rstd);
            }
        }
        if (s0 < s1) load_x(s0, 0, xa);
    } else if (s0 < s1) {
        load_x(s0, 0, xa);
        fetch(s0);
    }
    for (int s = s0; s < s1; s++) step(s);

    // ---- add the wavefronts' partial sums (the slabs are dead: reuse them) -------------------------
    __syncthreads();
    f32x4_t* red = reinterpret_cast<f32x4_t*>(lds);  // [waves][R][MT][64]
#pragma unroll
    for (int rg = 0; rg < R; rg++)
#pragma unroll
        for (int t = 0; t < MT; t++) red[((wave * R + rg) * MT + t) * 64 + lane] = acc[rg][t];
    __syncthreads();
    if (wave != 0) return;
    // D[i][j]: j = lane % 16 is the activation row (of operand t), register v holds weight row 4 * (lane / 16) + v
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const int m = 16 * t + r;
        if (m >= M) continue;
        uint64_t best = 0;   // arg-max form: best (value, column) of this workgroup's rows for activation row m
#pragma unroll
        for (int rg = 0; rg < R; rg++) {
            f32x4_t sum = red[(rg * MT + t) * 64 + lane];
            for (int w = 1; w < W; w++) {
                const f32x4_t p = red[((w * R + rg) * MT + t) * 64 + lane];
                sum[0] += p[0]; sum[1] += p[1]; sum[2] += p[2]; sum[3] += p[3];
            }
            const int64_t n = n0 + 16 * rg + 4 * g;
            float o[4];
            if constexpr (GATED) {
                f32x4_t up = red[((W * R + rg) * MT + t) * 64 + lane];
                for (int w = 1; w < W; w++) {
                    const f32x4_t p = red[(((W + w) * R + rg) * MT + t) * 64 + lane];
                    up[0] += p[0]; up[1] += p[1]; up[2] += p[2]; up[3] += p[3];
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
#pragma unroll
                    for (int v = 0; v < 4; v++)
                        if (n + v < N) best = u64_max(best, argmax_key(o[v], n + v));
                    continue;
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
        if constexpr (!GATED) {
            if (amax) argmax_store(best, g, amax, m, blockIdx.x, gridDim.x);
        }
    }
}

template <int QT, int NUM, int R>
int launch_r(const bf16_t* x, int M, const uint8_t* qa, const uint8_t* qb, int64_t N, int64_t K, const bf16_t* bias,
             const bf16_t* residual, bf16_t* y, bool gated, const bf16_t* gamma, float eps, hipStream_t stream, uint64_t* amax) {
    const int64_t groups = (N + 16 * R - 1) / (16 * R);
    const int nsb = (int)(K >> 8);
    const int mt = (M + 15) / 16;
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
    const size_t red = (size_t)waves * R * mt * 64 * sizeof(f32x4_t);
    const dim3 grid((unsigned)groups), block((unsigned)(64 * waves));
    // Q6_K streams its activations from LDS too when one or two rows of them fit there and the matrix is large
    // (12288 x 4096 at M = 1: 13.6 against 15.3 us; the other formats and small matrices lose by it)
    const bool stage = QT == SNGGUF_TYPE_Q6_K && !gamma && M <= 2 && N * K >= ((int64_t)32 << 20) &&
                       (size_t)M * (2 * (size_t)K + 64) <= 36 * 1024;
    if (gamma || stage) {
        // slabs, then every wavefront's share of the activations ([M][xrow_b]), then [M][waves] sums of squares; the
        // caller keeps M (2 K + 64) within 36 KB
        if (mt > 1) return SNGGUF_E_BADSHAPE;
        const size_t xrow_b = (size_t)((nsb + w - 1) / w) * 512 + 16;
        const size_t staged = slab + (size_t)waves * M * xrow_b + (((size_t)4 * M * waves + 15) & ~(size_t)15);
        const size_t lds_norm = staged > red ? staged : red;
        if (lds_norm > 160 * 1024) return SNGGUF_E_BADSHAPE;
        // slabs of two row groups per wavefront plus the staged activations can pass the default dynamic-LDS limit:
        // raise it once per kernel instance
#define SNGGUF_LAUNCH_XN(G, WM)                                                                                        \
    do {                                                                                                               \
        static const hipError_t attr = hipFuncSetAttribute(                                                            \
            reinterpret_cast<const void*>(&gemv_kq_mfma_kernel<QT, NUM, R, G, WM, 1, true>),                            \
            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);                                                    \
        if (attr != hipSuccess) return SNGGUF_E_LAUNCH;                                                                 \
        gemv_kq_mfma_kernel<QT, NUM, R, G, WM, 1, true><<<grid, block, lds_norm, stream>>>(x, M, qa, qb, N, K, bias,    \
                                                                                           residual, y, gamma, eps, amax); \
    } while (0)
        if (gated) {
            if (waves <= 4) SNGGUF_LAUNCH_XN(true, 4);
            else SNGGUF_LAUNCH_XN(true, 8);
        } else {
            if (waves <= 4) SNGGUF_LAUNCH_XN(false, 4);
            else SNGGUF_LAUNCH_XN(false, 8);
        }
#undef SNGGUF_LAUNCH_XN
        return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
    }
    const size_t lds_bytes = slab > red ? slab : red;
#define SNGGUF_LAUNCH(G, WM, MT_) \
    gemv_kq_mfma_kernel<QT, NUM, R, G, WM, MT_><<<grid, block, lds_bytes, stream>>>(x, M, qa, qb, N, K, bias, residual, y, nullptr, 0.f, amax)
    if (mt > 1) {
        // more than 16 activation rows: plain projections with one row group per wavefront only
        if constexpr (R == 1) {
            if (gated || mt > 4) return SNGGUF_E_BADSHAPE;
            if (mt == 2) SNGGUF_LAUNCH(false, 8, 2);
            else if (mt == 3) SNGGUF_LAUNCH(false, 8, 3);
            else SNGGUF_LAUNCH(false, 8, 4);
        } else {
            return SNGGUF_E_BADSHAPE;
        }
    } else if (gated) {
        if (waves <= 4) SNGGUF_LAUNCH(true, 4, 1);
        else SNGGUF_LAUNCH(true, 8, 1);
    } else {
        if (waves <= 4) SNGGUF_LAUNCH(false, 4, 1);
        else SNGGUF_LAUNCH(false, 8, 1);
    }
#undef SNGGUF_LAUNCH
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

// Row groups per wavefront (see launch_qt) as a function, so that the arg-max caller can size its slot array.
inline int rows_per_workgroup(int64_t M, int64_t N) { return (N >= 32768 && M <= 16) ? 32 : 16; }

template <int QT, int NUM>
int launch_qt(const bf16_t* x, int M, const uint8_t* qa, const uint8_t* qb, int64_t N, int64_t K, const bf16_t* bias,
              const bf16_t* residual, bf16_t* y, bool gated, const bf16_t* gamma, float eps, hipStream_t stream, uint64_t* amax) {
    // Two row groups per wavefront only when one per wavefront would already give far more
    // wavefronts than the chip holds (a vocabulary-sized projection): otherwise more, smaller
    // workgroups spread more evenly over the 256 compute units.
    if (rows_per_workgroup(M, N) == 32) return launch_r<QT, NUM, 2>(x, M, qa, qb, N, K, bias, residual, y, gated, gamma, eps, stream, amax);
    return launch_r<QT, NUM, 1>(x, M, qa, qb, N, K, bias, residual, y, gated, gamma, eps, stream, amax);
}

// ---- the SiLU-gated MLP of a decoder layer at decode sizes in ONE launch, K-quant weights ---------------------
// The organisation of mlp_q8_decode_kernel (gemv_q8_mfma.hip) with this file's decoders: 256 workgroups of twelve
// wavefronts, one per compute unit.  Phase A: workgroup b computes the gated activations of rows [48 b, +48) - three
// 16-row groups, each with four wavefronts as in the gated pair's own launch (gate / up x two K halves of eight
// super-blocks), the activations staged once per workgroup in LDS (normalized there if `gamma` is given) - and writes
// them as 8-byte words { two bf16, generation tag } with agent-scope stores, then the group's flag.  No barrier inside
// the phase: a wavefront leaves its partial sums in LDS and counts itself in for its row group; the group's storing
// wavefront waits for that count only.  Phase B: 16 rows of the down matrix, K = inter split over the twelve
// wavefronts, four super-blocks each; two of them are requested the moment the wavefront leaves phase A's loop, the
// other two when every wavefront of the workgroup has left it (a count in LDS; requested earlier, their traffic slows
// phase A's last wavefronts, which the whole device waits for), and all four wait as raw bytes in registers; the first is decoded into matrix-core operands
// while the activations are on their way.  Then the wavefront polls the flags of the 64 row groups its K range needs,
// reads the tagged words (every tag checked), contracts the decoded super-block, decodes and contracts the other three,
// and the twelve partial sums are added.  Bounded wait, status word, generation counter and workspace layout as in the
// Q8_0 kernel (MlpCtl).  Without `gamma` the gated activations are bit-identical to the gated pair's own launch (same
// fragments, same order of accumulation), and so is the output (the down projection's own launch splits K over eight
// wavefronts, not twelve: equal up to the order of twelve fp32 additions, which the tests allow for).
// The decode arithmetic, not memory, bounds these formats: the launch is 0 - 5 % ahead of the two separate ones by device
// and down type (32.3 against 33.9 us with a Q6_K down projection once the down projection's first requests are made
// behind phase A's epilogue instead of in front of it; 31.9 - 32.8 against 32.7 - 33.0 with Q4_K), where the Q8_0 kernel
// gains 10 %.
template <int QT>
struct SlabIo {
    typedef Slab<QT> S;
    static constexpr int kPieces = 16 * S::pieces;
    static constexpr int kLoads = (kPieces + 63) / 64;
    static constexpr int kSlab = 16 * S::stride;
    static constexpr bool kQ6 = QT == SNGGUF_TYPE_Q6_K;
    uint32_t off[kLoads], dst[kLoads];
    uint32_t doff;
    bool tail_lane;
    __device__ __forceinline__ void init(int lane, int64_t row_bytes) {
#pragma unroll
        for (int i = 0; i < kLoads; i++) {
            const int f = lane + 64 * i;
            const bool ok = f < kPieces;
            const int fr = ok ? f / S::pieces : 0, fp = ok ? f % S::pieces : 0;
            off[i] = (uint32_t)(fr * row_bytes + (fp == S::pieces - 1 ? S::last_src : 16 * fp));
            dst[i] = (uint32_t)(fr * S::stride + 16 * fp);
        }
        tail_lane = lane + 64 * (kLoads - 1) < kPieces;
        doff = (uint32_t)((lane < 16 ? lane : 0) * row_bytes + 208);
    }
    __device__ __forceinline__ void fetch(const uint8_t* __restrict__ base, int s, int lane, u32x4_t (&pre)[kLoads], uint16_t& pre_d) const {
        const uint8_t* p = base + (int64_t)s * S::ts;
#pragma unroll
        for (int i = 0; i < kLoads - 1; i++) pre[i] = ld_piece<S::align>(p + off[i]);
        if (tail_lane) pre[kLoads - 1] = ld_piece<S::align>(p + off[kLoads - 1]);
        if constexpr (kQ6) {
            if (lane < 16) pre_d = ld_u16(p + doff);
        }
    }
    __device__ __forceinline__ void store(uint8_t* slab, int lane, const u32x4_t (&pre)[kLoads], uint16_t pre_d) const {
#pragma unroll
        for (int i = 0; i < kLoads - 1; i++) *reinterpret_cast<u32x4_t*>(slab + dst[i]) = pre[i];
        if (tail_lane) *reinterpret_cast<u32x4_t*>(slab + dst[kLoads - 1]) = pre[kLoads - 1];
        if constexpr (kQ6) {
            if (lane < 16) *reinterpret_cast<uint16_t*>(slab + lane * S::stride + 208) = pre_d;
        }
    }
};

constexpr int kMlpKqWaves = 12;
// Super-blocks of the down matrix that a wavefront decodes into registers while it waits for the activations: one (32
// registers of operands beside a decoder's ~100 of temporaries is what 168 registers per lane hold; two spill).
#ifndef SNGGUF_MLPKQ_AHEAD
#define SNGGUF_MLPKQ_AHEAD 1
#endif
constexpr int kMlpKqSteps = 4;   // super-blocks of the down matrix per wavefront: inter = 12 x 4 x 256 (the launcher checks)

template <int QA, int QB>
struct MlpKqLds {
    // [12 slabs of phase A][x staged (M rows) + sums of squares][partial sums of phase A + counters][12 x (slab of phase B, two staged activation rows)]
    static constexpr int kSlabsA = kMlpKqWaves * SlabIo<QA>::kSlab;
    static constexpr int kWaveB = SlabIo<QB>::kSlab + 2 * kMlpKqSteps * 512;
    __host__ __device__ static size_t xs_bytes(int M, int64_t hidden, bool norm) {
        return (((size_t)M * (2 * (size_t)hidden + 64) + (norm ? (size_t)4 * M * kMlpKqWaves : 0)) + 255) & ~(size_t)255;
    }
    __host__ __device__ static size_t total(int M, int64_t hidden, bool norm) {
        return (size_t)kSlabsA + xs_bytes(M, hidden, norm) + (size_t)kMlpKqWaves * 64 * 16 + 64 + (size_t)kMlpKqWaves * kWaveB;
    }
};

template <int QA, int QB, int NUM>
__global__ __launch_bounds__(64 * kMlpKqWaves) void mlp_kq_decode_kernel(const bf16_t* __restrict__ x, int M, const uint8_t* __restrict__ q_gate,
                                                                         const uint8_t* __restrict__ q_up, const uint8_t* __restrict__ q_down,
                                                                         int64_t hidden, int64_t inter, const bf16_t* __restrict__ gamma, float eps,
                                                                         const bf16_t* residual, bf16_t* __restrict__ y, MlpCtl* ctl, uint64_t* ht,
                                                                         int spin_limit) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    typedef SlabIo<QA> IA;
    typedef SlabIo<QB> IB;
    typedef MlpKqLds<QA, QB> L;
    constexpr int kWaves = kMlpKqWaves, kSteps = kMlpKqSteps;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bid = (int)blockIdx.x, nb = (int)gridDim.x;
    const int r = lane & 15, g = lane >> 4;
    const half4_t ident = identity_row(lane);
    // this launch's tag: nobody advances the generation before every workgroup, this one included, has finished
    const uint32_t tag = __hip_atomic_load(&ctl->gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;

    uint8_t* const xs = lds + L::kSlabsA;
    const int64_t xs_stride = 2 * hidden + 64;
    f32x4_t* const red_a = reinterpret_cast<f32x4_t*>(xs + L::xs_bytes(M, hidden, gamma != nullptr));
    uint32_t* const cnt = reinterpret_cast<uint32_t*>(red_a + kWaves * 64);
    uint8_t* const slab_b = reinterpret_cast<uint8_t*>(cnt + 16) + wave * L::kWaveB;
    uint8_t* const xw = slab_b + IB::kSlab;   // [2][kSteps * 512] bytes

    // ---- phase A: row group 3 bid + grp, matrix mat (0 gate, 1 up), K half kh ----
    __builtin_amdgcn_s_setprio(2);
    const int grp = wave >> 2, lw = wave & 3, mat = lw >> 1, kh = lw & 1;
    const int nsb = (int)(hidden >> 8);
    const int sa0 = kh * (nsb >> 1), sa1 = sa0 + (nsb >> 1);
    const int64_t arow_bytes = (int64_t)nsb * IA::S::ts;
    const uint8_t* __restrict__ abase = (mat ? q_up : q_gate) + (int64_t)(3 * bid + grp) * 16 * arow_bytes;
    IA ia;
    ia.init(lane, arow_bytes);
    uint8_t* const slab_a = lds + wave * IA::kSlab;
    u32x4_t pre_a[IA::kLoads];
    uint16_t pre_ad = 0;
    ia.fetch(abase, sa0, lane, pre_a, pre_ad);
    if (tid < 16) cnt[tid] = 0;
    // the activations, staged once for the workgroup (normalized in place if gamma is given)
    {
        const int pieces_per_row = (int)(hidden >> 3);
        if (gamma == nullptr) {
            for (int f = tid; f < M * pieces_per_row; f += 64 * kWaves) {
                const int m = f / pieces_per_row, c = f - m * pieces_per_row;
                *reinterpret_cast<u32x4_t*>(xs + m * xs_stride + 16 * c) = *reinterpret_cast<const u32x4_t*>(x + (int64_t)m * hidden + 8 * c);
            }
        } else {
            float* ssum = reinterpret_cast<float*>(xs + M * xs_stride);   // [M][waves]
            for (int m = 0; m < M; m++) {
                float ss = 0.f;
                for (int c = tid; c < pieces_per_row; c += 64 * kWaves) {
                    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(x + (int64_t)m * hidden + 8 * c);
                    *reinterpret_cast<u32x4_t*>(xs + m * xs_stride + 16 * c) = v;
                    ss += sumsq_piece(v);
                }
                ss = wave_sum(ss);
                if (lane == 0) ssum[m * kWaves + wave] = ss;
            }
            __syncthreads();
            for (int m = 0; m < M; m++) {
                float tot = 0.f;
                for (int w = 0; w < kWaves; w++) tot += ssum[m * kWaves + w];
                const float rstd = rms_rstd(tot, hidden, eps);
                for (int c = tid; c < pieces_per_row; c += 64 * kWaves) {
                    u32x4_t* cell = reinterpret_cast<u32x4_t*>(xs + m * xs_stride + 16 * c);
                    *cell = rmsnorm_piece(*cell, *reinterpret_cast<const u32x4_t*>(gamma + 8 * c), rstd);
                }
            }
        }
        __syncthreads();
    }
    const bool has_x = r < M;
    const uint8_t* xsrow = xs + (has_x ? r : M - 1) * xs_stride + 16 * g;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int s = sa0; s < sa1; s++) {
        ia.store(slab_a, lane, pre_a, pre_ad);
        if (s + 1 < sa1) ia.fetch(abase, s + 1, lane, pre_a, pre_ad);
        const uint8_t* row = slab_a + r * IA::S::stride;
        auto emit0 = [&](int jj, const u32x4_t& a) {
            const u32x4_t xf = *reinterpret_cast<const u32x4_t*>(xsrow + (s * 8 + jj) * 64);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, xf), acc, 0, 0, 0);
        };
        decode_half<QA, NUM, 0>(ident, row, g, emit0);
        auto emit1 = [&](int jj, const u32x4_t& a) {
            const u32x4_t xf = *reinterpret_cast<const u32x4_t*>(xsrow + (s * 8 + 4 + jj) * 64);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, xf), acc, 0, 0, 0);
        };
        decode_half<QA, NUM, 1>(ident, row, g, emit1);
    }

    // ---- phase B geometry: rows [16 bid, +16) of down, super-blocks [4 wave, +4) ----
    const int sb0 = wave * kSteps;
    const int64_t brow_bytes = (inter >> 8) * IB::S::ts;
    const uint8_t* __restrict__ bbase = q_down + (int64_t)bid * 16 * brow_bytes;
    IB ib;
    ib.init(lane, brow_bytes);
    u32x4_t raw[kSteps][IB::kLoads];
    uint16_t raw_d[kSteps] = {};
    // ---- phase A epilogue: partial sums, per-group count, the storing wavefront's SiLU and tagged stores; the down
    // projection's first requests come behind it, so that they do not queue in front of what other workgroups wait for ----
    red_a[wave * 64 + lane] = acc;
    if (lane == 0) __hip_atomic_fetch_add(cnt + grp, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (lw == 0) {
        while (__hip_atomic_load(cnt + grp, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < 4u) __builtin_amdgcn_s_sleep(1);
        if (has_x) {
            // wavefronts 4 grp + {0, 1}: gate K halves, + {2, 3}: up K halves; D[i][j]: j = lane % 16 the activation row
            f32x4_t gs = red_a[(4 * grp) * 64 + lane], us = red_a[(4 * grp + 2) * 64 + lane];
            const f32x4_t g1 = red_a[(4 * grp + 1) * 64 + lane], u1 = red_a[(4 * grp + 3) * 64 + lane];
            float o[4];
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float gt = bf16_to_f32(f32_to_bf16(gs[v] + g1[v]));
                const float ut = bf16_to_f32(f32_to_bf16(us[v] + u1[v]));
                const float sl = bf16_to_f32(f32_to_bf16(gt / (1.0f + expf(-gt))));
                o[v] = sl * ut;
            }
            const int64_t n = (int64_t)(3 * bid + grp) * 16 + 4 * g;
            uint64_t* yt = ht + (((int64_t)r * inter + n) >> 1);
            __hip_atomic_store(yt, (uint64_t)pack_bf16(o[0], o[1]) | ((uint64_t)tag << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(yt + 1, (uint64_t)pack_bf16(o[2], o[3]) | ((uint64_t)tag << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (lane == 0) __hip_atomic_store(&ctl->flags[3 * bid + grp], tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    ib.fetch(bbase, sb0, lane, raw[0], raw_d[0]);
    ib.fetch(bbase, sb0 + 1, lane, raw[1], raw_d[1]);
    // counted as having left the loop: the other two steps are requested when that count is full
    uint32_t* const left_a = cnt + 8;
    if (lane == 0) __hip_atomic_fetch_add(left_a, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);

    __builtin_amdgcn_s_setprio(0);

    // ---- phase B: decode the first kAhead super-blocks into matrix-core operands while the activations are on their
    // way (what the register file holds beside a decoder's temporaries); the others wait as raw bytes in registers ----
    constexpr int kAhead = SNGGUF_MLPKQ_AHEAD;
    u32x4_t afrag[kAhead > 0 ? kAhead * 8 : 1];
    const uint8_t* const brow = slab_b + r * IB::S::stride;
    auto decode = [&](int i) {
        ib.store(slab_b, lane, raw[i], raw_d[i]);
        auto e0 = [&](int jj, const u32x4_t& a) { afrag[i * 8 + jj] = a; };
        decode_half<QB, NUM, 0>(ident, brow, g, e0);
        auto e1 = [&](int jj, const u32x4_t& a) { afrag[i * 8 + 4 + jj] = a; };
        decode_half<QB, NUM, 1>(ident, brow, g, e1);
    };
    if constexpr (kAhead > 0) decode(0);
    if constexpr (kAhead > 1) decode(1);
    // every wavefront of the workgroup has left phase A's loop: now the other two steps' traffic
    while (__hip_atomic_load(left_a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < (uint32_t)kWaves) __builtin_amdgcn_s_sleep(1);
    ib.fetch(bbase, sb0 + 2, lane, raw[2], raw_d[2]);
    ib.fetch(bbase, sb0 + 3, lane, raw[3], raw_d[3]);
    if constexpr (kAhead > 2) decode(2);
    if constexpr (kAhead > 3) decode(3);

    // ---- wait for this wavefront's K range of the activations: flags of its 64 row groups, then the tagged words ----
    constexpr int xrow_b = kSteps * 512;
    {
        const int pairs = kSteps * 64;                    // 16-byte pairs of words per row in this wavefront's K range
        const int64_t w0 = (int64_t)sb0 * 128;            // first word of the range within a row
        const int64_t row_words = inter >> 1;
        const int g0 = sb0 * 16, ng = kSteps * 16;        // row groups of 16 outputs
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
                    *reinterpret_cast<uint64_t*>(xw + m * xrow_b + 8 * c) = (uint64_t)(uint32_t)a | (b << 32);
                }
            if (gave_up || __builtin_amdgcn_ballot_w64(!all) == 0) break;
            if (++polls > spin_limit) { gave_up = true; break; }
        }
        if (gave_up && lane == 0) __hip_atomic_store(&ctl->status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- contract, add the twelve partial sums, residual, store ----
    __builtin_amdgcn_s_setprio(3);
    f32x4_t yacc = {0.f, 0.f, 0.f, 0.f};
    const uint8_t* xwrow = xw + (has_x ? r : M - 1) * xrow_b + 16 * g;
#pragma unroll
    for (int i = 0; i < kAhead * 8; i++) {
        const u32x4_t xf = *reinterpret_cast<const u32x4_t*>(xwrow + i * 64);
        yacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, afrag[i]), __builtin_bit_cast(bf16x8_t, xf), yacc, 0, 0, 0);
    }
    auto decode_contract = [&](int i) {
        ib.store(slab_b, lane, raw[i], raw_d[i]);
        auto e0 = [&](int jj, const u32x4_t& a) {
            const u32x4_t xf = *reinterpret_cast<const u32x4_t*>(xwrow + (i * 8 + jj) * 64);
            yacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, xf), yacc, 0, 0, 0);
        };
        decode_half<QB, NUM, 0>(ident, brow, g, e0);
        auto e1 = [&](int jj, const u32x4_t& a) {
            const u32x4_t xf = *reinterpret_cast<const u32x4_t*>(xwrow + (i * 8 + 4 + jj) * 64);
            yacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, xf), yacc, 0, 0, 0);
        };
        decode_half<QB, NUM, 1>(ident, brow, g, e1);
    };
    if constexpr (kAhead <= 0) decode_contract(0);
    if constexpr (kAhead <= 1) decode_contract(1);
    if constexpr (kAhead <= 2) decode_contract(2);
    if constexpr (kAhead <= 3) decode_contract(3);
    __syncthreads();   // every wavefront is past phase A's epilogue: its partial-sum area is free
    red_a[wave * 64 + lane] = yacc;
    __syncthreads();
    if (wave == 0 && has_x) {
        f32x4_t sum = red_a[lane];
        for (int w = 1; w < kWaves; w++) {
            const f32x4_t t = red_a[w * 64 + lane];
            sum[0] += t[0]; sum[1] += t[1]; sum[2] += t[2]; sum[3] += t[3];
        }
        const int64_t n = (int64_t)bid * 16 + 4 * g;
        float o[4];
#pragma unroll
        for (int v = 0; v < 4; v++) o[v] = add_residual(sum[v], residual, (int64_t)r * hidden + n + v);
        *reinterpret_cast<u32x2_t*>(y + (int64_t)r * hidden + n) = u32x2_t{pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3])};
    }
    if (tid == 0) {
        const uint32_t old = __hip_atomic_fetch_add(&ctl->done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old == (uint32_t)nb - 1u) {
            __hip_atomic_store(&ctl->done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&ctl->gen, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

template <int QA, int QB, int NUM>
int launch_mlp_kq(const void* x, int M, const void* gamma, float eps, const void* q_gate, const void* q_up, const void* q_down, int64_t hidden,
                  int64_t inter, const void* residual, void* y, void* workspace, int spin_limit, hipStream_t stream) {
    const size_t lds_bytes = MlpKqLds<QA, QB>::total(M, hidden, gamma != nullptr);
    if (lds_bytes > 160 * 1024) return SNGGUF_E_BADSHAPE;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&mlp_kq_decode_kernel<QA, QB, NUM>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess) return SNGGUF_E_LAUNCH;
    MlpCtl* ctl = static_cast<MlpCtl*>(workspace);
    uint64_t* h = reinterpret_cast<uint64_t*>(static_cast<uint8_t*>(workspace) + kMlpCtlBytes);
    const int limit = spin_limit == 0 ? 1 << 20 : spin_limit < 0 ? 0 : spin_limit;
    mlp_kq_decode_kernel<QA, QB, NUM><<<dim3((unsigned)(inter / 48)), dim3(64 * kMlpKqWaves), lds_bytes, stream>>>(
        static_cast<const bf16_t*>(x), M, static_cast<const uint8_t*>(q_gate), static_cast<const uint8_t*>(q_up),
        static_cast<const uint8_t*>(q_down), hidden, inter, static_cast<const bf16_t*>(gamma), eps, static_cast<const bf16_t*>(residual),
        static_cast<bf16_t*>(y), ctl, h, limit);
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

}  // namespace

// The K-quant mixes the one-launch MLP takes: Q4_K gate / up with a Q6_K or Q4_K down projection (the "Q4_K_M" recipe),
// hidden 4096, inter 12288 (48 rows of gate / up and 16 rows of down per workgroup, 12 x 4 super-blocks per down row),
// one or two rows, one resident workgroup per compute unit.
bool mlp_kq_decode_fits(int qtype_gate_up, int qtype_down, int64_t M, int64_t hidden, int64_t inter) {
    if (qtype_gate_up != SNGGUF_TYPE_Q4_K || (qtype_down != SNGGUF_TYPE_Q6_K && qtype_down != SNGGUF_TYPE_Q4_K)) return false;
    if (M < 1 || M > 2 || hidden != 4096 || inter != 12 * kMlpKqSteps * 256) return false;
    static const int cus = [] {
        int dev = 0, n = 0, per_cu = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        const void* k = reinterpret_cast<const void*>(&mlp_kq_decode_kernel<SNGGUF_TYPE_Q4_K, SNGGUF_TYPE_Q6_K, 1>);
        if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) return 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, mlp_kq_decode_kernel<SNGGUF_TYPE_Q4_K, SNGGUF_TYPE_Q6_K, 1>, 64 * kMlpKqWaves,
                                                         160 * 1024) != hipSuccess)
            return 0;
        return per_cu >= 1 ? n : 0;
    }();
    return cus >= inter / 48;
}

int launch_mlp_kq_decode(const void* x, int64_t M, const void* gamma, float eps, const void* q_gate, const void* q_up, const void* q_down,
                         int qtype_down, int64_t hidden, int64_t inter, const void* residual, void* y, void* workspace, int numerics,
                         int spin_limit, hipStream_t stream) {
    if (!mlp_kq_decode_fits(SNGGUF_TYPE_Q4_K, qtype_down, M, hidden, inter)) return SNGGUF_E_BADSHAPE;
#define SNGGUF_GO(QB, NUMV) \
    return launch_mlp_kq<SNGGUF_TYPE_Q4_K, QB, NUMV>(x, (int)M, gamma, eps, q_gate, q_up, q_down, hidden, inter, residual, y, workspace, spin_limit, stream)
    if (qtype_down == SNGGUF_TYPE_Q6_K) {
        if (numerics == SNGGUF_NUM_GGML_FP32) SNGGUF_GO(SNGGUF_TYPE_Q6_K, 0);
        SNGGUF_GO(SNGGUF_TYPE_Q6_K, 1);
    }
    if (numerics == SNGGUF_NUM_GGML_FP32) SNGGUF_GO(SNGGUF_TYPE_Q4_K, 0);
    SNGGUF_GO(SNGGUF_TYPE_Q4_K, 1);
#undef SNGGUF_GO
}

// Workgroups of a plain decode launch = (value, column) slots per activation row that its arg-max form writes.
int64_t gemv_argmax_slots(int qtype, int64_t M, int64_t N) {
    const int64_t rows = qtype == SNGGUF_TYPE_Q8_0 ? 16 : rows_per_workgroup(M, N);   // (Q8_0 has kernels of its own)
    return (N + rows - 1) / rows;
}

// 1 <= M <= 64 (SiLU-gated pair: M <= 16), K % 256 == 0, 16-byte aligned x and q (checked by the caller).  `gamma`
// (K bf16, 16-byte aligned) switches the fused RMSNorm on; the caller keeps M (2 K + 64) <= 36 KB then.
int launch_gemv_kq_mfma(const void* x, int64_t M, const void* qa, const void* qb, int qtype, int64_t N, int64_t K,
                        const void* bias, const void* residual, void* y, int numerics, bool gated, hipStream_t stream,
                        const void* gamma, float eps, uint64_t* amax) {
    if (amax && (gated || M > 16)) return SNGGUF_E_BADSHAPE;
    const bf16_t* gp = static_cast<const bf16_t*>(gamma);
    const bf16_t* xp = static_cast<const bf16_t*>(x);
    const uint8_t* a = static_cast<const uint8_t*>(qa);
    const uint8_t* b = static_cast<const uint8_t*>(qb);
    const bf16_t* bp = static_cast<const bf16_t*>(bias);
    const bf16_t* rp = static_cast<const bf16_t*>(residual);
    bf16_t* yp = static_cast<bf16_t*>(y);
#define SNGGUF_CASE(QT)                                                                                          \
    if (qtype == QT) {                                                                                           \
        if (numerics == SNGGUF_NUM_GGML_FP32)                                                                    \
            return launch_qt<QT, SNGGUF_NUM_GGML_FP32>(xp, (int)M, a, b, N, K, bp, rp, yp, gated, gp, eps, stream, amax);          \
        if (numerics == SNGGUF_NUM_UPSTREAM_FP16)                                                                \
            return launch_qt<QT, SNGGUF_NUM_UPSTREAM_FP16>(xp, (int)M, a, b, N, K, bp, rp, yp, gated, gp, eps, stream, amax);      \
        return SNGGUF_E_BADTYPE;                                                                                 \
    }
    SNGGUF_CASE(SNGGUF_TYPE_Q4_0)
    SNGGUF_CASE(SNGGUF_TYPE_Q4_1)
    SNGGUF_CASE(SNGGUF_TYPE_Q5_0)
    SNGGUF_CASE(SNGGUF_TYPE_Q5_1)
    SNGGUF_CASE(SNGGUF_TYPE_Q8_0)
    SNGGUF_CASE(SNGGUF_TYPE_Q2_K)
    SNGGUF_CASE(SNGGUF_TYPE_Q3_K)
    SNGGUF_CASE(SNGGUF_TYPE_Q4_K)
    SNGGUF_CASE(SNGGUF_TYPE_Q5_K)
    SNGGUF_CASE(SNGGUF_TYPE_Q6_K)
#undef SNGGUF_CASE
    return SNGGUF_E_BADTYPE;
}

}  // namespace sngguf
