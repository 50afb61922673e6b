/*
 * sngguf_oracle.c - CPU restatement of the GGUF quantized-linear path.  TEST INFRASTRUCTURE:
 * only tests, the smoke check and the bench's cpu_baseline leg may build or call this file;
 * the shipped library never does.
 *
 * What it restates.  The reference glue (src/sensenova_u1/utils/gguf_loader.py:17-85) hands
 * every quantized tensor to diffusers 0.37.1 (uv.lock:164-165), whose GGUFLinear.forward is
 *     w = dequantize_gguf_tensor(weight)      # dequantize_blocks_Q8_0 / _Q4_K / _Q6_K / ...
 *     w = w.to(compute_dtype)                 # bf16
 *     y = F.linear(x, w, bias)
 * and whose block decoders restate ggml's dequantize_row_q8_0 / q4_K / q6_K (and the other
 * q4_0 ... q5_K formats) and get_scale_min_k4.  Neither package's source is in the reference tree, so the functions
 * below restate the published ggml block formats (numerics 0) and the upstream torch op
 * sequence with its fp16 intermediates (numerics 1).
 *
 * Pinning.  Numerics 0 is pinned by closed forms: one-hot positional blocks, scale-packing
 * cases, encode->decode round trips through independently written packers, hand-written
 * known-answer blocks and a bitwise cross-check against the vectorised restatement in
 * oracle.py.  Numerics 1 is pinned, per type, against the recorded operation sequence written out as
 * numpy float16 operations, one rounding per tensor operation, with an alternative placement of a
 * rounding shown to give different bits on the same blocks (tests/test_oracle_fp16_chain.py), so a
 * moved or dropped rounding here fails.  That the recorded sequence is what the upstream package
 * executes rests on a reading of that package, which cannot be imported here: PARITY UNPINNED for
 * that one point (the order and kind of upstream's tensor operations), for every type.
 *
 * No dependency beyond libc; scalar loops; fp16/bf16 conversions written out by hand so that
 * they do not share code with numpy, torch or the device kernels.
 */
#include <stdint.h>
#include <string.h>
#include <math.h>

/* ---- scalar float formats ------------------------------------------------------------ */

static inline float u32_as_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_as_u32(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* IEEE binary16 -> binary32, exact (subnormals, inf, nan included). */
float sno_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return u32_as_f32(sign);
        /* subnormal: man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-8f;
        return sign ? -v : v;
    }
    if (exp == 31) return u32_as_f32(sign | 0x7F800000u | (man << 13));
    return u32_as_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* binary32 -> binary16, round to nearest even, subnormals produced, overflow -> inf. */
uint16_t sno_f32_to_f16(float f) {
    uint32_t x = f32_as_u32(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((ax > 0x7F800000u) ? (0x200u | ((ax >> 13) & 0x3FFu)) : 0u));
    }
    if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* >= 65520 rounds to inf */
    if (ax < 0x38800000u) { /* below the smallest normal half: result is subnormal or zero */
        if (ax < 0x33000000u) return sign; /* < 2^-25 rounds to zero (2^-25 itself ties to even = 0) */
        uint32_t e = ax >> 23;                         /* biased fp32 exponent, 102..112 */
        uint32_t m = (ax & 0x7FFFFFu) | 0x800000u;     /* 24-bit significand */
        uint32_t shift = 126u - e;                     /* drop so that the unit is 2^-24: 14..24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t e = (ax >> 23) - 112u;
    uint32_t m = ax & 0x7FFFFFu;
    uint32_t q = (e << 10) | (m >> 13);
    uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++; /* carry into the exponent is correct */
    return (uint16_t)(sign | q);
}

/* binary32 -> bfloat16, round to nearest even (nan kept quiet). */
uint16_t sno_f32_to_bf16(float f) {
    uint32_t x = f32_as_u32(f);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x40u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7FFFu + lsb;
    return (uint16_t)(x >> 16);
}

float sno_bf16_to_f32(uint16_t b) { return u32_as_f32((uint32_t)b << 16); }

/* one fp16 tensor-op rounding: the value an fp16 result tensor holds, widened again */
static inline float r16(float v) { return sno_f16_to_f32(sno_f32_to_f16(v)); }

static inline uint16_t rd16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* ---- block decoders ------------------------------------------------------------------ */
/* numerics 0: ggml fp32 semantics.  numerics 1: upstream fp16 op chain, result is the fp16
 * tensor value widened to fp32 (exactly representable). */

#define QK8_0 32
#define QK_K 256

/* ggml dequantize_row_q8_0: y[i] = d * qs[i].  Upstream: (d.view(f16) * x.view(i8)) -> f16. */
void sno_dequantize_row_q8_0(const uint8_t* src, float* y, int64_t k, int numerics) {
    int64_t nb = k / QK8_0;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = src + b * 34;
        float d = sno_f16_to_f32(rd16(blk));
        for (int i = 0; i < 32; i++) {
            float v = d * (float)(int8_t)blk[2 + i];
            y[b * 32 + i] = numerics ? r16(v) : v;
        }
    }
}

/* ggml get_scale_min_k4: sub-block j of a Q4_K super-block -> 6-bit scale and 6-bit min. */
static void scale_min_k4(int j, const uint8_t* s, uint8_t* sc, uint8_t* mn) {
    if (j < 4) {
        *sc = s[j] & 63;
        *mn = s[j + 4] & 63;
    } else {
        *sc = (uint8_t)((s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4));
        *mn = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}

/* ggml dequantize_row_q4_K: per 64 elements, low nibbles then high nibbles of 32 bytes;
 * y = d*sc*q - dmin*m.  Upstream: D=R(d*sc), DM=R(dmin*m), y = R(R(D*q) - DM). */
void sno_dequantize_row_q4_K(const uint8_t* src, float* y, int64_t k, int numerics) {
    int64_t nb = k / QK_K;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = src + b * 144;
        float d = sno_f16_to_f32(rd16(blk));
        float dmin = sno_f16_to_f32(rd16(blk + 2));
        const uint8_t* scales = blk + 4;
        const uint8_t* qs = blk + 16;
        float* out = y + b * QK_K;
        for (int c = 0; c < 4; c++) { /* 64-element chunk: sub-blocks 2c and 2c+1 */
            uint8_t sc0, m0, sc1, m1;
            scale_min_k4(2 * c, scales, &sc0, &m0);
            scale_min_k4(2 * c + 1, scales, &sc1, &m1);
            float d0 = d * (float)sc0, mm0 = dmin * (float)m0;
            float d1 = d * (float)sc1, mm1 = dmin * (float)m1;
            if (numerics) { d0 = r16(d0); mm0 = r16(mm0); d1 = r16(d1); mm1 = r16(mm1); }
            for (int l = 0; l < 32; l++) {
                float lo = (float)(qs[32 * c + l] & 0x0F);
                float hi = (float)(qs[32 * c + l] >> 4);
                if (numerics) {
                    out[64 * c + l] = r16(r16(d0 * lo) - mm0);
                    out[64 * c + 32 + l] = r16(r16(d1 * hi) - mm1);
                } else {
                    out[64 * c + l] = d0 * lo - mm0;
                    out[64 * c + 32 + l] = d1 * hi - mm1;
                }
            }
        }
    }
}

/* block_q5_K { f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128] } (176 bytes), ggml
 * dequantize_row_q5_K: as Q4_K with a fifth bit per quant, bit j of qh[l] for element l of
 * sub-block j.  upstream (numerics 1): dequantize_blocks_Q5_K, the rounding points of Q4_K. */
void sno_dequantize_row_q5_K(const uint8_t* src, float* y, int64_t k, int numerics) {
    int64_t nb = k / QK_K;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = src + b * 176;
        float d = sno_f16_to_f32(rd16(blk));
        float dmin = sno_f16_to_f32(rd16(blk + 2));
        const uint8_t* scales = blk + 4;
        const uint8_t* qh = blk + 16;
        const uint8_t* qs = blk + 48;
        float* out = y + b * QK_K;
        for (int c = 0; c < 4; c++) {
            uint8_t sc0, m0, sc1, m1;
            scale_min_k4(2 * c, scales, &sc0, &m0);
            scale_min_k4(2 * c + 1, scales, &sc1, &m1);
            float d0 = d * (float)sc0, mm0 = dmin * (float)m0;
            float d1 = d * (float)sc1, mm1 = dmin * (float)m1;
            if (numerics) { d0 = r16(d0); mm0 = r16(mm0); d1 = r16(d1); mm1 = r16(mm1); }
            for (int l = 0; l < 32; l++) {
                float lo = (float)((qs[32 * c + l] & 0x0F) | (((qh[l] >> (2 * c)) & 1) << 4));
                float hi = (float)((qs[32 * c + l] >> 4) | (((qh[l] >> (2 * c + 1)) & 1) << 4));
                if (numerics) {
                    out[64 * c + l] = r16(r16(d0 * lo) - mm0);
                    out[64 * c + 32 + l] = r16(r16(d1 * hi) - mm1);
                } else {
                    out[64 * c + l] = d0 * lo - mm0;
                    out[64 * c + 32 + l] = d1 * hi - mm1;
                }
            }
        }
    }
}

/* ggml dequantize_row_q6_K: per 128-element half, 32 lanes l give elements l, l+32, l+64,
 * l+96; y = d*scale[e/16]*(q-32).  Upstream: D=R(d*scale), y=R(D*(q-32)). */
void sno_dequantize_row_q6_K(const uint8_t* src, float* y, int64_t k, int numerics) {
    int64_t nb = k / QK_K;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = src + b * 210;
        const uint8_t* ql = blk;
        const uint8_t* qh = blk + 128;
        const int8_t* sc = (const int8_t*)(blk + 192);
        float d = sno_f16_to_f32(rd16(blk + 208));
        float* out = y + b * QK_K;
        for (int h = 0; h < 2; h++) {
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int q1 = (int)((ql[64 * h + l] & 0x0F) | (((qh[32 * h + l] >> 0) & 3) << 4)) - 32;
                int q2 = (int)((ql[64 * h + l + 32] & 0x0F) | (((qh[32 * h + l] >> 2) & 3) << 4)) - 32;
                int q3 = (int)((ql[64 * h + l] >> 4) | (((qh[32 * h + l] >> 4) & 3) << 4)) - 32;
                int q4 = (int)((ql[64 * h + l + 32] >> 4) | (((qh[32 * h + l] >> 6) & 3) << 4)) - 32;
                float s1 = d * (float)sc[8 * h + is + 0];
                float s2 = d * (float)sc[8 * h + is + 2];
                float s3 = d * (float)sc[8 * h + is + 4];
                float s4 = d * (float)sc[8 * h + is + 6];
                float v1, v2, v3, v4;
                if (numerics) {
                    v1 = r16(r16(s1) * (float)q1); v2 = r16(r16(s2) * (float)q2);
                    v3 = r16(r16(s3) * (float)q3); v4 = r16(r16(s4) * (float)q4);
                } else {
                    v1 = s1 * (float)q1; v2 = s2 * (float)q2; v3 = s3 * (float)q3; v4 = s4 * (float)q4;
                }
                out[128 * h + l] = v1;
                out[128 * h + l + 32] = v2;
                out[128 * h + l + 64] = v3;
                out[128 * h + l + 96] = v4;
            }
        }
    }
}

/* ---- legacy 32-element blocks --------------------------------------------------------- */

/* block_q4_0 { f16 d; u8 qs[16] } (18 bytes), ggml dequantize_row_q4_0: element l is the low
 * nibble of qs[l], element l+16 the high nibble; y = d * (q - 8).
 * upstream dequantize_blocks_Q4_0: R(d * (q - 8)). */
void sno_dequantize_row_q4_0(const uint8_t* src, float* y, int64_t k, int numerics) {
    int64_t nb = k / 32;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = src + b * 18;
        float d = sno_f16_to_f32(rd16(blk));
        for (int l = 0; l < 16; l++) {
            float v0 = d * (float)((int)(blk[2 + l] & 0x0F) - 8);
            float v1 = d * (float)((int)(blk[2 + l] >> 4) - 8);
            y[b * 32 + l] = numerics ? r16(v0) : v0;
            y[b * 32 + l + 16] = numerics ? r16(v1) : v1;
        }
    }
}

/* block_q4_1 { f16 d; f16 m; u8 qs[16] } (20 bytes), ggml dequantize_row_q4_1: y = d * q + m.
 * upstream dequantize_blocks_Q4_1: R(R(d * q) + m). */
void sno_dequantize_row_q4_1(const uint8_t* src, float* y, int64_t k, int numerics) {
    int64_t nb = k / 32;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = src + b * 20;
        float d = sno_f16_to_f32(rd16(blk));
        float m = sno_f16_to_f32(rd16(blk + 2));
        for (int l = 0; l < 16; l++) {
            float q0 = (float)(blk[4 + l] & 0x0F), q1 = (float)(blk[4 + l] >> 4);
            y[b * 32 + l] = numerics ? r16(r16(d * q0) + m) : d * q0 + m;
            y[b * 32 + l + 16] = numerics ? r16(r16(d * q1) + m) : d * q1 + m;
        }
    }
}

/* block_q5_0 { f16 d; u8 qh[4]; u8 qs[16] } (22 bytes), ggml dequantize_row_q5_0: bit e of the
 * little-endian 32-bit qh is the fifth bit of element e; y = d * (q - 16).
 * upstream dequantize_blocks_Q5_0: R(d * (q - 16)). */
void sno_dequantize_row_q5_0(const uint8_t* src, float* y, int64_t k, int numerics) {
    int64_t nb = k / 32;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = src + b * 22;
        float d = sno_f16_to_f32(rd16(blk));
        uint32_t qh = (uint32_t)blk[2] | ((uint32_t)blk[3] << 8) | ((uint32_t)blk[4] << 16) | ((uint32_t)blk[5] << 24);
        for (int l = 0; l < 16; l++) {
            int q0 = (int)((blk[6 + l] & 0x0F) | (((qh >> l) & 1u) << 4)) - 16;
            int q1 = (int)((blk[6 + l] >> 4) | (((qh >> (l + 16)) & 1u) << 4)) - 16;
            float v0 = d * (float)q0, v1 = d * (float)q1;
            y[b * 32 + l] = numerics ? r16(v0) : v0;
            y[b * 32 + l + 16] = numerics ? r16(v1) : v1;
        }
    }
}

/* block_q5_1 { f16 d; f16 m; u8 qh[4]; u8 qs[16] } (24 bytes), ggml dequantize_row_q5_1:
 * y = d * q + m with the 5-bit q of Q5_0 (no offset).  upstream: R(R(d * q) + m). */
void sno_dequantize_row_q5_1(const uint8_t* src, float* y, int64_t k, int numerics) {
    int64_t nb = k / 32;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = src + b * 24;
        float d = sno_f16_to_f32(rd16(blk));
        float m = sno_f16_to_f32(rd16(blk + 2));
        uint32_t qh = (uint32_t)blk[4] | ((uint32_t)blk[5] << 8) | ((uint32_t)blk[6] << 16) | ((uint32_t)blk[7] << 24);
        for (int l = 0; l < 16; l++) {
            float q0 = (float)((blk[8 + l] & 0x0F) | (((qh >> l) & 1u) << 4));
            float q1 = (float)((blk[8 + l] >> 4) | (((qh >> (l + 16)) & 1u) << 4));
            y[b * 32 + l] = numerics ? r16(r16(d * q0) + m) : d * q0 + m;
            y[b * 32 + l + 16] = numerics ? r16(r16(d * q1) + m) : d * q1 + m;
        }
    }
}

/* ---- 2- and 3-bit super-blocks ---------------------------------------------------------- */

/* block_q2_K { u8 scales[16]; u8 qs[64]; f16 d; f16 dmin } (84 bytes), ggml dequantize_row_q2_K:
 * per 128-element half, bit pair j of qs[32*half + l] is element 32*j + l; 16-element group g
 * has scale scales[g] & 15 and min scales[g] >> 4; y = d*sc*q - dmin*mn.
 * upstream dequantize_blocks_Q2_K: DL = R(d*sc), ML = R(dmin*mn), y = R(R(DL*q) - ML). */
void sno_dequantize_row_q2_K(const uint8_t* src, float* y, int64_t k, int numerics) {
    int64_t nb = k / QK_K;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = src + b * 84;
        const uint8_t* scales = blk;
        const uint8_t* qs = blk + 16;
        float d = sno_f16_to_f32(rd16(blk + 80));
        float dmin = sno_f16_to_f32(rd16(blk + 82));
        float* out = y + b * QK_K;
        int is = 0;
        for (int half = 0; half < 2; half++) {
            for (int j = 0; j < 4; j++) {
                for (int part = 0; part < 2; part++) {
                    uint8_t sc = scales[is++];
                    float dl = d * (float)(sc & 0x0F), ml = dmin * (float)(sc >> 4);
                    if (numerics) { dl = r16(dl); ml = r16(ml); }
                    for (int l = 0; l < 16; l++) {
                        float q = (float)((qs[32 * half + 16 * part + l] >> (2 * j)) & 3);
                        out[128 * half + 32 * j + 16 * part + l] = numerics ? r16(r16(dl * q) - ml) : dl * q - ml;
                    }
                }
            }
        }
    }
}

/* block_q3_K { u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d } (110 bytes), ggml
 * dequantize_row_q3_K: the 6-bit scale of 16-element group g has its low nibble in
 * scales[g % 8] (upper nibble for g >= 8) and its two high bits in scales[8 + g % 4] at bit
 * 2*(g/4), offset by -32; the quant is the bit pair as in Q2_K minus 4 unless bit
 * (4*half + j) of hmask[l] is set; y = d*(sc-32)*q.
 * upstream dequantize_blocks_Q3_K: DL = R(d*(sc-32)), y = R(DL*q). */
void sno_dequantize_row_q3_K(const uint8_t* src, float* y, int64_t k, int numerics) {
    int64_t nb = k / QK_K;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = src + b * 110;
        const uint8_t* hm = blk;
        const uint8_t* qs = blk + 32;
        const uint8_t* sp = blk + 96;
        float d = sno_f16_to_f32(rd16(blk + 108));
        float* out = y + b * QK_K;
        int sc[16];
        for (int g = 0; g < 16; g++) {
            int lo = g < 8 ? (sp[g] & 0x0F) : (sp[g - 8] >> 4);
            int hi = (sp[8 + (g & 3)] >> (2 * (g >> 2))) & 3;
            sc[g] = (lo | (hi << 4)) - 32;
        }
        int is = 0;
        for (int half = 0; half < 2; half++) {
            for (int j = 0; j < 4; j++) {
                for (int part = 0; part < 2; part++) {
                    float dl = d * (float)sc[is++];
                    if (numerics) dl = r16(dl);
                    for (int l = 0; l < 16; l++) {
                        int ll = 16 * part + l;
                        int q = (int)((qs[32 * half + ll] >> (2 * j)) & 3) - (((hm[ll] >> (4 * half + j)) & 1) ? 0 : 4);
                        float v = dl * (float)q;
                        out[128 * half + 32 * j + ll] = numerics ? r16(v) : v;
                    }
                }
            }
        }
    }
}


/* BF16 (type 30; upstream dequantize_blocks_BF16): "blocks" of one element, two bytes; the
 * value is the bf16 bit pattern shifted into the upper half of an fp32 word - exact, no
 * rounding in either numerics mode. */
void sno_dequantize_row_bf16(const uint8_t* src, float* y, int64_t k, int numerics) {
    (void)numerics;
    for (int64_t i = 0; i < k; i++) y[i] = u32_as_f32((uint32_t)rd16(src + 2 * i) << 16);
}

/* ggml type enum -> bytes / elements per block (0: not restated here) */
int64_t sno_type_size(int qtype) {
    switch (qtype) {
    case 2: return 18; case 3: return 20; case 6: return 22; case 7: return 24; case 8: return 34;
    case 10: return 84; case 11: return 110; case 12: return 144; case 13: return 176; case 14: return 210;
    case 30: return 2;
    default: return 0;
    }
}
int64_t sno_block_size(int qtype) {
    switch (qtype) {
    case 2: case 3: case 6: case 7: case 8: return 32;
    case 10: case 11: case 12: case 13: case 14: return 256;
    case 30: return 1;
    default: return 0;
    }
}

static int dequant_row(const uint8_t* src, int qtype, float* y, int64_t k, int numerics) {
    switch (qtype) {
    case 2: sno_dequantize_row_q4_0(src, y, k, numerics); return 0;
    case 3: sno_dequantize_row_q4_1(src, y, k, numerics); return 0;
    case 6: sno_dequantize_row_q5_0(src, y, k, numerics); return 0;
    case 7: sno_dequantize_row_q5_1(src, y, k, numerics); return 0;
    case 8: sno_dequantize_row_q8_0(src, y, k, numerics); return 0;
    case 10: sno_dequantize_row_q2_K(src, y, k, numerics); return 0;
    case 11: sno_dequantize_row_q3_K(src, y, k, numerics); return 0;
    case 12: sno_dequantize_row_q4_K(src, y, k, numerics); return 0;
    case 13: sno_dequantize_row_q5_K(src, y, k, numerics); return 0;
    case 14: sno_dequantize_row_q6_K(src, y, k, numerics); return 0;
    case 30: sno_dequantize_row_bf16(src, y, k, numerics); return 0;
    default: return -1;
    }
}

/*
 * dequantize_gguf_tensor: bytes [rows][cols/bs*ts] -> [rows][cols] of out_dtype
 * (0 = fp32, 1 = fp16 bits, 2 = bf16 bits).  `scratch` holds cols floats.
 */
int sno_dequantize(const uint8_t* q, int qtype, int64_t rows, int64_t cols, void* out, int out_dtype,
                   int numerics, float* scratch) {
    int64_t bs = sno_block_size(qtype), ts = sno_type_size(qtype);
    if (!bs || cols % bs) return -2;
    int64_t row_bytes = cols / bs * ts;
    for (int64_t r = 0; r < rows; r++) {
        float* dst = out_dtype == 0 ? (float*)out + r * cols : scratch;
        if (dequant_row(q + r * row_bytes, qtype, dst, cols, numerics)) return -1;
        if (out_dtype == 1) {
            uint16_t* o = (uint16_t*)out + r * cols;
            for (int64_t i = 0; i < cols; i++) o[i] = sno_f32_to_f16(dst[i]);
        } else if (out_dtype == 2) {
            uint16_t* o = (uint16_t*)out + r * cols;
            for (int64_t i = 0; i < cols; i++) o[i] = sno_f32_to_bf16(dst[i]);
        }
    }
    return 0;
}

/*
 * GGUFLinear.forward_native on bf16 bit patterns: the weight row is decoded, rounded to bf16,
 * and dotted with each bf16 activation row.  The accumulator is a double, i.e. the exact sum
 * up to 2^-53 - the value every fp32 summation order of F.linear scatters around - and the
 * result (plus bias) is rounded to fp32 and then to bf16.  `scratch` holds K floats.
 */
int sno_linear(const uint16_t* x, int64_t M, const uint8_t* q, int qtype, int64_t N, int64_t K,
               const uint16_t* bias, uint16_t* y, int numerics, float* scratch) {
    int64_t bs = sno_block_size(qtype), ts = sno_type_size(qtype);
    if (!bs || K % bs) return -2;
    int64_t row_bytes = K / bs * ts;
    for (int64_t n = 0; n < N; n++) {
        if (dequant_row(q + n * row_bytes, qtype, scratch, K, numerics)) return -1;
        for (int64_t i = 0; i < K; i++) scratch[i] = sno_bf16_to_f32(sno_f32_to_bf16(scratch[i]));
        for (int64_t m = 0; m < M; m++) {
            const uint16_t* xr = x + m * K;
            double acc = 0.0;
            for (int64_t i = 0; i < K; i++) acc += (double)sno_bf16_to_f32(xr[i]) * (double)scratch[i];
            if (bias) acc += (double)sno_bf16_to_f32(bias[n]);
            y[m * N + n] = sno_f32_to_bf16((float)acc);
        }
    }
    return 0;
}

/* SiLU gating with the bf16 rounding after every torch op of
 * `act_fn(gate_proj(x)) * up_proj(x)` (modeling_qwen3.py:215): inputs are the two bf16
 * projection outputs. */
void sno_silu_mul(const uint16_t* gate, const uint16_t* up, uint16_t* h, int64_t n) {
    for (int64_t i = 0; i < n; i++) {
        float g = sno_bf16_to_f32(gate[i]);
        float s = sno_bf16_to_f32(sno_f32_to_bf16(g / (1.0f + expf(-g))));
        h[i] = sno_f32_to_bf16(s * sno_bf16_to_f32(up[i]));
    }
}

/*
 * Mixed-modality routing as the unreachable branch at modeling_qwen3.py:779-783 defines it:
 * out = zeros; out[~ind] = proj(x[~ind]); out[ind] = proj_mot_gen(x[ind]).
 */
int sno_grouped_linear(const uint16_t* x, int64_t M, const uint8_t* indicator, const uint8_t* q_und,
                       int qtype_und, const uint8_t* q_gen, int qtype_gen, int64_t N, int64_t K,
                       const uint16_t* bias_und, const uint16_t* bias_gen, uint16_t* y, int numerics,
                       float* scratch) {
    memset(y, 0, (size_t)(M * N) * sizeof(uint16_t));
    for (int tower = 0; tower < 2; tower++) {
        const uint8_t* q = tower ? q_gen : q_und;
        const uint16_t* bias = tower ? bias_gen : bias_und;
        int qtype = tower ? qtype_gen : qtype_und;
        int64_t bs = sno_block_size(qtype), ts = sno_type_size(qtype);
        if (!bs || K % bs) return -2;
        int64_t row_bytes = K / bs * ts;
        for (int64_t n = 0; n < N; n++) {
            if (dequant_row(q + n * row_bytes, qtype, scratch, K, numerics)) return -1;
            for (int64_t i = 0; i < K; i++) scratch[i] = sno_bf16_to_f32(sno_f32_to_bf16(scratch[i]));
            for (int64_t m = 0; m < M; m++) {
                if ((indicator[m] != 0) != tower) continue;
                const uint16_t* xr = x + m * K;
                double acc = 0.0;
                for (int64_t i = 0; i < K; i++) acc += (double)sno_bf16_to_f32(xr[i]) * (double)scratch[i];
                if (bias) acc += (double)sno_bf16_to_f32(bias[n]);
                y[m * N + n] = sno_f32_to_bf16((float)acc);
            }
        }
    }
    return 0;
}
