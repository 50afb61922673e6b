"""Writes kat_blocks.json: known-answer GGUF blocks typed in by hand.

No decoder and no packer is called here.  Every block is spelled as hex bytes straight from the
struct layouts of the ggml format, and every expected value is worked out on paper in the
comments, so the file pins the oracle against the format definition itself.

    block_q8_0 { f16 d; int8 qs[32]; }                                   34 bytes
    block_q4_K { f16 d; f16 dmin; u8 scales[12]; u8 qs[128]; }          144 bytes
    block_q5_K { f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]; } 176 bytes
    block_q6_K { u8 ql[128]; u8 qh[64]; int8 scales[16]; f16 d; }       210 bytes
    block_q4_0 { f16 d; u8 qs[16]; }                                     18 bytes
    block_q4_1 { f16 d; f16 m; u8 qs[16]; }                              20 bytes
    block_q5_0 { f16 d; u8 qh[4]; u8 qs[16]; }                           22 bytes
    block_q5_1 { f16 d; f16 m; u8 qh[4]; u8 qs[16]; }                    24 bytes
    block_q2_K { u8 scales[16]; u8 qs[64]; f16 d; f16 dmin; }            84 bytes
    block_q3_K { u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d; }       110 bytes

Run from this directory: ``python make_kat.py``.
"""
import json

kats = []

# --- Q8_0, d = 1.0 (f16 0x3C00, little endian "003c"); value = d * qs[i]
# qs[0..3] = 0,1,2,3; qs[30] = 0xFF = -1; qs[31] = 0x80 = -128
hexs = "003c" + "00010203" + "00" * 26 + "ff80"
kats.append({"name": "q8_0 d=1 first bytes and sign", "type": 8, "hex": hexs, "fill": 0.0,
             "expect": {"1": 1.0, "2": 2.0, "3": 3.0, "30": -1.0, "31": -128.0},
             "how": "f16 0x3C00 = 1.0; int8 0xFF = -1, 0x80 = -128"})

# --- Q8_0, subnormal scale: f16 0x0001 = 2^-24; qs[5] = 127 -> 127 * 2^-24 (exact in fp32)
hexs = "0100" + "00" * 5 + "7f" + "00" * 26
kats.append({"name": "q8_0 subnormal scale", "type": 8, "hex": hexs, "fill": 0.0,
             "expect": {"5": 127 * 2.0 ** -24}, "how": "f16 0x0001 is 2^-24"})

# --- Q8_0, the fp16 chain rounds: d = f16 0x3555 = 1365/4096, q = 3 -> 4095/4096.
# Halves just below 1.0 are spaced 1/2048, so 4095/4096 is exactly halfway between
# 2047/2048 (0x3BFF, odd mantissa) and 1.0 (0x3C00, even): ties-to-even gives 1.0.
hexs = "5535" + "03" + "00" * 31
kats.append({"name": "q8_0 fp16-chain tie rounds to even", "type": 8, "numerics": 1, "hex": hexs, "fill": 0.0,
             "expect": {"0": 1.0}, "how": "0x3555 * 3 = 4095/4096, a tie between 0x3BFF and 0x3C00 -> 1.0"})
kats.append({"name": "q8_0 same block exact in fp32", "type": 8, "numerics": 0, "hex": hexs, "fill": 0.0,
             "expect": {"0": 4095 / 4096}, "how": "no rounding in fp32"})

# --- Q4_K: d = 1.0 ("003c"), dmin = 0.5 (f16 0x3800, "0038").
# 6-bit scales sc = [1,2,3,4, 21,6,7,8], mins m = [0,0,0,2, 0,0,0,35].
# scales[0..3] hold sc0..3 in bits 0-5 and the top two bits of sc4..7 in bits 6-7:
#   s0 = 1 | (21 >> 4 = 1) << 6 = 0x41, s1 = 0x02, s2 = 0x03, s3 = 0x04
# scales[4..7] hold m0..3 in bits 0-5 and the top two bits of m4..7 in bits 6-7:
#   s4 = s5 = s6 = 0x00, s7 = 2 | (35 >> 4 = 2) << 6 = 0x82
# scales[8..11]: low nibble = sc4..7 & 15, high nibble = m4..7 & 15:
#   s8 = 0x05, s9 = 0x06, s10 = 0x07, s11 = 8 | (35 & 15 = 3) << 4 = 0x38
# qs: chunk c (32 bytes) carries elements 64c..64c+31 in low nibbles (sub-block 2c) and
# 64c+32..64c+63 in high nibbles (sub-block 2c+1).
#   qs[0] = 0xA3   -> element 0 = 3 (sub-block 0), element 32 = 10 (sub-block 1)
#   qs[127] = 0xF0 -> element 223 = 0 (sub-block 6), element 255 = 15 (sub-block 7)
# value = d*sc_j*q - dmin*m_j: every element of sub-block 3 is -0.5*2 = -1, of sub-block 7 is
# -0.5*35 = -17.5; element 0 = 1*3 = 3; element 32 = 2*10 = 20; element 255 = 8*15 - 17.5.
qs = ["00"] * 128
qs[0] = "a3"
qs[127] = "f0"
hexs = "003c" + "0038" + "41020304" + "00000082" + "05060738" + "".join(qs)
exp = {}
for e in range(96, 128):
    exp[str(e)] = -1.0
for e in range(224, 256):
    exp[str(e)] = -17.5
exp["0"] = 3.0
exp["32"] = 20.0
exp["255"] = 8 * 15 - 17.5
kats.append({"name": "q4_k high scale bits and nibble order", "type": 12, "hex": hexs, "fill": 0.0, "expect": exp,
             "how": "see make_kat.py"})

# --- Q5_K: the Q4_K head above (d = 1, dmin = 0.5, sc = [1,2,3,4,21,6,7,8], m = [0,0,0,2,0,0,0,35]), then
# qh[32], then qs[128].  Element l of sub-block j takes its fifth bit from bit j of qh[l]:
#   qs[0] = 0xA3, qh[0] = 0b00000011 -> element 0 = 3 + 16 = 19 (sub-block 0), element 32 = 10 + 16 = 26 (sub-block 1)
#   qs[127] = 0xF0 (chunk 3, l = 31), qh[31] = 0b10000000 -> element 223 = 0 (sub-block 6, bit 6 clear),
#                                                          element 255 = 15 + 16 = 31 (sub-block 7)
#   qh[5] = 0b00010000 with qs[64 + 5] = 0x00 -> element 128 + 5 = 133 (sub-block 4, l = 5) = 16
# value = d*sc_j*q - dmin*m_j: element 0 = 19, element 32 = 2*26 = 52, element 133 = 21*16 = 336,
# element 255 = 8*31 - 17.5 = 230.5; the rest of sub-block 3 is -1, the rest of sub-block 7 is -17.5.
qs = ["00"] * 128
qs[0] = "a3"
qs[127] = "f0"
qh = ["00"] * 32
qh[0] = "03"
qh[31] = "80"
qh[5] = "10"
hexs = "003c" + "0038" + "41020304" + "00000082" + "05060738" + "".join(qh) + "".join(qs)
exp = {}
for e in range(96, 128):
    exp[str(e)] = -1.0
for e in range(224, 256):
    exp[str(e)] = -17.5
exp["0"] = 19.0
exp["32"] = 52.0
exp["133"] = 336.0
exp["255"] = 8 * 31 - 17.5
kats.append({"name": "q5_k fifth bit by sub-block", "type": 13, "hex": hexs, "fill": 0.0, "expect": exp,
             "how": "see make_kat.py"})

# --- Q6_K: d = 2.0 (f16 0x4000, "0040"); scales all 1 except scales[9] = 0xFD = -3.
# A quant is 6 bits: low nibble from ql, top two bits from qh; value = d * scale[e/16] * (q - 32).
# Per 128-element half h and l in 0..31: elements l, l+32, l+64, l+96 take
#   ql[64h+l] low, ql[64h+32+l] low, ql[64h+l] high, ql[64h+32+l] high   and qh[32h+l] bits 0-1, 2-3, 4-5, 6-7.
# Background: every quant = 32 (-> 0): all ql nibbles 0, every qh field 0b10 -> qh bytes 0xAA.
#   element 146 = half 1, l = 18, first quarter, scale index 146/16 = 9 (-3): q = 63:
#       ql[64+18] = 0x0F, qh[32+18] fields (q1=3, others 2) = 0b10101011 = 0xAB -> 2 * -3 * 31 = -186
#   element 5 = half 0, l = 5, first quarter, scale 1: q = 0: qh[5] field 0 = 0
#   element 101 = half 0, l = 5, fourth quarter (96..127), scale index 6 (1): q = 48: low nibble 0,
#       top bits 3 -> qh[5] field 3 = 3.  qh[5] = fields (0, 2, 2, 3) = 0b11101000 = 0xE8
#       -> element 5 = 2 * 1 * (0 - 32) = -64, element 101 = 2 * 1 * (48 - 32) = 32
ql = ["00"] * 128
qh = ["aa"] * 64
ql[64 + 18] = "0f"
qh[32 + 18] = "ab"
qh[5] = "e8"
sc = ["01"] * 16
sc[9] = "fd"
hexs = "".join(ql) + "".join(qh) + "".join(sc) + "0040"
kats.append({"name": "q6_k quadrants, high bits, signed scale", "type": 14, "hex": hexs, "fill": 0.0,
             "expect": {"146": -186.0, "5": -64.0, "101": 32.0}, "how": "see make_kat.py"})

# --- Q4_0: d = 2.0 ("0040"); value = d * (nibble - 8); byte l carries element l (low) and l + 16 (high).
# Background nibble 8 (-> 0): bytes 0x88.  qs[3] = 0x1F: element 3 = 15 - 8 = 7 -> 14, element 19 = 1 - 8 = -7 -> -14.
hexs = "0040" + "88" * 3 + "1f" + "88" * 12
kats.append({"name": "q4_0 nibble order and offset", "type": 2, "hex": hexs, "fill": 0.0,
             "expect": {"3": 14.0, "19": -14.0}, "how": "see make_kat.py"})

# --- Q4_1: d = 0.5 ("0038"), m = -1.0 (f16 0xBC00, "00bc"); value = d * nibble + m.
# Background nibble 0 -> -1.  qs[15] = 0x92: element 15 = 2 -> 0.0, element 31 = 9 -> 3.5.
hexs = "0038" + "00bc" + "00" * 15 + "92"
kats.append({"name": "q4_1 minimum is added", "type": 3, "hex": hexs, "fill": -1.0,
             "expect": {"15": 0.0, "31": 3.5}, "how": "see make_kat.py"})

# --- Q5_0: d = 1.0; value = d * ((nibble | fifth << 4) - 16), fifth bit of element e = bit e of the
# little-endian 32-bit qh.  Background stored 16 (-> 0): nibbles 0, qh all ones.
#   element 9: bit 9 (byte 1, bit 1) cleared -> qh bytes ff fd ff ff; low nibble of qs[9] = 3 -> 3 - 16 = -13
#   element 30: bit 30 stays set; high nibble of qs[14] = 0xA -> (10 | 16) - 16 = 10
qs = ["00"] * 16
qs[9] = "03"
qs[14] = "a0"
hexs = "003c" + "fffdffff" + "".join(qs)
kats.append({"name": "q5_0 fifth-bit word, bit order", "type": 6, "hex": hexs, "fill": 0.0,
             "expect": {"9": -13.0, "30": 10.0}, "how": "see make_kat.py"})

# --- Q5_1: d = 0.25 (f16 0x3400, "0034"), m = 1.0; value = d * (nibble | fifth << 4) + m.
# Only bit 17 of qh set (byte 2 = 0x02); qs[1] = 0x70: element 1 = 0 -> 1.0, element 17 = 7 + 16 = 23 -> 6.75.
hexs = "0034" + "003c" + "00000200" + "00" + "70" + "00" * 14
kats.append({"name": "q5_1 fifth bit of a high-nibble element", "type": 7, "hex": hexs, "fill": 1.0,
             "expect": {"17": 6.75}, "how": "see make_kat.py"})

# --- Q2_K: d = 1.0, dmin = 0.5; scales[g] = scale | min << 4 for the 16-element group g; per 128-element half,
# bit pair j of qs[32 * half + l] is element 128 * half + 32 * j + l; value = d * scale * q - dmin * min.
# All scales 0x01 (scale 1, min 0) except scales[10] = 0x23 (scale 3, min 2): elements 160..175.
# qs[32 + 5] = 0b01_00_11_10 = 0x4E (half 1, l = 5): element 133 = 2 -> 2; element 165 = 3 -> 3 * 3 - 1 = 8;
# element 197 = 0; element 229 = 1 -> 1.  The rest of group 10 is 0 * 3 - 0.5 * 2 = -1.
hexs = "01" * 10 + "23" + "01" * 5 + "00" * 37 + "4e" + "00" * 26 + "003c" + "0038"
exp = {str(e): -1.0 for e in range(160, 176)}
exp.update({"133": 2.0, "165": 8.0, "229": 1.0})
kats.append({"name": "q2_k bit pairs, group scale and min", "type": 10, "hex": hexs, "fill": 0.0, "expect": exp,
             "how": "see make_kat.py"})

# --- Q3_K: d = 1.0; quant = bit pair (as Q2_K) minus 4 unless bit (4 * half + j) of hmask[l] is set;
# value = d * (scale6 - 32) * quant.  Background: quant stored 4 (mask bit set, low bits 0) -> 0.
# Scales: all 1 -> stored 33 = 0b10_0001: low nibble 1 (scales[0..7] = 0x11: low nibble for groups 0..7, high
# nibble for groups 8..15), high bits 2 (scales[8..11] = 0b10101010 = 0xAA: byte k holds groups k, k+4, k+8,
# k+12 at bits 0-1, 2-3, 4-5, 6-7).  Group 13 = -3 -> stored 29 = 0b01_1101: low nibble 0xD in the high nibble
# of scales[5] (0xD1), high bits 1 at bits 6-7 of scales[9] (0b01101010 = 0x6A).
#   element 210 (half 1, j = 2, l = 18, group 13): quant -4 -> stored 0: clear bit 6 of hmask[18] (0xBF) -> -3 * -4 = 12
#   element 211 (l = 19): quant 3 -> stored 7: mask bit set, qs[32 + 19] bits 4-5 = 3 (0x30) -> -3 * 3 = -9
#   element 7 (half 0, j = 0, group 0): quant -2 -> stored 2: clear bit 0 of hmask[7] (0xFE), qs[7] = 0x02 -> -2
hm = ["ff"] * 32
hm[7] = "fe"
hm[18] = "bf"
qs = ["00"] * 64
qs[7] = "02"
qs[51] = "30"
hexs = "".join(hm) + "".join(qs) + "11" * 5 + "d1" + "11" * 2 + "aa" + "6a" + "aa" + "aa" + "003c"
kats.append({"name": "q3_k mask bit, split scales", "type": 11, "hex": hexs, "fill": 0.0,
             "expect": {"210": 12.0, "211": -9.0, "7": -2.0}, "how": "see make_kat.py"})

with open("kat_blocks.json", "w") as f:
    json.dump(kats, f, indent=1)
print(f"wrote {len(kats)} known-answer blocks")
