"""Writes kat_blocks.json: known-answer GGUF blocks typed in by hand.

No decoder and no packer is called here.  Every block is spelled as hex bytes straight from the
struct layouts of the ggml format, and every expected value is worked out on paper in the
comments, so the file pins the oracle against the format definition itself.

    block_q8_0 { f16 d; int8 qs[32]; }                                   34 bytes
    block_q4_K { f16 d; f16 dmin; u8 scales[12]; u8 qs[128]; }          144 bytes
    block_q5_K { f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]; } 176 bytes
    block_q6_K { u8 ql[128]; u8 qh[64]; int8 scales[16]; f16 d; }       210 bytes

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

with open("kat_blocks.json", "w") as f:
    json.dump(kats, f, indent=1)
print(f"wrote {len(kats)} known-answer blocks")
