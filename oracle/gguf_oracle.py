"""CPU oracle for the GGUF quantized-linear path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this module; the shipped package never does.

Two independent restatements live here:

* a vectorised torch-CPU one that follows, op by op, what the reference executes for a
  quantized projection: ``src/sensenova_u1/utils/gguf_loader.py:43`` wraps the raw bytes in a
  ``GGUFParameter`` and ``:64-81`` swaps ``nn.Linear`` for diffusers' ``GGUFLinear``
  (diffusers 0.37.1, ``uv.lock:164-165``), whose forward is ``dequantize_gguf_tensor(weight)
  .to(compute_dtype)`` followed by ``torch.nn.functional.linear``.  The per-type decoders
  below (``dequantize_blocks_*``) keep upstream's names, arguments and tensor-op sequence, so
  that with ``dtype=None`` every intermediate is the fp16 tensor upstream produces, and with
  ``dtype=torch.float32`` they are ggml's exact fp32 values;
* the scalar C file ``sngguf_oracle.c`` (ggml ``dequantize_row_*`` loops with hand-written
  fp16/bf16 rounding), reached through ``COracle``.

Pinning (see tests/test_oracle_*.py): one-hot positional blocks, scale-packing cases, the
encode->decode round trip through the packers below (written from ggml's *quantize* side, not
from the decoders), hand-written known-answer blocks in tests/golden, C-vs-torch bitwise
agreement, and the fp16 chain of every type step by step against numpy float16 with an
alternative rounding placement shown to differ (tests/test_oracle_fp16_chain.py).  PARITY
UNPINNED: that the operation sequence restated here (``dtype=None``: every tensor op in fp16) is
the one the upstream package executes is taken from reading that package, which is neither in
the reference tree nor installed; no reference test or fixture covers it.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 2, 3, 6, 7, 8, 10, 11, 12, 13, 14
BF16 = 30
QK_K = 256
K_SCALE_SIZE = 12
# gguf.GGML_QUANT_SIZES: type -> (elements per block, bytes per block)
GGML_QUANT_SIZES = {Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q8_0: (32, 34),
                    Q2_K: (256, 84), Q3_K: (256, 110), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210), BF16: (1, 2)}
TYPE_NAMES = {Q4_0: "Q4_0", Q4_1: "Q4_1", Q5_0: "Q5_0", Q5_1: "Q5_1", Q8_0: "Q8_0", Q2_K: "Q2_K", Q3_K: "Q3_K",
              Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", BF16: "BF16"}

NUM_GGML_FP32 = 0
NUM_UPSTREAM_FP16 = 1


# --------------------------------------------------------------------------------------
# vectorised restatement (upstream op sequence)
# --------------------------------------------------------------------------------------

def split_block_dims(blocks: torch.Tensor, *args: int):
    """Split the byte columns of [n_blocks, type_size] into the struct members."""
    n_max = blocks.shape[1]
    dims = list(args) + [n_max - sum(args)]
    return torch.split(blocks, dims, dim=1)


def _to(t: torch.Tensor, dtype):
    # Tensor.to(None) is the identity in torch; spelled out so the fp16 path is visible.
    return t if dtype is None else t.to(dtype)


def dequantize_blocks_Q8_0(blocks, block_size, type_size, dtype=None):
    d, x = split_block_dims(blocks, 2)
    d = _to(d.contiguous().view(torch.float16), dtype)
    x = x.contiguous().view(torch.int8)
    return d * x


def to_uint32(x: torch.Tensor) -> torch.Tensor:
    """Four little-endian bytes per row -> one int32 column."""
    x = x.contiguous().view(torch.uint8).to(torch.int32)
    return (x[:, 0] | x[:, 1] << 8 | x[:, 2] << 16 | x[:, 3] << 24).unsqueeze(1)


def _nibbles(qs: torch.Tensor, n_blocks: int, block_size: int) -> torch.Tensor:
    """16 bytes -> 32 values: all low nibbles, then all high nibbles."""
    ql = qs.reshape((n_blocks, -1, 1, block_size // 2)) >> torch.tensor([0, 4], dtype=torch.uint8).reshape((1, 1, 2, 1))
    return (ql & 0x0F).reshape((n_blocks, -1))


def _fifth_bits(qh: torch.Tensor, n_blocks: int) -> torch.Tensor:
    qh = to_uint32(qh)
    qh = qh.reshape((n_blocks, 1)) >> torch.arange(32, dtype=torch.int32).reshape((1, 32))
    return (qh & 1).to(torch.uint8)


def dequantize_blocks_Q4_0(blocks, block_size, type_size, dtype=None):
    n_blocks = blocks.shape[0]
    d, qs = split_block_dims(blocks, 2)
    d = _to(d.contiguous().view(torch.float16), dtype)
    qs = _nibbles(qs, n_blocks, block_size).to(torch.int8) - 8
    return d * qs


def dequantize_blocks_Q4_1(blocks, block_size, type_size, dtype=None):
    n_blocks = blocks.shape[0]
    d, m, qs = split_block_dims(blocks, 2, 2)
    d = _to(d.contiguous().view(torch.float16), dtype)
    m = _to(m.contiguous().view(torch.float16), dtype)
    qs = _nibbles(qs, n_blocks, block_size)
    return (d * qs) + m


def dequantize_blocks_Q5_0(blocks, block_size, type_size, dtype=None):
    n_blocks = blocks.shape[0]
    d, qh, qs = split_block_dims(blocks, 2, 4)
    d = _to(d.contiguous().view(torch.float16), dtype)
    qs = (_nibbles(qs, n_blocks, block_size) | (_fifth_bits(qh, n_blocks) << 4)).to(torch.int8) - 16
    return d * qs


def dequantize_blocks_Q5_1(blocks, block_size, type_size, dtype=None):
    n_blocks = blocks.shape[0]
    d, m, qh, qs = split_block_dims(blocks, 2, 2, 4)
    d = _to(d.contiguous().view(torch.float16), dtype)
    m = _to(m.contiguous().view(torch.float16), dtype)
    qs = _nibbles(qs, n_blocks, block_size) | (_fifth_bits(qh, n_blocks) << 4)
    return (d * qs) + m


def dequantize_blocks_Q2_K(blocks, block_size, type_size, dtype=None):
    n_blocks = blocks.shape[0]
    scales, qs, d, dmin = split_block_dims(blocks, QK_K // 16, QK_K // 4, 2)
    d = _to(d.contiguous().view(torch.float16), dtype)
    dmin = _to(dmin.contiguous().view(torch.float16), dtype)
    dl = (d * (scales & 0xF)).reshape((n_blocks, QK_K // 16, 1))
    ml = (dmin * (scales >> 4)).reshape((n_blocks, QK_K // 16, 1))
    shift = torch.tensor([0, 2, 4, 6], dtype=torch.uint8).reshape((1, 1, 4, 1))
    qs = (qs.reshape((n_blocks, -1, 1, 32)) >> shift) & 3
    qs = qs.reshape((n_blocks, QK_K // 16, 16))
    qs = dl * qs - ml
    return qs.reshape((n_blocks, -1))


def dequantize_blocks_Q3_K(blocks, block_size, type_size, dtype=None):
    n_blocks = blocks.shape[0]
    hmask, qs, scales, d = split_block_dims(blocks, QK_K // 8, QK_K // 4, 12)
    d = _to(d.contiguous().view(torch.float16), dtype)
    lscales, hscales = scales[:, :8], scales[:, 8:]
    lscales = lscales.reshape((n_blocks, 1, 8)) >> torch.tensor([0, 4], dtype=torch.uint8).reshape((1, 2, 1))
    lscales = lscales.reshape((n_blocks, 16))
    hscales = hscales.reshape((n_blocks, 1, 4)) >> torch.tensor([0, 2, 4, 6], dtype=torch.uint8).reshape((1, 4, 1))
    hscales = hscales.reshape((n_blocks, 16))
    scales = (lscales & 0x0F) | ((hscales & 0x03) << 4)
    scales = scales.to(torch.int8) - 32
    dl = (d * scales).reshape((n_blocks, 16, 1))
    ql = qs.reshape((n_blocks, -1, 1, 32)) >> torch.tensor([0, 2, 4, 6], dtype=torch.uint8).reshape((1, 1, 4, 1))
    qh = hmask.reshape((n_blocks, -1, 1, 32)) >> torch.arange(8, dtype=torch.uint8).reshape((1, 1, 8, 1))
    ql = ql.reshape((n_blocks, 16, QK_K // 16)) & 3
    qh = (qh.reshape((n_blocks, 16, QK_K // 16)) & 1) ^ 1
    q = ql.to(torch.int8) - (qh << 2).to(torch.int8)
    return (dl * q).reshape((n_blocks, QK_K))


def get_scale_min(scales: torch.Tensor):
    """12 packed bytes per super-block -> eight 6-bit scales and eight 6-bit mins."""
    n_blocks = scales.shape[0]
    scales = scales.contiguous().view(torch.uint8).reshape((n_blocks, 3, 4))
    d, m, m_d = torch.split(scales, scales.shape[-2] // 3, dim=-2)
    sc = torch.cat([d & 0x3F, (m_d & 0x0F) | ((d >> 2) & 0x30)], dim=-1)
    mn = torch.cat([m & 0x3F, (m_d >> 4) | ((m >> 2) & 0x30)], dim=-1)
    return sc.reshape((n_blocks, 8)), mn.reshape((n_blocks, 8))


def dequantize_blocks_Q4_K(blocks, block_size, type_size, dtype=None):
    n_blocks = blocks.shape[0]
    d, dmin, scales, qs = split_block_dims(blocks, 2, 2, K_SCALE_SIZE)
    d = _to(d.contiguous().view(torch.float16), dtype)
    dmin = _to(dmin.contiguous().view(torch.float16), dtype)
    sc, m = get_scale_min(scales)
    d = (d * sc).reshape((n_blocks, -1, 1))
    dm = (dmin * m).reshape((n_blocks, -1, 1))
    shifts = torch.tensor([0, 4], dtype=torch.uint8).reshape((1, 1, 2, 1))
    qs = qs.reshape((n_blocks, -1, 1, 32)) >> shifts
    qs = (qs & 0x0F).reshape((n_blocks, -1, 32))
    return (d * qs - dm).reshape((n_blocks, QK_K))


def dequantize_blocks_Q5_K(blocks, block_size, type_size, dtype=None):
    n_blocks = blocks.shape[0]
    d, dmin, scales, qh, qs = split_block_dims(blocks, 2, 2, K_SCALE_SIZE, QK_K // 8)
    d = _to(d.contiguous().view(torch.float16), dtype)
    dmin = _to(dmin.contiguous().view(torch.float16), dtype)
    sc, m = get_scale_min(scales)
    d = (d * sc).reshape((n_blocks, -1, 1))
    dm = (dmin * m).reshape((n_blocks, -1, 1))
    ql = qs.reshape((n_blocks, -1, 1, 32)) >> torch.tensor([0, 4], dtype=torch.uint8).reshape((1, 1, 2, 1))
    qh = qh.reshape((n_blocks, -1, 1, 32)) >> torch.arange(8, dtype=torch.uint8).reshape((1, 1, 8, 1))
    ql = (ql & 0x0F).reshape((n_blocks, -1, 32))
    qh = (qh & 0x01).reshape((n_blocks, -1, 32))
    q = ql | (qh << 4)
    return (d * q - dm).reshape((n_blocks, QK_K))


def dequantize_blocks_Q6_K(blocks, block_size, type_size, dtype=None):
    n_blocks = blocks.shape[0]
    ql, qh, scales, d = split_block_dims(blocks, QK_K // 2, QK_K // 4, QK_K // 16)
    scales = _to(scales.contiguous().view(torch.int8), dtype)
    d = _to(d.contiguous().view(torch.float16), dtype)
    d = (d * scales).reshape((n_blocks, QK_K // 16, 1))
    ql = ql.reshape((n_blocks, -1, 1, 64)) >> torch.tensor([0, 4], dtype=torch.uint8).reshape((1, 1, 2, 1))
    ql = (ql & 0x0F).reshape((n_blocks, -1, 32))
    qh = qh.reshape((n_blocks, -1, 1, 32)) >> torch.tensor([0, 2, 4, 6], dtype=torch.uint8).reshape((1, 1, 4, 1))
    qh = (qh & 0x03).reshape((n_blocks, -1, 32))
    q = (ql | (qh << 4)).to(torch.int8) - 32
    q = q.reshape((n_blocks, QK_K // 16, -1))
    return (d * q).reshape((n_blocks, QK_K))


def dequantize_blocks_BF16(blocks, block_size, type_size, dtype=None):
    """bf16 bit patterns widened to fp32 (exact): the result is fp32 whatever ``dtype`` says, as upstream's is."""
    return (blocks.contiguous().view(torch.int16).to(torch.int32) << 16).view(torch.float32)


dequantize_functions = {BF16: dequantize_blocks_BF16, Q4_0: dequantize_blocks_Q4_0, Q4_1: dequantize_blocks_Q4_1, Q5_0: dequantize_blocks_Q5_0,
                        Q5_1: dequantize_blocks_Q5_1, Q8_0: dequantize_blocks_Q8_0, Q2_K: dequantize_blocks_Q2_K,
                        Q3_K: dequantize_blocks_Q3_K, Q4_K: dequantize_blocks_Q4_K, Q5_K: dequantize_blocks_Q5_K,
                        Q6_K: dequantize_blocks_Q6_K}


def dequantize_gguf_tensor(packed: torch.Tensor, quant_type: int, numerics: int = NUM_UPSTREAM_FP16) -> torch.Tensor:
    """uint8 [N, K/bs*ts] -> [N, K]; fp16 tensor (numerics 1, upstream) or fp32 (numerics 0)."""
    block_size, type_size = GGML_QUANT_SIZES[quant_type]
    packed = packed.detach().cpu().view(torch.uint8)
    shape = (*packed.shape[:-1], packed.shape[-1] // type_size * block_size)
    n_blocks = packed.numel() // type_size
    blocks = packed.reshape((n_blocks, type_size))
    dtype = None if numerics == NUM_UPSTREAM_FP16 else torch.float32
    return dequantize_functions[quant_type](blocks, block_size, type_size, dtype).reshape(shape)


def gguf_linear_forward(x: torch.Tensor, packed: torch.Tensor, quant_type: int, bias: torch.Tensor | None = None,
                        compute_dtype: torch.dtype = torch.bfloat16, numerics: int = NUM_UPSTREAM_FP16) -> torch.Tensor:
    """GGUFLinear.forward_native on the CPU: decode -> cast to compute dtype -> F.linear."""
    w = dequantize_gguf_tensor(packed, quant_type, numerics).to(compute_dtype)
    b = bias.detach().cpu().to(compute_dtype) if bias is not None else None
    return torch.nn.functional.linear(x.detach().cpu().to(compute_dtype), w, b)


def qwen3_rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """Qwen3RMSNorm.forward, op by op (src/sensenova_u1/models/neo_unify/modeling_qwen3.py:192-197): upcast to
    fp32, variance = mean of squares over the last dim, x * rsqrt(variance + eps), cast back to the input dtype,
    then the product with the weight in the input dtype.  Pinned in tests/test_oracle_rmsnorm.py against closed
    forms (constant rows, one-hot rows, scale invariance) and torch.nn.functional.rms_norm."""
    input_dtype = x.dtype
    h = x.to(torch.float32)
    variance = h.pow(2).mean(-1, keepdim=True)
    h = h * torch.rsqrt(variance + eps)
    return weight * h.to(input_dtype)


def mlp_forward(x, gate, up, down, quant_types, numerics=NUM_UPSTREAM_FP16):
    """Qwen3MLP.forward (modeling_qwen3.py:214-216): down(silu(gate(x)) * up(x)), each a GGUFLinear."""
    g = gguf_linear_forward(x, gate, quant_types[0], numerics=numerics)
    u = gguf_linear_forward(x, up, quant_types[1], numerics=numerics)
    h = torch.nn.functional.silu(g) * u
    return gguf_linear_forward(h, down, quant_types[2], numerics=numerics), h


def grouped_linear_forward(x, indicator, packed_und, qt_und, packed_gen, qt_gen, bias_und=None, bias_gen=None,
                           numerics=NUM_UPSTREAM_FP16):
    """Mixed routing as written (unreachable) at modeling_qwen3.py:779-783."""
    x = x.detach().cpu()
    ind = indicator.detach().cpu().bool()
    n_out = packed_und.shape[0]
    out = torch.zeros((x.shape[0], n_out), dtype=torch.bfloat16)
    if (~ind).any():
        out[~ind] = gguf_linear_forward(x[~ind], packed_und, qt_und, bias_und, numerics=numerics)
    if ind.any():
        out[ind] = gguf_linear_forward(x[ind], packed_gen, qt_gen, bias_gen, numerics=numerics)
    return out


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a = a.detach().cpu().double().flatten()
    b = b.detach().cpu().double().flatten()
    den = float(b.norm())
    return float((a - b).norm()) / (den if den > 0 else 1.0)


# --------------------------------------------------------------------------------------
# packers: the *encode* side of the formats, written from ggml's quantize_row_*_ref packing
# loops (numpy, one block at a time, no code shared with the decoders above)
# --------------------------------------------------------------------------------------

def _f16_bytes(v) -> bytes:
    return np.asarray(v, dtype=np.float16).tobytes()


def pack_q8_0(d, qs) -> bytes:
    """block_q8_0 {f16 d; int8 qs[32]}."""
    qs = np.asarray(qs, dtype=np.int8)
    assert qs.shape == (32,)
    return _f16_bytes(d) + qs.tobytes()


def _pack_nibbles_32(q) -> bytes:
    """ggml quantize_row_q4_0_ref packing: byte j holds element j (low) and element j + 16 (high)."""
    return bytes((q[j] & 0x0F) | ((q[j + 16] & 0x0F) << 4) for j in range(16))


def _pack_fifth_bits_32(q) -> bytes:
    """ggml quantize_row_q5_0_ref: bit j of the 32-bit qh is bit 4 of element j."""
    qh = 0
    for j in range(32):
        qh |= ((q[j] >> 4) & 1) << j
    return int(qh).to_bytes(4, "little")


def pack_q4_0(d, q) -> bytes:
    """block_q4_0 {f16 d; u8 qs[16]} from 32 signed quants (-8..7), stored with offset 8."""
    q = [int(v) + 8 for v in q]
    assert len(q) == 32 and all(0 <= v < 16 for v in q)
    return _f16_bytes(d) + _pack_nibbles_32(q)


def pack_q4_1(d, m, q) -> bytes:
    """block_q4_1 {f16 d; f16 m; u8 qs[16]} from 32 quants (0..15)."""
    q = [int(v) for v in q]
    assert len(q) == 32 and all(0 <= v < 16 for v in q)
    return _f16_bytes(d) + _f16_bytes(m) + _pack_nibbles_32(q)


def pack_q5_0(d, q) -> bytes:
    """block_q5_0 {f16 d; u8 qh[4]; u8 qs[16]} from 32 signed quants (-16..15), stored with offset 16."""
    q = [int(v) + 16 for v in q]
    assert len(q) == 32 and all(0 <= v < 32 for v in q)
    return _f16_bytes(d) + _pack_fifth_bits_32(q) + _pack_nibbles_32(q)


def pack_q5_1(d, m, q) -> bytes:
    """block_q5_1 {f16 d; f16 m; u8 qh[4]; u8 qs[16]} from 32 quants (0..31)."""
    q = [int(v) for v in q]
    assert len(q) == 32 and all(0 <= v < 32 for v in q)
    return _f16_bytes(d) + _f16_bytes(m) + _pack_fifth_bits_32(q) + _pack_nibbles_32(q)


def _pack_bit_pairs_256(q) -> bytes:
    """ggml quantize_row_q2_K_ref / q3_K packing of the two low bits: per 128 elements, byte l holds
    elements l, l + 32, l + 64, l + 96 at bits 0, 2, 4, 6."""
    out = []
    for j in range(0, 256, 128):
        for l in range(32):
            out.append((q[j + l] & 3) | ((q[j + l + 32] & 3) << 2) | ((q[j + l + 64] & 3) << 4) | ((q[j + l + 96] & 3) << 6))
    return bytes(out)


def pack_q2_k(d, dmin, sc, mn, q) -> bytes:
    """block_q2_K {u8 scales[16]; u8 qs[64]; f16 d, dmin} from 16 scales, 16 mins (0..15), 256 quants (0..3)."""
    sc = [int(v) for v in sc]
    mn = [int(v) for v in mn]
    q = [int(v) for v in q]
    assert len(sc) == 16 and len(mn) == 16 and len(q) == 256
    assert all(0 <= v < 16 for v in sc + mn) and all(0 <= v < 4 for v in q)
    scales = bytes(sc[j] | (mn[j] << 4) for j in range(16))
    return scales + _pack_bit_pairs_256(q) + _f16_bytes(d) + _f16_bytes(dmin)


def pack_q3_k(d, sc, q) -> bytes:
    """block_q3_K {u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d} from 16 signed scales (-32..31) and 256
    signed quants (-4..3); stored as ggml's quantize_row_q3_K_ref does: scale + 32 split 4 + 2 bits, quant + 4
    with bit 2 in hmask and bits 0..1 in qs."""
    sc = [int(v) + 32 for v in sc]
    q = [int(v) + 4 for v in q]
    assert len(sc) == 16 and len(q) == 256
    assert all(0 <= v < 64 for v in sc) and all(0 <= v < 8 for v in q)
    scales = [0] * 12
    for j in range(16):
        l = sc[j]
        if j < 8:
            scales[j] = l & 0xF
        else:
            scales[j - 8] |= (l & 0xF) << 4
        scales[8 + j % 4] |= (l >> 4) << (2 * (j // 4))
    hmask = [0] * 32
    m, hm = 0, 1
    for j in range(256):
        if q[j] > 3:
            hmask[m] |= hm
        m += 1
        if m == 32:
            m, hm = 0, hm << 1
    return bytes(hmask) + _pack_bit_pairs_256([v & 3 for v in q]) + bytes(scales) + _f16_bytes(d)


def pack_q4_k(d, dmin, sc, mn, q) -> bytes:
    """block_q4_K {f16 d, dmin; u8 scales[12]; u8 qs[128]} from 8 scales, 8 mins (0..63), 256 quants (0..15)."""
    sc = [int(v) for v in sc]
    mn = [int(v) for v in mn]
    q = [int(v) for v in q]
    assert len(sc) == 8 and len(mn) == 8 and len(q) == 256
    assert all(0 <= v < 64 for v in sc + mn) and all(0 <= v < 16 for v in q)
    scales = [0] * 12
    for j in range(8):
        ls, lm = sc[j], mn[j]
        if j < 4:
            scales[j] = ls
            scales[j + 4] = lm
        else:
            scales[j + 4] = (ls & 0xF) | ((lm & 0xF) << 4)
            scales[j - 4] |= (ls >> 4) << 6
            scales[j] |= (lm >> 4) << 6
    qs = []
    for j in range(0, 256, 64):
        for l in range(32):
            qs.append(q[j + l] | (q[j + l + 32] << 4))
    return _f16_bytes(d) + _f16_bytes(dmin) + bytes(scales) + bytes(qs)


def pack_q5_k(d, dmin, sc, mn, q) -> bytes:
    """block_q5_K {f16 d, dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]} from 8 scales, 8 mins (0..63), 256 quants (0..31)."""
    q = [int(v) for v in q]
    assert len(q) == 256 and all(0 <= v < 32 for v in q)
    low = pack_q4_k(d, dmin, sc, mn, [v & 0x0F for v in q])   # same head, scale packing and nibble order
    qh = [0] * 32
    for j in range(8):
        for l in range(32):
            qh[l] |= (q[32 * j + l] >> 4) << j
    return low[:16] + bytes(qh) + low[16:]


def pack_q6_k(d, scales, q) -> bytes:
    """block_q6_K {u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d} from 16 int8 scales and 256 quants (0..63)."""
    scales = np.asarray(scales, dtype=np.int8)
    q = [int(v) for v in q]
    assert scales.shape == (16,) and len(q) == 256 and all(0 <= v < 64 for v in q)
    ql = [0] * 128
    qh = [0] * 64
    for j in range(0, 256, 128):
        for l in range(32):
            q1, q2, q3, q4 = q[j + l] & 0xF, q[j + l + 32] & 0xF, q[j + l + 64] & 0xF, q[j + l + 96] & 0xF
            ql[j // 2 + l] = q1 | (q3 << 4)
            ql[j // 2 + l + 32] = q2 | (q4 << 4)
            qh[j // 4 + l] = ((q[j + l] >> 4) | ((q[j + l + 32] >> 4) << 2) | ((q[j + l + 64] >> 4) << 4)
                              | ((q[j + l + 96] >> 4) << 6))
    return bytes(ql) + bytes(qh) + scales.tobytes() + _f16_bytes(d)


def quantize_q8_0(w: np.ndarray) -> np.ndarray:
    """ggml quantize_row_q8_0_ref over the last axis: d = amax/127, q = round-half-away(x/d)."""
    w = np.asarray(w, dtype=np.float32)
    assert w.shape[-1] % 32 == 0
    blk = w.reshape(*w.shape[:-1], -1, 32)
    amax = np.abs(blk).max(axis=-1, keepdims=True)
    d = (amax / np.float32(127.0)).astype(np.float32)
    inv = np.where(d > 0, np.float32(1.0) / np.where(d > 0, d, 1), np.float32(0)).astype(np.float32)
    x = blk * inv
    q = np.where(x >= 0, np.floor(x + np.float32(0.5)), np.ceil(x - np.float32(0.5))).astype(np.int8)
    out = np.empty((*blk.shape[:-1], 34), dtype=np.uint8)
    out[..., :2] = d.astype(np.float16).view(np.uint8).reshape(*blk.shape[:-1], 2)
    out[..., 2:] = q.view(np.uint8)
    return out.reshape(*w.shape[:-1], -1)


# --------------------------------------------------------------------------------------
# C oracle
# --------------------------------------------------------------------------------------

_HERE = os.path.dirname(os.path.abspath(__file__))
_C_LIB = os.path.join(_HERE, "libsngguf_oracle.so")


def build_c_oracle(force: bool = False) -> str:
    src = os.path.join(_HERE, "sngguf_oracle.c")
    if force or not os.path.exists(_C_LIB) or os.path.getmtime(_C_LIB) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE, "-B", "libsngguf_oracle.so"], check=True, capture_output=True)
    return _C_LIB


class COracle:
    """ctypes view of sngguf_oracle.c."""

    def __init__(self):
        self.lib = ctypes.CDLL(build_c_oracle())
        L = self.lib
        vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        L.sno_dequantize.argtypes = [vp, ci, i64, i64, vp, ci, ci, vp]
        L.sno_dequantize.restype = ci
        L.sno_linear.argtypes = [vp, i64, vp, ci, i64, i64, vp, vp, ci, vp]
        L.sno_linear.restype = ci
        L.sno_grouped_linear.argtypes = [vp, i64, vp, vp, ci, vp, ci, i64, i64, vp, vp, vp, ci, vp]
        L.sno_grouped_linear.restype = ci
        L.sno_silu_mul.argtypes = [vp, vp, vp, i64]
        L.sno_silu_mul.restype = None
        L.sno_f32_to_f16.argtypes = [ctypes.c_float]
        L.sno_f32_to_f16.restype = ctypes.c_uint16
        L.sno_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.sno_f16_to_f32.restype = ctypes.c_float
        L.sno_f32_to_bf16.argtypes = [ctypes.c_float]
        L.sno_f32_to_bf16.restype = ctypes.c_uint16

    @staticmethod
    def _ptr(t: torch.Tensor | None):
        return None if t is None else ctypes.c_void_p(t.data_ptr())

    def dequantize(self, packed: torch.Tensor, quant_type: int, out_dtype: torch.dtype = torch.float32,
                   numerics: int = NUM_GGML_FP32) -> torch.Tensor:
        bs, ts = GGML_QUANT_SIZES[quant_type]
        packed = packed.detach().cpu().contiguous().view(torch.uint8)
        rows = packed.numel() // packed.shape[-1]
        cols = packed.shape[-1] // ts * bs
        out = torch.empty((rows, cols), dtype=out_dtype)
        scratch = torch.empty(cols, dtype=torch.float32)
        code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[out_dtype]
        rc = self.lib.sno_dequantize(self._ptr(packed), quant_type, rows, cols, self._ptr(out), code, numerics,
                                     self._ptr(scratch))
        if rc:
            raise RuntimeError(f"sno_dequantize failed: {rc}")
        return out.reshape(*packed.shape[:-1], cols)

    def linear(self, x: torch.Tensor, packed: torch.Tensor, quant_type: int, bias: torch.Tensor | None = None,
               numerics: int = NUM_UPSTREAM_FP16) -> torch.Tensor:
        bs, ts = GGML_QUANT_SIZES[quant_type]
        x = x.detach().cpu().to(torch.bfloat16).contiguous()
        packed = packed.detach().cpu().contiguous().view(torch.uint8)
        n, k = packed.shape[0], packed.shape[1] // ts * bs
        m = x.numel() // k
        y = torch.empty((m, n), dtype=torch.bfloat16)
        b = bias.detach().cpu().to(torch.bfloat16).contiguous() if bias is not None else None
        scratch = torch.empty(k, dtype=torch.float32)
        rc = self.lib.sno_linear(self._ptr(x), m, self._ptr(packed), quant_type, n, k, self._ptr(b), self._ptr(y),
                                 numerics, self._ptr(scratch))
        if rc:
            raise RuntimeError(f"sno_linear failed: {rc}")
        return y.reshape(*x.shape[:-1], n)

    def grouped_linear(self, x, indicator, packed_und, qt_und, packed_gen, qt_gen, bias_und=None, bias_gen=None,
                       numerics: int = NUM_UPSTREAM_FP16) -> torch.Tensor:
        bs, ts = GGML_QUANT_SIZES[qt_und]
        x = x.detach().cpu().to(torch.bfloat16).contiguous()
        ind = indicator.detach().cpu().to(torch.uint8).contiguous()
        pu = packed_und.detach().cpu().contiguous().view(torch.uint8)
        pg = packed_gen.detach().cpu().contiguous().view(torch.uint8)
        n, k = pu.shape[0], pu.shape[1] // ts * bs
        m = x.shape[0]
        y = torch.empty((m, n), dtype=torch.bfloat16)
        bu = bias_und.detach().cpu().to(torch.bfloat16).contiguous() if bias_und is not None else None
        bg = bias_gen.detach().cpu().to(torch.bfloat16).contiguous() if bias_gen is not None else None
        scratch = torch.empty(k, dtype=torch.float32)
        rc = self.lib.sno_grouped_linear(self._ptr(x), m, self._ptr(ind), self._ptr(pu), qt_und, self._ptr(pg),
                                         qt_gen, n, k, self._ptr(bu), self._ptr(bg), self._ptr(y), numerics,
                                         self._ptr(scratch))
        if rc:
            raise RuntimeError(f"sno_grouped_linear failed: {rc}")
        return y

    def silu_mul(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        gate = gate.detach().cpu().to(torch.bfloat16).contiguous()
        up = up.detach().cpu().to(torch.bfloat16).contiguous()
        h = torch.empty_like(gate)
        self.lib.sno_silu_mul(self._ptr(gate), self._ptr(up), self._ptr(h), gate.numel())
        return h
