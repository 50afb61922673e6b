"""Seeded synthetic GGUF blocks and activations with the distributions the benchmark
configurations name.  Works on any torch device, so full-size weights can be generated directly
in HBM.

* Q8_0: int8 quants uniform in [-127, 127], ``d = fp16(|N(0, 0.02)| / 127)``.
* Q4_K: 4-bit quants uniform (all 128 quant bytes uniform), the 12 scale bytes uniform (so the
  eight 6-bit scales and mins are uniform over 0..63), ``d, dmin = fp16(|N(0, 0.01)|)``.
* Q5_K: as Q4_K, with the 32 high-bit bytes uniform as well.
* Q4_0 / Q4_1 / Q5_0 / Q5_1: quant and high-bit bytes uniform, ``d = fp16(|N(0, 0.01)|)``,
  ``m = fp16(N(0, 0.01))`` for the two formats that carry a block minimum.
* Q2_K: scale and quant bytes uniform, ``d, dmin = fp16(|N(0, 0.01)|)``.
* Q3_K: mask, quant and scale bytes uniform, ``d = fp16(|N(0, 0.01)|)``.
* Q6_K: 6-bit quants uniform (ql, qh bytes uniform), int8 sub-scales uniform over the signed
  6-bit range [-32, 31], ``d = fp16(|N(0, 0.01)|)``.
* BF16 (plain rows): bf16(N(0, 0.02)).
* activations: bf16 N(0, 1).
"""
from __future__ import annotations

import torch

from .ops import BF16, GGML_QUANT_SIZES, Q2_K, Q3_K, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0


def _gen(seed: int, device) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def _f16_bytes(v: torch.Tensor) -> torch.Tensor:
    return v.to(torch.float16).contiguous().view(torch.uint8).reshape(*v.shape, 2)


def make_packed(quant_type: int, n: int, k: int, seed: int = 0, device="cpu") -> torch.Tensor:
    """uint8 ``[n, k / block * type_size]`` of random blocks of ``quant_type``."""
    bs, ts = GGML_QUANT_SIZES[quant_type]
    if k % bs:
        raise ValueError(f"k={k} is not a multiple of the block size {bs}")
    g = _gen(seed, device)
    if quant_type == BF16:
        w = torch.randn((n, k), generator=g, device=device, dtype=torch.float32) * 0.02
        return w.to(torch.bfloat16).view(torch.uint8).reshape(n, 2 * k)
    nb = k // bs
    blocks = torch.empty((n, nb, ts), dtype=torch.uint8, device=device)

    def absnormal(std):
        return torch.randn((n, nb), generator=g, device=device, dtype=torch.float32).abs() * std

    def uniform_bytes(count):
        return torch.randint(0, 256, (n, nb, count), generator=g, device=device, dtype=torch.int16).to(torch.uint8)

    if quant_type in (Q4_0, Q5_0):
        blocks[..., 0:2] = _f16_bytes(absnormal(0.01))
        blocks[..., 2:] = uniform_bytes(ts - 2)
    elif quant_type in (Q4_1, Q5_1):
        blocks[..., 0:2] = _f16_bytes(absnormal(0.01))
        blocks[..., 2:4] = _f16_bytes(torch.randn((n, nb), generator=g, device=device, dtype=torch.float32) * 0.01)
        blocks[..., 4:] = uniform_bytes(ts - 4)
    elif quant_type == Q2_K:
        blocks[..., 0:80] = uniform_bytes(80)
        blocks[..., 80:82] = _f16_bytes(absnormal(0.01))
        blocks[..., 82:84] = _f16_bytes(absnormal(0.01))
    elif quant_type == Q3_K:
        blocks[..., 0:108] = uniform_bytes(108)
        blocks[..., 108:110] = _f16_bytes(absnormal(0.01))
    elif quant_type == Q8_0:
        blocks[..., 0:2] = _f16_bytes(absnormal(0.02) / 127.0)
        q = torch.randint(-127, 128, (n, nb, 32), generator=g, device=device, dtype=torch.int16)
        blocks[..., 2:] = q.to(torch.int8).view(torch.uint8)
    elif quant_type == Q4_K:
        blocks[..., 0:2] = _f16_bytes(absnormal(0.01))
        blocks[..., 2:4] = _f16_bytes(absnormal(0.01))
        blocks[..., 4:] = torch.randint(0, 256, (n, nb, 140), generator=g, device=device, dtype=torch.int16).to(torch.uint8)
    elif quant_type == Q5_K:
        blocks[..., 0:2] = _f16_bytes(absnormal(0.01))
        blocks[..., 2:4] = _f16_bytes(absnormal(0.01))
        blocks[..., 4:] = torch.randint(0, 256, (n, nb, 172), generator=g, device=device, dtype=torch.int16).to(torch.uint8)
    elif quant_type == Q6_K:
        blocks[..., 0:192] = torch.randint(0, 256, (n, nb, 192), generator=g, device=device, dtype=torch.int16).to(torch.uint8)
        sc = torch.randint(-32, 32, (n, nb, 16), generator=g, device=device, dtype=torch.int16)
        blocks[..., 192:208] = sc.to(torch.int8).view(torch.uint8)
        blocks[..., 208:210] = _f16_bytes(absnormal(0.01))
    else:
        raise ValueError(f"no synthetic generator for quant type {quant_type}")
    return blocks.reshape(n, nb * ts)


def make_activations(m: int, k: int, seed: int = 1, device="cpu") -> torch.Tensor:
    g = _gen(seed, device)
    return torch.randn((m, k), generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
