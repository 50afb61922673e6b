"""The fp16 rounding chain (numerics 1) of every format, step by step with numpy float16.

Each format's upstream decode is a short sequence of tensor operations on fp16 tensors, each of
which rounds its result to fp16 once (the published diffusers 0.37 ``dequantize_blocks_*`` with
``dtype=None``).  The chains are restated here from the struct members the block was packed from
- the packers are written from ggml's quantize side and share no code with the decoders - using
numpy's float16, an implementation of IEEE half that is neither torch's nor the C file's, and are
compared bit for bit with both restatements of the oracle on random blocks.  For every format
whose chain has more than one rounding the test also evaluates the chain with an operation
order or rounding placement that a reader of the upstream code could plausibly pick instead and
asserts that it gives different bits on the same blocks: the check can tell the placements apart.

This pins the oracle's arithmetic to the published operation sequence; that the absent upstream
package really follows that sequence stays unverifiable here.
"""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as go

f16 = np.float16
N_BLOCKS = 96


def R(v):
    """One tensor-op rounding: the exact result (held in float64) rounded to half, nearest-even."""
    return np.asarray(v, dtype=np.float64).astype(f16)


def mul(a, b):
    # fp16 x (fp16 | small integer) is exact in float64
    return R(np.asarray(a, dtype=np.float64) * np.asarray(b, dtype=np.float64))


def sub(a, b):
    return R(np.asarray(a, dtype=np.float64) - np.asarray(b, dtype=np.float64))


def add(a, b):
    return R(np.asarray(a, dtype=np.float64) + np.asarray(b, dtype=np.float64))


def _rand_scale(rng, sigma):
    # a positive fp16 scale with a full mantissa; now and then tiny, so that products go subnormal
    v = abs(rng.normal(0.0, sigma)) + 1e-7
    if rng.random() < 0.15:
        v *= 2.0 ** -rng.integers(4, 12)
    return f16(v)


def _decode_both(c_oracle, raw: bytes, qt: int):
    packed = torch.frombuffer(bytearray(raw), dtype=torch.uint8).reshape(1, -1)
    t = go.dequantize_gguf_tensor(packed, qt, go.NUM_UPSTREAM_FP16)
    assert t.dtype == torch.float16
    c = c_oracle.dequantize(packed, qt, torch.float16, go.NUM_UPSTREAM_FP16)
    assert torch.equal(t.view(torch.int16), c.view(torch.int16)), "C and torch restatements disagree"
    return t.numpy().reshape(-1)


def _bits(a):
    return np.asarray(a, dtype=f16).view(np.uint16)


def _run(c_oracle, qt, make_block, seed):
    """make_block(rng) -> (raw bytes, chain values, alternative-placement values or None)."""
    rng = np.random.default_rng(seed)
    differs = 0
    any_alt = False
    for _ in range(N_BLOCKS):
        raw, want, alt = make_block(rng)
        got = _decode_both(c_oracle, raw, qt)
        assert np.array_equal(_bits(got), _bits(want)), f"{go.TYPE_NAMES[qt]}: fp16 chain differs from the numpy restatement"
        if alt is not None:
            any_alt = True
            differs += int(np.count_nonzero(_bits(alt) != _bits(want)))
    if any_alt:
        assert differs > 0, f"{go.TYPE_NAMES[qt]}: the alternative rounding placement gives the same bits; the test pins nothing"


def test_q8_0_chain(c_oracle):
    # w = R(d * q): a single tensor op, so there is no placement to tell apart
    def make(rng):
        d, q = _rand_scale(rng, 0.02 / 127), rng.integers(-127, 128, 32)
        return go.pack_q8_0(d, q), mul(d, q), None
    _run(c_oracle, go.Q8_0, make, 11)
    # the rounding matters: some products of an 11-bit scale and a 7-bit quant need more than 11 bits
    d, q = f16(0.000123), np.arange(-127, 128)
    assert np.any(mul(d, q).astype(np.float64) != np.float64(d) * q)


@pytest.mark.parametrize("qt,offset,hi", [(go.Q4_0, 8, 16), (go.Q5_0, 16, 32)])
def test_q4_0_q5_0_chain(c_oracle, qt, offset, hi):
    # w = R(d * (q - offset)) with the offset taken in integers before the product
    pack = go.pack_q4_0 if qt == go.Q4_0 else go.pack_q5_0

    def make(rng):
        d, q = _rand_scale(rng, 0.01), rng.integers(-offset, hi - offset, 32)
        # alternative: R(R(d * u) - R(d * offset)) with the stored unsigned quant u
        alt = sub(mul(d, q + offset), mul(d, offset))
        return pack(d, q), mul(d, q), alt
    _run(c_oracle, qt, make, 12 + qt)


@pytest.mark.parametrize("qt,hi", [(go.Q4_1, 16), (go.Q5_1, 32)])
def test_q4_1_q5_1_chain(c_oracle, qt, hi):
    # w = R(R(d * q) + m): the product and the sum are separate tensor ops
    pack = go.pack_q4_1 if qt == go.Q4_1 else go.pack_q5_1

    def make(rng):
        d, m, q = _rand_scale(rng, 0.01), f16(rng.normal(0.0, 0.05)), rng.integers(0, hi, 32)
        alt = R(np.float64(d) * q + np.float64(m))   # one fused rounding
        return pack(d, m, q), add(mul(d, q), m), alt
    _run(c_oracle, qt, make, 20 + qt)


def test_q2_k_chain(c_oracle):
    # dl = R(d * sc), ml = R(dmin * mn) per 16 elements; w = R(R(dl * q) - ml)
    def make(rng):
        d, dmin = _rand_scale(rng, 0.01), _rand_scale(rng, 0.01)
        sc, mn, q = rng.integers(0, 16, 16), rng.integers(0, 16, 16), rng.integers(0, 4, 256)
        dl, ml = mul(d, sc).repeat(16), mul(dmin, mn).repeat(16)
        want = sub(mul(dl, q), ml)
        alt = sub(mul(d, sc.repeat(16) * q), ml)      # scale and quant multiplied as integers first
        return go.pack_q2_k(d, dmin, sc, mn, q), want, alt
    _run(c_oracle, go.Q2_K, make, 31)


def test_q3_k_chain(c_oracle):
    # dl = R(d * (scale - 32)) per 16 elements; w = R(dl * q), q in -4..3
    def make(rng):
        d = _rand_scale(rng, 0.01)
        sc, q = rng.integers(-32, 32, 16), rng.integers(-4, 4, 256)
        want = mul(mul(d, sc).repeat(16), q)
        alt = mul(d, sc.repeat(16) * q)
        return go.pack_q3_k(d, sc, q), want, alt
    _run(c_oracle, go.Q3_K, make, 32)


@pytest.mark.parametrize("qt,hi", [(go.Q4_K, 16), (go.Q5_K, 32)])
def test_q4_k_q5_k_chain(c_oracle, qt, hi):
    # D = R(d * sc), DM = R(dmin * mn) per 32 elements; w = R(R(D * q) - DM)
    pack = go.pack_q4_k if qt == go.Q4_K else go.pack_q5_k

    def make(rng):
        d, dmin = _rand_scale(rng, 0.01), _rand_scale(rng, 0.01)
        sc, mn, q = rng.integers(0, 64, 8), rng.integers(0, 64, 8), rng.integers(0, hi, 256)
        D, DM = mul(d, sc).repeat(32), mul(dmin, mn).repeat(32)
        want = sub(mul(D, q), DM)
        alt = R(D.astype(np.float64) * q - DM.astype(np.float64))   # product and difference fused into one rounding
        return pack(d, dmin, sc, mn, q), want, alt
    _run(c_oracle, qt, make, 40 + qt)


def test_q4_k_scale_rounding_is_separate(c_oracle):
    # a second alternative for Q4_K: the sub-block scale left unrounded, w = R(R(d * sc * q) - DM)
    def make(rng):
        d, dmin = _rand_scale(rng, 0.01), _rand_scale(rng, 0.01)
        sc, mn, q = rng.integers(0, 64, 8), rng.integers(0, 64, 8), rng.integers(0, 16, 256)
        D, DM = mul(d, sc).repeat(32), mul(dmin, mn).repeat(32)
        alt = sub(mul(d, sc.repeat(32) * q), DM)
        return go.pack_q4_k(d, dmin, sc, mn, q), sub(mul(D, q), DM), alt
    _run(c_oracle, go.Q4_K, make, 55)


def test_q6_k_chain(c_oracle):
    # D = R(d * scale) per 16 elements (int8 scale, exact as fp16); w = R(D * (q - 32))
    def make(rng):
        d = _rand_scale(rng, 0.01)
        sc, q = rng.integers(-128, 128, 16), rng.integers(0, 64, 256)
        want = mul(mul(d, sc).repeat(16), q - 32)
        alt = mul(d, sc.repeat(16) * (q - 32))        # one rounding of d * scale * q
        return go.pack_q6_k(d, sc, q), want, alt
    _run(c_oracle, go.Q6_K, make, 60)


def test_q6_k_offset_is_taken_in_integers(c_oracle):
    # the -32 is applied to the int8 quant before it meets the scale, not as R(R(D * q) - R(D * 32))
    def make(rng):
        d = _rand_scale(rng, 0.01)
        sc, q = rng.integers(-128, 128, 16), rng.integers(0, 64, 256)
        D = mul(d, sc).repeat(16)
        return go.pack_q6_k(d, sc, q), mul(D, q - 32), sub(mul(D, q), mul(D, 32))
    _run(c_oracle, go.Q6_K, make, 61)


@pytest.mark.parametrize("qt", [go.Q8_0, go.Q4_K, go.Q6_K])
def test_chain_then_bf16_is_what_the_linear_contracts(c_oracle, qt):
    """``GGUFLinear.forward_native`` casts the fp16 tensor to the compute dtype: a second rounding, fp16 -> bf16,
    nearest-even.  Checked against an integer restatement of that rounding on the oracle's own fp16 output."""
    from sensenova_u1_amd import synthetic
    packed = synthetic.make_packed(qt, 8, 1024, seed=3)
    h = go.dequantize_gguf_tensor(packed, qt, go.NUM_UPSTREAM_FP16)
    got = h.to(torch.bfloat16).view(torch.int16).numpy().astype(np.uint16).reshape(-1)
    bits = h.float().numpy().reshape(-1).view(np.uint32).astype(np.uint64)   # fp16 -> fp32 is exact
    want = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(got, want)
    # and the weights the C oracle's linear contracts are those bf16 values
    c = c_oracle.dequantize(packed, qt, torch.bfloat16, go.NUM_UPSTREAM_FP16)
    assert np.array_equal(c.view(torch.int16).numpy().astype(np.uint16).reshape(-1), want)
