"""GPU parity: standalone dequantize op vs the CPU oracle, bit for bit."""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import ops, synthetic

pytestmark = pytest.mark.gpu

TYPES = [go.Q4_0, go.Q4_1, go.Q5_0, go.Q5_1, go.Q8_0, go.Q2_K, go.Q3_K, go.Q4_K, go.Q5_K, go.Q6_K]


def _bits(t):
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


@pytest.mark.parametrize("qt", TYPES)
@pytest.mark.parametrize("numerics", [0, 1])
def test_dequantize_bit_exact_fp32(dev, c_oracle, qt, numerics):
    print(f"case dequantize fp32 qt={qt} numerics={numerics}", flush=True)
    packed = synthetic.make_packed(qt, 96, 2048, seed=3 + qt)
    want = c_oracle.dequantize(packed, qt, torch.float32, numerics)
    got = ops.dequantize(packed.to(dev), qt, torch.float32, numerics).cpu()
    assert got.shape == want.shape
    assert torch.equal(_bits(got), _bits(want))
    # the vectorised restatement says the same
    want2 = go.dequantize_gguf_tensor(packed, qt, numerics).float()
    assert torch.equal(_bits(got), _bits(want2))


@pytest.mark.parametrize("qt", TYPES)
@pytest.mark.parametrize("numerics", [0, 1])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16])
def test_dequantize_bit_exact_narrow(dev, c_oracle, qt, numerics, out_dtype):
    print(f"case dequantize {out_dtype} qt={qt} numerics={numerics}", flush=True)
    packed = synthetic.make_packed(qt, 33, 1024, seed=11 + qt)
    want = c_oracle.dequantize(packed, qt, out_dtype, numerics)
    got = ops.dequantize(packed.to(dev), qt, out_dtype, numerics).cpu()
    assert torch.equal(_bits(got), _bits(want))
    if numerics == 1 and out_dtype == torch.float16:
        # this is the tensor upstream's dequantize_gguf_tensor returns
        assert torch.equal(_bits(got), _bits(go.dequantize_gguf_tensor(packed, qt, 1)))
    if numerics == 1 and out_dtype == torch.bfloat16:
        assert torch.equal(_bits(got), _bits(go.dequantize_gguf_tensor(packed, qt, 1).to(torch.bfloat16)))


@pytest.mark.parametrize("qt", TYPES)
def test_dequantize_random_bytes_extremes(dev, c_oracle, qt):
    """Uniformly random bytes: every nibble / high-bit / sign combination, scales of any
    magnitude (inf / nan scale bit patterns are replaced: nan payloads are not compared)."""
    print(f"case dequantize random bytes qt={qt}", flush=True)
    bs, ts = go.GGML_QUANT_SIZES[qt]
    g = torch.Generator().manual_seed(99 + qt)
    packed = torch.randint(0, 256, (64, 1024 // bs * ts), dtype=torch.uint8, generator=g)
    blocks = packed.view(-1, ts)
    for off in {go.Q4_0: [0], go.Q4_1: [0, 2], go.Q5_0: [0], go.Q5_1: [0, 2], go.Q8_0: [0], go.Q2_K: [80, 82], go.Q3_K: [108],
                go.Q4_K: [0, 2], go.Q5_K: [0, 2], go.Q6_K: [208]}[qt]:
        h = blocks[:, off:off + 2].contiguous().view(torch.int16)
        bad = (h & 0x7C00) == 0x7C00
        h[bad] = h[bad] & ~0x4000  # clear one exponent bit: finite, keeps sign and mantissa
        blocks[:, off:off + 2] = h.view(torch.uint8)
    for numerics in (0, 1):
        want = c_oracle.dequantize(packed, qt, torch.float32, numerics)
        got = ops.dequantize(packed.to(dev), qt, torch.float32, numerics).cpu()
        both_nan = got.isnan() & want.isnan()
        assert torch.equal(_bits(got)[~both_nan], _bits(want)[~both_nan])


def test_dequantize_full_size_matches_row_sample(dev, c_oracle):
    """12288 x 4096 Q8_0 (the MLP gate shape): sample rows against the oracle."""
    print("case dequantize full size", flush=True)
    packed = synthetic.make_packed(go.Q8_0, 12288, 4096, seed=5, device=dev)
    got = ops.dequantize(packed, go.Q8_0, torch.float32, 0)
    rows = torch.tensor([0, 1, 4095, 7777, 12287])
    want = c_oracle.dequantize(packed[rows.to(dev)].cpu(), go.Q8_0, torch.float32, 0)
    assert torch.equal(_bits(got[rows.to(dev)].cpu()), _bits(want))


def test_dequantize_empty_and_errors(dev):
    out = ops.dequantize(torch.empty((0, 34), dtype=torch.uint8, device=dev), go.Q8_0, torch.float32, 0)
    assert out.shape == (0, 32)
    with pytest.raises(ops.SnGgufError):
        ops.dequantize(torch.zeros((2, 35), dtype=torch.uint8, device=dev), go.Q8_0, torch.float32, 0)
    with pytest.raises(ops.SnGgufError):
        ops.dequantize(torch.zeros((2, 34), dtype=torch.uint8, device=dev), 13, torch.float32, 0)
    with pytest.raises(ops.SnGgufError):
        ops.dequantize(torch.zeros((2, 34), dtype=torch.uint8), go.Q8_0, torch.float32, 0)  # CPU tensor
