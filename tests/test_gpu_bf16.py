"""GPU parity for GGUF tensors of type BF16 (ggml type 30): plain bfloat16 rows that upstream wraps and decodes like a
quantized type.  The decode is exact, so dequantize is bit-exact in every output type and both numerics modes."""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import GGUFLinear, GGUFParameter, grouped_linear, ops, synthetic

pytestmark = pytest.mark.gpu
TOL = 1e-3


def test_dequantize_bf16_rows_bit_exact(dev, c_oracle):
    print("case bf16 dequantize", flush=True)
    for n, k in [(7, 33), (64, 4096), (3, 1)]:
        packed = synthetic.make_packed(go.BF16, n, k, seed=n + k)
        # include values fp16 cannot hold, and signed zeros
        vals = packed.view(torch.bfloat16).clone()
        vals.view(-1)[0] = 1e30
        vals.view(-1)[-1] = -0.0
        packed = vals.view(torch.uint8).reshape(n, 2 * k)
        for numerics in (0, 1):
            for dt in (torch.float32, torch.float16, torch.bfloat16):
                got = ops.dequantize(packed.to(dev), go.BF16, dt, numerics).cpu()
                want = c_oracle.dequantize(packed, go.BF16, dt, numerics)
                assert got.shape == (n, k)
                iv = torch.int32 if dt == torch.float32 else torch.int16
                assert torch.equal(got.view(iv), want.view(iv)), (n, k, numerics, dt)
        assert torch.equal(ops.dequantize(packed.to(dev), go.BF16, torch.float32, 1).cpu(), go.dequantize_gguf_tensor(packed, go.BF16, 1))


@pytest.mark.parametrize("m,n,k", [(1, 130, 4096), (5, 37, 520), (16, 64, 100), (3, 9, 7), (40, 200, 512), (300, 515, 1024),
                                   (33, 50, 72), (2048, 1024, 256)])
def test_linear_bf16_rows(dev, m, n, k):
    """Decode-sized kernel (vector and single-element form), 16-row chunks for ragged K, the dense tile kernel from 17
    rows on when K is a multiple of 64; bias and residual."""
    print(f"case bf16 linear {m}x{n}x{k}", flush=True)
    packed = synthetic.make_packed(go.BF16, n, k, seed=m + n)
    x = synthetic.make_activations(m, k, seed=k)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.bfloat16)
    res = synthetic.make_activations(m, n, seed=n)
    xd, pd = x.to(dev), packed.to(dev)
    for b in (None, bias):
        want = go.gguf_linear_forward(x, packed, go.BF16, b)
        got = ops.linear(xd, pd, go.BF16, b.to(dev) if b is not None else None)
        assert go.rel_l2(got.cpu(), want) <= TOL
        got_r = ops.linear_residual(xd, pd, go.BF16, res.to(dev), b.to(dev) if b is not None else None)
        assert torch.equal(got_r, res.to(dev) + got)
    ws = torch.empty(ops.linear_workspace_bytes(n, k), dtype=torch.uint8, device=dev)
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.linear_ws_into(xd, pd, go.BF16, None, y, ws, 1)
    assert torch.equal(y, ops.linear(xd, pd, go.BF16))


def test_gate_up_silu_and_grouped_with_bf16_rows(dev, c_oracle):
    print("case bf16 gated / grouped", flush=True)
    n, k = 96, 512
    gate, up = synthetic.make_packed(go.BF16, n, k, seed=1), synthetic.make_packed(go.BF16, n, k, seed=2)
    for m in (1, 7, 16):
        x = synthetic.make_activations(m, k, seed=m)
        want = c_oracle.silu_mul(go.gguf_linear_forward(x, gate, go.BF16), go.gguf_linear_forward(x, up, go.BF16))
        got = ops.gate_up_silu(x.to(dev), gate.to(dev), up.to(dev), go.BF16).cpu()
        assert go.rel_l2(got, want) <= TOL
    m = 333
    x = synthetic.make_activations(m, k, seed=3)
    wq = synthetic.make_packed(go.Q8_0, n, k, seed=4)
    ind = torch.rand(m, generator=torch.Generator().manual_seed(5)) < 0.4
    for (wu, qu, wg, qg) in ((gate, go.BF16, up, go.BF16), (gate, go.BF16, wq, go.Q8_0), (wq, go.Q8_0, up, go.BF16)):
        want = go.grouped_linear_forward(x, ind, wu, qu, wg, qg)
        got = ops.grouped_linear(x.to(dev), ind.to(dev), 0, wu.to(dev), qu, wg.to(dev), qg).cpu()
        assert go.rel_l2(got, want) <= TOL
    # ragged K has no grouped kernel for plain rows: refused, not mis-computed
    with pytest.raises(ops.SnGgufError):
        ops.grouped_linear(synthetic.make_activations(m, 100).to(dev), ind.to(dev), 0, synthetic.make_packed(go.BF16, n, 100).to(dev),
                           go.BF16, synthetic.make_packed(go.BF16, n, 100).to(dev), go.BF16)


def test_module_with_bf16_weight(dev):
    print("case bf16 module", flush=True)
    n, k = 128, 256
    packed = synthetic.make_packed(go.BF16, n, k, seed=9)
    lin = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16, device="meta")
    lin.weight = GGUFParameter(packed.to(dev), quant_type=go.BF16)
    for m in (1, 100):
        x = synthetic.make_activations(m, k, seed=m)
        assert go.rel_l2(lin(x.to(dev)).cpu(), go.gguf_linear_forward(x, packed, go.BF16)) <= TOL
    und = GGUFLinear(k, n, compute_dtype=torch.bfloat16, device="meta")
    und.weight = GGUFParameter(synthetic.make_packed(go.Q8_0, n, k, seed=1).to(dev), quant_type=go.Q8_0)
    x = synthetic.make_activations(96, k, seed=2)
    ind = torch.arange(96) >= 40
    got = grouped_linear(x.to(dev), ind.to(dev), und, lin).cpu()
    want = go.grouped_linear_forward(x, ind, und.weight.as_tensor().cpu(), go.Q8_0, packed, go.BF16)
    assert go.rel_l2(got, want) <= TOL
