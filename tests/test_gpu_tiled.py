"""GPU: the operand-order ("tiled") copy of Q8_0 weights and the decode entry points that read it - the copy holds
exactly the bits of the GGUF rows in the documented order, and linear / residual / gated results agree with the oracle
(and, up to the summation order over K, with the GGUF-native kernels)."""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import ops, synthetic

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _tiled_reference(packed, n, k):
    """The layout in tensor operations: quants [G][B/2][g][r][pair member][8], scales [G][B/8][r][8], rows padded with zeros."""
    nb, groups = k // 32, (n + 15) // 16
    padded = torch.zeros((groups * 16, nb, 34), dtype=torch.uint8)
    padded[:n] = packed.view(n, nb, 34)
    quants = padded[:, :, 2:].reshape(groups, 16, nb // 2, 2, 4, 8).permute(0, 2, 4, 1, 3, 5).reshape(-1)
    scales = padded[:, :, :2].reshape(groups, 16, nb // 8, 8, 2).permute(0, 2, 1, 3, 4).reshape(-1)
    return torch.cat([quants, scales])


@pytest.mark.parametrize("shape", [(16, 256), (33, 512), (160, 1024), (4100, 2048)])
def test_tiled_copy_is_a_permutation_of_the_gguf_rows(dev, shape):
    n, k = shape
    print(f"case tile n={n} k={k}", flush=True)
    packed = synthetic.make_packed(go.Q8_0, n, k, seed=n + k)
    tiled = ops.q8_0_tile(packed.to(dev)).cpu()
    assert tiled.numel() == ((n + 15) // 16) * 16 * (k // 32) * 34
    assert torch.equal(tiled, _tiled_reference(packed, n, k))


@pytest.mark.parametrize("numerics", [0, 1])
@pytest.mark.parametrize("m", [1, 2, 3, 7, 8, 16])
def test_linear_tiled_parity(dev, numerics, m):
    print(f"case linear_tiled m={m} numerics={numerics}", flush=True)
    for n, k, use_bias, use_res in [(4096, 4096, False, False), (1030, 512, True, False), (37, 256, True, True), (12288, 2048, False, True)]:
        packed = synthetic.make_packed(go.Q8_0, n, k, seed=m + n)
        x = synthetic.make_activations(m, k, seed=3 * m)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(k)) * 0.5).to(torch.bfloat16) if use_bias else None
        res = synthetic.make_activations(m, n, seed=5 * m) if use_res else None
        want = go.gguf_linear_forward(x, packed, go.Q8_0, bias, numerics=numerics)
        if res is not None:
            want = (res.float() + want.float()).to(torch.bfloat16)
        pd = packed.to(dev)
        tiled = ops.q8_0_tile(pd)
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.linear_tiled_into(x.to(dev), tiled, bias.to(dev) if use_bias else None, res.to(dev) if use_res else None, y, numerics)
        assert bool(torch.isfinite(y.float()).all())
        assert go.rel_l2(y.cpu(), want) <= TOL, (n, k)
        native = ops.linear_residual(x.to(dev), pd, go.Q8_0, res.to(dev), bias.to(dev) if use_bias else None, numerics) if use_res \
            else ops.linear(x.to(dev), pd, go.Q8_0, bias.to(dev) if use_bias else None, numerics)
        # same weights, same rounding chain: only the way K is split over wavefronts differs, which moves a few sums
        # across a bf16 rounding boundary (one flipped output in a thousand is 1e-4 here)
        assert go.rel_l2(y.cpu(), native.cpu()) <= 4e-4, (n, k)


@pytest.mark.parametrize("m", [1, 4, 13, 16])
def test_gate_up_silu_tiled_parity(dev, c_oracle, m):
    print(f"case gate_up_tiled m={m}", flush=True)
    for n, k in [(12288, 4096), (1000, 768), (48, 256)]:
        gate = synthetic.make_packed(go.Q8_0, n, k, seed=71)
        up = synthetic.make_packed(go.Q8_0, n, k, seed=72)
        x = synthetic.make_activations(m, k, seed=73 + m)
        g = go.gguf_linear_forward(x, gate, go.Q8_0)
        u = go.gguf_linear_forward(x, up, go.Q8_0)
        h = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.gate_up_silu_tiled_into(x.to(dev), ops.q8_0_tile(gate.to(dev)), ops.q8_0_tile(up.to(dev)), h, 1)
        assert go.rel_l2(h.cpu(), torch.nn.functional.silu(g) * u) <= TOL
        assert go.rel_l2(h.cpu(), c_oracle.silu_mul(g, u)) <= TOL


def test_tiled_argument_errors(dev):
    packed = synthetic.make_packed(go.Q8_0, 32, 288, seed=1).to(dev)
    with pytest.raises(ops.SnGgufError):
        ops.q8_0_tile(packed)                      # K % 256
    packed = synthetic.make_packed(go.Q8_0, 32, 256, seed=1).to(dev)
    tiled = ops.q8_0_tile(packed)
    x = synthetic.make_activations(17, 256, seed=2).to(dev)
    y = torch.empty((17, 32), dtype=torch.bfloat16, device=dev)
    with pytest.raises(ops.SnGgufError):
        ops.linear_tiled_into(x, tiled, None, None, y, 1)   # decode rows only
