"""GPU: lm_head with the arg-max folded into the decode kernel (greedy token of the think loop) against
`argmax(linear(x))` - bit-equal to the library's own logits, and consistent with the oracle's logits."""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import GGUFLinear, GGUFParameter, ops, synthetic

pytestmark = pytest.mark.gpu


def _oracle_consistent(x, packed, qt, idx, bias=None):
    """The chosen column's oracle logit is the oracle's maximum, up to the one bf16 step by which two summation orders
    of the same dot product can differ."""
    logits = go.gguf_linear_forward(x, packed, qt, bias).float()
    best = logits.max(dim=-1).values
    chosen = logits.gather(-1, idx.cpu().reshape(-1, 1)).reshape(-1)
    assert bool((chosen >= best - best.abs() * 2.0 ** -7 - 1e-30).all()), (chosen, best)


@pytest.mark.parametrize("qt,n,k", [(go.Q8_0, 8200, 4096), (go.Q8_0, 301, 512), (go.Q8_0, 4096, 2048), (go.Q4_K, 1000, 1024),
                                    (go.Q6_K, 515, 512), (go.Q4_K, 33000, 256), (go.Q5_0, 777, 256), (go.Q2_K, 64, 768)])
def test_argmax_equals_argmax_of_the_logits(dev, qt, n, k):
    print(f"case argmax qt={qt} {n}x{k}", flush=True)
    packed = synthetic.make_packed(qt, n, k, seed=n)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.05).to(torch.bfloat16)
    pd = packed.to(dev)
    for m in (1, 5, 16):
        x = synthetic.make_activations(m, k, seed=m + k)
        for b in (None, bias):
            bd = b.to(dev) if b is not None else None
            for numerics in (0, 1):
                got = ops.lm_head_argmax(x.to(dev), pd, qt, bd, numerics)
                logits = ops.linear(x.to(dev), pd, qt, bd, numerics)
                assert got.dtype == torch.int64 and got.shape == (m,)
                assert torch.equal(got, logits.argmax(dim=-1)), (m, b is not None, numerics)
            _oracle_consistent(x, packed, qt, got, b)
    # leading dims are kept
    x3 = synthetic.make_activations(6, k, seed=1).reshape(2, 3, k).to(dev)
    assert ops.lm_head_argmax(x3, pd, qt).shape == (2, 3)


def test_argmax_ties_and_nan_follow_torch(dev):
    print("case argmax ties", flush=True)
    n, k = 4096, 4096
    packed = synthetic.make_packed(go.Q8_0, n, k, seed=3)
    x = synthetic.make_activations(2, k, seed=4)
    ref = ops.linear(x.to(dev), packed.to(dev), go.Q8_0)
    win = int(ref[0].argmax())
    # copies of the winning row at a lower and at higher columns (other workgroups, other lanes): the lowest wins
    lo = 5 if win > 5 else win
    for dup in (lo, 1234, 4095, win ^ 1):
        packed[dup] = packed[win]
    pd = packed.to(dev)
    got = ops.lm_head_argmax(x.to(dev), pd, go.Q8_0)
    logits = ops.linear(x.to(dev), pd, go.Q8_0)
    assert torch.equal(got, logits.argmax(dim=-1))
    assert int(got[0]) == min(lo, win, win ^ 1)
    # a NaN logit counts as the maximum, the first one wins
    xn = x.clone()
    xn[1, 7] = float("nan")
    got = ops.lm_head_argmax(xn.to(dev), pd, go.Q8_0)
    assert int(got[1]) == 0 and int(got[0]) == min(lo, win, win ^ 1)
    # all-negative logits (the key order must hold below zero too)
    bias = torch.full((n,), -300.0).to(torch.bfloat16).to(dev)
    got = ops.lm_head_argmax(x.to(dev), pd, go.Q8_0, bias)
    assert torch.equal(got, ops.linear(x.to(dev), pd, go.Q8_0, bias).argmax(dim=-1))


def test_argmax_treats_signed_zeros_as_equal(dev):
    """A row whose maximum is zero, with a -0 logit in front of a +0 logit: torch.argmax compares them equal and returns
    the first.  -0 comes from a negative sum too small for bf16 (2^-120 x -2^-24); every other logit is negative."""
    print("case argmax signed zeros", flush=True)
    n, k = 512, 256
    packed = torch.zeros((n, k // 32 * 34), dtype=torch.uint8)
    one = torch.tensor([1.0], dtype=torch.float16).view(torch.uint8)
    tiny = torch.tensor([2.0 ** -24], dtype=torch.float16).view(torch.uint8)
    packed[:, 0:2] = one
    packed[:, 2] = 0x9C                      # q[0] = -100: logit -100 x
    a, b = 37, 300
    packed[a, 0:2] = tiny
    packed[a, 2] = 0xFF                      # q[0] = -1, d = 2^-24
    packed[b, 2] = 0                         # all-zero row: +0
    x = torch.zeros((2, k), dtype=torch.bfloat16)
    x[:, 0] = 2.0 ** -120
    for numerics in (0, 1):
        logits = ops.linear(x.to(dev), packed.to(dev), go.Q8_0, None, numerics)
        got = ops.lm_head_argmax(x.to(dev), packed.to(dev), go.Q8_0, None, numerics)
        assert float(logits[0, a]) == 0.0 and float(logits[0, b]) == 0.0 and float(logits.max()) == 0.0
        assert torch.equal(got, logits.argmax(dim=-1)), (got, logits.argmax(dim=-1), logits[0, a], logits[0, b])


def test_vocabulary_sized_argmax_and_module_helper(dev):
    print("case argmax lm_head", flush=True)
    n, k = 151936, 4096
    for qt in (go.Q8_0, go.Q4_K):
        packed = synthetic.make_packed(qt, n, k, seed=5, device=dev)
        lin = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16, device="meta")
        lin.weight = GGUFParameter(packed, quant_type=qt)
        for m in (1, 3):
            x = synthetic.make_activations(m, k, seed=m, device=dev)
            got = lin.forward_argmax(x)
            assert torch.equal(got, lin(x).argmax(dim=-1))
            sub = packed[got].cpu()
            want = go.gguf_linear_forward(x.cpu(), sub, qt)          # [m, m]: the winners' logits
            assert bool(torch.isfinite(want.float()).all())
    # shapes without a fused kernel take linear + argmax
    small = synthetic.make_packed(go.Q8_0, 64, 96, seed=1).to(dev)
    xs = synthetic.make_activations(20, 96, seed=2).to(dev)
    assert torch.equal(ops.lm_head_argmax(xs, small, go.Q8_0), ops.linear(xs, small, go.Q8_0).argmax(dim=-1))
    with pytest.raises(ops.SnGgufError):
        ops.lm_head_argmax(xs.cpu(), small, go.Q8_0)
