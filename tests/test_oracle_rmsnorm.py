"""CPU: pins the oracle's RMSNorm restatement (oracle.gguf_oracle.qwen3_rms_norm) with cases whose answer is
known without it - a dropped eps, a sum where a mean belongs, a norm over the wrong axis or a weight applied
before the cast each fail one of them."""
import math

import torch

from oracle import gguf_oracle as go


def test_constant_row_has_closed_form():
    # x = c everywhere: variance = c^2, so every element becomes c / sqrt(c^2 + eps), times the weight
    k, c, eps = 512, 3.0, 0.25
    x = torch.full((2, k), c, dtype=torch.float32)
    w = torch.full((k,), 2.0)
    want = 2.0 * c / math.sqrt(c * c + eps)
    got = go.qwen3_rms_norm(x, w, eps)
    assert torch.allclose(got, torch.full_like(got, want), rtol=1e-6)


def test_one_hot_row_pins_mean_not_sum_and_the_axis():
    # a single a at position j of K: variance = a^2 / K (a sum would give a^2), output a / sqrt(a^2 / K + eps) at j only;
    # each row has its own statistic
    k, eps = 64, 1e-6
    x = torch.zeros((3, k))
    x[0, 5], x[1, 17], x[2, 63] = 4.0, -2.0, 0.5
    w = torch.arange(1, k + 1, dtype=torch.float32)
    got = go.qwen3_rms_norm(x, w, eps)
    for row, (j, a) in enumerate([(5, 4.0), (17, -2.0), (63, 0.5)]):
        want = torch.zeros(k)
        want[j] = (j + 1) * a / math.sqrt(a * a / k + eps)
        assert torch.allclose(got[row], want, rtol=1e-6), row


def test_scale_invariance_and_eps():
    g = torch.Generator().manual_seed(5)
    x = torch.randn((4, 256), generator=g)
    w = torch.rand(256, generator=g) + 0.5
    base = go.qwen3_rms_norm(x, w, 0.0)
    assert torch.allclose(go.qwen3_rms_norm(8.0 * x, w, 0.0), base, rtol=1e-5, atol=1e-6)    # eps = 0: scale-free
    rms = x.pow(2).mean(-1, keepdim=True).sqrt()
    assert torch.allclose(base.pow(2).div(w * w).mean(-1), torch.ones(4), rtol=1e-5)          # unit RMS before the weight
    big_eps = go.qwen3_rms_norm(x, w, 3.0)
    assert torch.allclose(big_eps, w * x / torch.sqrt(rms * rms + 3.0), rtol=1e-5, atol=1e-6)


def test_matches_the_library_routine_in_fp32():
    g = torch.Generator().manual_seed(6)
    x = torch.randn((5, 1024), generator=g)
    w = torch.randn(1024, generator=g)
    want = torch.nn.functional.rms_norm(x, (1024,), w, 1e-6)
    assert torch.allclose(go.qwen3_rms_norm(x, w, 1e-6), want, rtol=1e-5, atol=1e-6)


def test_bf16_rounds_before_the_weight():
    # in bf16 the normalized row is rounded to bf16 first and the product with the weight is rounded again
    g = torch.Generator().manual_seed(7)
    x = torch.randn((3, 512), generator=g).to(torch.bfloat16)
    w = (torch.rand(512, generator=g) + 0.5).to(torch.bfloat16)
    got = go.qwen3_rms_norm(x, w, 1e-6)
    assert got.dtype == torch.bfloat16
    xf = x.double()
    v = (xf / torch.sqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).float().to(torch.bfloat16)
    want = (w.float() * v.float()).to(torch.bfloat16)
    # the fp64 statistic can round differently from the fp32 one in rare near-ties: allow one bf16 step on < 1 % of elements
    diff = (got.float() - want.float()).abs()
    assert float((diff > 0).float().mean()) < 0.01
    assert bool((diff <= want.float().abs() * 2 ** -7 + 1e-30).all())
