"""The allocation-free entry point: sngguf_linear_static is sngguf_linear_ws with the library's own static device
area as the workspace.  Through the C ABI, against the existing entry point given a workspace of the same size, bit
for bit, on consecutive calls of which the later ones are smaller (the area keeps the earlier call's contents)."""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import ops, synthetic

pytestmark = pytest.mark.gpu


def _pair(dev, qt, m, n, k, seed, bias=False, numerics=1):
    packed = synthetic.make_packed(qt, n, k, seed=seed).to(dev)
    x = synthetic.make_activations(m, k, seed=seed + 1).to(dev)
    b = (torch.randn(n, generator=torch.Generator().manual_seed(seed)) * 0.5).to(torch.bfloat16).to(dev) if bias else None
    ws = torch.full((64 << 20,), 0xA5, dtype=torch.uint8, device=dev)       # same size as the static area
    want = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.linear_ws_into(x, packed, qt, b, want, ws, numerics)
    got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.linear_static_into(x, packed, qt, b, got, numerics)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(got.float()).all())
    assert torch.equal(got, want), (qt, m, n, k)
    return x, packed, b, got


def test_linear_static_matches_workspace_entry_point_on_consecutive_calls(dev):
    print("case no-alloc entry point", flush=True)
    assert ops.linear_static_max_outputs() == (64 << 20) // 8
    # K split with the sums in the static area (Q8_0: no weight pass), then a smaller problem right behind it
    x, packed, b, got = _pair(dev, go.Q8_0, 512, 1024, 4096, seed=1, bias=True)
    assert go.rel_l2(got[:16].cpu(), go.gguf_linear_forward(x[:16].cpu(), packed.cpu(), go.Q8_0, b.cpu())) <= 1e-3
    x2, packed2, _, got2 = _pair(dev, go.Q8_0, 130, 515, 1024, seed=2)
    assert go.rel_l2(got2.cpu(), go.gguf_linear_forward(x2.cpu(), packed2.cpu(), go.Q8_0)) <= 1e-3
    # a type whose K split keeps its decoded weights in the area too, again larger first
    _pair(dev, go.Q6_K, 300, 2048, 2048, seed=3, numerics=0)
    x4, packed4, _, got4 = _pair(dev, go.Q6_K, 70, 256, 512, seed=4)
    assert go.rel_l2(got4.cpu(), go.gguf_linear_forward(x4.cpu(), packed4.cpu(), go.Q6_K)) <= 1e-3
    # decode-sized and plain tile-GEMM problems pass through without touching the area
    _pair(dev, go.Q8_0, 1, 4096, 4096, seed=5)
    _pair(dev, go.Q4_K, 2048, 4096, 1024, seed=6)


def test_linear_static_refuses_what_does_not_fit(dev):
    packed = synthetic.make_packed(go.Q8_0, 8192, 64, seed=7).to(dev)
    x = synthetic.make_activations(2048, 64, seed=8).to(dev)
    y = torch.zeros((2048, 8192), dtype=torch.bfloat16, device=dev)          # 16 Mi outputs
    with pytest.raises(ops.SnGgufError, match="static scratch"):
        ops.linear_static_into(x, packed, go.Q8_0, None, y, 1)
    assert int(y.float().abs().sum()) == 0                                    # refused before any launch
    ops.linear_static_into(x[:1024], packed, go.Q8_0, None, y[:1024], 1)     # exactly at the limit: taken
    torch.cuda.synchronize()
    assert go.rel_l2(y[:8].cpu(), go.gguf_linear_forward(x[:8].cpu(), packed.cpu(), go.Q8_0)) <= 1e-3


def test_linear_static_under_graph_capture(dev):
    """The call allocates nothing, so it can be captured; every replay equals the eager result."""
    packed = synthetic.make_packed(go.Q8_0, 1024, 2048, seed=9).to(dev)
    x = synthetic.make_activations(256, 2048, seed=10).to(dev)
    y = torch.empty((256, 1024), dtype=torch.bfloat16, device=dev)
    ops.linear_static_into(x, packed, go.Q8_0, None, y, 1)                   # first call on the device: address lookup
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.linear_static_into(x, packed, go.Q8_0, None, y, 1)
    for seed in (11, 12, 13):
        x.copy_(synthetic.make_activations(256, 2048, seed=seed).to(dev))
        eager = torch.empty_like(y)
        ops.linear_static_into(x, packed, go.Q8_0, None, eager, 1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), seed
