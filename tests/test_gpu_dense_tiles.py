"""GPU parity of the two dense bf16 tile kernels behind weights that are already bf16 rows (GGUF type 30) and behind
the workspace routes of quantized weights.

A launch whose workgroups get an even number of 64-wide K steps runs on the four-wavefront kernel, every other one on
the dense form of the eight-wavefront tile kernel; both accumulate a row's K steps in the same order with the same
matrix instruction, so an output must not depend on which of the two computed it.  The cases below put the same
weights through both (K and K + 64, the extra columns zero) and compare bit for bit, and check each against the CPU
oracle (rel-L2 <= 1e-3).  Shapes cover all three epilogues: staged bf16 tile (N % 8 == 0), direct stores (any N),
fp32 partial sums of a K split (few output tiles)."""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import ops, synthetic

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _bf16_rows(n, k, seed, dev):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16)
    return w, w.view(torch.uint8).to(dev)


@pytest.mark.parametrize("m,n,k", [(65, 256, 128), (300, 520, 256), (257, 264, 512), (1000, 1001, 128), (513, 77, 1024),
                                   (4096, 512, 4096), (256, 256, 64 * 6)])
def test_both_dense_kernels_agree_and_match_the_oracle(dev, m, n, k):
    print(f"case dense tiles {m}x{n}x{k}", flush=True)
    w, wd = _bf16_rows(n, k, 7 * n + k, dev)
    x = synthetic.make_activations(m, k, seed=m + k)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.bfloat16)
    res = synthetic.make_activations(m, n, seed=n + 1)
    xd = x.to(dev)
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.linear_into(xd, wd, go.BF16, bias.to(dev), y, 1)          # K / 64 even: four wavefronts
    # one more K step of zeros (odd count: eight wavefronts); zeros add nothing, so the bits must be the same
    w1 = torch.cat([w, torch.zeros(n, 64, dtype=torch.bfloat16)], dim=1).contiguous()
    x1 = torch.cat([x, torch.zeros(m, 64, dtype=torch.bfloat16)], dim=1).contiguous()
    y1 = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.linear_into(x1.to(dev), w1.view(torch.uint8).to(dev), go.BF16, bias.to(dev), y1, 1)
    assert torch.equal(y, y1)
    rows = torch.randperm(m, generator=torch.Generator().manual_seed(1))[:48]
    rows[0], rows[1] = 0, m - 1
    want = go.gguf_linear_forward(x[rows], w.view(torch.uint8), go.BF16, bias)
    assert go.rel_l2(y[rows.to(dev)].cpu(), want) <= TOL
    assert bool(torch.isfinite(y.float()).all())
    if n % 8 == 0:
        got_r = ops.linear_residual(xd, wd, go.BF16, res.to(dev), bias.to(dev))
        assert torch.equal(got_r, res.to(dev) + y)


@pytest.mark.parametrize("m,n,k", [(128, 4096, 12288), (512, 1024, 4096), (96, 512, 2048)])
def test_k_split_partial_sums_of_the_workspace_route(dev, m, n, k):
    """Few output tiles: the workspace route cuts K over workgroups, the slices go out as fp32 partial sums and a
    second kernel adds them up.  Against the oracle on sampled rows, and against the same launch with one more
    (zero) K step, which changes the slice boundaries and the kernel."""
    print(f"case dense split-K {m}x{n}x{k}", flush=True)
    packed = synthetic.make_packed(go.Q8_0, n, k, seed=n + k, device=dev)
    x = synthetic.make_activations(m, k, seed=m, device=dev)
    ws = torch.empty(ops.linear_workspace_bytes(n, k), dtype=torch.uint8, device=dev)
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.linear_ws_into(x, packed, go.Q8_0, None, y, ws, ops.NUM_UPSTREAM_FP16)
    cols = torch.randperm(n, generator=torch.Generator().manual_seed(2))[:64]
    want = go.gguf_linear_forward(x.cpu(), packed[cols.to(dev)].cpu(), go.Q8_0)
    assert go.rel_l2(y[:, cols.to(dev)].cpu(), want) <= TOL
    assert bool(torch.isfinite(y.float()).all())


@pytest.mark.parametrize("m,n,k", [(512, 1024, 4096), (4096, 1024, 1024), (300, 520, 2048)])
def test_k_split_of_plain_bf16_rows_with_a_workspace(dev, m, n, k):
    """Weights that are bf16 rows already (GGUF type 30, and the kept weights of the module's "resident" policy) need no
    weight pass; with a workspace that has room for fp32 partial sums a shape with few output tiles still gets the K
    split.  Against the oracle, and against the same call without a workspace (the dense kernel unsplit: another order
    of the fp32 sums, same bf16 weights)."""
    print(f"case dense split-K of bf16 rows {m}x{n}x{k}", flush=True)
    w, wd = _bf16_rows(n, k, 3 * n + k, dev)
    x = synthetic.make_activations(m, k, seed=m + 1)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n + 2)) * 0.5).to(torch.bfloat16)
    xd = x.to(dev)
    outs = []
    for ws_bytes in (0, 16 * m * n):
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.linear_ws_into(xd, wd, go.BF16, bias.to(dev), y, ws, ops.NUM_UPSTREAM_FP16)
        assert bool(torch.isfinite(y.float()).all())
        outs.append(y)
    rows = torch.randperm(m, generator=torch.Generator().manual_seed(3))[:48]
    rows[0], rows[1] = 0, m - 1
    want = go.gguf_linear_forward(x[rows], w.view(torch.uint8), go.BF16, bias)
    for y in outs:
        assert go.rel_l2(y[rows.to(dev)].cpu(), want) <= TOL
    assert go.rel_l2(outs[1].cpu(), outs[0].cpu()) <= 5e-4
