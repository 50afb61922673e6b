"""GPU parity of the SiLU-gated pair beyond decode sizes: ``sngguf_gate_up_silu_ws`` - one weight pass per matrix into
an interleaved bf16 workspace and one launch of the dense tile kernel with the gated epilogue
(``act_fn(gate_proj(x)) * up_proj(x)``, modeling_qwen3.py:214-216).

The launch adds up each output's K steps exactly as the plain workspace route does, so against
``silu(linear_ws(gate)) * linear_ws(up)`` on bf16 tensors only the last place of exp() can differ; against the CPU
oracle the bar is rel-L2 <= 1e-3.  Shapes cover ragged row and column counts (rows past the end of the last tile,
columns past the end of the last 128-wide block), every packed format family, and the model's MLP shape."""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import GGUFLinear, GGUFParameter, ops, synthetic
from sensenova_u1_amd import modality
from sensenova_u1_amd.modality import gated_mlp

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _pair(dev, qt, m, n, k, seed):
    gate = synthetic.make_packed(qt, n, k, seed=seed, device=dev)
    up = synthetic.make_packed(qt, n, k, seed=seed + 1, device=dev)
    x = synthetic.make_activations(m, k, seed=seed + 2, device=dev)
    return gate, up, x


def _fused(x, gate, up, qt, n, k, num=ops.NUM_UPSTREAM_FP16, extra=0):
    ws = torch.empty(ops.gate_up_silu_workspace_bytes(n, k) + extra, dtype=torch.uint8, device=x.device)
    h = torch.full((x.shape[0], n), float("nan"), dtype=torch.bfloat16, device=x.device)
    ops.gate_up_silu_ws_into(x, gate, up, qt, h, ws, num)
    return h


@pytest.mark.parametrize("qt,m,n,k", [(go.Q8_0, 65, 256, 128), (go.Q8_0, 300, 520, 256), (go.Q4_0, 257, 136, 384),
                                      (go.Q5_1, 1000, 1000, 128), (go.Q4_K, 513, 72, 1024), (go.Q6_K, 17, 384, 256),
                                      (go.Q2_K, 700, 128, 512), (go.Q8_0, 2049, 640, 4096)])
@pytest.mark.parametrize("num", [ops.NUM_GGML_FP32, ops.NUM_UPSTREAM_FP16])
def test_gated_pair_on_the_dense_tile_kernel(dev, c_oracle, qt, m, n, k, num):
    print(f"case gated tiles qt={qt} {m}x{n}x{k} num={num}", flush=True)
    gate, up, x = _pair(dev, qt, m, n, k, seed=11 * n + k)
    h = _fused(x, gate, up, qt, n, k, num)
    assert bool(torch.isfinite(h.float()).all())
    # the two projections on the plain workspace route, then the product as bf16 tensors give it
    ws = torch.empty(ops.linear_workspace_bytes(n, k), dtype=torch.uint8, device=dev)
    g = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    u = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    ops.linear_ws_into(x, gate, qt, None, g, ws, num)
    ops.linear_ws_into(x, up, qt, None, u, ws, num)
    ref = torch.nn.functional.silu(g) * u
    assert go.rel_l2(h.cpu(), ref.cpu()) <= 1e-4
    # the oracle on sampled rows
    rows = torch.randperm(m, generator=torch.Generator().manual_seed(m))[:24]
    rows[0], rows[1] = 0, m - 1
    xs = x[rows.to(dev)].cpu()
    want = c_oracle.silu_mul(go.gguf_linear_forward(xs, gate.cpu(), qt, None, numerics=num),
                             go.gguf_linear_forward(xs, up.cpu(), qt, None, numerics=num))
    assert go.rel_l2(h[rows.to(dev)].cpu(), want) <= TOL


def test_overflowed_and_huge_gates_follow_silu_on_bf16_tensors(dev, c_oracle):
    """Gate sums that overflow to +-inf, or are finite and huge: silu(+inf) = +inf, silu(-inf) = NaN (-inf / inf, as
    torch computes it), silu(-1e30) = -0.  The dense launch's own exp / reciprocal must give what the oracle and the
    decode kernels' gated pair give on the same sums."""
    print("case gated tiles overflow", flush=True)
    qt, n, k = go.Q8_0, 256, 256
    gate = synthetic.make_packed(qt, n, k, seed=71)
    up = synthetic.make_packed(qt, n, k, seed=72)
    big = torch.tensor([100.0], dtype=torch.float16).view(torch.uint8)
    gate[:64, 0:2] = big                       # first block of the first 64 gate rows: weights 100 q
    for m in (4, 130):                         # the decode kernels' pair and the dense launch
        x = torch.zeros((m, k), dtype=torch.bfloat16)
        x[0, 0], x[1, 0], x[2, 0] = 1e38, -1e38, 1e30
        x[3:] = synthetic.make_activations(m - 3, k, seed=5)
        g = go.gguf_linear_forward(x, gate, qt)
        u = go.gguf_linear_forward(x, up, qt)
        want = c_oracle.silu_mul(g, u)
        assert bool(torch.isinf(g[0, :64].float()).any()) and bool(torch.isnan(want[:2].float()).any())
        if m <= 16:
            h = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
            ops.gate_up_silu_into(x.to(dev), gate.to(dev), up.to(dev), qt, h, 1)
        else:
            h = _fused(x.to(dev), gate.to(dev), up.to(dev), qt, n, k)
        h = h.cpu()
        assert torch.equal(torch.isnan(h.float()), torch.isnan(want.float())), m
        inf_w = torch.isinf(want.float())
        assert torch.equal(torch.isinf(h.float()), inf_w) and torch.equal(h[inf_w].float(), want[inf_w].float()), m
        fin = torch.isfinite(want.float())
        assert torch.equal(torch.signbit(h[:3][fin[:3]].float()), torch.signbit(want[:3][fin[:3]].float()))
        assert go.rel_l2(torch.where(fin, h.float(), 0.0), torch.where(fin, want.float(), 0.0)) <= TOL, m


@pytest.mark.parametrize("seed", range(16))
def test_random_gated_cases(dev, c_oracle, seed):
    """Seeded random shapes across the tile boundaries: any of the ten packed formats, 17 ... 1300 rows, output widths
    that are any multiple of 8, K any admissible multiple of 128; the whole output against the oracle."""
    gen = torch.Generator().manual_seed(1000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=gen))
    qt = [go.Q4_0, go.Q4_1, go.Q5_0, go.Q5_1, go.Q8_0, go.Q2_K, go.Q3_K, go.Q4_K, go.Q5_K, go.Q6_K][r(0, 9)]
    m = [r(17, 64), r(65, 300), r(250, 520), r(500, 1300)][r(0, 3)]
    n = 8 * r(1, 70)
    k = 256 * r(1, 6) if qt in (go.Q2_K, go.Q3_K, go.Q4_K, go.Q5_K, go.Q6_K) else 128 * r(1, 12)
    num = [ops.NUM_GGML_FP32, ops.NUM_UPSTREAM_FP16][r(0, 1)]
    print(f"case random gated seed={seed} qt={qt} {m}x{n}x{k} num={num}", flush=True)
    gate, up, x = _pair(dev, qt, m, n, k, seed=seed)
    h = _fused(x, gate, up, qt, n, k, num)
    want = c_oracle.silu_mul(go.gguf_linear_forward(x.cpu(), gate.cpu(), qt, None, numerics=num),
                             go.gguf_linear_forward(x.cpu(), up.cpu(), qt, None, numerics=num))
    assert bool(torch.isfinite(h.float()).all())
    assert go.rel_l2(h.cpu(), want) <= TOL


def test_gated_pair_at_the_mlp_shape_over_image_rows(dev, c_oracle):
    """gate / up 4096 -> 12288 at M = 4096: the generation tower's MLP.  Sampled columns against the oracle, the whole
    output against the two plain workspace launches."""
    qt, m, n, k = go.Q8_0, 4096, 12288, 4096
    print("case gated tiles full size", flush=True)
    gate, up, x = _pair(dev, qt, m, n, k, seed=77)
    h = _fused(x, gate, up, qt, n, k, extra=4096)
    assert bool(torch.isfinite(h.float()).all())
    gen = torch.Generator().manual_seed(5)
    cols = torch.randint(0, n, (48,), generator=gen)
    cols[0], cols[1] = 0, n - 1
    rows = torch.randint(0, m, (24,), generator=gen)
    rows[0] = m - 1
    xs = x[rows.to(dev)].cpu()
    want = c_oracle.silu_mul(go.gguf_linear_forward(xs, gate[cols.to(dev)].cpu(), qt),
                             go.gguf_linear_forward(xs, up[cols.to(dev)].cpu(), qt))
    assert go.rel_l2(h[rows.to(dev)][:, cols.to(dev)].cpu(), want) <= TOL
    ws = torch.empty(ops.linear_workspace_bytes(n, k), dtype=torch.uint8, device=dev)
    g = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    u = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    ops.linear_ws_into(x, gate, qt, None, g, ws, ops.NUM_UPSTREAM_FP16)
    ops.linear_ws_into(x, up, qt, None, u, ws, ops.NUM_UPSTREAM_FP16)
    assert go.rel_l2(h.cpu(), (torch.nn.functional.silu(g) * u).cpu()) <= 1e-4


def test_gated_pair_entry_point_routes_and_refusals(dev):
    """Up to 16 rows the entry point is the decode kernel's gated pair (bit for bit, workspace untouched); shapes the
    dense kernel's epilogue does not take are refused before anything is launched."""
    qt, n, k = go.Q8_0, 512, 256
    gate, up, x = _pair(dev, qt, 16, n, k, seed=3)
    assert torch.equal(_fused(x, gate, up, qt, n, k), ops.gate_up_silu(x, gate, up, qt))
    assert ops.gate_up_silu_ws_fits(qt, 4096, 12288, 4096)
    assert not ops.gate_up_silu_ws_fits(qt, 16, n, k)          # decode sizes belong to the other kernel
    assert not ops.gate_up_silu_ws_fits(qt, 300, n, 192)       # odd number of 64-wide K steps
    assert not ops.gate_up_silu_ws_fits(qt, 300, 516, k)       # output rows of whole 16-byte pieces only
    assert not ops.gate_up_silu_ws_fits(go.BF16, 300, n, k)
    gate, up, x = _pair(dev, qt, 300, n, 192, seed=4)
    with pytest.raises(ops.SnGgufError):
        _fused(x, gate, up, qt, n, 192)
    gate, up, x = _pair(dev, qt, 300, n, k, seed=5)
    h = torch.empty((300, n), dtype=torch.bfloat16, device=dev)
    small = torch.empty(ops.gate_up_silu_workspace_bytes(n, k) - 16, dtype=torch.uint8, device=dev)
    with pytest.raises(ops.SnGgufError):
        ops.gate_up_silu_ws_into(x, gate, up, qt, h, small, ops.NUM_UPSTREAM_FP16)


def test_gated_mlp_takes_the_tile_route_when_its_tiles_fill_the_chip(dev, monkeypatch):
    """``modality.gated_mlp`` (what the loader points ``Qwen3MLP.forward`` at) with enough rows and tiles: same result as
    the three module calls and the product on bf16 tensors, and the gated entry point is what ran."""
    n, k, m = 6144, 256, 1024
    assert modality.gated_tile_fill(m, n) >= modality.GATED_TILE_MIN_FILL > modality.gated_tile_fill(768, 12288)
    mods = []
    for j, (o, i) in enumerate(((n, k), (n, k), (k, n))):
        lin = GGUFLinear(i, o, bias=False, compute_dtype=torch.bfloat16, device="meta")
        lin.weight = GGUFParameter(synthetic.make_packed(go.Q8_0, o, i, seed=90 + j, device=dev), quant_type=go.Q8_0)
        mods.append(lin)
    gate, up, down = mods
    x = synthetic.make_activations(m, k, seed=9, device=dev).view(2, m // 2, k)
    calls = []
    real = ops.gate_up_silu_ws_into
    monkeypatch.setattr(ops, "gate_up_silu_ws_into", lambda *a, **kw: (calls.append(a[0].shape[0]), real(*a, **kw))[1])
    got = gated_mlp(x, gate, up, down)
    assert calls == [m]
    want = down(torch.nn.functional.silu(gate(x)) * up(x))
    assert got.shape == want.shape
    # (the separate launches of this shape have few tiles and split K over workgroups: another order of the fp32 sums)
    assert go.rel_l2(got.cpu(), want.cpu()) <= 5e-4
    # few tiles: the separate launches (with their K split) stay
    calls.clear()
    gated_mlp(x[:, :128], gate, up, down)
    assert calls == []
