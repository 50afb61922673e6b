"""GPU parity at the benchmark configurations' real shapes, so that every headline launch geometry is checked.

An output element depends on one activation row and one weight row only, so at sizes the CPU oracle cannot finish a
random sample of output rows x columns is compared with the oracle run on exactly those weight rows (rel-L2 <= 1e-3).
"""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import ops, synthetic

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _sample_check(y, x, packed, qt, gen, what, bias=None, n_cols=48, n_rows=24):
    m, n = y.shape
    dev = y.device
    cols = torch.randint(0, n, (n_cols,), generator=gen)
    cols[0], cols[1] = 0, n - 1
    rows = torch.randint(0, m, (min(m, n_rows),), generator=gen)
    rows[0] = m - 1
    sub = packed[cols.to(dev)].cpu()
    b = bias.cpu()[cols] if bias is not None else None
    want = go.gguf_linear_forward(x[rows.to(dev)].cpu(), sub, qt, b)
    err = go.rel_l2(y[rows.to(dev)][:, cols.to(dev)].cpu(), want)
    assert err <= TOL, f"{what}: rel-L2 {err:.3e}"
    assert bool(torch.isfinite(y.float()).all()), what


def test_q8_0_square_projection_decode_and_image_rows(dev):
    """Single Q8_0 linear 4096 -> 4096 at M = 1 (the one-linear configuration) and M = 4096 (q / o of the generation
    tower), plain entry point and workspace route."""
    n = k = 4096
    gen = torch.Generator().manual_seed(10)
    packed = synthetic.make_packed(go.Q8_0, n, k, seed=40, device=dev)
    ws = torch.empty(ops.linear_workspace_bytes(n, k), dtype=torch.uint8, device=dev)
    for m in (1, 4096):
        print(f"case full q8_0 4096x4096 m={m}", flush=True)
        x = synthetic.make_activations(m, k, seed=m, device=dev)
        y = ops.linear(x, packed, go.Q8_0)
        _sample_check(y, x, packed, go.Q8_0, gen, f"linear m={m}")
        y2 = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.linear_ws_into(x, packed, go.Q8_0, None, y2, ws, ops.NUM_UPSTREAM_FP16)
        _sample_check(y2, x, packed, go.Q8_0, gen, f"linear_ws m={m}")


@pytest.mark.parametrize("qt", [go.Q8_0, go.Q4_K])
def test_gate_up_silu_at_the_mlp_shape(dev, c_oracle, qt):
    """The fused gate / up / SiLU launch at 4096 -> 12288 for M = 1, 4, 16: the headline kernel's own grid."""
    n, k = 12288, 4096
    gen = torch.Generator().manual_seed(11 + qt)
    gate = synthetic.make_packed(qt, n, k, seed=41, device=dev)
    up = synthetic.make_packed(qt, n, k, seed=42, device=dev)
    for m in (1, 4, 16):
        print(f"case full gate_up qt={qt} m={m}", flush=True)
        x = synthetic.make_activations(m, k, seed=50 + m, device=dev)
        h = ops.gate_up_silu(x, gate, up, qt)
        cols = torch.randint(0, n, (64,), generator=gen)
        cols[0], cols[1] = 0, n - 1
        g = go.gguf_linear_forward(x.cpu(), gate[cols.to(dev)].cpu(), qt)
        u = go.gguf_linear_forward(x.cpu(), up[cols.to(dev)].cpu(), qt)
        want = c_oracle.silu_mul(g, u)
        err = go.rel_l2(h[:, cols.to(dev)].cpu(), want)
        assert err <= TOL, f"gate_up m={m}: rel-L2 {err:.3e}"
        assert bool(torch.isfinite(h.float()).all())
        # and the two halves computed separately through the plain entry point give the same bits
        g_full = ops.linear(x, gate, qt)
        u_full = ops.linear(x, up, qt)
        ref = torch.nn.functional.silu(g_full) * u_full
        assert go.rel_l2(h.cpu(), ref.cpu()) <= TOL    # same roundings; exp() of the two implementations may differ in the last place


@pytest.mark.parametrize("qt,n,k", [(go.Q4_K, 12288, 4096), (go.Q6_K, 4096, 12288), (go.Q4_K, 4096, 4096), (go.Q4_K, 1024, 4096)])
def test_k_quant_mix_at_full_size(dev, qt, n, k):
    """The K-quant configuration: Q4_K for q / k / v / o / gate / up, Q6_K for down, at M = 1 and M = 4096, on the plain
    entry point and on the workspace route."""
    gen = torch.Generator().manual_seed(12 + n)
    packed = synthetic.make_packed(qt, n, k, seed=43, device=dev)
    ws = torch.empty(ops.linear_workspace_bytes(n, k), dtype=torch.uint8, device=dev)
    for m in (1, 4096):
        print(f"case full kquant qt={qt} {n}x{k} m={m}", flush=True)
        x = synthetic.make_activations(m, k, seed=60 + m, device=dev)
        y = ops.linear(x, packed, qt)
        _sample_check(y, x, packed, qt, gen, f"linear qt={qt} m={m}")
        y2 = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.linear_ws_into(x, packed, qt, None, y2, ws, ops.NUM_UPSTREAM_FP16)
        _sample_check(y2, x, packed, qt, gen, f"linear_ws qt={qt} m={m}")


@pytest.mark.parametrize("qt", [go.Q8_0, go.Q4_K])
def test_narrow_projection_over_image_rows_with_room_for_a_k_split(dev, qt):
    """k / v of the generation tower (4096 -> 1024 at M = 4096: 64 output tiles) with a workspace that has room for fp32
    partial sums behind the decoded weight, as the module's pooled workspace has: weight pass + dense kernel with K split
    over workgroups.  The same call with the minimal workspace (no room: no split) must give the same sampled values."""
    n, k, m = 1024, 4096, 4096
    gen = torch.Generator().manual_seed(13 + qt)
    packed = synthetic.make_packed(qt, n, k, seed=44, device=dev)
    x = synthetic.make_activations(m, k, seed=61, device=dev)
    bias = synthetic.make_activations(1, n, seed=62, device=dev).reshape(n)
    outs = []
    for extra in (0, 4 * 4 * m * n):
        print(f"case full narrow qt={qt} extra workspace {extra}", flush=True)
        ws = torch.empty(ops.linear_workspace_bytes(n, k) + extra, dtype=torch.uint8, device=dev)
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.linear_ws_into(x, packed, qt, bias, y, ws, ops.NUM_UPSTREAM_FP16)
        _sample_check(y, x, packed, qt, gen, f"narrow qt={qt} extra={extra}", bias=bias)
        outs.append(y)
    assert go.rel_l2(outs[1].cpu(), outs[0].cpu()) <= 1e-4   # same bf16 weights; only the order of the fp32 sums differs


def test_q8_0_down_projection_with_residual_at_decode(dev):
    """down_proj 12288 -> 4096 with the residual add in the epilogue, M = 1, 4, 16."""
    n, k = 4096, 12288
    gen = torch.Generator().manual_seed(13)
    packed = synthetic.make_packed(go.Q8_0, n, k, seed=44, device=dev)
    for m in (1, 4, 16):
        print(f"case full down residual m={m}", flush=True)
        x = synthetic.make_activations(m, k, seed=70 + m, device=dev)
        res = synthetic.make_activations(m, n, seed=80 + m, device=dev)
        y = ops.linear_residual(x, packed, go.Q8_0, res)
        assert torch.equal(y, res + ops.linear(x, packed, go.Q8_0))
        _sample_check(ops.linear(x, packed, go.Q8_0), x, packed, go.Q8_0, gen, f"down m={m}")


@pytest.mark.parametrize("num", [ops.NUM_GGML_FP32, ops.NUM_UPSTREAM_FP16])
def test_q6_k_large_projection_with_activations_staged_in_lds(dev, c_oracle, num):
    """Q6_K at 12288 x 4096: with one or two activation rows the decode kernel streams them from LDS, with three it
    reads them from global memory.  Plain projection with bias and residual, and the gated pair; the rows that both
    routes compute must agree bit for bit (same fragments, same order of accumulation)."""
    n, k = 12288, 4096
    qt = go.Q6_K
    gen = torch.Generator().manual_seed(14 + num)
    gate = synthetic.make_packed(qt, n, k, seed=45, device=dev)
    up = synthetic.make_packed(qt, n, k, seed=46, device=dev)
    bias = synthetic.make_activations(1, n, seed=47, device=dev).reshape(n)
    x3 = synthetic.make_activations(3, k, seed=90, device=dev)
    y3 = torch.empty((3, n), dtype=torch.bfloat16, device=dev)
    ops.linear_into(x3, gate, qt, bias, y3, num)
    h3 = torch.empty((3, n), dtype=torch.bfloat16, device=dev)
    ops.gate_up_silu_into(x3, gate, up, qt, h3, num)
    for m in (1, 2):
        print(f"case full q6_k staged num={num} m={m}", flush=True)
        x = x3[:m].contiguous()
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.linear_into(x, gate, qt, bias, y, num)
        assert torch.equal(y, y3[:m])
        if num == ops.NUM_UPSTREAM_FP16:
            _sample_check(y, x, gate, qt, gen, f"staged linear m={m}", bias=bias)
        h = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.gate_up_silu_into(x, gate, up, qt, h, num)
        assert torch.equal(h, h3[:m])
        if num == ops.NUM_UPSTREAM_FP16:
            cols = torch.randint(0, n, (64,), generator=gen)
            cols[0], cols[1] = 0, n - 1
            g = go.gguf_linear_forward(x.cpu(), gate[cols.to(dev)].cpu(), qt)
            u = go.gguf_linear_forward(x.cpu(), up[cols.to(dev)].cpu(), qt)
            assert go.rel_l2(h[:, cols.to(dev)].cpu(), c_oracle.silu_mul(g, u)) <= TOL
    # the 12288 -> 4096 projection with a residual, one row (two rows of K = 12288 do not fit and take the other route)
    down = synthetic.make_packed(qt, 4096, 12288, seed=48, device=dev)
    xd = synthetic.make_activations(2, 12288, seed=91, device=dev)
    res = synthetic.make_activations(2, 4096, seed=92, device=dev)
    y2 = ops.linear_residual(xd, down, qt, res)
    y1 = ops.linear_residual(xd[:1].contiguous(), down, qt, res[:1].contiguous())
    assert torch.equal(y1, y2[:1])
    _sample_check(ops.linear(xd[:1].contiguous(), down, qt), xd[:1].contiguous(), down, qt, gen, "staged down m=1")
