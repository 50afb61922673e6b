"""GPU parity of the routes the host layer takes by default at the benchmark configurations' real shapes.

Beyond 64 rows ``GGUFLinear.forward`` (policy "auto") and ``modality.grouped_linear`` with ``n_text`` run the
workspace routes (``sngguf_linear_ws`` / ``sngguf_grouped_linear_ws`` on the pooled workspace): a weight pass + the
dense tile kernel for thousands of rows, a K split over workgroups for a few hundred.  These tests launch those routes
with the mixed layer's real geometry - 512 text rows + 4096 image rows on the four projection shapes - and compare a
sample of output rows x columns of either group with the CPU oracle on exactly those weight rows (rel-L2 <= 1e-3)."""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import GGUFLinear, GGUFParameter, grouped_linear, ops, synthetic

pytestmark = pytest.mark.gpu
TOL = 1e-3
SHAPES = [(4096, 4096), (1024, 4096), (12288, 4096), (4096, 12288)]


def _sample(y, x, packed, qt, rows, gen, what, n_cols=40):
    n = y.shape[1]
    dev = y.device
    cols = torch.randint(0, n, (n_cols,), generator=gen)
    cols[0], cols[1] = 0, n - 1
    want = go.gguf_linear_forward(x[rows.to(dev)].cpu(), packed[cols.to(dev)].cpu(), qt)
    err = go.rel_l2(y[rows.to(dev)][:, cols.to(dev)].cpu(), want)
    assert err <= TOL, f"{what}: rel-L2 {err:.3e}"


def _module(packed, n, k, qt=go.Q8_0):
    lin = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16, device="meta")
    lin.weight = GGUFParameter(packed, quant_type=qt)
    return lin


@pytest.mark.parametrize("n,k", SHAPES)
def test_grouped_workspace_route_at_the_mixed_layer_geometry(dev, n, k):
    """sngguf_grouped_linear_ws, 512 text rows -> understanding weights, 4096 image rows -> generation weights."""
    print(f"case default route grouped {n}x{k}", flush=True)
    n_text, m = 512, 4608
    gen = torch.Generator().manual_seed(n + k)
    und = synthetic.make_packed(go.Q8_0, n, k, seed=31, device=dev)
    gnr = synthetic.make_packed(go.Q8_0, n, k, seed=32, device=dev)
    x = synthetic.make_activations(m, k, seed=33, device=dev)
    dws = torch.empty(2 * ops.linear_workspace_bytes(12288, 4096), dtype=torch.uint8, device=dev)   # the bench's shared workspace
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.grouped_linear_ws_into(x, None, n_text, und, go.Q8_0, gnr, go.Q8_0, None, None, y, None, dws, ops.NUM_UPSTREAM_FP16)
    assert bool(torch.isfinite(y.float()).all())
    text_rows = torch.randint(0, n_text, (12,), generator=gen)
    text_rows[0], text_rows[1] = 0, n_text - 1
    image_rows = torch.randint(n_text, m, (12,), generator=gen)
    image_rows[0], image_rows[1] = n_text, m - 1
    _sample(y, x, und, go.Q8_0, text_rows, gen, "text group")
    _sample(y, x, gnr, go.Q8_0, image_rows, gen, "image group")
    # the definition of the launcher: two independent linears on the two row ranges
    ya = torch.empty((n_text, n), dtype=torch.bfloat16, device=dev)
    yb = torch.empty((m - n_text, n), dtype=torch.bfloat16, device=dev)
    ops.linear_ws_into(x[:n_text], und, go.Q8_0, None, ya, dws, ops.NUM_UPSTREAM_FP16)
    ops.linear_ws_into(x[n_text:], gnr, go.Q8_0, None, yb, dws, ops.NUM_UPSTREAM_FP16)
    ref = torch.cat([ya, yb], dim=0)
    assert go.rel_l2(y.cpu(), ref.cpu()) <= 1e-4     # same bf16 weights and products; K may be cut differently
    # ... and through the host layer's own entry (pooled workspace)
    got = grouped_linear(x, None, _module(und, n, k), _module(gnr, n, k), n_text=n_text)
    assert go.rel_l2(got.cpu(), y.cpu()) <= 1e-4


@pytest.mark.parametrize("n,k", [(12288, 4096), (4096, 12288)])
def test_module_forward_and_workspace_route_over_image_rows(dev, n, k):
    """GGUFLinear.forward under policy "auto" and sngguf_linear_ws at M = 4096 on the two MLP shapes (Q8_0)."""
    print(f"case default route module {n}x{k}", flush=True)
    m = 4096
    gen = torch.Generator().manual_seed(n - k)
    packed = synthetic.make_packed(go.Q8_0, n, k, seed=34, device=dev)
    x = synthetic.make_activations(m, k, seed=35, device=dev)
    rows = torch.randint(0, m, (16,), generator=gen)
    rows[0], rows[1] = 0, m - 1
    lin = _module(packed, n, k)
    assert lin.gemm_policy == "auto"
    y = lin(x)
    assert y.shape == (m, n) and bool(torch.isfinite(y.float()).all())
    _sample(y, x, packed, go.Q8_0, rows, gen, "module forward")
    ws = torch.empty(ops.linear_workspace_bytes(n, k), dtype=torch.uint8, device=dev)
    y2 = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.linear_ws_into(x, packed, go.Q8_0, None, y2, ws, ops.NUM_UPSTREAM_FP16)
    _sample(y2, x, packed, go.Q8_0, rows, gen, "linear_ws")
    assert torch.equal(y, y2)
