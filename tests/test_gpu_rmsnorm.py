"""GPU: RMSNorm fused in front of the decode projections (sngguf_rmsnorm_linear, sngguf_rmsnorm_gate_up_silu)
against the oracle's norm followed by the oracle's projection, and against the library's own unfused entry points
fed with the oracle's normalized rows."""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import ops, synthetic

pytestmark = pytest.mark.gpu
TOL = 1e-3   # rel-L2 of the bf16 outputs
EPS = 1e-6   # rms_norm_eps of the 8B configuration


def _gamma(k, seed):
    return (torch.rand(k, generator=torch.Generator().manual_seed(seed)) * 1.5 + 0.25).to(torch.bfloat16)


# (m, n, k): the stacked q|k|v and single projections (block-aligned kernel), the lm_head-like wide matrix
# (line-aligned kernel), small K with several rows, N not a multiple of 16
LINEAR_SHAPES = [(1, 6144, 4096), (1, 4096, 4096), (1, 1024, 4096), (1, 40000, 4096), (3, 2048, 2048), (2, 1000, 2048),
                 (7, 530, 512), (16, 64, 256), (1, 37, 256), (1, 4096, 6144)]


@pytest.mark.parametrize("numerics", [0, 1])
@pytest.mark.parametrize("shape", LINEAR_SHAPES)
def test_rmsnorm_linear_parity(dev, numerics, shape):
    m, n, k = shape
    print(f"case rmsnorm_linear m={m} n={n} k={k} numerics={numerics}", flush=True)
    assert ops.rmsnorm_fits(go.Q8_0, m, k)
    packed = synthetic.make_packed(go.Q8_0, n, k, seed=n + k)
    x = (synthetic.make_activations(m, k, seed=m + k).float() * 3.0).to(torch.bfloat16)   # rows off unit RMS
    gamma = _gamma(k, k)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.bfloat16) if n % 2 else None
    normed = go.qwen3_rms_norm(x, gamma, EPS)
    want = go.gguf_linear_forward(normed, packed, go.Q8_0, bias, numerics=numerics)
    pd = packed.to(dev)
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.rmsnorm_linear_into(x.to(dev), gamma.to(dev), EPS, pd, go.Q8_0, bias.to(dev) if bias is not None else None, y, numerics)
    assert bool(torch.isfinite(y.float()).all())
    assert go.rel_l2(y.cpu(), want) <= TOL
    # against the unfused kernel on the oracle's normalized rows: the same weights and rounding chain; what differs is
    # the summation order and, rarely, one bf16 step in a normalized value
    unfused = ops.linear(normed.to(dev), pd, go.Q8_0, bias.to(dev) if bias is not None else None, numerics)
    assert go.rel_l2(y.cpu(), unfused.cpu()) <= 5e-4


@pytest.mark.parametrize("shape", [(1, 12288, 4096), (1, 1000, 4096), (3, 4096, 2048), (2, 48, 256), (1, 12288, 6144)])
def test_rmsnorm_gate_up_silu_parity(dev, c_oracle, shape):
    m, n, k = shape
    print(f"case rmsnorm_gate_up m={m} n={n} k={k}", flush=True)
    gate = synthetic.make_packed(go.Q8_0, n, k, seed=81)
    up = synthetic.make_packed(go.Q8_0, n, k, seed=82)
    x = (synthetic.make_activations(m, k, seed=83 + m).float() * 0.3).to(torch.bfloat16)
    gamma = _gamma(k, 84)
    normed = go.qwen3_rms_norm(x, gamma, EPS)
    g = go.gguf_linear_forward(normed, gate, go.Q8_0)
    u = go.gguf_linear_forward(normed, up, go.Q8_0)
    h = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.rmsnorm_gate_up_silu_into(x.to(dev), gamma.to(dev), EPS, gate.to(dev), up.to(dev), go.Q8_0, h, 1)
    assert bool(torch.isfinite(h.float()).all())
    assert go.rel_l2(h.cpu(), torch.nn.functional.silu(g) * u) <= TOL
    assert go.rel_l2(h.cpu(), c_oracle.silu_mul(g, u)) <= TOL


OTHER_TYPES = [go.Q4_0, go.Q4_1, go.Q5_0, go.Q5_1, go.Q2_K, go.Q3_K, go.Q4_K, go.Q5_K, go.Q6_K]


@pytest.mark.parametrize("qt", OTHER_TYPES)
def test_rmsnorm_other_formats_parity(dev, c_oracle, qt):
    """The fused norm in the kernel of the nine other formats: projection with bias (both numerics), a vocabulary-wide
    one (two row groups per wavefront) and the gated pair."""
    for m, n, k in [(1, 6144, 4096), (3, 530, 2048), (16, 37, 256)] + ([(1, 40000, 1024)] if qt in (go.Q4_K, go.Q6_K) else []) \
            + ([(1, 33000, 4096)] if qt in (go.Q6_K, go.Q5_1) else []):   # lm_head-like: the largest slabs + staged activations
        print(f"case rmsnorm_kq qt={qt} m={m} n={n} k={k}", flush=True)
        assert ops.rmsnorm_fits(qt, m, k)
        gate = synthetic.make_packed(qt, n, k, seed=111)
        up = synthetic.make_packed(qt, n, k, seed=112)
        x = (synthetic.make_activations(m, k, seed=113 + m).float() * 2.5).to(torch.bfloat16)
        gamma = _gamma(k, 114)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.bfloat16)
        normed = go.qwen3_rms_norm(x, gamma, EPS)
        gd, ud = gate.to(dev), up.to(dev)
        for numerics in (0, 1):
            want = go.gguf_linear_forward(normed, gate, qt, bias, numerics=numerics)
            y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
            ops.rmsnorm_linear_into(x.to(dev), gamma.to(dev), EPS, gd, qt, bias.to(dev), y, numerics)
            assert bool(torch.isfinite(y.float()).all())
            assert go.rel_l2(y.cpu(), want) <= TOL, (m, n, k, numerics)
        g = go.gguf_linear_forward(normed, gate, qt)
        u = go.gguf_linear_forward(normed, up, qt)
        h = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.rmsnorm_gate_up_silu_into(x.to(dev), gamma.to(dev), EPS, gd, ud, qt, h, 1)
        assert go.rel_l2(h.cpu(), c_oracle.silu_mul(g, u)) <= TOL, (m, n, k)


def test_normalized_rows_match_the_oracle_elementwise(dev):
    """An identity-like weight (scale 1.0, one quant of 1 per row) makes the projection return the normalized row itself:
    every element must equal the oracle's, up to one bf16 step in the rare near-tie of the first rounding."""
    for m, k in [(1, 4096), (3, 2048), (1, 256)]:
        print(f"case rmsnorm_identity m={m} k={k}", flush=True)
        blocks = torch.zeros((k, k // 32, 34), dtype=torch.uint8)
        blocks[:, :, 0:2] = torch.tensor([0x00, 0x3C], dtype=torch.uint8)     # fp16 1.0, little-endian
        idx = torch.arange(k)
        blocks[idx, idx // 32, 2 + idx % 32] = 1
        packed = blocks.view(k, -1).contiguous()
        x = (synthetic.make_activations(m, k, seed=91 + k).float() * 5.0).to(torch.bfloat16)
        gamma = _gamma(k, 92)
        want = go.qwen3_rms_norm(x, gamma, EPS)
        y = torch.empty((m, k), dtype=torch.bfloat16, device=dev)
        ops.rmsnorm_linear_into(x.to(dev), gamma.to(dev), EPS, packed.to(dev), go.Q8_0, None, y, 1)
        diff = (y.cpu().float() - want.float()).abs()
        assert float((diff > 0).float().mean()) < 0.01
        assert bool((diff <= want.float().abs() * 2 ** -6 + 1e-30).all())


def test_rmsnorm_argument_errors(dev):
    packed = synthetic.make_packed(go.Q8_0, 64, 4096, seed=1).to(dev)
    gamma = _gamma(4096, 2).to(dev)
    x = synthetic.make_activations(5, 4096, seed=3).to(dev)
    y = torch.empty((5, 64), dtype=torch.bfloat16, device=dev)
    assert not ops.rmsnorm_fits(go.Q8_0, 5, 4096)           # five rows of 4096 do not fit the staging area
    assert ops.rmsnorm_fits(go.Q4_K, 1, 4096) and not ops.rmsnorm_fits(go.Q4_0, 1, 4096 + 32)
    with pytest.raises(ops.SnGgufError):
        ops.rmsnorm_linear_into(x, gamma, EPS, packed, go.Q8_0, None, y, 1)
    with pytest.raises(ops.SnGgufError):
        ops.rmsnorm_linear_into(x[:1], None, EPS, packed, go.Q8_0, None, y[:1], 1)          # gamma required
    q40 = synthetic.make_packed(go.Q4_0, 64, 4096 + 32, seed=4).to(dev)
    with pytest.raises(ops.SnGgufError):
        ops.rmsnorm_linear_into(synthetic.make_activations(1, 4096 + 32, seed=5).to(dev), gamma, EPS, q40, go.Q4_0, None, y[:1], 1)   # K % 256
    with pytest.raises(ops.SnGgufError):
        ops.rmsnorm_linear_into(x[:1], gamma, -1.0, packed, go.Q8_0, None, y[:1], 1)        # eps < 0


@pytest.mark.parametrize("shape", [(1, 6144, 4096), (1, 1030, 4096), (3, 2048, 2048), (5, 37, 256)])
def test_rmsnorm_tiled_parity(dev, c_oracle, shape):
    """The same fusion on the operand-order copy of the weights: linear (with bias) and the gated pair."""
    m, n, k = shape
    print(f"case rmsnorm_tiled m={m} n={n} k={k}", flush=True)
    gate = synthetic.make_packed(go.Q8_0, n, k, seed=101)
    up = synthetic.make_packed(go.Q8_0, n, k, seed=102)
    x = (synthetic.make_activations(m, k, seed=103 + m).float() * 1.7).to(torch.bfloat16)
    gamma = _gamma(k, 104)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.bfloat16)
    normed = go.qwen3_rms_norm(x, gamma, EPS)
    tg, tu = ops.q8_0_tile(gate.to(dev)), ops.q8_0_tile(up.to(dev))
    for numerics in (0, 1):
        want = go.gguf_linear_forward(normed, gate, go.Q8_0, bias, numerics=numerics)
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.rmsnorm_linear_tiled_into(x.to(dev), gamma.to(dev), EPS, tg, bias.to(dev), y, numerics)
        assert go.rel_l2(y.cpu(), want) <= TOL
    g = go.gguf_linear_forward(normed, gate, go.Q8_0)
    u = go.gguf_linear_forward(normed, up, go.Q8_0)
    h = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.rmsnorm_gate_up_silu_tiled_into(x.to(dev), gamma.to(dev), EPS, tg, tu, h, 1)
    assert go.rel_l2(h.cpu(), c_oracle.silu_mul(g, u)) <= TOL
    # the fused norm of the two layouts works on the same staged rows: same normalized values, another summation order
    h_native = torch.empty_like(h)
    ops.rmsnorm_gate_up_silu_into(x.to(dev), gamma.to(dev), EPS, gate.to(dev), up.to(dev), go.Q8_0, h_native, 1)
    assert go.rel_l2(h.cpu(), h_native.cpu()) <= 5e-4
    if 16 * (2 * k + 64) > 36864:      # sixteen rows of this width do not fit the staging area
        big = synthetic.make_activations(16, k, seed=1).to(dev)
        with pytest.raises(ops.SnGgufError):
            ops.rmsnorm_linear_tiled_into(big, gamma.to(dev), EPS, tg, None, torch.empty((16, n), dtype=torch.bfloat16, device=dev), 1)


@pytest.mark.parametrize("m,k", [(1, 4096), (4, 4096), (16, 4096), (3, 264), (40, 12288), (2, 16384), (2, 20480), (0, 64)])
def test_standalone_rmsnorm_launch(dev, m, k):
    """sngguf_rmsnorm against the oracle's Qwen3RMSNorm: the row statistic is summed in another order, so a normalized
    value may sit one bf16 step off on a near tie; everything else is the same two roundings."""
    print(f"case rmsnorm standalone m={m} k={k}", flush=True)
    x = (synthetic.make_activations(max(m, 1), k, seed=m + k).float() * 2.5).to(torch.bfloat16)[:m]
    gamma = _gamma(k, k + 1)
    got = ops.rms_norm(x.to(dev), gamma.to(dev), EPS).cpu()
    assert got.shape == x.shape and got.dtype == torch.bfloat16
    if m == 0:
        return
    want = go.qwen3_rms_norm(x, gamma, EPS)
    assert go.rel_l2(got, want) <= 1e-3
    frac = (got.view(torch.int16) != want.view(torch.int16)).float().mean().item()
    assert frac < 0.01, frac
    step = (got.float() - want.float()).abs() <= want.float().abs() * 2.0 ** -7 + 1e-30
    assert bool(step.all())
    # identity weight: the normalized rows themselves
    one = torch.ones(k, dtype=torch.bfloat16)
    got1 = ops.rms_norm(x.to(dev), one.to(dev), EPS).cpu()
    assert (got1.view(torch.int16) != go.qwen3_rms_norm(x, one, EPS).view(torch.int16)).float().mean().item() < 0.01


@pytest.mark.parametrize("k", [4096, 16384, 20480])
def test_standalone_rmsnorm_in_place(dev, k):
    """y may be x: rows held in registers (K <= 16384) and rows re-read while they are written (K > 16384)."""
    print(f"case rmsnorm in place k={k}", flush=True)
    x = (synthetic.make_activations(3, k, seed=k).float() * 1.9).to(torch.bfloat16).to(dev)
    gamma = _gamma(k, 4).to(dev)
    want = ops.rms_norm(x, gamma, EPS)
    buf = x.clone()
    lib = ops.load_library()
    import ctypes
    rc = lib.sngguf_rmsnorm(ctypes.c_void_p(buf.data_ptr()), 3, k, ctypes.c_void_p(gamma.data_ptr()), ctypes.c_float(EPS),
                            ctypes.c_void_p(buf.data_ptr()), ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(buf, want)


def test_module_helpers_use_the_library_norm_beyond_the_fused_row_count(dev):
    from sensenova_u1_amd import GGUFLinear, GGUFParameter
    from sensenova_u1_amd.quantized_linear import rms_norm
    n, k = 512, 4096
    packed = synthetic.make_packed(go.Q8_0, n, k, seed=7)
    lin = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16, device="meta")
    lin.weight = GGUFParameter(packed.to(dev), quant_type=go.Q8_0)
    gamma = _gamma(k, 3)
    for m in (5, 16, 100):
        x = (synthetic.make_activations(m, k, seed=m).float() * 1.7).to(torch.bfloat16)
        assert not ops.rmsnorm_fits(go.Q8_0, m, k)
        got = lin.forward_normed(x.to(dev), gamma.to(dev), EPS).cpu()
        want = go.gguf_linear_forward(go.qwen3_rms_norm(x, gamma, EPS), packed, go.Q8_0)
        assert go.rel_l2(got, want) <= TOL
        assert torch.equal(rms_norm(x.to(dev), gamma.to(dev), EPS), ops.rms_norm(x.to(dev), gamma.to(dev), EPS))


@pytest.mark.parametrize("qt", [go.Q8_0, go.Q4_K, go.Q6_K])
@pytest.mark.parametrize("m", [2, 3, 4])
def test_fused_norm_for_a_few_decode_rows_at_hidden_4096(dev, c_oracle, qt, m):
    """Two to four decode rows at K = 4096 (the MLP configuration's M = 4): the norm rides inside the q|k|v-shaped
    projection (block-aligned kernel), the vocabulary-sized one and the gate / up pair (line-aligned kernel for Q8_0)."""
    print(f"case rmsnorm few rows qt={qt} m={m}", flush=True)
    k = 4096
    assert ops.rmsnorm_fits(qt, m, k) and not ops.rmsnorm_fits(qt, 5, k)
    gamma = _gamma(k, 9)
    x = (synthetic.make_activations(m, k, seed=90 + m).float() * 1.3).to(torch.bfloat16)
    normed = go.qwen3_rms_norm(x, gamma, EPS)
    for n in (6144, 530, 40000):
        packed = synthetic.make_packed(qt, n, k, seed=n)
        cols = torch.randint(0, n, (96,), generator=torch.Generator().manual_seed(n))
        want = go.gguf_linear_forward(normed, packed[cols], qt)
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.rmsnorm_linear_into(x.to(dev), gamma.to(dev), EPS, packed.to(dev), qt, None, y, 1)
        assert bool(torch.isfinite(y.float()).all())
        assert go.rel_l2(y[:, cols.to(dev)].cpu(), want) <= TOL, n
    n = 12288
    gate, up = synthetic.make_packed(qt, n, k, seed=1, device=dev), synthetic.make_packed(qt, n, k, seed=2, device=dev)
    cols = torch.randint(0, n, (96,), generator=torch.Generator().manual_seed(3))
    g = go.gguf_linear_forward(normed, gate[cols.to(dev)].cpu(), qt)
    u = go.gguf_linear_forward(normed, up[cols.to(dev)].cpu(), qt)
    h = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.rmsnorm_gate_up_silu_into(x.to(dev), gamma.to(dev), EPS, gate, up, qt, h, 1)
    assert go.rel_l2(h[:, cols.to(dev)].cpu(), c_oracle.silu_mul(g, u)) <= TOL
