"""GPU parity: fused dequant-GEMV, dequant-GEMM, SiLU-gated pair and the modality-grouped
launcher against the CPU oracle (rel-L2 <= 1e-3 in bf16, the tolerance of the task)."""
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import ops, synthetic

pytestmark = pytest.mark.gpu

TOL = 1e-3          # rel-L2 bound on bf16 outputs
TYPES = [go.Q4_0, go.Q4_1, go.Q5_0, go.Q5_1, go.Q8_0, go.Q2_K, go.Q3_K, go.Q4_K, go.Q5_K, go.Q6_K]


def _check(got, want, tol=TOL):
    err = go.rel_l2(got, want)
    assert err <= tol, f"rel-L2 {err:.3e} > {tol}"
    return err


@pytest.mark.parametrize("qt", TYPES)
def test_linear_with_workspace_split_k(dev, qt):
    """sngguf_linear_ws on problems with few output tiles (some hundred rows, or a narrow matrix): K is split over
    several workgroups per tile and the fp32 partial sums are added in a second pass.  Q8_0 / Q4_K keep the sums in
    the plain 2 N K workspace, the other formats behind the decoded weights when the workspace is larger."""
    print(f"case linear_ws_splitk qt={qt}", flush=True)
    for numerics, (m, n, k) in [(1, (128, 1024, 4096)), (0, (300, 2050, 1024)), (1, (65, 37, 512)), (1, (512, 4096, 2048)),
                                (0, (1000, 515, 768))]:
        packed = synthetic.make_packed(qt, n, k, seed=m + n + k + qt)
        x = synthetic.make_activations(m, k, seed=m)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(k)) * 0.5).to(torch.bfloat16) if n % 2 else None
        want = go.gguf_linear_forward(x, packed, qt, bias, numerics=numerics)
        xd, pd = x.to(dev), packed.to(dev)
        bd = bias.to(dev) if bias is not None else None
        for extra in (0, 4 * 16 * m * n):
            ws = torch.full(((ops.linear_workspace_bytes(n, k) + extra) // 2,), float("nan"), dtype=torch.bfloat16, device=dev)
            y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
            ops.linear_ws_into(xd, pd, qt, bd, y, ws, numerics)
            assert bool(torch.isfinite(y.float()).all())
            _check(y.cpu(), want)


@pytest.mark.parametrize("qt", TYPES)
@pytest.mark.parametrize("numerics", [0, 1])
@pytest.mark.parametrize("m", [1, 2, 3, 4, 7, 8, 16])
def test_gemv_parity(dev, qt, numerics, m):
    print(f"case gemv qt={qt} numerics={numerics} m={m}", flush=True)
    n, k = 192, 4096
    packed = synthetic.make_packed(qt, n, k, seed=qt * 10 + m)
    x = synthetic.make_activations(m, k, seed=100 + m)
    want = go.gguf_linear_forward(x, packed, qt, numerics=numerics)
    got = ops.linear(x.to(dev), packed.to(dev), qt, None, numerics).cpu()
    err = _check(got, want)
    # with the other rounding chain the weights differ in a few percent of positions: the
    # kernel must follow the chain it was asked for, so it sits closer to its own oracle
    other = go.gguf_linear_forward(x, packed, qt, numerics=1 - numerics)
    assert err <= go.rel_l2(got, other) + 1e-6


@pytest.mark.parametrize("qt", TYPES)
def test_gemv_shapes_bias_ragged(dev, c_oracle, qt):
    print(f"case gemv ragged qt={qt}", flush=True)
    for n, k, m in [(1, 256, 1), (5, 512, 3), (131, 768, 16), (64, 12288, 4)]:
        packed = synthetic.make_packed(qt, n, k, seed=n + k)
        x = synthetic.make_activations(m, k, seed=7)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.bfloat16)
        want = go.gguf_linear_forward(x, packed, qt, bias)
        got = ops.linear(x.to(dev), packed.to(dev), qt, bias.to(dev)).cpu()
        _check(got, want)
        _check(got, c_oracle.linear(x, packed, qt, bias))


@pytest.mark.parametrize("qt", [t for t in TYPES if t != go.Q8_0])
@pytest.mark.parametrize("numerics", [0, 1])
def test_gemv_k_quants_two_row_groups(dev, c_oracle, qt, numerics):
    """N >= 32768 puts two 16-row groups on one wavefront: ragged N (last group half empty, last
    row group missing), bias, one and several super-blocks per wavefront, plain and SiLU-gated."""
    print(f"case gemv k-quant wide qt={qt} numerics={numerics}", flush=True)
    for n, k, m in [(32776, 256, 16), (32791, 768, 5), (32768, 1024, 1)]:
        packed = synthetic.make_packed(qt, n, k, seed=n + k)
        x = synthetic.make_activations(m, k, seed=9)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.bfloat16)
        got = ops.linear(x.to(dev), packed.to(dev), qt, bias.to(dev), numerics).cpu()
        _check(got, c_oracle.linear(x, packed, qt, bias, numerics))
    n, k, m = 32784, 512, 3
    gate = synthetic.make_packed(qt, n, k, seed=21)
    up = synthetic.make_packed(qt, n, k, seed=22)
    x = synthetic.make_activations(m, k, seed=23)
    g = go.gguf_linear_forward(x, gate, qt, numerics=numerics)
    u = go.gguf_linear_forward(x, up, qt, numerics=numerics)
    got = ops.gate_up_silu(x.to(dev), gate.to(dev), up.to(dev), qt, numerics).cpu()
    _check(got, c_oracle.silu_mul(g, u))


@pytest.mark.parametrize("qt", [go.Q4_0, go.Q4_1, go.Q5_0, go.Q5_1])
@pytest.mark.parametrize("numerics", [0, 1])
def test_gemv_32_element_formats_ragged_k(dev, c_oracle, qt, numerics):
    """K a multiple of 32 but not of 256 (the vector-ALU path; rows only 2-byte aligned for the 18- and
    22-byte blocks), plain with bias and SiLU-gated."""
    print(f"case gemv ragged K qt={qt} numerics={numerics}", flush=True)
    for n, k, m in [(37, 32, 1), (130, 96, 16), (9, 4128, 5)]:
        packed = synthetic.make_packed(qt, n, k, seed=n + k)
        x = synthetic.make_activations(m, k, seed=k + 1)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.bfloat16)
        got = ops.linear(x.to(dev), packed.to(dev), qt, bias.to(dev), numerics).cpu()
        _check(got, c_oracle.linear(x, packed, qt, bias, numerics))
        up = synthetic.make_packed(qt, n, k, seed=n + k + 1)
        g = go.gguf_linear_forward(x, packed, qt, numerics=numerics)
        u = go.gguf_linear_forward(x, up, qt, numerics=numerics)
        got = ops.gate_up_silu(x.to(dev), packed.to(dev), up.to(dev), qt, numerics).cpu()
        _check(got, c_oracle.silu_mul(g, u))


@pytest.mark.parametrize("qt", TYPES)
@pytest.mark.parametrize("numerics", [0, 1])
def test_gemv_17_to_64_rows(dev, c_oracle, qt, numerics):
    """17 .. 64 activation rows with K % 256 == 0 stay on the decode kernel (2 .. 4 matrix operands per
    decoded weight fragment): every operand count, partly filled last operand, ragged N, bias, one and
    several super-blocks per wavefront."""
    print(f"case gemv 17..64 rows qt={qt} numerics={numerics}", flush=True)
    for n, k, m in [(192, 4096, 17), (131, 768, 32), (37, 256, 33), (64, 1024, 48), (20, 512, 49), (192, 2048, 64)]:
        packed = synthetic.make_packed(qt, n, k, seed=n + k + m)
        x = synthetic.make_activations(m, k, seed=m)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.bfloat16)
        got = ops.linear(x.to(dev), packed.to(dev), qt, bias.to(dev), numerics).cpu()
        err = _check(got, go.gguf_linear_forward(x, packed, qt, bias, numerics=numerics))
        other = go.gguf_linear_forward(x, packed, qt, bias, numerics=1 - numerics)
        assert err <= go.rel_l2(got, other) + 1e-6
    rows = torch.tensor([0, 15, 16, 47, 63])
    _check(got[rows], c_oracle.linear(x[rows], packed, qt, bias, numerics))


def test_gemv_q8_0_odd_block_count(dev):
    """K = 32 * odd: rows are 2-byte aligned and not a whole number of 64-element units."""
    print("case gemv odd blocks", flush=True)
    for k in (32, 96, 4128):
        packed = synthetic.make_packed(go.Q8_0, 37, k, seed=k)
        x = synthetic.make_activations(5, k, seed=k + 1)
        _check(ops.linear(x.to(dev), packed.to(dev), go.Q8_0).cpu(), go.gguf_linear_forward(x, packed, go.Q8_0))


@pytest.mark.parametrize("numerics", [0, 1])
@pytest.mark.parametrize("m", [1, 16, 512])
def test_q8_0_fp16_subnormal_products(dev, numerics, m):
    """Block scales so small that every d * q is an fp16 subnormal (d = 3 * 2^-24, |q| <= 127):
    the decode must keep them (a path that flushes fp16 subnormals would return zeros).  K covers
    the line-aligned (2048) and the block-aligned (256) GEMV fetch schemes and both GEMM kernels."""
    import numpy as np
    print(f"case fp16 subnormal products numerics={numerics} m={m}", flush=True)
    for n, k in [(2048, 2048), (48, 256), (512, 512)]:
        rng = np.random.default_rng(n + k)
        raw = np.empty((n, k // 32, 34), dtype=np.uint8)
        raw[..., :2] = np.array([3], dtype=np.uint16).view(np.uint8)      # fp16 bits 0x0003 = 3 * 2^-24
        raw[..., 2:] = rng.integers(-127, 128, size=(n, k // 32, 32), dtype=np.int8).view(np.uint8)
        packed = torch.from_numpy(raw.reshape(n, -1))
        x = (synthetic.make_activations(m, k, seed=k).float() * 4096).to(torch.bfloat16)
        want = go.gguf_linear_forward(x, packed, go.Q8_0, None, numerics=numerics)
        assert want.float().abs().max() > 0
        got = ops.linear(x.to(dev), packed.to(dev), go.Q8_0, None, numerics).cpu()
        _check(got, want)


@pytest.mark.parametrize("qt", [go.Q4_K, go.Q5_K])
@pytest.mark.parametrize("numerics", [0, 1])
def test_k_quant_decode_with_scale_products_on_both_sides_of_64(dev, c_oracle, qt, numerics):
    """The decode kernel of Q4_K / Q5_K forms q * D as one fused multiply-add around the constant -1024 * D where every
    |D| = |d * scale| of a wavefront is below 64 (so that the constant is exact in fp16), and keeps the separate
    subtraction and product elsewhere.  Super-block scales d of 2^-10, 1.5 and 24 with the 6-bit sub-scales put D far
    below 64, on both sides of it within one wavefront, and beyond the range where 1024 * D would still be finite:
    all must follow the oracle's chain; one and sixteen rows, the plain projection and the gated pair."""
    import numpy as np
    print(f"case k-quant scale products qt={qt} numerics={numerics}", flush=True)
    n, k = 96, 2048
    for m in (1, 16):
        for case, d_values in enumerate(([2.0 ** -10], [1.5], [24.0], [2.0 ** -10, 1.5, 24.0])):
            mats = []
            for which in range(2):
                raw = synthetic.make_packed(qt, n, k, seed=7 * case + which + m).numpy().copy()
                blocks = raw.reshape(n, k // 256, -1)
                rng = np.random.default_rng(case + which)
                d = rng.choice(np.array(d_values, dtype=np.float16), size=(n, k // 256))
                blocks[..., 0:2] = d.view(np.uint16)[..., None].view(np.uint8)
                blocks[..., 2:4] = np.array([0.25], dtype=np.float16).view(np.uint8)      # dmin
                mats.append(torch.from_numpy(raw))
            x = (synthetic.make_activations(m, k, seed=case + 3).float() / 64).to(torch.bfloat16)
            want = go.gguf_linear_forward(x, mats[0], qt, None, numerics=numerics)
            assert bool(torch.isfinite(want.float()).all()) and want.float().abs().max() > 0
            _check(ops.linear(x.to(dev), mats[0].to(dev), qt, None, numerics).cpu(), want)
            up = go.gguf_linear_forward(x, mats[1], qt, None, numerics=numerics)
            _check(ops.gate_up_silu(x.to(dev), mats[0].to(dev), mats[1].to(dev), qt, numerics).cpu(), c_oracle.silu_mul(want, up))


def test_gemv_fp64_bruteforce_tiny(dev):
    """Independent of torch's matmul: exact fp64 dot products on the bf16-rounded weights."""
    print("case gemv fp64", flush=True)
    for qt in TYPES:
        packed = synthetic.make_packed(qt, 16, 256, seed=qt)
        x = synthetic.make_activations(2, 256, seed=3)
        w = go.dequantize_gguf_tensor(packed, qt, 1).to(torch.bfloat16).double()
        want = (x.double() @ w.T).to(torch.bfloat16)
        _check(ops.linear(x.to(dev), packed.to(dev), qt).cpu(), want)


@pytest.mark.parametrize("qt", TYPES)
@pytest.mark.parametrize("numerics", [0, 1])
def test_gemm_parity(dev, qt, numerics):
    print(f"case gemm qt={qt} numerics={numerics}", flush=True)
    m, n, k = 300, 384, 1024
    packed = synthetic.make_packed(qt, n, k, seed=qt + 40)
    x = synthetic.make_activations(m, k, seed=41)
    want = go.gguf_linear_forward(x, packed, qt, numerics=numerics)
    got = ops.linear(x.to(dev), packed.to(dev), qt, None, numerics).cpu()
    err = _check(got, want)
    other = go.gguf_linear_forward(x, packed, qt, numerics=1 - numerics)
    assert err <= go.rel_l2(got, other) + 1e-6


@pytest.mark.parametrize("qt", TYPES)
def test_gemm_ragged_bias(dev, qt):
    print(f"case gemm ragged qt={qt}", flush=True)
    for m, n, k in [(17, 1, 256), (129, 130, 512), (64, 257, 768), (513, 100, 256)]:
        packed = synthetic.make_packed(qt, n, k, seed=m + n)
        x = synthetic.make_activations(m, k, seed=m)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(m)) * 0.5).to(torch.bfloat16)
        want = go.gguf_linear_forward(x, packed, qt, bias)
        got = ops.linear(x.to(dev), packed.to(dev), qt, bias.to(dev)).cpu()
        _check(got, want)


@pytest.mark.parametrize("numerics", [0, 1])
def test_gemm_q8_0_large_tile_kernel(dev, c_oracle, numerics):
    """M >= 384 with K % 64 == 0 takes the 256 x 256 tile kernel: ragged M / N, bias, one K step,
    odd and even step counts, a tile grid that divides into 4 x 8 blocks (blocked tile order) and
    grids that do not."""
    print(f"case gemm tiles numerics={numerics}", flush=True)
    for m, n, k in [(2816, 2816, 64), (2048, 4096, 128), (3000, 2904, 320), (3000, 2900, 192), (4100, 2050, 128), (8300, 1030, 64)]:
        packed = synthetic.make_packed(go.Q8_0, n, k, seed=m + n + k)
        x = synthetic.make_activations(m, k, seed=m)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(k)) * 0.5).to(torch.bfloat16)
        want = go.gguf_linear_forward(x, packed, go.Q8_0, bias, numerics=numerics)
        got = ops.linear(x.to(dev), packed.to(dev), go.Q8_0, bias.to(dev), numerics).cpu()
        _check(got, want)
    rows = torch.tensor([0, 255, 256, 8299])
    sub = c_oracle.linear(x[rows], packed, go.Q8_0, bias, numerics)
    _check(got[rows], sub)


@pytest.mark.parametrize("qt", TYPES)
def test_linear_with_workspace(dev, qt):
    """sngguf_linear_ws: with a large enough workspace big problems go through the weight pass + the dense tile
    kernel (every type; ragged M / N, bias, one K step and many, odd and even step counts, blocked and plain tile
    order); with no or too small a workspace, or a problem below the thresholds, it is sngguf_linear."""
    print(f"case linear_ws qt={qt}", flush=True)
    bs = go.GGML_QUANT_SIZES[qt][0]
    for numerics, (m, n, k) in [(1, (3072, 2816, 256)), (0, (3000, 2904, 768)), (1, (2048, 4096, 512)), (1, (8300, 1030, 256))]:
        packed = synthetic.make_packed(qt, n, k, seed=m + n + k + qt)
        x = synthetic.make_activations(m, k, seed=m)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(k)) * 0.5).to(torch.bfloat16)
        want = go.gguf_linear_forward(x, packed, qt, bias, numerics=numerics)
        xd, pd, bd = x.to(dev), packed.to(dev), bias.to(dev)
        ws = torch.full((ops.linear_workspace_bytes(n, k) // 2,), float("nan"), dtype=torch.bfloat16, device=dev)
        y = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
        ops.linear_ws_into(xd, pd, qt, bd, y, ws, numerics)
        _check(y.cpu(), want)
        # the workspace now holds the decoded weight: bit-identical to the standalone dequantize
        assert torch.equal(ws.view(n, k), ops.dequantize(pd, qt, torch.bfloat16, numerics))
        fused = ops.linear(xd, pd, qt, bd, numerics)
        for small in (None, ws[:n * k - 8]):
            y2 = torch.empty_like(y)
            ops.linear_ws_into(xd, pd, qt, bd, y2, small, numerics)
            assert torch.equal(y2, fused)
    # below the thresholds (few rows): the fused path although a workspace is there
    x = synthetic.make_activations(40, k, seed=4).to(dev)
    y3 = torch.empty((40, n), dtype=torch.bfloat16, device=dev)
    ws.fill_(float("nan"))
    ops.linear_ws_into(x, pd, qt, None, y3, ws, 1)
    assert torch.equal(y3, ops.linear(x, pd, qt, None, 1)) and bool(torch.isnan(ws.float()).all())
    assert bs in (32, 256)


@pytest.mark.parametrize("numerics", [0, 1])
def test_gemm_q4_k_large_tile_kernel(dev, c_oracle, numerics):
    """Q4_K through the 256 x 256 tile kernel (M >= 384, at least 128 tiles): every chunk position of
    a super-block (K steps 0..3 and beyond), ragged M / N, both output paths, bias."""
    print(f"case gemm q4_k tiles numerics={numerics}", flush=True)
    for m, n, k in [(2048, 4096, 256), (3000, 2904, 256), (4100, 2050, 512), (3072, 3080, 1280)]:
        packed = synthetic.make_packed(go.Q4_K, n, k, seed=m + n + k)
        x = synthetic.make_activations(m, k, seed=m)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(k)) * 0.5).to(torch.bfloat16)
        want = go.gguf_linear_forward(x, packed, go.Q4_K, bias, numerics=numerics)
        got = ops.linear(x.to(dev), packed.to(dev), go.Q4_K, bias.to(dev), numerics).cpu()
        err = _check(got, want)
        other = go.gguf_linear_forward(x, packed, go.Q4_K, bias, numerics=1 - numerics)
        assert err <= go.rel_l2(got, other) + 1e-6
    rows = torch.tensor([0, 255, 256, 3071])
    sub = c_oracle.linear(x[rows], packed, go.Q4_K, bias, numerics)
    _check(got[rows], sub)


def test_grouped_linear_large_tiles(dev):
    """Grouped routing through the tile kernel: indicator form and contiguous split, group sizes
    that are not multiples of the tile."""
    print("case grouped tiles", flush=True)
    _grouped_large_tiles(dev, 4500, 2100, 128)   # rows of y 8-byte aligned
    _grouped_large_tiles(dev, 4500, 2104, 256)   # rows of y 16-byte aligned: coalesced store path


def _grouped_large_tiles(dev, m, n, k):
    wu = synthetic.make_packed(go.Q8_0, n, k, seed=11)
    wg = synthetic.make_packed(go.Q8_0, n, k, seed=12)
    x = synthetic.make_activations(m, k, seed=13)
    ind = torch.rand(m, generator=torch.Generator().manual_seed(14)) < 0.7
    got = ops.grouped_linear(x.to(dev), ind.to(dev), 0, wu.to(dev), go.Q8_0, wg.to(dev), go.Q8_0).cpu()
    _check(got, go.grouped_linear_forward(x, ind, wu, go.Q8_0, wg, go.Q8_0))
    split = torch.arange(m) >= 530
    got = ops.grouped_linear(x.to(dev), None, 530, wu.to(dev), go.Q8_0, wg.to(dev), go.Q8_0).cpu()
    _check(got, go.grouped_linear_forward(x, split, wu, go.Q8_0, wg, go.Q8_0))
    yu = ops.linear(x.to(dev), wu.to(dev), go.Q8_0).cpu()
    yg = ops.linear(x.to(dev), wg.to(dev), go.Q8_0).cpu()
    assert torch.equal(got[~split], yu[~split]) and torch.equal(got[split], yg[split])


@pytest.mark.parametrize("qt", [go.Q8_0, go.Q4_K])
def test_grouped_linear_split_k(dev, qt):
    """sngguf_grouped_linear_ws on a narrow matrix (few output tiles) of a type the large-tile kernel decodes: K split over
    workgroups, partial sums in the dense workspace, the reduce pass adding each row's own group bias - with a row map
    and with the contiguous split, ragged N, an empty group."""
    print(f"case grouped_splitk qt={qt}", flush=True)
    for m, n, k, n_text in [(700, 1024, 1024, 300), (4608, 1030, 512, 512), (130, 257, 2048, 0), (1000, 515, 768, 1000)]:
        und = synthetic.make_packed(qt, n, k, seed=61)
        gen = synthetic.make_packed(qt, n, k, seed=62)
        x = synthetic.make_activations(m, k, seed=63)
        g = torch.Generator().manual_seed(64)
        ind = torch.rand(m, generator=g) < 0.6
        bu = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16)
        bg = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16)
        want = torch.empty((m, n), dtype=torch.bfloat16)
        want[~ind] = go.gguf_linear_forward(x[~ind], und, qt, bu)
        want[ind] = go.gguf_linear_forward(x[ind], gen, qt, bg)
        xd, ud, gd, bud, bgd = x.to(dev), und.to(dev), gen.to(dev), bu.to(dev), bg.to(dev)
        ws = torch.empty(ops.grouped_workspace_bytes(m), dtype=torch.uint8, device=dev)
        dw = torch.full((4 * 16 * m * n // 2,), float("nan"), dtype=torch.bfloat16, device=dev)   # room for 16 slices
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.grouped_linear_ws_into(xd, ind.to(torch.uint8).to(dev), 0, ud, qt, gd, qt, bud, bgd, y, ws, dw, 1)
        assert bool(torch.isfinite(y.float()).all())
        _check(y.cpu(), want)
        want2 = torch.cat([go.gguf_linear_forward(x[:n_text], und, qt, bu), go.gguf_linear_forward(x[n_text:], gen, qt, bg)])
        y2 = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ops.grouped_linear_ws_into(xd, None, n_text, ud, qt, gd, qt, bud, bgd, y2, None, dw, 0)
        want2 = torch.cat([go.gguf_linear_forward(x[:n_text], und, qt, bu, numerics=0), go.gguf_linear_forward(x[n_text:], gen, qt, bg, numerics=0)])
        _check(y2.cpu(), want2)


@pytest.mark.parametrize("qt_pair", [(go.Q8_0, go.Q8_0), (go.Q4_K, go.Q6_K), (go.Q5_0, go.Q3_K)])
def test_grouped_linear_with_dense_workspace(dev, qt_pair):
    """sngguf_grouped_linear_ws: both weight sets decoded once into the workspace, one dense launch over both row
    groups - equal quant types or not, with an indicator (row map) and with the contiguous split, biases; and the
    plain grouped launcher when the workspace is missing or too small."""
    qu, qg = qt_pair
    print(f"case grouped_ws {qu} {qg}", flush=True)
    m, n, k = 3100, 2904, 512
    und = synthetic.make_packed(qu, n, k, seed=51)
    gen = synthetic.make_packed(qg, n, k, seed=52)
    x = synthetic.make_activations(m, k, seed=53)
    g = torch.Generator().manual_seed(54)
    ind = torch.rand(m, generator=g) < 0.6
    bu = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16)
    bg = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16)
    want = torch.empty((m, n), dtype=torch.bfloat16)
    want[~ind] = go.gguf_linear_forward(x[~ind], und, qu, bu)
    want[ind] = go.gguf_linear_forward(x[ind], gen, qg, bg)
    xd, ud, gd, bud, bgd = x.to(dev), und.to(dev), gen.to(dev), bu.to(dev), bg.to(dev)
    indd = ind.to(torch.uint8).to(dev)
    ws = torch.empty(ops.grouped_workspace_bytes(m), dtype=torch.uint8, device=dev)
    dw = torch.empty(2 * ops.linear_workspace_bytes(n, k) // 2, dtype=torch.bfloat16, device=dev)
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.grouped_linear_ws_into(xd, indd, 0, ud, qu, gd, qg, bud, bgd, y, ws, dw, 1)
    _check(y.cpu(), want)
    assert torch.equal(dw[:n * k].view(n, k), ops.dequantize(ud, qu, torch.bfloat16, 1))
    assert torch.equal(dw[n * k:].view(n, k), ops.dequantize(gd, qg, torch.bfloat16, 1))
    # contiguous [text | image] layout, no row map
    n_text = 1300
    want2 = torch.cat([go.gguf_linear_forward(x[:n_text], und, qu, bu), go.gguf_linear_forward(x[n_text:], gen, qg, bg)])
    y2 = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.grouped_linear_ws_into(xd, None, n_text, ud, qu, gd, qg, bud, bgd, y2, None, dw, 1)
    _check(y2.cpu(), want2)
    # no / short dense workspace: the plain grouped launcher
    plain = torch.empty_like(y)
    ops.grouped_linear_into(xd, indd, 0, ud, qu, gd, qg, bud, bgd, plain, ws, 1)
    for short in (None, dw[:2 * n * k - 8]):
        y3 = torch.empty_like(y)
        ops.grouped_linear_ws_into(xd, indd, 0, ud, qu, gd, qg, bud, bgd, y3, ws, short, 1)
        assert torch.equal(y3, plain)


def test_gemm_q8_0_odd_block_count(dev):
    print("case gemm odd blocks", flush=True)
    packed = synthetic.make_packed(go.Q8_0, 70, 96, seed=1)
    x = synthetic.make_activations(40, 96, seed=2)
    _check(ops.linear(x.to(dev), packed.to(dev), go.Q8_0).cpu(), go.gguf_linear_forward(x, packed, go.Q8_0))


def test_gemm_leading_dims_and_linearity(dev):
    """[B, S, K] input keeps its leading dims; y(a) + y(b) == y(a + b) up to bf16 rounding."""
    print("case gemm leading dims", flush=True)
    packed = synthetic.make_packed(go.Q8_0, 256, 512, seed=8).to(dev)
    a = synthetic.make_activations(2 * 50, 512, seed=1).reshape(2, 50, 512).to(dev)
    y = ops.linear(a, packed, go.Q8_0)
    assert y.shape == (2, 50, 256)
    y2 = ops.linear(a.reshape(100, 512), packed, go.Q8_0)
    assert torch.equal(y.reshape(100, 256), y2)
    two = ops.linear((a * 2).contiguous(), packed, go.Q8_0)   # exact in bf16: power-of-two scaling
    assert torch.equal(two, y * 2)


@pytest.mark.parametrize("qt", TYPES)
@pytest.mark.parametrize("m", [1, 4, 16])
def test_gate_up_silu(dev, c_oracle, qt, m):
    print(f"case gate_up qt={qt} m={m}", flush=True)
    n, k = 160, 1024
    gate = synthetic.make_packed(qt, n, k, seed=1)
    up = synthetic.make_packed(qt, n, k, seed=2)
    x = synthetic.make_activations(m, k, seed=3)
    g = go.gguf_linear_forward(x, gate, qt)
    u = go.gguf_linear_forward(x, up, qt)
    want = torch.nn.functional.silu(g) * u
    got = ops.gate_up_silu(x.to(dev), gate.to(dev), up.to(dev), qt).cpu()
    _check(got, want)
    _check(got, c_oracle.silu_mul(g, u))


@pytest.mark.parametrize("m", [1, 2, 11, 12, 13, 16])
def test_gate_up_silu_line_aligned_kernel(dev, m):
    """Q8_0 gate/up with K a multiple of 2048 and enough row groups takes the line-aligned kernel: activations staged
    in LDS (m = 1), fetched per wavefront (m < 12), and from 12 rows on one wavefront working on both matrices of
    its K range; ragged N."""
    print(f"case gate_up span m={m}", flush=True)
    n, k = 8200, 4096
    gate = synthetic.make_packed(go.Q8_0, n, k, seed=61)
    up = synthetic.make_packed(go.Q8_0, n, k, seed=62)
    x = synthetic.make_activations(m, k, seed=63 + m)
    g = go.gguf_linear_forward(x, gate, go.Q8_0)
    u = go.gguf_linear_forward(x, up, go.Q8_0)
    got = ops.gate_up_silu(x.to(dev), gate.to(dev), up.to(dev), go.Q8_0).cpu()
    _check(got, torch.nn.functional.silu(g) * u)


@pytest.mark.parametrize("qt_pair", [(go.Q8_0, go.Q8_0), (go.Q4_K, go.Q4_K), (go.Q6_K, go.Q6_K), (go.Q4_K, go.Q6_K), (go.Q5_K, go.Q8_0),
                                     (go.Q4_0, go.Q3_K), (go.Q5_1, go.Q2_K)])
def test_grouped_linear_indicator(dev, qt_pair):
    print(f"case grouped indicator {qt_pair}", flush=True)
    qu, qg = qt_pair
    m, n, k = 333, 256, 512
    wu = synthetic.make_packed(qu, n, k, seed=1)
    wg = synthetic.make_packed(qg, n, k, seed=2)
    x = synthetic.make_activations(m, k, seed=3)
    gen = torch.Generator().manual_seed(4)
    for ind in (torch.rand(m, generator=gen) < 0.6, torch.zeros(m, dtype=torch.bool), torch.ones(m, dtype=torch.bool)):
        want = go.grouped_linear_forward(x, ind, wu, qu, wg, qg)
        got = ops.grouped_linear(x.to(dev), ind.to(dev), 0, wu.to(dev), qu, wg.to(dev), qg).cpu()
        _check(got, want)
        # definition: each row equals the plain linear of its own tower, bit for bit
        yu = ops.linear(x.to(dev), wu.to(dev), qu).cpu()
        yg = ops.linear(x.to(dev), wg.to(dev), qg).cpu()
        assert torch.equal(got[~ind], yu[~ind]) and torch.equal(got[ind], yg[ind])


def test_grouped_linear_contiguous_split_with_bias(dev, c_oracle):
    print("case grouped split", flush=True)
    m, n, k, n_text = 200, 128, 256, 72
    wu = synthetic.make_packed(go.Q8_0, n, k, seed=5)
    wg = synthetic.make_packed(go.Q8_0, n, k, seed=6)
    x = synthetic.make_activations(m, k, seed=7)
    bu = torch.linspace(-1, 1, n).to(torch.bfloat16)
    bg = torch.linspace(2, 3, n).to(torch.bfloat16)
    ind = torch.arange(m) >= n_text
    want = go.grouped_linear_forward(x, ind, wu, go.Q8_0, wg, go.Q8_0, bu, bg)
    got = ops.grouped_linear(x.to(dev), None, n_text, wu.to(dev), go.Q8_0, wg.to(dev), go.Q8_0, bu.to(dev),
                             bg.to(dev)).cpu()
    _check(got, want)
    _check(got, c_oracle.grouped_linear(x, ind, wu, go.Q8_0, wg, go.Q8_0, bu, bg))
    for edge in (0, m):
        ind = torch.arange(m) >= edge
        got = ops.grouped_linear(x.to(dev), None, edge, wu.to(dev), go.Q8_0, wg.to(dev), go.Q8_0).cpu()
        _check(got, go.grouped_linear_forward(x, ind, wu, go.Q8_0, wg, go.Q8_0))


def test_full_size_shapes_row_sample(dev):
    """The 8B backbone's projection shapes at full size; a sample of output rows / columns is checked against the
    oracle run on exactly those weight rows (an output element depends on one x row and one
    weight row only)."""
    print("case full size", flush=True)
    g = torch.Generator().manual_seed(0)
    for (n, k) in [(12288, 4096), (4096, 12288), (1024, 4096)]:
        packed = synthetic.make_packed(go.Q8_0, n, k, seed=n, device=dev)
        cols = torch.randint(0, n, (48,), generator=g)
        sub = packed[cols.to(dev)].cpu()
        for m in (1, 16, 4096):
            x = synthetic.make_activations(m, k, seed=m, device=dev)
            y = ops.linear(x, packed, go.Q8_0)
            rows = torch.randint(0, m, (min(m, 24),), generator=g)
            want = go.gguf_linear_forward(x[rows.to(dev)].cpu(), sub, go.Q8_0)
            _check(y[rows.to(dev)][:, cols.to(dev)].cpu(), want)


@pytest.mark.parametrize("qt", [go.Q8_0, go.Q4_K])
def test_vocabulary_sized_projection(dev, qt):
    """The largest linear of the model: lm_head, 151936 x 4096, at decode.  A sample of output
    columns is checked against the oracle run on exactly those weight rows; the row count is not a
    multiple of 256 and the byte offsets of the last rows exceed 2^29."""
    print(f"case lm_head qt={qt}", flush=True)
    n, k = 151936, 4096
    packed = synthetic.make_packed(qt, n, k, seed=5, device=dev)
    g = torch.Generator().manual_seed(1)
    cols = torch.cat([torch.randint(0, n, (60,), generator=g), torch.tensor([0, n - 1, n - 17, 75967])])
    sub = packed[cols.to(dev)].cpu()
    for m in (1, 5):
        x = synthetic.make_activations(m, k, seed=m, device=dev)
        y = ops.linear(x, packed, qt)
        assert y.shape == (m, n)
        _check(y[:, cols.to(dev)].cpu(), go.gguf_linear_forward(x.cpu(), sub, qt))
    assert torch.isfinite(y.float()).all()


@pytest.mark.parametrize("qt", TYPES)
def test_linear_residual(dev, qt):
    """residual + linear in one launch equals the two bf16 tensor operations, bit for bit against the library's own
    plain linear followed by torch's add (same kernel, same accumulation order), and within tolerance of the oracle:
    every kernel family (decode kernels, 17..64 rows, 128- and 256-tile GEMM, ragged N, odd K)."""
    print(f"case linear residual qt={qt}", flush=True)
    bs = go.GGML_QUANT_SIZES[qt][0]
    shapes = [(1, 192, 4096), (5, 37, 512), (16, 130, 768), (40, 64, 1024), (100, 131, 512), (513, 260, 256)]
    if bs == 32:
        shapes += [(3, 50, 96), (70, 33, 160)]
    if qt in (go.Q8_0, go.Q4_K):
        shapes += [(2048, 4096, 256)]
    for m, n, k in shapes:
        packed = synthetic.make_packed(qt, n, k, seed=m + n + k).to(dev)
        x = synthetic.make_activations(m, k, seed=m).to(dev)
        res = synthetic.make_activations(m, n, seed=n).to(dev)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.bfloat16).to(dev)
        for b in (None, bias):
            got = ops.linear_residual(x, packed, qt, res, b)
            plain = ops.linear(x, packed, qt, b)
            assert torch.equal(got, res + plain), (m, n, k, b is not None)
        want = res.cpu() + go.gguf_linear_forward(x.cpu(), packed.cpu(), qt, bias.cpu())
        _check(got.cpu(), want)
    with pytest.raises(ops.SnGgufError):
        ops.linear_residual(x, packed, qt, res[:, :-1].contiguous())


def test_linear_errors(dev):
    packed = synthetic.make_packed(go.Q8_0, 8, 64).to(dev)
    with pytest.raises(ops.SnGgufError):
        ops.linear(torch.zeros(2, 64, device=dev), packed, go.Q8_0)            # fp32 activations
    with pytest.raises(ops.SnGgufError):
        ops.linear(torch.zeros(2, 32, device=dev, dtype=torch.bfloat16), packed, go.Q8_0)  # wrong K
    with pytest.raises(ops.SnGgufError):
        ops.linear(torch.zeros(2, 64, dtype=torch.bfloat16), packed.cpu(), go.Q8_0)       # CPU
    y = ops.linear(torch.zeros(0, 64, device=dev, dtype=torch.bfloat16), packed, go.Q8_0)
    assert y.shape == (0, 8)


def test_workspace_routes_replay_in_a_graph(dev):
    """The multi-launch routes (split-K + reduce pass; weight pass + dense kernel; row partition + grouped launch)
    captured in a HIP graph: every replay, with eager launches and new inputs in between, equals the eager result."""
    print("case ws_graph", flush=True)
    qt, n, k = go.Q8_0, 1024, 2048
    packed = synthetic.make_packed(qt, n, k, seed=5).to(dev)
    gen = synthetic.make_packed(qt, n, k, seed=6).to(dev)
    big = synthetic.make_packed(qt, 8192, 512, seed=7).to(dev)
    ws = torch.empty(4 * 16 * 700 * n, dtype=torch.uint8, device=dev)
    rowws = torch.empty(ops.grouped_workspace_bytes(700), dtype=torch.uint8, device=dev)
    sx = synthetic.make_activations(700, k, seed=1).to(dev)
    sx_big = synthetic.make_activations(4096, 512, seed=2).to(dev)
    sind = torch.zeros(700, dtype=torch.uint8, device=dev)
    y1 = torch.empty((128, n), dtype=torch.bfloat16, device=dev)
    y2 = torch.empty((700, n), dtype=torch.bfloat16, device=dev)
    y3 = torch.empty((4096, 8192), dtype=torch.bfloat16, device=dev)

    def run(o1, o2, o3):
        ops.linear_ws_into(sx[:128], packed, qt, None, o1, ws, 1)                                   # split-K
        ops.grouped_linear_ws_into(sx, sind, 0, packed, qt, gen, qt, None, None, o2, rowws, ws, 1)  # partition + split-K
        ops.linear_ws_into(sx_big, big, qt, None, o3, ws, 1)                                        # weight pass + dense

    run(y1, y2, y3)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(y1, y2, y3)
    for seed in (21, 22, 23):
        sx.copy_(synthetic.make_activations(700, k, seed=seed).to(dev))
        sx_big.copy_(synthetic.make_activations(4096, 512, seed=seed + 10).to(dev))
        sind.copy_((torch.rand(700, generator=torch.Generator().manual_seed(seed)) < 0.5).to(torch.uint8).to(dev))
        e1, e2, e3 = torch.empty_like(y1), torch.empty_like(y2), torch.empty_like(y3)
        run(e1, e2, e3)                      # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y1, e1) and torch.equal(y2, e2) and torch.equal(y3, e3), seed


@pytest.mark.parametrize("qt", [go.Q8_0, go.Q4_K, go.Q6_K, go.Q5_0])
def test_linear_row_chunks_between_65_and_512_rows(dev, c_oracle, qt):
    """A few hundred rows on matrices with few output tiles run as 64-row chunks through the decode kernel (no
    workspace): whole and partial last chunks, bias, residual, ragged N, both numerics."""
    print(f"case row_chunks qt={qt}", flush=True)
    for numerics, (m, n, k) in [(1, (65, 1024, 4096)), (0, (128, 4096, 4096)), (1, (200, 515, 2048)), (1, (256, 1030, 12288)),
                                (0, (321, 64, 4096))]:
        packed = synthetic.make_packed(qt, n, k, seed=m + n + qt)
        x = synthetic.make_activations(m, k, seed=m)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.bfloat16) if n % 2 else None
        res = synthetic.make_activations(m, n, seed=m + 1)
        want = go.gguf_linear_forward(x, packed, qt, bias, numerics=numerics)
        xd, pd = x.to(dev), packed.to(dev)
        bd = bias.to(dev) if bias is not None else None
        got = ops.linear(xd, pd, qt, bd, numerics)
        _check(got.cpu(), want)
        got_r = ops.linear_residual(xd, pd, qt, res.to(dev), bd, numerics)
        _check(got_r.cpu(), (res.float() + want.float()).to(torch.bfloat16))
        if (m, n, k) in ((65, 1024, 4096), (128, 4096, 4096)):
            # these two are chunked for certain (19 - 47 us of decode kernel against ~100 us of tile kernel): the chunks
            # are the decode kernel's own results on those rows
            hi = min(m, 128)
            assert torch.equal(got[64:hi], ops.linear(xd[64:hi].contiguous(), pd, qt, bd, numerics))
