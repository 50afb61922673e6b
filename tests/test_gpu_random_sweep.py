"""GPU: seeded random sweep over the dispatch boundaries of the linear entry points (row counts around 16 / 64 /
384, ragged N, K down to one block, the line-aligned and the large-tile shapes, every type, both numerics modes,
bias, residual, gated pair, workspace route) and of the grouped launcher (indicator / contiguous split / one empty
group, equal and different types, with and without the dense workspace), each case against the oracle."""
import random

import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import ops, synthetic

pytestmark = pytest.mark.gpu
TOL = 1e-3
TYPES = [go.Q4_0, go.Q4_1, go.Q5_0, go.Q5_1, go.Q8_0, go.Q2_K, go.Q3_K, go.Q4_K, go.Q5_K, go.Q6_K]
ROWS = [1, 2, 3, 5, 8, 11, 12, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 100, 129, 383, 384, 385, 512, 700]


def _ok(got, want, tag):
    assert bool(torch.isfinite(got.float()).all()), tag
    assert go.rel_l2(got, want) <= TOL, tag


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_linear_cases(dev, seed):
    rnd = random.Random(seed)
    for it in range(70):
        qt = rnd.choice(TYPES)
        bs = go.GGML_QUANT_SIZES[qt][0]
        m = rnd.choice(ROWS)
        mode = rnd.random()
        if mode < 0.15:      # Q8_0 rows that are whole 2048-element spans, many row groups
            qt, k, n = go.Q8_0, rnd.choice([2048, 4096, 6144]), rnd.choice([8192, 8200, 9000, 16400])
        elif mode < 0.3:     # enough 256 x 256 tiles for the large-tile kernels
            m = rnd.choice([384, 500, 1000, 2100])
            n = rnd.choice([5632, 4100, 8200, 33000 if m < 600 else 3000])
            k = bs * rnd.randint(1, max(1, 1024 // bs))
        else:
            n, k = rnd.randint(1, 2500), bs * rnd.randint(1, max(1, 3072 // bs))
        if m * n > 6_000_000:
            n = max(1, 6_000_000 // m)
        numerics = rnd.choice([0, 1])
        kind = rnd.choice(["linear", "linear", "residual", "gate_up", "ws", "tiled"])
        if kind == "gate_up" and m > 16:
            kind = "linear"
        if kind == "tiled":   # the operand-order copy: Q8_0, decode rows, whole 256-element runs
            qt, bs, m = go.Q8_0, 32, rnd.choice([r for r in ROWS if r <= 16])
            k = 256 * max(1, k // 256)
        use_bias = kind != "gate_up" and rnd.random() < 0.4
        tag = f"seed={seed} it={it} kind={kind} qt={qt} m={m} n={n} k={k} numerics={numerics} bias={use_bias}"
        print("case", tag, flush=True)
        packed = synthetic.make_packed(qt, n, k, seed=it)
        x = synthetic.make_activations(m, k, seed=1000 + it)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(it)) * 0.5).to(torch.bfloat16) if use_bias else None
        xd, pd = x.to(dev), packed.to(dev)
        bd = bias.to(dev) if bias is not None else None
        want = go.gguf_linear_forward(x, packed, qt, bias, numerics=numerics)
        if kind == "linear":
            got = ops.linear(xd, pd, qt, bd, numerics)
        elif kind == "ws":
            got = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
            ws = torch.empty(n * k + 8, dtype=torch.bfloat16, device=dev)
            ops.linear_ws_into(xd, pd, qt, bd, got, ws, numerics)
        elif kind == "tiled":
            res = synthetic.make_activations(m, n, seed=5000 + it) if rnd.random() < 0.5 else None
            got = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
            ops.linear_tiled_into(xd, ops.q8_0_tile(pd), bd, res.to(dev) if res is not None else None, got, numerics)
            if res is not None:
                want = (res.float() + want.float()).to(torch.bfloat16)
        elif kind == "residual":
            res = synthetic.make_activations(m, n, seed=5000 + it)
            got = ops.linear_residual(xd, pd, qt, res.to(dev), bd, numerics)
            want = (res.float() + want.float()).to(torch.bfloat16)
        else:
            up = synthetic.make_packed(qt, n, k, seed=9000 + it)
            want = torch.nn.functional.silu(want) * go.gguf_linear_forward(x, up, qt, None, numerics=numerics)
            got = ops.gate_up_silu(xd, pd, up.to(dev), qt, numerics)
        _ok(got.cpu(), want, tag)


@pytest.mark.parametrize("seed", [21, 22])
def test_random_grouped_cases(dev, seed):
    rnd = random.Random(seed)
    for it in range(50):
        qu, qg = rnd.choice(TYPES), rnd.choice(TYPES)
        if rnd.random() < 0.4:
            qg = qu
        step = max(go.GGML_QUANT_SIZES[qu][0], go.GGML_QUANT_SIZES[qg][0])
        m = rnd.choice([1, 7, 17, 64, 65, 200, 383, 384, 600, 1500, 3000])
        big = rnd.random() < 0.3
        n = rnd.choice([2816, 4100, 8200]) if big else rnd.randint(1, 1500)
        k = step * rnd.randint(1, max(1, (512 if big else 2048) // step))
        if m * n > 6_000_000:
            n = 6_000_000 // m
        numerics = rnd.choice([0, 1])
        form = rnd.choice(["indicator", "split", "all_text", "all_image"])
        dense = rnd.random() < 0.5
        tag = f"seed={seed} it={it} qu={qu} qg={qg} m={m} n={n} k={k} numerics={numerics} form={form} dense_ws={dense}"
        print("case", tag, flush=True)
        und, gen = synthetic.make_packed(qu, n, k, seed=it), synthetic.make_packed(qg, n, k, seed=7000 + it)
        x = synthetic.make_activations(m, k, seed=100 + it)
        g = torch.Generator().manual_seed(it)
        n_text = rnd.randint(0, m)
        ind = {"indicator": torch.rand(m, generator=g) < rnd.random(), "split": torch.arange(m) >= n_text,
               "all_text": torch.zeros(m, dtype=torch.bool), "all_image": torch.ones(m, dtype=torch.bool)}[form]
        bu = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16) if rnd.random() < 0.5 else None
        bg = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16) if rnd.random() < 0.5 else None
        want = torch.empty((m, n), dtype=torch.bfloat16)
        if bool((~ind).any()):
            want[~ind] = go.gguf_linear_forward(x[~ind], und, qu, bu, numerics=numerics)
        if bool(ind.any()):
            want[ind] = go.gguf_linear_forward(x[ind], gen, qg, bg, numerics=numerics)
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        row_ws = torch.empty(ops.grouped_workspace_bytes(m), dtype=torch.uint8, device=dev)
        dense_ws = torch.empty(2 * n * k, dtype=torch.bfloat16, device=dev) if dense else None

        def put(t):
            return t.to(dev) if t is not None else None

        if form == "split":
            ops.grouped_linear_ws_into(put(x), None, n_text, put(und), qu, put(gen), qg, put(bu), put(bg), y, None, dense_ws, numerics)
        else:
            ops.grouped_linear_ws_into(put(x), put(ind.to(torch.uint8)), 0, put(und), qu, put(gen), qg, put(bu), put(bg), y,
                                       row_ws, dense_ws, numerics)
        _ok(y.cpu(), want, tag)


def _draw_rmsnorm_case(rnd, seed, it):
    """One fused-norm case from the generator's stream (every draw in a fixed order, so that a case is named by
    (seed, it) alone)."""
    qt = rnd.choice(TYPES)
    k = 256 * rnd.randint(1, 24)
    m = rnd.randint(1, min(16, 36864 // (2 * k + 64)))
    n = rnd.choice([rnd.randint(1, 2500), rnd.randint(1, 2500), 6144, 33000 + rnd.randint(0, 40)])
    numerics = rnd.choice([0, 1])
    kind = rnd.choice(["linear", "gate_up", "tiled", "tiled_gate_up"])
    if kind.startswith("tiled"):
        qt = go.Q8_0
    eps = rnd.choice([1e-6, 1e-5, 0.0])
    tag = f"seed={seed} it={it} kind={kind} qt={qt} m={m} n={n} k={k} numerics={numerics} eps={eps}"
    scale = rnd.choice([0.05, 1.0, 7.0])
    use_bias = kind in ("linear", "tiled") and rnd.random() < 0.4
    return qt, k, m, n, numerics, kind, eps, scale, use_bias, tag


def _run_rmsnorm_case(dev, case, it, normed_fn):
    """Runs the drawn case on the device; returns (got, want_fn) where want_fn(normed) is the oracle's projection (or
    gated pair) of normalized rows."""
    qt, k, m, n, numerics, kind, eps, scale, use_bias, tag = case
    assert ops.rmsnorm_fits(qt, m, k), tag
    packed = synthetic.make_packed(qt, n, k, seed=it)
    x = (synthetic.make_activations(m, k, seed=2000 + it).float() * scale).to(torch.bfloat16)
    gamma = (torch.rand(k, generator=torch.Generator().manual_seed(it)) * 1.5 + 0.25).to(torch.bfloat16)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(it)) * 0.5).to(torch.bfloat16) if use_bias else None
    up = synthetic.make_packed(qt, n, k, seed=9000 + it) if kind.endswith("gate_up") else None

    def want_fn(normed):
        want = go.gguf_linear_forward(normed, packed, qt, bias, numerics=numerics)
        if up is not None:
            want = torch.nn.functional.silu(want) * go.gguf_linear_forward(normed, up, qt, None, numerics=numerics)
        return want

    xd, gd, pd = x.to(dev), gamma.to(dev), packed.to(dev)
    bd = bias.to(dev) if bias is not None else None
    got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    if kind == "linear":
        ops.rmsnorm_linear_into(xd, gd, eps, pd, qt, bd, got, numerics)
    elif kind == "tiled":
        ops.rmsnorm_linear_tiled_into(xd, gd, eps, ops.q8_0_tile(pd), bd, got, numerics)
    elif kind == "gate_up":
        ops.rmsnorm_gate_up_silu_into(xd, gd, eps, pd, up.to(dev), qt, got, numerics)
    else:
        ops.rmsnorm_gate_up_silu_tiled_into(xd, gd, eps, ops.q8_0_tile(pd), ops.q8_0_tile(up.to(dev)), got, numerics)
    return got.cpu(), want_fn, normed_fn(x, gamma, eps)


@pytest.mark.parametrize("seed", [31, 32])
def test_random_rmsnorm_cases(dev, seed):
    """RMSNorm folded into the projection / the gated pair: every type (and the tiled Q8_0 copy), row counts up to what
    the staging area takes for the drawn K, ragged N, wide N, both numerics, against oracle norm + oracle projection."""
    rnd = random.Random(seed)
    for it in range(40):
        case = _draw_rmsnorm_case(rnd, seed, it)
        print("case", case[-1], flush=True)
        got, want_fn, normed = _run_rmsnorm_case(dev, case, it, go.qwen3_rms_norm)
        _ok(got, want_fn(normed), case[-1])


def _rms_norm_with_rstd_steps(x, weight, eps, steps):
    """Qwen3RMSNorm.forward with the row statistic moved by `steps` fp32 units in the last place: what the same norm
    gives when the squares of a row are added up in another order (the sum of some thousand squares differs in its last
    places between orders of addition, and rsqrt carries that into rstd)."""
    h = x.to(torch.float32)
    rstd = torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + eps)
    rstd = (rstd.view(torch.int32) + steps).view(torch.float32)
    return weight * (h * rstd).to(x.dtype)


@pytest.mark.parametrize("seed,it", [(502, 10), (2010, 8), (2012, 23), (125, 8)])
def test_fused_norm_cases_with_many_exact_ties(dev, seed, it):
    """Four cases that one-off runs of the generator above (other seeds) ended above 1e-3 against the oracle, at
    1.05e-3 ... 1.9e-3.  In each, one row has dozens of activations for which x * rstd lies within two fp32 units of
    the midpoint between two bf16 values (activations with 8-bit mantissas share mantissas, so one unlucky rstd makes
    many ties at once); they round as the oracle's only if rstd has the oracle's bits, and rstd depends on the order in
    which the row's squares are added.  The kernel is right if, row by row, its outputs are the oracle's for SOME rstd
    within two units of the oracle's: that is what is checked, at the ordinary tolerance.  (Two of the four are short
    rows in which a few outputs one bf16 step off already make up 1e-3 of the row's norm, whatever rstd is taken.)"""
    rnd = random.Random(seed)
    for i in range(it + 1):
        case = _draw_rmsnorm_case(rnd, seed, i)
    print("case", case[-1], flush=True)
    got, want_fn, _ = _run_rmsnorm_case(dev, case, it, go.qwen3_rms_norm)
    qt, k, m = case[0], case[1], case[2]
    x = (synthetic.make_activations(m, k, seed=2000 + it).float() * case[7]).to(torch.bfloat16)
    gamma = (torch.rand(k, generator=torch.Generator().manual_seed(it)) * 1.5 + 0.25).to(torch.bfloat16)
    wants = {s: want_fn(_rms_norm_with_rstd_steps(x, gamma, case[6], s)) for s in (0, -1, 1, -2, 2)}
    for r in range(m):
        errs = {s: go.rel_l2(got[r:r + 1], w[r:r + 1]) for s, w in wants.items()}
        step = min(errs, key=errs.get)
        # outputs that differ from that oracle row at all, and by how many bf16 steps (sign-magnitude order of the bits)
        a, b = got[r].view(torch.int16).int(), wants[step][r].view(torch.int16).int()
        a, b = torch.where(a < 0, -(a & 0x7FFF), a), torch.where(b < 0, -(b & 0x7FFF), b)
        off = (a - b).abs()
        print(f"  row {r}: rel-L2 by rstd step {({s: round(e, 6) for s, e in errs.items()})}; with step {step}: "
              f"{int((off > 0).sum())} of {off.numel()} outputs differ, by at most {int(off.max())} bf16 steps", flush=True)
        # either the row is within the ordinary tolerance of the oracle for that rstd, or (the two short-output cases,
        # where a handful of one-step differences IS 1e-3 of the row's norm) at most 1 % of it differs, by one step
        assert errs[step] <= TOL or (int(off.max()) <= 1 and int((off > 0).sum()) <= max(3, off.numel() // 100)), (case[-1], r, errs)
    assert bool(torch.isfinite(got.float()).all())


@pytest.mark.parametrize("seed", [41])
def test_random_split_k_cases(dev, seed):
    """The K-split routes on random shapes with few output tiles: plain (all ten types, the partial sums behind the decoded
    weights where the kernel does not decode the type itself) and grouped (Q8_0 / Q4_K, all four row-group forms)."""
    rnd = random.Random(seed)
    for it in range(40):
        grouped = rnd.random() < 0.5
        qt = rnd.choice([go.Q8_0, go.Q4_K]) if grouped else rnd.choice(TYPES)
        m = rnd.choice([65, 66, 100, 255, 256, 257, 511, 700, 1500])
        n = rnd.randint(1, 1500)
        k = 256 * rnd.randint(1, 10) if rnd.random() < 0.7 else 64 * rnd.randint(2, 40) if qt == go.Q8_0 else 256
        numerics = rnd.choice([0, 1])
        tag = f"seed={seed} it={it} grouped={grouped} qt={qt} m={m} n={n} k={k} numerics={numerics}"
        print("case", tag, flush=True)
        g = torch.Generator().manual_seed(it)
        x = synthetic.make_activations(m, k, seed=300 + it)
        und = synthetic.make_packed(qt, n, k, seed=it)
        bu = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16) if rnd.random() < 0.5 else None
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
        ws = torch.empty(2 * n * k + 4 * 16 * m * n, dtype=torch.uint8, device=dev)

        def put(t):
            return t.to(dev) if t is not None else None

        if not grouped:
            want = go.gguf_linear_forward(x, und, qt, bu, numerics=numerics)
            ops.linear_ws_into(put(x), put(und), qt, put(bu), y, ws, numerics)
        else:
            gen = synthetic.make_packed(qt, n, k, seed=7000 + it)
            bg = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16) if rnd.random() < 0.5 else None
            form = rnd.choice(["indicator", "split", "all_text", "all_image"])
            n_text = rnd.randint(0, m)
            ind = {"indicator": torch.rand(m, generator=g) < rnd.random(), "split": torch.arange(m) >= n_text,
                   "all_text": torch.zeros(m, dtype=torch.bool), "all_image": torch.ones(m, dtype=torch.bool)}[form]
            want = torch.empty((m, n), dtype=torch.bfloat16)
            if bool((~ind).any()):
                want[~ind] = go.gguf_linear_forward(x[~ind], und, qt, bu, numerics=numerics)
            if bool(ind.any()):
                want[ind] = go.gguf_linear_forward(x[ind], gen, qt, bg, numerics=numerics)
            row_ws = torch.empty(ops.grouped_workspace_bytes(m), dtype=torch.uint8, device=dev)
            if form == "split":
                ops.grouped_linear_ws_into(put(x), None, n_text, put(und), qt, put(gen), qt, put(bu), put(bg), y, None, ws, numerics)
            else:
                ops.grouped_linear_ws_into(put(x), put(ind.to(torch.uint8)), 0, put(und), qt, put(gen), qt, put(bu), put(bg), y,
                                           row_ws, ws, numerics)
            tag += f" form={form}"
        _ok(y.cpu(), want, tag)


@pytest.mark.parametrize("seed", [51, 52])
def test_random_bf16_static_argmax_cases(dev, seed):
    """The later entry points over random shapes: BF16 (type 30) weights through every linear form (K of any length -
    odd K takes the element-wise loads, K % 64 != 0 above 16 rows the chunked decode route), the allocation-free
    sngguf_linear_static on every type, and the arg-max form of the projection against the arg-max of the library's
    own logits (same kernels, so equal indices, ties included)."""
    rnd = random.Random(seed)
    for it in range(60):
        kind = rnd.choice(["bf16_linear", "bf16_residual", "bf16_gate_up", "bf16_ws", "static", "argmax"])
        numerics = rnd.choice([0, 1])
        m = rnd.choice(ROWS)
        if kind.startswith("bf16"):
            qt = go.BF16
            k = rnd.choice([rnd.randint(1, 3072), 8 * rnd.randint(1, 384), 64 * rnd.randint(1, 48)])
            n = rnd.choice([rnd.randint(1, 2500), 4100, 5632])
            if kind == "bf16_gate_up":
                m = rnd.choice([r for r in ROWS if r <= 16])
        elif kind == "static":
            qt = rnd.choice(TYPES + [go.BF16])
            bs = go.GGML_QUANT_SIZES[qt][0]
            k = bs * rnd.randint(1, max(1, 3072 // bs)) if qt != go.BF16 else 64 * rnd.randint(1, 48)
            n = rnd.choice([rnd.randint(1, 2500), 4100, 8200])
        else:
            qt = rnd.choice(TYPES)
            m = rnd.choice([r for r in ROWS if r <= 16])
            k = 256 * rnd.randint(1, 16)
            n = rnd.choice([rnd.randint(1, 2500), 8200, 33000 + rnd.randint(0, 40)])
            if qt == go.Q8_0 and rnd.random() < 0.5:
                k = rnd.choice([2048, 4096])
        if m * n > 6_000_000:
            n = max(1, 6_000_000 // m)
        use_bias = kind != "bf16_gate_up" and rnd.random() < 0.4
        tag = f"seed={seed} it={it} kind={kind} qt={qt} m={m} n={n} k={k} numerics={numerics} bias={use_bias}"
        print("case", tag, flush=True)
        packed = synthetic.make_packed(qt, n, k, seed=it)
        x = synthetic.make_activations(m, k, seed=1000 + it)
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(it)) * 0.5).to(torch.bfloat16) if use_bias else None
        xd, pd = x.to(dev), packed.to(dev)
        bd = bias.to(dev) if bias is not None else None
        if kind == "argmax":
            got = ops.lm_head_argmax(xd, pd, qt, bd, numerics)
            logits = ops.linear(xd, pd, qt, bd, numerics)
            assert got.dtype == torch.int64 and got.shape == (m,), tag
            assert torch.equal(got, torch.argmax(logits, dim=-1)), tag
            _ok(logits.cpu(), go.gguf_linear_forward(x, packed, qt, bias, numerics=numerics), tag)
            continue
        want = go.gguf_linear_forward(x, packed, qt, bias, numerics=numerics)
        if kind == "bf16_linear":
            got = ops.linear(xd, pd, qt, bd, numerics)
        elif kind == "bf16_ws":
            got = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
            ws = torch.empty(n * k + 8, dtype=torch.bfloat16, device=dev)
            ops.linear_ws_into(xd, pd, qt, bd, got, ws, numerics)
        elif kind == "bf16_residual":
            res = synthetic.make_activations(m, n, seed=5000 + it)
            got = ops.linear_residual(xd, pd, qt, res.to(dev), bd, numerics)
            want = (res.float() + want.float()).to(torch.bfloat16)
        elif kind == "bf16_gate_up":
            up = synthetic.make_packed(qt, n, k, seed=9000 + it)
            want = torch.nn.functional.silu(want) * go.gguf_linear_forward(x, up, qt, None, numerics=numerics)
            got = ops.gate_up_silu(xd, pd, up.to(dev), qt, numerics)
        else:
            assert m * n <= ops.linear_static_max_outputs(), tag
            got = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
            ops.linear_static_into(xd, pd, qt, bd, got, numerics)
        _ok(got.cpu(), want, tag)
