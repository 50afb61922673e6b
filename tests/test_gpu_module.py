"""GPU: the module / loader boundary end to end - file -> load -> GGUFLinear.forward on the HIP
kernels, against the oracle's GGUFLinear.forward_native restatement."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as go
from sensenova_u1_amd import ops
from sensenova_u1_amd import (FusedProjections, GGUFLinear, GGUFParameter, gated_mlp, grouped_linear, load_gguf_checkpoint,
                              set_gguf2meta_model, synthetic)
from tests.test_loader import H, I, TinyModel, _make_file

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _load(tmp_path, dev, quant=8):
    path = str(tmp_path / "m.gguf")
    ref, packed = _make_file(path, quant)
    sd = load_gguf_checkpoint(path)
    with torch.device("meta"):
        model = TinyModel()
    return set_gguf2meta_model(model, sd, torch.bfloat16, dev).eval(), packed


@pytest.mark.parametrize("quant", [8, 12, 13, 14])
def test_loaded_model_projections(tmp_path, dev, quant):
    print(f"case module quant={quant}", flush=True)
    model, packed = _load(tmp_path, dev, quant)
    assert model.layers[0].q_proj.weight.device.type == "cuda"
    for m in (1, 5, 16, 40):
        x = synthetic.make_activations(m, H, seed=m)
        for name in ("layers.0.q_proj", "layers.1.mlp.gate_proj_mot_gen", "timestep_embedder"):
            mod = model.get_submodule(name)
            want = go.gguf_linear_forward(x, torch.from_numpy(packed[name + ".weight"]), quant,
                                          mod.bias.cpu() if mod.bias is not None else None)
            got = mod(x.to(dev).reshape(1, m, H))
            assert got.shape == (1, m, mod.out_features) and got.dtype == torch.bfloat16
            assert go.rel_l2(got.cpu().reshape(m, -1), want) <= TOL


def test_mlp_decode_and_prefill(tmp_path, dev):
    """Qwen3MLP.forward through the modules: fused gate/up GEMV at decode, three GEMMs above."""
    print("case module mlp", flush=True)
    model, packed = _load(tmp_path, dev)
    mlp = model.layers[0].mlp
    w = {n: torch.from_numpy(packed[f"layers.0.mlp.{n}.weight"]) for n in ("gate_proj", "up_proj", "down_proj")}
    for m in (1, 4, 16, 33):
        x = synthetic.make_activations(m, H, seed=20 + m)
        want, _ = go.mlp_forward(x, w["gate_proj"], w["up_proj"], w["down_proj"], (8, 8, 8))
        got = gated_mlp(x.to(dev), mlp.gate_proj, mlp.up_proj, mlp.down_proj)
        assert go.rel_l2(got.cpu(), want) <= 2 * TOL   # two chained projections


def test_grouped_modules(tmp_path, dev):
    print("case module grouped", flush=True)
    model, packed = _load(tmp_path, dev)
    layer = model.layers[1]
    x = synthetic.make_activations(2 * 30, H, seed=5).reshape(2, 30, H)
    ind = torch.zeros(2, 30, dtype=torch.bool)
    ind[0, 10:] = True
    ind[1, ::3] = True
    got = grouped_linear(x.to(dev), ind.to(dev), layer.q_proj, layer.q_proj_mot_gen)
    assert got.shape == (2, 30, H)
    want = go.grouped_linear_forward(x.reshape(60, H), ind.reshape(60), torch.from_numpy(packed["layers.1.q_proj.weight"]),
                                     8, torch.from_numpy(packed["layers.1.q_proj_mot_gen.weight"]), 8)
    assert go.rel_l2(got.cpu().reshape(60, H), want) <= TOL
    # the reference's production cases: all text -> understanding weights only, all image -> generation only
    # (bit for bit when both sides run the library's fused kernels)
    layer.q_proj.gemm_policy = layer.q_proj_mot_gen.gemm_policy = "fused"
    all_und = grouped_linear(x.to(dev), torch.zeros(2, 30, dtype=torch.bool, device=dev), layer.q_proj, layer.q_proj_mot_gen)
    assert torch.equal(all_und, layer.q_proj(x.to(dev)))
    all_gen = grouped_linear(x.to(dev), None, layer.q_proj, layer.q_proj_mot_gen, n_text=0)
    assert torch.equal(all_gen, layer.q_proj_mot_gen(x.to(dev)))
    # contiguous [text | image] layout under both policies: fused kernel, and weight pass + dense GEMM per group
    split = torch.arange(60) >= 22
    want = go.grouped_linear_forward(x.reshape(60, H), split, torch.from_numpy(packed["layers.1.q_proj.weight"]),
                                     8, torch.from_numpy(packed["layers.1.q_proj_mot_gen.weight"]), 8)
    for policy in ("fused", "auto"):
        layer.q_proj.gemm_policy = layer.q_proj_mot_gen.gemm_policy = policy
        for n_text in (22, 0, 60, 5, 50):
            got = grouped_linear(x.to(dev), None, layer.q_proj, layer.q_proj_mot_gen, n_text=n_text)
            ind = (torch.arange(60) >= n_text)
            want = go.grouped_linear_forward(x.reshape(60, H), ind, torch.from_numpy(packed["layers.1.q_proj.weight"]),
                                             8, torch.from_numpy(packed["layers.1.q_proj_mot_gen.weight"]), 8)
            assert got.shape == (2, 30, H) and go.rel_l2(got.cpu().reshape(60, H), want) <= TOL, (policy, n_text)


@pytest.mark.parametrize("quant", [8, 12, 2, 11])
def test_gemm_policies_agree_with_the_oracle(tmp_path, dev, quant):
    """More than 16 rows: "auto" (library workspace route), "fused" (library fused kernels), "resident" (the library's
    dense kernel on a kept bf16 weight) and "two_pass" (bf16 weight pass + the device library's dense GEMM) all reproduce
    the oracle; with and without bias; 3-d inputs keep their leading dims."""
    print(f"case module gemm policies quant={quant}", flush=True)
    model, packed = _load(tmp_path, dev, quant)
    for name in ("layers.0.mlp.down_proj", "timestep_embedder"):
        mod = model.get_submodule(name)
        assert mod.gemm_policy == "auto"
        for m in (17, 300):
            x = synthetic.make_activations(2 * m, mod.in_features, seed=m)
            want = go.gguf_linear_forward(x, torch.from_numpy(packed[name + ".weight"]), quant,
                                          mod.bias.cpu() if mod.bias is not None else None)
            outs = {}
            for policy in ("auto", "two_pass", "fused", "resident"):
                mod.gemm_policy = policy
                got = mod(x.to(dev).reshape(2, m, -1))
                assert got.shape == (2, m, mod.out_features) and got.dtype == torch.bfloat16
                assert go.rel_l2(got.cpu().reshape(2 * m, -1), want) <= TOL, (name, m, policy)
                outs[policy] = got
            # all four contract the same bf16 weights; they differ in the order of the fp32 sums only
            for policy in ("two_pass", "fused", "resident"):
                assert go.rel_l2(outs[policy].cpu(), outs["auto"].cpu()) <= TOL, (name, m, policy)
        mod.gemm_policy = "sometimes"
        with pytest.raises(ValueError):
            mod(x.to(dev))
        mod.gemm_policy = "auto"


def test_resident_policy_keeps_the_bf16_weight_until_the_packed_bytes_change(tmp_path, dev):
    print("case module resident policy", flush=True)
    model, packed = _load(tmp_path, dev, 8)
    mod = model.get_submodule("layers.0.mlp.down_proj")
    other = model.get_submodule("layers.1.mlp.down_proj")
    mod.gemm_policy = "resident"
    x = synthetic.make_activations(200, mod.in_features, seed=9).to(dev)
    y0 = mod(x)
    kept = mod._dense_cache[1]
    assert kept.dtype == torch.bfloat16 and kept.shape == (mod.out_features, mod.in_features)
    assert torch.equal(mod(x), y0) and mod._dense_cache[1] is kept          # second call: no new weight pass
    assert torch.equal(mod(x[:3]), y0[:3])                                  # decode rows do not touch the kept weight
    old = mod.weight.data
    mod.weight.data = other.weight.data.clone()                             # the offloader's kind of rebinding
    other.gemm_policy = "resident"
    assert torch.equal(mod(x), other(x)) and mod._dense_cache[1] is not kept
    mod.weight.data = old
    y_old = mod(x)                                                          # the cache now holds `old`'s address
    assert torch.equal(y_old, y0)
    mod.weight.data.copy_(other.weight.data)                                # in-place change at the same address:
    assert torch.equal(mod(x), y0)                                          # invisible to the key (documented) ...
    mod.weights_changed()                                                   # ... until the module is told
    assert torch.equal(mod(x), other(x))
    mod.drop_dense_cache()
    assert mod._dense_cache is None


def test_tiled_decode_layout(tmp_path, dev):
    """decode_layout = "tiled": decode calls read the operand-order copy (built once, rebuilt when the packed bytes move),
    larger inputs and other formats take the usual routes; results agree with the oracle and, closely, with the native layout."""
    print("case module tiled decode layout", flush=True)
    model, packed = _load(tmp_path, dev, 8)
    mlp = model.layers[0].mlp
    w = {n: torch.from_numpy(packed[f"layers.0.mlp.{n}.weight"]) for n in ("gate_proj", "up_proj", "down_proj")}
    for m in (1, 5, 16):
        x = synthetic.make_activations(m, H, seed=30 + m)
        want, _ = go.mlp_forward(x, w["gate_proj"], w["up_proj"], w["down_proj"], (8, 8, 8))
        native = gated_mlp(x.to(dev), mlp.gate_proj, mlp.up_proj, mlp.down_proj)
        for mod in (mlp.gate_proj, mlp.up_proj, mlp.down_proj):
            mod.decode_layout = "tiled"
        got = gated_mlp(x.to(dev), mlp.gate_proj, mlp.up_proj, mlp.down_proj)
        assert go.rel_l2(got.cpu(), want) <= 2 * TOL and go.rel_l2(got.cpu(), native.cpu()) <= 1e-3
        kept = mlp.down_proj._tiled_cache[1]
        h = synthetic.make_activations(m, I, seed=40 + m).to(dev)
        res = synthetic.make_activations(m, H, seed=41 + m).to(dev)
        y = mlp.down_proj(h.reshape(1, m, I))
        assert y.shape == (1, m, H) and mlp.down_proj._tiled_cache[1] is kept
        wantd = go.gguf_linear_forward(h.cpu(), w["down_proj"], 8)
        assert go.rel_l2(y.cpu().reshape(m, H), wantd) <= TOL
        yr = mlp.down_proj.forward_residual(h, res)
        assert go.rel_l2(yr.cpu(), (res.cpu().float() + wantd.float()).to(torch.bfloat16)) <= TOL
        for mod in (mlp.gate_proj, mlp.up_proj, mlp.down_proj):
            mod.decode_layout = "native"
    mod = mlp.down_proj
    mod.decode_layout = "tiled"
    big = synthetic.make_activations(40, I, seed=9).to(dev)
    assert go.rel_l2(mod(big).cpu(), go.gguf_linear_forward(big.cpu(), w["down_proj"], 8)) <= TOL   # beyond 16 rows: native routes
    other = model.layers[1].mlp.down_proj
    mod.weight.data = other.weight.data.clone()                                     # packed bytes move: the copy follows
    x1 = synthetic.make_activations(1, I, seed=3).to(dev)
    assert go.rel_l2(mod(x1).cpu(), other(x1).cpu()) <= 1e-3
    mod.drop_tiled_cache()
    assert mod._tiled_cache is None
    mod.decode_layout = "sideways"
    with pytest.raises(ValueError):
        mod(x1)
    mod.decode_layout = "native"
    q4 = _load(tmp_path, dev, 12)[0].layers[0].mlp.down_proj
    q4.decode_layout = "tiled"                                                       # not Q8_0: stays on the native path
    assert q4.tiled_weight() is None and q4(x1).shape == (1, H)


@pytest.mark.parametrize("quant", [8, 12, 3])
def test_fused_qkv_projections(tmp_path, dev, quant):
    """Projections that read the same hidden states (q / k / v in the model; here the four H-input projections the
    test model has) stacked row-wise into one launch: each output equals its own projection's oracle result, at
    decode and above 64 rows; sources can be released afterwards."""
    print(f"case module fused qkv quant={quant}", flush=True)
    model, packed = _load(tmp_path, dev, quant)
    layer = model.layers[0]
    names = ("q_proj", "q_proj_mot_gen", "mlp.gate_proj", "mlp.up_proj")
    fused = FusedProjections([layer.get_submodule(n) for n in names])
    assert fused.fused.out_features == sum(layer.get_submodule(n).out_features for n in names)
    for m in (1, 7, 16, 40, 100):
        x = synthetic.make_activations(m, H, seed=50 + m)
        outs = fused(x.to(dev))
        assert len(outs) == 4
        for n, got in zip(names, outs):
            want = go.gguf_linear_forward(x, torch.from_numpy(packed[f"layers.0.{n}.weight"]), quant)
            assert got.shape == (m, layer.get_submodule(n).out_features)
            assert go.rel_l2(got.cpu(), want) <= TOL, (n, m)
    released = FusedProjections([layer.get_submodule(n) for n in names], release_sources=True)
    assert all(layer.get_submodule(n).weight.numel() == 0 for n in names)
    x = synthetic.make_activations(3, H, seed=9)
    for a, b in zip(fused(x.to(dev)), released(x.to(dev))):
        assert torch.equal(a, b)
    with pytest.raises(ValueError):
        FusedProjections([model.layers[1].q_proj, model.layers[1].mlp.down_proj])    # different in_features


def test_weight_data_rebinding_between_forwards(dev):
    """The offloader swaps weight.data between a pinned CPU copy and a fresh device tensor around
    every forward (layer_offload.py:349-356,373-375)."""
    print("case module rebinding", flush=True)
    packed = synthetic.make_packed(8, 64, 256, seed=1)
    lin = GGUFLinear(256, 64, bias=False, compute_dtype=torch.bfloat16, device="meta")
    lin.weight = GGUFParameter(packed.pin_memory(), quant_type=8)
    x = synthetic.make_activations(3, 256, seed=2).to(dev)
    want = go.gguf_linear_forward(x, packed, 8)
    cpu_copy = lin.weight.data
    for _ in range(3):
        lin.weight.data = cpu_copy.to(dev, non_blocking=True)
        y = lin(x)
        lin.weight.data = cpu_copy
        assert go.rel_l2(y.cpu(), want) <= TOL


def test_other_compute_dtypes_use_hip_dequantize(dev):
    print("case module fp16 compute", flush=True)
    packed = synthetic.make_packed(12, 64, 512, seed=3)
    for dt in (torch.float16, torch.float32):
        lin = GGUFLinear(512, 64, bias=True, compute_dtype=dt, device="meta")
        lin.weight = GGUFParameter(packed.to(dev), quant_type=12)
        lin.bias = torch.nn.Parameter(torch.linspace(-1, 1, 64, device=dev, dtype=dt), requires_grad=False)
        x = synthetic.make_activations(9, 512, seed=4).to(dev).to(dt)
        want = go.gguf_linear_forward(x, packed, 12, lin.bias, compute_dtype=dt)
        got = lin(x)
        assert got.dtype == dt and go.rel_l2(got.cpu(), want) <= TOL


def test_mlp_forward_under_hip_graph(tmp_path, dev):
    """The modules launch on torch's current stream, allocate only through torch's allocator and
    never synchronise, so a decode step can be captured into a HIP graph.  The replay is checked
    against the eager result three times with fresh inputs (and eager work between replays)."""
    print("case module graph capture", flush=True)
    from sensenova_u1_amd import modality
    from sensenova_u1_amd.quantized_linear import GGUFLinear, GGUFParameter
    torch.manual_seed(0)
    hidden, inter = 512, 1536
    mods = {}
    for name, (n, k) in {"gate": (inter, hidden), "up": (inter, hidden), "down": (hidden, inter)}.items():
        m = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16, device=dev)
        m.weight = GGUFParameter(synthetic.make_packed(go.Q8_0, n, k, seed=len(name)).to(dev), quant_type=go.Q8_0)
        mods[name] = m

    def mlp(x):
        return modality.gated_mlp(x, mods["gate"], mods["up"], mods["down"])

    static_x = synthetic.make_activations(4, hidden, seed=1).to(dev)
    for _ in range(3):
        mlp(static_x)                       # warm-up outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = mlp(static_x)
    for seed in (11, 12, 13):
        x = synthetic.make_activations(4, hidden, seed=seed).to(dev)
        want = mlp(x)                       # eager work between replays
        torch.cuda.synchronize()
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, want)


def test_fused_rmsnorm_through_the_module_helpers(dev):
    """FusedProjections / gated_mlp with a norm weight: one decode row takes the fused-norm kernels, more rows the torch
    norm in front of the projection; both agree with the oracle's norm + projection."""
    from sensenova_u1_amd import FusedProjections, gated_mlp
    from sensenova_u1_amd.quantized_linear import rms_norm
    k, eps = 2048, 1e-6
    gamma = (torch.rand(k, generator=torch.Generator().manual_seed(3)) + 0.5).to(torch.bfloat16)

    def lin(n, kk, qt, seed):
        mod = GGUFLinear(kk, n, bias=False, compute_dtype=torch.bfloat16, device="meta")
        mod.weight = GGUFParameter(synthetic.make_packed(qt, n, kk, seed=seed).to(dev), quant_type=qt)
        return mod

    for qt, layout in ((go.Q8_0, "native"), (go.Q4_K, "native"), (go.Q8_0, "tiled")):
        q, kp, v = lin(512, k, qt, 1), lin(128, k, qt, 2), lin(128, k, qt, 3)
        stack = FusedProjections([q, kp, v])
        gate, up, down = lin(1024, k, qt, 4), lin(1024, k, qt, 5), lin(k, 1024, qt, 6)
        for mod in (stack.fused, gate, up, down):
            mod.decode_layout = layout
        for rows in (1, 5):
            print(f"case module_rmsnorm qt={qt} layout={layout} rows={rows}", flush=True)
            x = (synthetic.make_activations(rows, k, seed=10 + rows).float() * 2.0).to(torch.bfloat16)
            normed = go.qwen3_rms_norm(x, gamma, eps)
            # the package's own torch norm (the unfused route) against the oracle's: the reduction order on the device can
            # move a near-tie by one bf16 step
            dn = (rms_norm(x.to(dev), gamma.to(dev), eps).cpu().float() - normed.float()).abs()
            assert float((dn > 0).float().mean()) < 0.01 and bool((dn <= normed.float().abs() * 2 ** -6).all())
            outs = stack(x.to(dev), gamma.to(dev), eps)
            for mod, got in zip((q, kp, v), outs):
                want = go.gguf_linear_forward(normed, mod.weight.as_tensor().cpu(), qt)
                assert go.rel_l2(got.cpu(), want) <= 1e-3
            got = gated_mlp(x.to(dev), gate, up, down, gamma.to(dev), eps)
            want, _ = go.mlp_forward(normed, gate.weight.as_tensor().cpu(), up.weight.as_tensor().cpu(),
                                     down.weight.as_tensor().cpu(), (qt, qt, qt))
            assert go.rel_l2(got.cpu(), want) <= 2e-3     # two chained projections


@pytest.mark.parametrize("qt", [go.Q8_0, go.Q4_K, go.Q6_K])
def test_auto_policy_between_65_and_256_rows(dev, qt):
    """65 ... 256 rows under gemm_policy 'auto': Q8_0 / Q4_K through the library's split-K route, other formats
    through the weight pass + dense GEMM; every policy agrees with the oracle."""
    n, k = 1000, 2048
    mod = GGUFLinear(k, n, bias=True, compute_dtype=torch.bfloat16, device="meta")
    packed = synthetic.make_packed(qt, n, k, seed=31)
    mod.weight = GGUFParameter(packed.to(dev), quant_type=qt)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(32)) * 0.5).to(torch.bfloat16)
    mod.bias = torch.nn.Parameter(bias.to(dev), requires_grad=False)
    for rows in (65, 200, 256, 300):
        print(f"case module_mid_rows qt={qt} rows={rows}", flush=True)
        x = synthetic.make_activations(rows, k, seed=rows)
        want = go.gguf_linear_forward(x, packed, qt, bias)
        for policy in ("auto", "two_pass", "fused"):
            mod.gemm_policy = policy
            got = mod(x.to(dev))
            assert go.rel_l2(got.cpu(), want) <= TOL, (rows, policy)


def test_set_decode_layout_on_a_loaded_model(tmp_path, dev):
    """The whole model switched to the tiled decode layout: copies built at once, decode outputs as on the GGUF rows up
    to the summation order, larger inputs untouched."""
    from sensenova_u1_amd import set_decode_layout
    model, _ = _load(tmp_path, dev, 8)
    x = synthetic.make_activations(3, H, seed=5).to(dev)
    big = synthetic.make_activations(70, H, seed=6).to(dev)
    mods = [m for m in model.modules() if type(m).__name__ == "GGUFLinear" and m.in_features == H]
    before = [m(x) for m in mods]
    before_big = [m(big) for m in mods]
    assert set_decode_layout(model, "tiled", build_now=True) >= len(mods)
    assert any(m.tiled_weight() is not None for m in mods) == (H % 256 == 0)
    for m, want, want_big in zip(mods, before, before_big):
        assert go.rel_l2(m(x).cpu(), want.cpu()) <= 2e-4
        assert torch.equal(m(big), want_big)
    set_decode_layout(model, "native")
    assert all(m._tiled_cache is None for m in mods)


def test_module_paths_refuse_host_tensors_and_wrong_widths(dev):
    """The module routes that hand raw pointers to the library (split-K workspace route, fused norm, tiled decode,
    fused gated MLP) raise a clean error for a weight / norm weight / residual left on the host and for an input
    whose last dim is not in_features, instead of launching a kernel on a host pointer or re-rowing the input."""
    print("case module host-tensor refusal", flush=True)
    n, k = 512, 256
    packed = synthetic.make_packed(8, n, k, seed=3)
    lin = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16, device="meta")
    lin.weight = GGUFParameter(packed, quant_type=8)                        # still on the host
    gamma_dev = torch.ones(k, dtype=torch.bfloat16, device=dev)
    for rows in (1, 100, 200):
        x = synthetic.make_activations(rows, k, seed=rows).to(dev)
        with pytest.raises(ops.SnGgufError):
            lin(x)
    with pytest.raises(ops.SnGgufError):
        lin.forward_normed(synthetic.make_activations(1, k).to(dev), gamma_dev, 1e-6)
    lin.weight = GGUFParameter(packed.to(dev), quant_type=8)
    with pytest.raises(ops.SnGgufError):
        lin.forward_normed(synthetic.make_activations(1, k).to(dev), gamma_dev.cpu(), 1e-6)   # norm weight on the host
    with pytest.raises(ops.SnGgufError):
        lin(synthetic.make_activations(100, 2 * k).to(dev))                 # 100 rows of the wrong width, not 200 rows
    with pytest.raises(ops.SnGgufError):
        lin.forward_normed(synthetic.make_activations(1, 2 * k).to(dev), gamma_dev, 1e-6)
    up = GGUFLinear(k, n, bias=False, compute_dtype=torch.bfloat16, device="meta")
    up.weight = GGUFParameter(synthetic.make_packed(8, n, k, seed=4), quant_type=8)           # host
    down = GGUFLinear(n, k, bias=False, compute_dtype=torch.bfloat16, device="meta")
    down.weight = GGUFParameter(synthetic.make_packed(8, k, n, seed=5).to(dev), quant_type=8)
    with pytest.raises(ops.SnGgufError):
        gated_mlp(synthetic.make_activations(1, k).to(dev), lin, up, down, gamma_dev, 1e-6)
    lin.decode_layout = "tiled"
    lin.tiled_weight()
    with pytest.raises(ops.SnGgufError):
        lin.forward_residual(synthetic.make_activations(2, k).to(dev), synthetic.make_activations(2, n))   # residual on the host
    torch.cuda.synchronize()


def test_loader_fused_mlp_forward_matches_the_three_module_calls(tmp_path, dev):
    """A Qwen3MLP-shaped module loaded through load_gguf_model runs gate / up / SiLU as one launch at decode row counts:
    its output holds the tolerance against the oracle and against its own unfused forward, at 1, 4 and 16 rows; beyond
    16 rows the fused forward IS the three module calls (bit-equal); a captured graph of the fused forward replays."""
    from sensenova_u1_amd import load_gguf_model, unfuse_gated_mlps
    from sensenova_u1_amd.gguf_file import write_gguf
    from tests.test_loader import _GatedMLP
    print("case loader-fused mlp", flush=True)

    class Wrap(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.mlp = _GatedMLP()

    torch.manual_seed(3)
    ref = Wrap()
    packed = {n: go.quantize_q8_0(t.detach().numpy()) for n, t in ref.state_dict().items()}
    path = str(tmp_path / "w.gguf")
    write_gguf(path, [(n, p, 8) for n, p in packed.items()])
    with torch.device("meta"):
        meta = Wrap()
    model = load_gguf_model(meta, path, dtype=torch.bfloat16, device=dev)
    outs = {}
    for m in (1, 4, 16, 40):
        x = (torch.randn(m, H, generator=torch.Generator().manual_seed(m)) * 0.7).to(torch.bfloat16)
        outs[m] = model.mlp(x.to(dev))
        g = go.gguf_linear_forward(x, torch.from_numpy(packed["mlp.gate_proj.weight"]), go.Q8_0)
        u = go.gguf_linear_forward(x, torch.from_numpy(packed["mlp.up_proj.weight"]), go.Q8_0)
        want = go.gguf_linear_forward(torch.nn.functional.silu(g) * u, torch.from_numpy(packed["mlp.down_proj.weight"]), go.Q8_0)
        assert go.rel_l2(outs[m].cpu(), want) <= 1e-3, m
    xg = (torch.randn(2, H, generator=torch.Generator().manual_seed(9)) * 0.7).to(torch.bfloat16).to(dev)
    eager = model.mlp(xg)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        yg = model.mlp(xg)
    for _ in range(3):
        yg.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(yg, eager)
    assert unfuse_gated_mlps(model) == 1
    for m in (1, 4, 16, 40):
        x = (torch.randn(m, H, generator=torch.Generator().manual_seed(m)) * 0.7).to(torch.bfloat16)
        plain = model.mlp(x.to(dev))
        if m > 16:
            assert torch.equal(plain, outs[m])
        else:
            assert go.rel_l2(outs[m].cpu(), plain.cpu()) <= 1e-3, m


def test_loader_stacks_qkv_into_one_decode_launch(tmp_path, dev):
    """q_proj / k_proj / v_proj of an attention-shaped module loaded through load_gguf_model share one weight tensor; at
    the q call runs one launch over all rows and k / v return their ranges of it (contiguous tensors for one row, strided
    column ranges of one buffer for several).  Every output holds the tolerance against the oracle; other inputs, an
    input changed in place between the calls and a weight moved away from the stack all take the member's own launch."""
    from sensenova_u1_amd import load_gguf_model
    from sensenova_u1_amd.gguf_file import write_gguf
    print("case loader-stacked qkv", flush=True)
    NQ, NKV, HK = 512, 128, 256

    class Attn(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj = torch.nn.Linear(HK, NQ, bias=False)
            self.k_proj = torch.nn.Linear(HK, NKV, bias=False)
            self.v_proj = torch.nn.Linear(HK, NKV, bias=False)
            self.o_proj = torch.nn.Linear(NQ, HK, bias=False)

    class Wrap(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.self_attn = Attn()

    torch.manual_seed(4)
    ref = Wrap()
    packed = {n: go.quantize_q8_0(t.detach().numpy()) for n, t in ref.state_dict().items()}
    path = str(tmp_path / "a.gguf")
    write_gguf(path, [(n, p, 8) for n, p in packed.items()])
    with torch.device("meta"):
        meta = Wrap()
    model = load_gguf_model(meta, path, dtype=torch.bfloat16, device=dev)
    att = model.self_attn
    stack = att.q_proj.__dict__["_shared_stack"]
    assert stack is att.k_proj.__dict__["_shared_stack"] is att.v_proj.__dict__["_shared_stack"] and "_shared_stack" not in att.o_proj.__dict__
    assert stack.intact() and att.k_proj.weight.data_ptr() == att.q_proj.weight.data_ptr() + NQ * (HK // 32) * 34

    def want(name, x):
        return go.gguf_linear_forward(x.cpu(), torch.from_numpy(packed[f"self_attn.{name}.weight"]), go.Q8_0)

    for seed in (1, 2):
        m = 1
        x = (torch.randn(1, m, HK, generator=torch.Generator().manual_seed(seed)) * 0.8).to(torch.bfloat16).to(dev)
        q = att.q_proj(x)
        assert stack._pending is not None
        k, v = att.k_proj(x), att.v_proj(x)
        assert stack._pending is None                                  # consumed by the last member
        assert q.shape == (1, m, NQ) and k.shape == (1, m, NKV) and v.shape == (1, m, NKV)
        assert k.data_ptr() == q.data_ptr() + 2 * NQ and v.data_ptr() == k.data_ptr() + 2 * NKV   # ranges of one buffer
        assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
        q.view(1, m, -1, 64), k.view(-1)                               # any reshape of the outputs works
        for name, got in (("q_proj", q), ("k_proj", k), ("v_proj", v)):
            assert go.rel_l2(got.cpu().reshape(m, -1), want(name, x.reshape(m, HK))) <= 1e-3, (name, m)
    # several rows (decode kernel, decode kernel's 17 .. 64-row form, workspace route): still one launch; the outputs are
    # column ranges of one buffer, whose last dimension splits into heads as the model code does it
    for m in (5, 40, 300):
        xm = (torch.randn(1, m, HK, generator=torch.Generator().manual_seed(m)) * 0.8).to(torch.bfloat16).to(dev)
        q = att.q_proj(xm)
        assert stack._pending is not None
        k, v = att.k_proj(xm), att.v_proj(xm)
        assert stack._pending is None
        assert q.shape == (1, m, NQ) and k.shape == (1, m, NKV) and q.stride(-2) == NQ + 2 * NKV and not k.is_contiguous()
        assert k.data_ptr() == q.data_ptr() + 2 * NQ and v.data_ptr() == k.data_ptr() + 2 * NKV
        assert q.view(1, m, -1, 64).shape == (1, m, NQ // 64, 64) and v.view(1, m, -1, 64).transpose(1, 2).shape == (1, NKV // 64, m, 64)
        for name, got in (("q_proj", q), ("k_proj", k), ("v_proj", v)):
            assert go.rel_l2(got.cpu().reshape(m, -1), want(name, xm.reshape(m, HK))) <= 1e-3, (name, m)
    # ... unless told not to: the members' own launches, separate contiguous tensors
    x5 = (torch.randn(1, 5, HK, generator=torch.Generator().manual_seed(5)) * 0.8).to(torch.bfloat16).to(dev)
    stack.MULTI_ROW = False
    q, k = att.q_proj(x5), att.k_proj(x5)
    assert stack._pending is None and q.is_contiguous() and k.is_contiguous()
    assert go.rel_l2(k.cpu().reshape(5, -1), want("k_proj", x5.reshape(5, HK))) <= 1e-3
    stack.MULTI_ROW = True
    # another tensor for k: its own launch on that tensor
    x1 = (torch.randn(1, HK, generator=torch.Generator().manual_seed(50)) * 0.8).to(torch.bfloat16).to(dev)
    x2 = (torch.randn(1, HK, generator=torch.Generator().manual_seed(51)) * 0.8).to(torch.bfloat16).to(dev)
    q = att.q_proj(x1)
    k = att.k_proj(x2)
    assert go.rel_l2(k.cpu(), want("k_proj", x2)) <= 1e-3 and k.data_ptr() != q.data_ptr() + 2 * NQ
    # the same tensor changed in place between the calls: the version counter moved, k reads the new values
    q = att.q_proj(x1)
    x1.mul_(0.5)
    k = att.k_proj(x1)
    assert go.rel_l2(k.cpu(), want("k_proj", x1)) <= 1e-3
    # a weight that left the stack (an offloader's rebinding): no stacked launch, same results
    att.k_proj.weight.data = att.k_proj.weight.data.clone()
    assert not stack.intact()
    q, k = att.q_proj(x2), att.k_proj(x2)
    assert stack._pending is None and go.rel_l2(q.cpu(), want("q_proj", x2)) <= 1e-3 and go.rel_l2(k.cpu(), want("k_proj", x2)) <= 1e-3
    stack.dissolve()
    assert "_shared_stack" not in att.q_proj.__dict__ and go.rel_l2(att.v_proj(x2).cpu(), want("v_proj", x2)) <= 1e-3


def test_registered_ops_and_direct_eager_route_agree(dev):
    """ops.linear / gate_up_silu / linear_residual go straight to the HIP implementation in plain eager calls and through
    the registered sn_gguf ops otherwise (torch.compile, export, dispatch modes): both routes give the same bits."""
    print("case eager route vs registered ops", flush=True)
    n, k = 320, 512
    w = synthetic.make_packed(go.Q8_0, n, k, seed=1).to(dev)
    u = synthetic.make_packed(go.Q8_0, n, k, seed=2).to(dev)
    x = synthetic.make_activations(3, k, seed=3).to(dev).reshape(1, 3, k)
    res = synthetic.make_activations(3, n, seed=4).to(dev).reshape(1, 3, n)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(5)) * 0.5).to(torch.bfloat16).to(dev)
    assert ops._eager(x)
    assert torch.equal(ops.linear(x, w, go.Q8_0, bias), torch.ops.sn_gguf.linear(x, w, go.Q8_0, bias, 1))
    assert torch.equal(ops.gate_up_silu(x, w, u, go.Q8_0), torch.ops.sn_gguf.gate_up_silu(x, w, u, go.Q8_0, 1))
    assert torch.equal(ops.linear_residual(x, w, go.Q8_0, res, bias), torch.ops.sn_gguf.linear_residual(x, w, go.Q8_0, bias, res, 1))
    # a non-contiguous input and a tagged parameter as the weight take the same route
    xt = synthetic.make_activations(k, 3, seed=6).to(dev).t()
    wp = GGUFParameter(w, quant_type=go.Q8_0)
    assert not xt.is_contiguous()
    assert torch.equal(ops.linear(xt, wp, go.Q8_0), torch.ops.sn_gguf.linear(xt.contiguous(), w, go.Q8_0, None, 1))
    # under a dispatch mode the registered op is used (the mode sees it)
    from torch.utils._python_dispatch import TorchDispatchMode

    seen = []

    class Spy(TorchDispatchMode):
        def __torch_dispatch__(self, func, types, args=(), kwargs=None):
            seen.append(str(func))
            return func(*args, **(kwargs or {}))

    with Spy():
        y = ops.linear(x, w, go.Q8_0, bias)
    assert any("sn_gguf.linear" in f for f in seen) and torch.equal(y, ops.linear(x, w, go.Q8_0, bias))
