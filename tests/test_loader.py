"""Loader and module boundary on the CPU: file -> state dict -> meta model, with the reference's
mapping rules (src/sensenova_u1/utils/gguf_loader.py) and error behaviour.  A tiny MoT-shaped
model stands in for the 8B backbone (the pattern of the reference's tests/test_transformers_compat.py:
real torch modules, hidden sizes small but multiples of the block sizes)."""
import copy

import numpy as np
import pytest
import torch
from torch import nn

from oracle import gguf_oracle as go
from sensenova_u1_amd import (GGUFLinear, GGUFParameter, count_gguf_linear, find_mot_pairs, load_gguf_checkpoint,
                              match_state_dict, set_gguf2meta_model, synthetic)
from sensenova_u1_amd import ops
from sensenova_u1_amd.gguf_file import GGMLQuantizationType, write_gguf

H, I = 256, 512


class TinyMLP(nn.Module):
    def __init__(self):
        super().__init__()
        self.gate_proj = nn.Linear(H, I, bias=False)
        self.up_proj = nn.Linear(H, I, bias=False)
        self.down_proj = nn.Linear(I, H, bias=False)
        self.gate_proj_mot_gen = nn.Linear(H, I, bias=False)
        self.up_proj_mot_gen = nn.Linear(H, I, bias=False)
        self.down_proj_mot_gen = nn.Linear(I, H, bias=False)


class TinyLayer(nn.Module):
    def __init__(self):
        super().__init__()
        self.q_proj = nn.Linear(H, H, bias=False)
        self.q_proj_mot_gen = nn.Linear(H, H, bias=False)
        self.mlp = TinyMLP()
        self.input_layernorm = nn.LayerNorm(H)


class TinyModel(nn.Module):
    def __init__(self):
        super().__init__()
        self.embed_tokens = nn.Embedding(32, H)
        self.layers = nn.ModuleList([TinyLayer(), TinyLayer()])
        self.timestep_embedder = nn.Linear(H, H, bias=True)      # non-backbone linear with a bias
        self.lm_head = nn.Linear(H, 32, bias=False)              # stays unquantized (F16 in the file)
        self.register_buffer("inv_freq", torch.ones(4))


def _make_file(path, quant=GGMLQuantizationType.Q8_0, skip=(), extra=()):
    torch.manual_seed(0)
    ref = TinyModel()
    tensors = []
    packed = {}
    for name, t in ref.state_dict().items():
        if name in skip:
            continue
        arr = t.detach().numpy()
        if name.endswith("_proj.weight") or name.endswith("_mot_gen.weight") or name == "timestep_embedder.weight":
            if quant == GGMLQuantizationType.Q8_0:
                p = go.quantize_q8_0(arr)
            else:
                p = synthetic.make_packed(int(quant), arr.shape[0], arr.shape[1], seed=len(tensors)).numpy()
            packed[name] = p
            tensors.append((name, p, int(quant)))
        elif name == "lm_head.weight":
            tensors.append((name, arr.astype(np.float16), 1))
        else:
            tensors.append((name, arr.astype(np.float32), 0))
    tensors.extend(extra)
    write_gguf(path, tensors)
    return ref, packed


def test_load_gguf_checkpoint_types_and_names(tmp_path):
    path = str(tmp_path / "m.gguf")
    ref, packed = _make_file(path)
    sd = load_gguf_checkpoint(path)
    assert set(sd) == set(ref.state_dict())                       # names verbatim
    w = sd["layers.0.mlp.gate_proj.weight"]
    assert isinstance(w, GGUFParameter) and w.dtype == torch.uint8 and w.quant_type == GGMLQuantizationType.Q8_0
    assert tuple(w.shape) == (I, H // 32 * 34) and tuple(w.quant_shape) == (I, H)
    assert np.array_equal(w.as_tensor().numpy(), packed["layers.0.mlp.gate_proj.weight"])
    assert not isinstance(sd["lm_head.weight"], GGUFParameter) and sd["lm_head.weight"].dtype == torch.float16
    assert sd["layers.0.input_layernorm.weight"].dtype == torch.float32
    assert not w.requires_grad


def test_unsupported_quant_type_raises_value_error(tmp_path):
    path = str(tmp_path / "u.gguf")
    _make_file(path, extra=[("odd.weight", np.zeros((2, 36), dtype=np.uint8), int(GGMLQuantizationType.Q8_1))])
    with pytest.raises(ValueError, match="odd.weight has unsupported quant type") as exc:
        load_gguf_checkpoint(path)
    assert "Supported" in str(exc.value) and "Q8_0" in str(exc.value)


@pytest.mark.parametrize("quant", [GGMLQuantizationType.Q8_0, GGMLQuantizationType.Q4_K, GGMLQuantizationType.Q5_K,
                                   GGMLQuantizationType.Q6_K, GGMLQuantizationType.Q4_0, GGMLQuantizationType.Q5_1,
                                   GGMLQuantizationType.Q3_K])
def test_set_gguf2meta_model_replaces_and_places(tmp_path, quant):
    path = str(tmp_path / "m.gguf")
    ref, packed = _make_file(path, quant)
    sd = load_gguf_checkpoint(path)
    with torch.device("meta"):
        model = TinyModel()
    report = match_state_dict(model, sd)
    assert report["matching"] == len(sd) and not report["extra"] and not report["missing"]
    model = set_gguf2meta_model(model, sd, torch.bfloat16, torch.device("cpu"))
    # every Linear whose weight is quantized in the file was swapped, by the generic rule
    n_expected = 2 * (2 + 6) + 1
    assert count_gguf_linear(model) == n_expected
    assert type(model.lm_head) is nn.Linear and model.lm_head.weight.dtype == torch.bfloat16
    assert type(model.embed_tokens) is nn.Embedding and model.embed_tokens.weight.dtype == torch.bfloat16
    te = model.timestep_embedder
    assert type(te).__name__ == "GGUFLinear" and te.bias is not None and te.bias.dtype == torch.bfloat16
    assert te.compute_dtype == torch.bfloat16 and (te.in_features, te.out_features) == (H, H)
    for name, mod in model.named_modules():
        if isinstance(mod, GGUFLinear):
            w = mod.weight
            assert isinstance(w, GGUFParameter) and w.dtype == torch.uint8 and w.device.type == "cpu"
            assert w.quant_type == quant and tuple(w.quant_shape) == (mod.out_features, mod.in_features)
            assert np.array_equal(w.as_tensor().numpy(), packed[name + ".weight"])
            assert not w.requires_grad
    assert not any(p.device.type == "meta" for p in model.parameters())
    assert model.layers[0].input_layernorm.weight.dtype == torch.bfloat16
    assert torch.equal(model.inv_freq, torch.ones(4))


def test_missing_and_extra_keys(tmp_path, capsys):
    path = str(tmp_path / "m.gguf")
    _make_file(path, skip=("layers.1.q_proj.weight",), extra=[("stray.weight", np.zeros((2, 34), dtype=np.uint8), 8)])
    sd = load_gguf_checkpoint(path)
    with torch.device("meta"):
        model = TinyModel()
    report = match_state_dict(model, sd, show_num=3)
    assert report["extra"] == {"stray.weight"} and report["missing"] == {"layers.1.q_proj.weight"}
    out = capsys.readouterr().out
    assert "[gguf] matching keys" in out and "+ stray.weight" in out and "- layers.1.q_proj.weight" in out
    model = set_gguf2meta_model(model, sd, torch.bfloat16, None)
    assert type(model.layers[1].q_proj) is nn.Linear                  # not in the file: left alone, still on meta
    assert model.layers[1].q_proj.weight.device.type == "meta"
    assert type(model.layers[0].q_proj).__name__ == "GGUFLinear"


def test_shape_mismatch_raises(tmp_path):
    path = str(tmp_path / "m.gguf")
    _make_file(path, skip=("layers.0.q_proj.weight",),
               extra=[("layers.0.q_proj.weight", np.zeros((H, (H // 32 - 1) * 34), dtype=np.uint8), 8)])
    sd = load_gguf_checkpoint(path)
    with torch.device("meta"):
        model = TinyModel()
    with pytest.raises(ValueError, match="layers.0.q_proj.weight"):
        set_gguf2meta_model(model, sd, torch.bfloat16, torch.device("cpu"))


def test_parameter_tag_survives_offloader_style_handling():
    """What the layer offloader does to a weight (layer_offload.py:313-320,349-356,373-375): keep a
    CPU copy, rebind .data to another tensor and back.  The tag lives on the Parameter object."""
    packed = synthetic.make_packed(8, 16, 64)
    p = GGUFParameter(packed, quant_type=8)
    assert p.quant_type == GGMLQuantizationType.Q8_0 and p.quant_shape == (16, 64)
    moved = p.to("cpu", copy=True)
    assert isinstance(moved, GGUFParameter) and moved.quant_type == p.quant_type and moved.quant_shape == (16, 64)
    viewed = p.view(torch.uint8)
    assert getattr(viewed, "quant_type", None) == p.quant_type
    keep = p.data
    p.data = torch.zeros_like(keep)
    assert p.quant_type == GGMLQuantizationType.Q8_0 and int(p.sum()) == 0
    p.data = keep
    assert torch.equal(p.as_tensor(), packed)
    plain = p.as_tensor()
    assert type(plain) is torch.Tensor and not hasattr(plain, "quant_type")
    q = copy.deepcopy(p)
    assert isinstance(q, GGUFParameter) and q.quant_type == p.quant_type and torch.equal(q.as_tensor(), packed)
    lin = GGUFLinear(64, 16, bias=False, compute_dtype=torch.bfloat16, device="meta")
    lin.weight = p
    lin = lin.to(dtype=torch.float16)                                  # Module.to(dtype) leaves uint8 alone
    assert lin.weight.dtype == torch.uint8 and lin.weight.quant_type == GGMLQuantizationType.Q8_0
    assert "quant_type=Q8_0" in repr(lin)
    with pytest.raises(ValueError):
        GGUFParameter(packed)                                           # no quant type


def test_forward_on_cpu_fails_loudly():
    """There is no CPU arithmetic behind the module: a CPU forward raises instead of silently
    computing something else."""
    lin = GGUFLinear(64, 16, bias=False, compute_dtype=torch.bfloat16, device="meta")
    lin.weight = GGUFParameter(synthetic.make_packed(8, 16, 64), quant_type=8)
    with pytest.raises(ops.SnGgufError, match="no CPU implementation"):
        lin(torch.zeros(2, 64, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="dtype"):
        lin(torch.zeros(2, 64, dtype=torch.float32))
    plain = GGUFLinear(64, 16, device="meta")
    with pytest.raises(RuntimeError, match="GGUFParameter"):
        plain(torch.zeros(2, 64, device="meta"))


def test_meta_shape_inference():
    x = torch.empty(3, 5, 64, dtype=torch.bfloat16, device="meta")
    w = torch.empty(16, 68, dtype=torch.uint8, device="meta")
    assert torch.ops.sn_gguf.linear(x, w, 8, None, 1).shape == (3, 5, 16)
    assert torch.ops.sn_gguf.dequantize(w, 8, torch.float32, 0).shape == (16, 64)
    assert torch.ops.sn_gguf.gate_up_silu(x, w, w, 8, 1).shape == (3, 5, 16)
    assert torch.ops.sn_gguf.grouped_linear(x, None, 4, w, 8, w, 8, None, None, 1).shape == (3, 5, 16)


def test_find_mot_pairs(tmp_path):
    """Generation twins are found by the `_mot_gen` suffix rule (layer_offload.py:195-222; the
    reference pins the same partition in tests/test_layer_offload.py:267-281)."""
    path = str(tmp_path / "m.gguf")
    _make_file(path)
    sd = load_gguf_checkpoint(path)
    with torch.device("meta"):
        model = TinyModel()
    model = set_gguf2meta_model(model, sd, torch.bfloat16, torch.device("cpu"))
    pairs = find_mot_pairs(model)
    assert set(pairs) == {f"layers.{i}.{n}" for i in (0, 1) for n in
                          ("q_proj", "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")}
    und, gen = pairs["layers.1.mlp.down_proj"]
    assert und is model.layers[1].mlp.down_proj and gen is model.layers[1].mlp.down_proj_mot_gen


def test_set_decode_layout_walks_the_model(tmp_path):
    """set_decode_layout switches every GGUFLinear (and nothing else); on a CPU host nothing is built."""
    from sensenova_u1_amd import set_decode_layout
    path = str(tmp_path / "m.gguf")
    _make_file(path, 8)
    sd = load_gguf_checkpoint(path)
    with torch.device("meta"):
        model = TinyModel()
    model = set_gguf2meta_model(model, sd, torch.bfloat16, "cpu")
    n = count_gguf_linear(model)
    assert set_decode_layout(model, "tiled") == n > 0
    assert all(m.decode_layout == "tiled" for m in model.modules() if type(m).__name__ == "GGUFLinear")
    assert all(m.tiled_weight() is None for m in model.modules() if type(m).__name__ == "GGUFLinear")   # weights on the CPU
    assert set_decode_layout(model, "native") == n
    with pytest.raises(ValueError):
        set_decode_layout(model, "blocked")


def _bf16_rows(t: torch.Tensor) -> np.ndarray:
    """A float tensor as the uint8 rows a GGUF file stores for type BF16 (two bytes per element)."""
    b = t.detach().to(torch.bfloat16).contiguous()
    return b.view(torch.uint8).reshape(*b.shape[:-1], 2 * b.shape[-1]).numpy()


def test_bf16_tensors_are_wrapped_and_placed(tmp_path):
    """BF16 is a GGUF tensor type like the quantized ones (only F32 / F16 are exempt in the reference,
    gguf_loader.py:37-41): a Linear weight stored as BF16 becomes a GGUFLinear of type BF16, a BF16 side tensor
    (here a norm weight) is decoded into its plain slot."""
    torch.manual_seed(0)
    ref = TinyModel()
    bf = GGMLQuantizationType.BF16
    skip = ("lm_head.weight", "layers.0.input_layernorm.weight")
    extra = [("lm_head.weight", _bf16_rows(ref.lm_head.weight), int(bf)),
             ("layers.0.input_layernorm.weight", _bf16_rows(ref.layers[0].input_layernorm.weight), int(bf))]
    path = str(tmp_path / "b.gguf")
    _make_file(path, skip=skip, extra=extra)
    sd = load_gguf_checkpoint(path)
    w = sd["lm_head.weight"]
    assert isinstance(w, GGUFParameter) and w.quant_type == bf and tuple(w.shape) == (32, 2 * H) and tuple(w.quant_shape) == (32, H)
    g = sd["layers.0.input_layernorm.weight"]
    assert isinstance(g, GGUFParameter) and tuple(g.quant_shape) == (H,)
    with torch.device("meta"):
        model = TinyModel()
    model = set_gguf2meta_model(model, sd, torch.bfloat16, torch.device("cpu"))
    assert type(model.lm_head).__name__ == "GGUFLinear" and model.lm_head.weight.quant_type == bf
    assert torch.equal(model.lm_head.weight.as_tensor().view(torch.bfloat16), ref.lm_head.weight.detach().to(torch.bfloat16))
    norm = model.layers[0].input_layernorm.weight
    assert type(norm) is nn.Parameter and norm.dtype == torch.bfloat16
    assert torch.equal(norm.detach(), ref.layers[0].input_layernorm.weight.detach().to(torch.bfloat16))
    # the oracle decodes type 30 exactly, in both modes and both restatements
    want = ref.lm_head.weight.detach().to(torch.bfloat16).float()
    for numerics in (0, 1):
        assert torch.equal(go.dequantize_gguf_tensor(w.as_tensor(), go.BF16, numerics), want)
        assert torch.equal(go.COracle().dequantize(w.as_tensor(), go.BF16, torch.float32, numerics), want)


def test_load_gguf_model_one_call(tmp_path, capsys):
    """The sequence of checkpoint_loading.py:288-323 in one call: meta model (or config + factory) -> parsed file ->
    swapped and placed -> count reported -> eval mode; and the warning when nothing was quantized."""
    from sensenova_u1_amd import load_gguf_model
    path = str(tmp_path / "m.gguf")
    ref, packed = _make_file(path)
    with torch.device("meta"):
        meta = TinyModel()
    model = load_gguf_model(meta, path, dtype=torch.bfloat16, device="cpu")
    out = capsys.readouterr().out
    assert f"[gguf] loading quantized checkpoint from {path}" in out and "[gguf] parsed" in out
    assert f"[gguf] {2 * (2 + 6) + 1} GGUFLinear modules active" in out and "WARNING" not in out
    assert model is meta and not model.training
    assert not any(p.device.type == "meta" for p in model.parameters())
    # a config and a factory
    model2 = load_gguf_model({"unused": 1}, path, dtype=torch.bfloat16, device=torch.device("cpu"), model_factory=lambda cfg: TinyModel())
    assert count_gguf_linear(model2) == count_gguf_linear(model)
    assert np.array_equal(model2.layers[1].mlp.up_proj.weight.as_tensor().numpy(), packed["layers.1.mlp.up_proj.weight"])
    # a model that already holds storage is refused
    with pytest.raises(ValueError, match="meta-initialized"):
        load_gguf_model(TinyModel(), path, dtype=torch.bfloat16, device="cpu")
    # a file without quantized tensors: loads, and says so
    plain_path = str(tmp_path / "p.gguf")
    torch.manual_seed(0)
    plain = TinyModel()
    write_gguf(plain_path, [(n, t.detach().numpy().astype(np.float32), 0) for n, t in plain.state_dict().items()])
    capsys.readouterr()
    model3 = load_gguf_model(None, plain_path, dtype=torch.float32, device="cpu", model_factory=lambda cfg: TinyModel())
    out = capsys.readouterr().out
    assert "[gguf] 0 GGUFLinear modules active" in out and "WARNING: no GGUFLinear modules found" in out
    assert torch.equal(model3.lm_head.weight, plain.lm_head.weight)


@pytest.mark.parametrize("rows", [1, 100, 300])
def test_module_with_host_weight_raises_before_any_launch(rows):
    """Every row count - decode, the split-K workspace route, the weight-pass route - refuses host tensors with the
    library's own error type; nothing reaches a kernel with a host pointer."""
    lin = GGUFLinear(256, 512, bias=False, compute_dtype=torch.bfloat16, device="meta")
    lin.weight = GGUFParameter(synthetic.make_packed(8, 512, 256), quant_type=8)
    with pytest.raises(ops.SnGgufError):
        lin(torch.zeros(rows, 256, dtype=torch.bfloat16))
    with pytest.raises(ops.SnGgufError):
        lin._checked_rows(torch.zeros(rows, 256, dtype=torch.bfloat16), torch.ones(256, dtype=torch.bfloat16))


class _GatedMLP(nn.Module):
    """The shape of the reference's Qwen3MLP (modeling_qwen3.py:203-216)."""

    def __init__(self, act=None):
        super().__init__()
        self.gate_proj = nn.Linear(H, I, bias=False)
        self.up_proj = nn.Linear(H, I, bias=False)
        self.down_proj = nn.Linear(I, H, bias=False)
        self.act_fn = act if act is not None else nn.SiLU()

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


class _TwoArgMLP(_GatedMLP):
    def forward(self, x, scale):
        return super().forward(x) * scale


class _MLPModel(nn.Module):
    def __init__(self):
        super().__init__()
        self.a = _GatedMLP()
        self.b = _GatedMLP(act=nn.GELU())
        self.c = _TwoArgMLP()
        self.d = _GatedMLP(act=torch.nn.functional.silu)


def test_gated_mlps_are_fused_by_the_one_call_loader(tmp_path, capsys):
    """load_gguf_model points the forward of Qwen3MLP-shaped modules (three GGUFLinear projections, a SiLU act_fn, a
    forward of one argument) at the fused gated MLP; other activations and other signatures keep their own forward;
    fuse_mlp=False and unfuse_gated_mlps leave / restore the class's forward."""
    from sensenova_u1_amd import fuse_gated_mlps, load_gguf_model, modality, unfuse_gated_mlps
    torch.manual_seed(1)
    ref = _MLPModel()
    tensors = [(n, go.quantize_q8_0(t.detach().numpy()), int(GGMLQuantizationType.Q8_0)) for n, t in ref.state_dict().items()]
    path = str(tmp_path / "mlp.gguf")
    write_gguf(path, tensors)

    def fused(m):
        return getattr(m.forward, "__func__", None) is modality._fused_mlp_forward

    with torch.device("meta"):
        meta = _MLPModel()
    model = load_gguf_model(meta, path, dtype=torch.bfloat16, device="cpu")
    out = capsys.readouterr().out
    assert "[gguf] 12 GGUFLinear modules active" in out
    assert "[gguf] 2 gated MLP modules run gate / up / SiLU as one launch at decode" in out
    assert fused(model.a) and fused(model.d) and not fused(model.b) and not fused(model.c)
    assert fuse_gated_mlps(model) == 2                     # idempotent
    assert unfuse_gated_mlps(model) == 2
    assert not fused(model.a) and model.a.forward.__func__ is _GatedMLP.forward
    with torch.device("meta"):
        meta2 = _MLPModel()
    model2 = load_gguf_model(meta2, path, dtype=torch.bfloat16, device="cpu", fuse_mlp=False)
    assert "gated MLP modules" not in capsys.readouterr().out
    assert not fused(model2.a) and not fused(model2.d)
