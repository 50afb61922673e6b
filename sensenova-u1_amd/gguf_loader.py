"""GGUF checkpoint loader: the loader half of the drop-in boundary.

Same three functions, signatures, tensor-name mapping (identity) and error behaviour as
``src/sensenova_u1/utils/gguf_loader.py`` of the reference, with the third-party ``gguf`` /
``diffusers`` machinery replaced by this package's own reader and ``GGUFLinear``:

    load_gguf_checkpoint(path) -> dict[str, Tensor | GGUFParameter]        (reference :17-47)
    set_gguf2meta_model(meta_model, state_dict, dtype, device) -> nn.Module (reference :50-85)
    match_state_dict(meta_model, state_dict, show_num=10) -> dict           (reference :88-114)

plus ``load_gguf_model``, the one-call form of the sequence the reference's model loader runs around them
(``src/sensenova_u1/utils/checkpoint_loading.py:288-323``).
"""
from __future__ import annotations

import gc

import torch
from torch import nn

from .gguf_file import GGML_QUANT_SIZES, GGMLQuantizationType, NativeGGUFReader
from .quantized_linear import (
    SUPPORTED_GGUF_QUANT_TYPES,
    GGUFLinear,
    GGUFParameter,
    _quant_shape_from_byte_shape,
    _replace_with_gguf_linear,
)


_TORCH_PLAIN = {GGMLQuantizationType.F32: torch.float32, GGMLQuantizationType.F16: torch.float16}


def load_gguf_checkpoint(gguf_checkpoint_path: str, pin_memory: bool = False, threads: int = 8) -> dict:
    """Parse a .gguf file into a state-dict-compatible mapping.

    F32 / F16 tensors come back as plain torch tensors; every other type must be one the HIP
    kernels decode and is wrapped in ``GGUFParameter`` (packed bytes, copied out of the file
    mapping).  That includes BF16, as in the reference (``gguf_loader.py:37-43``: only F32 and F16
    are exempt from the supported-types check and the wrapping).  Tensor names are used
    verbatim: GGUF names are the model's state-dict keys.

    The file is parsed by the library's C++ reader and all payloads are copied in one
    multi-threaded pass into freshly allocated host tensors - page-locked ones with
    ``pin_memory=True``, ready for asynchronous upload.
    """
    reader = NativeGGUFReader(gguf_checkpoint_path)
    parsed: dict = {}
    try:
        kinds = []
        for tensor in reader.tensors:
            quant_type = tensor.tensor_type
            is_quant = quant_type not in _TORCH_PLAIN
            if is_quant and quant_type not in SUPPORTED_GGUF_QUANT_TYPES:
                supported = "\n".join(str(t) for t in SUPPORTED_GGUF_QUANT_TYPES)
                raise ValueError(f"{tensor.name} has unsupported quant type {quant_type!s}.\nSupported:\n{supported}")
            kinds.append(is_quant)
        buffers = []
        for tensor, is_quant in zip(reader.tensors, kinds):
            dtype = torch.uint8 if is_quant else _TORCH_PLAIN[tensor.tensor_type]
            buffers.append(torch.empty(tuple(tensor.data.shape), dtype=dtype, pin_memory=pin_memory))
        reader.read_into(list(range(len(buffers))), buffers, threads=threads)
        for tensor, is_quant, weights in zip(reader.tensors, kinds, buffers):
            parsed[tensor.name] = GGUFParameter(weights, quant_type=tensor.tensor_type) if is_quant else weights
    finally:
        reader.close()
        del reader
        gc.collect()
    return parsed


def _split_param_name(model: nn.Module, full_name: str):
    module_path, _, leaf = full_name.rpartition(".")
    module = model.get_submodule(module_path) if module_path else model
    return module, leaf


def _load_state_dict_into_meta(model: nn.Module, state_dict: dict, dtype: torch.dtype | None, device) -> list[str]:
    """Place every tensor of ``state_dict`` that the model has a slot for.  Quantized entries
    keep their bytes and tag (after a shape check against the slot); plain entries are cast to
    ``dtype`` when they are floating point.  Returns the keys the model had no slot for."""
    expected = set(model.state_dict().keys())
    unexpected = []
    target = torch.device(device) if device is not None else torch.device("cpu")
    for name, value in state_dict.items():
        if name not in expected:
            unexpected.append(name)
            continue
        module, leaf = _split_param_name(model, name)
        is_buffer = leaf in module._buffers
        slot = module._buffers[leaf] if is_buffer else module._parameters[leaf]
        if isinstance(value, GGUFParameter) and value.quant_type == GGMLQuantizationType.BF16 \
                and not (type(module).__name__ == GGUFLinear.__name__ and leaf == "weight"):
            # a BF16 tensor outside a quantized linear (norm weight, embedding, bias ...): nothing would decode it at
            # forward time, so it is decoded here - a reinterpretation of the two-byte elements, no arithmetic
            value = value.as_tensor().view(torch.bfloat16)
        if isinstance(value, GGUFParameter):
            block_size, type_size = GGML_QUANT_SIZES[value.quant_type]
            inferred = _quant_shape_from_byte_shape(value.shape, type_size, block_size)
            if slot is not None and tuple(inferred) != tuple(slot.shape):
                raise ValueError(
                    f"{name} has an expected quantized shape of: {tuple(inferred)}, but received shape: {tuple(slot.shape)}")
            placed = value.to(target)
            if not isinstance(placed, GGUFParameter) or not hasattr(placed, "quant_type"):
                placed = GGUFParameter(placed, quant_type=value.quant_type)
            placed.requires_grad_(False)
            module._parameters[leaf] = placed
            continue
        if slot is not None and tuple(value.shape) != tuple(slot.shape):
            raise ValueError(
                f"Cannot load {name} because its shape {tuple(value.shape)} does not match the model's "
                f"{tuple(slot.shape)}")
        tensor = value.to(device=target, dtype=dtype if (dtype is not None and value.is_floating_point()) else None)
        if is_buffer:
            module._buffers[leaf] = tensor
        else:
            module._parameters[leaf] = nn.Parameter(tensor, requires_grad=False)
    return unexpected


def set_gguf2meta_model(
    meta_model: nn.Module,
    model_state_dict: dict,
    dtype: torch.dtype,
    device: torch.device | None,
) -> nn.Module:
    """Inject GGUF weights into a meta-initialized model.

    The model must have been built on the meta device (``accelerate.init_empty_weights()`` or
    ``torch.device("meta")``).  This function:
      1. replaces every ``nn.Linear`` whose ``<prefix>weight`` is quantized in the dict with
         ``GGUFLinear(in, out, bias is not None, compute_dtype=dtype or bf16)``;
      2. loads the parsed state dict into the model on ``device``;
      3. returns the model cast to ``dtype`` (floating-point, i.e. non-quantized, params only).
    """
    compute_dtype = dtype or torch.bfloat16
    _replace_with_gguf_linear(meta_model, compute_dtype, model_state_dict)
    _load_state_dict_into_meta(meta_model, model_state_dict, dtype, device)
    del model_state_dict
    gc.collect()
    return meta_model.to(dtype=dtype)


def match_state_dict(meta_model: nn.Module, sd: dict, show_num: int = 10) -> dict:
    """Debug helper: compare the keys of a parsed state dict with the model's.

    Prints a short report and returns ``{"matching": int, "extra": set, "missing": set}``
    (``extra``: in the file only, ``missing``: in the model only)."""
    wanted = set(meta_model.state_dict())
    given = set(sd)
    report = {"matching": len(wanted & given), "extra": given - wanted, "missing": wanted - given}

    def show(title: str, keys: set, mark: str) -> None:
        if keys:
            print(f"[gguf] {title}: {len(keys)}")
            for key in sorted(keys)[:show_num]:
                print(f"  {mark} {key}")

    print(f"[gguf] matching keys: {report['matching']}")
    show("extra in state_dict (not in model)", report["extra"], "+")
    show("missing in state_dict (in model only)", report["missing"], "-")
    print(f"[gguf] sample matches: {sorted(wanted & given)[:5]}")
    return report


def count_gguf_linear(model: nn.Module) -> int:
    """Number of active ``GGUFLinear`` modules, found by type name as the reference's sanity
    check does (``src/sensenova_u1/utils/checkpoint_loading.py:315``)."""
    return sum(1 for m in model.modules() if type(m).__name__ == GGUFLinear.__name__)


def load_gguf_model(config_or_meta_model, gguf_checkpoint: str, *, dtype: torch.dtype,
                    device: str | torch.device | None, model_factory=None, fuse_mlp: bool = True,
                    stack_qkv: bool = True) -> nn.Module:
    """The whole GGUF branch of the reference's model loader in one call
    (``_load_from_gguf``, ``src/sensenova_u1/utils/checkpoint_loading.py:288-323``): build the model without
    storage, parse the file, swap the quantized linears in and place the tensors on ``device``, report how many
    ``GGUFLinear`` modules are active - with the reference's warning when there are none - and return the model
    in eval mode.

    ``config_or_meta_model`` is either a model that already lives on the meta device, or a config: then
    ``model_factory(config)`` is called under ``torch.device("meta")``, and without a factory the reference's own
    construction is used (``transformers.AutoModel.from_config`` under ``accelerate.init_empty_weights``).

    ``fuse_mlp`` (an addition to the reference's behaviour, on by default): the SiLU-gated MLPs whose three
    projections became ``GGUFLinear`` get ``modality.fuse_gated_mlps``'s forward, i.e. gate, up and the SiLU product in
    one launch at decode row counts; the results keep every rounding of the three module calls.
    ``stack_qkv`` (likewise, when the model lands on a HIP device): ``q_proj`` / ``k_proj`` / ``v_proj`` of every
    attention module share one weight tensor (``modality.SharedInputStack``) and one decode launch.
    """
    print(f"[gguf] loading quantized checkpoint from {gguf_checkpoint}")
    if isinstance(config_or_meta_model, nn.Module):
        model = config_or_meta_model
        on_storage = [n for n, p in model.named_parameters() if p.device.type != "meta"]
        if on_storage:
            raise ValueError(f"load_gguf_model needs a meta-initialized model; {on_storage[0]} already has storage")
    elif model_factory is not None:
        with torch.device("meta"):
            model = model_factory(config_or_meta_model)
    else:
        try:
            from accelerate import init_empty_weights
        except ImportError as exc:
            raise RuntimeError("GGUF loading requires `accelerate`; install it in your environment.") from exc
        from transformers import AutoModel

        with init_empty_weights():
            model = AutoModel.from_config(config_or_meta_model)

    state_dict = load_gguf_checkpoint(gguf_checkpoint)
    print(f"[gguf] parsed {len(state_dict)} tensors")
    target_device = torch.device(device) if isinstance(device, str) else device
    set_gguf2meta_model(model, state_dict, dtype, target_device)

    n_gguf_linear = count_gguf_linear(model)
    print(f"[gguf] {n_gguf_linear} GGUFLinear modules active (HIP dequant-GEMV / dequant-GEMM at forward time)")
    if n_gguf_linear == 0:
        print("[gguf] WARNING: no GGUFLinear modules found — no Linear of the model has a quantized weight in the file")
    if fuse_mlp and n_gguf_linear:
        from .modality import fuse_gated_mlps

        print(f"[gguf] {fuse_gated_mlps(model)} gated MLP modules run gate / up / SiLU as one launch at decode")
    if stack_qkv and n_gguf_linear and target_device is not None and torch.device(target_device).type == "cuda":
        from .modality import stack_shared_input_projections

        print(f"[gguf] {stack_shared_input_projections(model)} q / k / v groups share one weight tensor and one decode launch")

    del state_dict
    gc.collect()
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return model.eval()
