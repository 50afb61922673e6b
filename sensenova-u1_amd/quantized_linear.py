"""``GGUFParameter`` and ``GGUFLinear``: the module half of the drop-in boundary.

The reference gets both from ``diffusers.quantizers.gguf.utils``
(``src/sensenova_u1/utils/gguf_loader.py:30,43,64-81``) and recognises the module by its type
name (``src/sensenova_u1/utils/checkpoint_loading.py:315``).  Same constructor, same
``forward(inputs)``; the arithmetic behind it is the HIP library, not torch elementwise ops.

``weight`` keeps the GGUF-native bytes ``uint8 [out_features, in_features / block * type_size]``
and carries ``quant_type`` / ``quant_shape`` on the Parameter object itself, so they survive
``weight.data = <other storage>`` - which the layer offloader does around every forward
(``src/sensenova_u1/utils/layer_offload.py:349-356,373-375``).
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from . import ops
from .gguf_file import GGML_QUANT_SIZES, GGMLQuantizationType

# quant types the HIP kernels decode
SUPPORTED_GGUF_QUANT_TYPES = (
    GGMLQuantizationType.Q4_0,
    GGMLQuantizationType.Q4_1,
    GGMLQuantizationType.Q5_0,
    GGMLQuantizationType.Q5_1,
    GGMLQuantizationType.Q8_0,
    GGMLQuantizationType.Q2_K,
    GGMLQuantizationType.Q3_K,
    GGMLQuantizationType.Q4_K,
    GGMLQuantizationType.Q5_K,
    GGMLQuantizationType.Q6_K,
    GGMLQuantizationType.BF16,   # upstream lists it too: a BF16 tensor is wrapped and decoded like a quantized one
)


def _quant_shape_from_byte_shape(shape, type_size: int, block_size: int):
    return (*shape[:-1], shape[-1] // type_size * block_size)


class GGUFParameter(torch.nn.Parameter):
    """uint8 parameter holding packed GGUF blocks, tagged with its ggml type."""

    def __new__(cls, data, requires_grad: bool = False, quant_type=None):
        if quant_type is None:
            raise ValueError("GGUFParameter needs a quant_type")
        data = data if data is not None else torch.empty(0, dtype=torch.uint8)
        self = torch.Tensor._make_subclass(cls, data, requires_grad)
        self.quant_type = GGMLQuantizationType(int(quant_type))
        block_size, type_size = GGML_QUANT_SIZES[self.quant_type]
        self.quant_shape = _quant_shape_from_byte_shape(self.shape, type_size, block_size)
        return self

    def as_tensor(self) -> torch.Tensor:
        """The same storage as a plain tensor (no subclass, no tag)."""
        return torch.Tensor._make_subclass(torch.Tensor, self, self.requires_grad)

    @staticmethod
    def _tag_source(args):
        for a in args:
            if isinstance(a, GGUFParameter):
                return a
            if isinstance(a, (list, tuple)):
                for b in a:
                    if isinstance(b, GGUFParameter):
                        return b
        return None

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        result = super().__torch_function__(func, types, args, kwargs)
        # .to() / .cuda() / .pin_memory() / views hand back the subclass without Python attributes
        src = cls._tag_source(args)
        if src is None:
            return result

        def retag(t):
            if isinstance(t, torch.Tensor) and t.dtype == torch.uint8 and t.dim() >= 1 and not hasattr(t, "quant_type"):
                _, ts = GGML_QUANT_SIZES[src.quant_type]
                if t.shape[-1] % ts == 0:
                    if not isinstance(t, GGUFParameter):
                        t = torch.Tensor._make_subclass(cls, t, False)
                    t.quant_type = src.quant_type
                    t.quant_shape = _quant_shape_from_byte_shape(t.shape, ts, GGML_QUANT_SIZES[src.quant_type][0])
            return t

        if isinstance(result, torch.Tensor):
            return retag(result)
        if isinstance(result, (tuple, list)):
            return type(result)(retag(r) for r in result)
        return result

    def __deepcopy__(self, memo):
        if id(self) in memo:
            return memo[id(self)]
        clone = GGUFParameter(self.as_tensor().detach().clone(memory_format=torch.preserve_format),
                              requires_grad=self.requires_grad, quant_type=self.quant_type)
        memo[id(self)] = clone
        return clone

    def __reduce_ex__(self, proto):
        return (_rebuild_gguf_parameter, (self.as_tensor().detach(), int(self.quant_type)))


def _rebuild_gguf_parameter(data, quant_type):
    return GGUFParameter(data, quant_type=quant_type)


def dequantize_gguf_tensor(tensor: torch.Tensor, dtype: Optional[torch.dtype] = None,
                           numerics: int = ops.NUM_UPSTREAM_FP16) -> torch.Tensor:
    """Packed parameter -> dense ``quant_shape`` tensor on the same (HIP) device.

    With the default numerics the result is the fp16 tensor the reference's
    ``dequantize_gguf_tensor`` returns; ``numerics=ops.NUM_GGML_FP32`` gives ggml's exact fp32
    values.  Tensors without a ``quant_type`` pass through unchanged, as upstream does.
    """
    if not hasattr(tensor, "quant_type"):
        return tensor
    if dtype is None:
        # (upstream's BF16 decode returns fp32 whatever the mode)
        plain = int(tensor.quant_type) == ops.BF16
        dtype = torch.float16 if numerics == ops.NUM_UPSTREAM_FP16 and not plain else torch.float32
    return ops.dequantize(tensor, int(tensor.quant_type), dtype, numerics)


def set_decode_layout(model: nn.Module, layout: str = "tiled", build_now: bool = False) -> int:
    """Set ``decode_layout`` on every ``GGUFLinear`` below ``model`` (including ``model`` itself) and return how many
    were switched.  ``"tiled"`` makes the decode path (at most 16 rows) of Q8_0 modules whose ``in_features`` is a
    multiple of 256 read an operand-order copy of the weight, built on first use - or right away with ``build_now``
    for weights that are already on the device - and kept beside the GGUF rows (the same number of bytes again);
    ``"native"`` switches back and releases the copies."""
    if layout not in ("native", "tiled"):
        raise ValueError(f"decode layout is {layout!r}; expected 'native' or 'tiled'")
    count = 0
    for mod in model.modules():
        if type(mod).__name__ != "GGUFLinear":
            continue
        mod.decode_layout = layout
        if layout == "native":
            mod.drop_tiled_cache()
        elif build_now:
            mod.tiled_weight()
        count += 1
    return count


def rms_norm(hidden_states: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNorm as the decoder layers compute it (``Qwen3RMSNorm.forward``, ``modeling_qwen3.py:192-197``): statistic
    and scaling in fp32, one rounding to the input dtype, then the product with the weight in that dtype.  bf16 rows
    on the device run as one library launch (``sngguf_rmsnorm``), anything else as the tensor operations."""
    if (hidden_states.is_cuda and weight.is_cuda and hidden_states.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
            and hidden_states.shape[-1] % 8 == 0 and weight.numel() == hidden_states.shape[-1]):
        return ops.rms_norm(hidden_states, weight, eps)        # the library's one-launch form
    h = hidden_states.float()
    h = h * torch.rsqrt(h.square().mean(dim=-1, keepdim=True) + eps)
    return weight * h.to(hidden_states.dtype)


class GGUFLinear(nn.Linear):
    """``nn.Linear`` whose weight is a :class:`GGUFParameter`.

    ``forward`` computes ``F.linear(x, dequantize(weight).to(compute_dtype), bias)`` with the
    reference's rounding chain.  With bf16 activations and at most 16 rows (decode) - at most 64 rows
    when ``in_features`` is a multiple of 256 - it is one fused dequant-GEMV launch that streams and
    decodes the weights once.  With more rows ``gemm_policy`` decides:

    * ``"auto"`` (default): the library's own kernels through ``sngguf_linear_ws`` with a pooled workspace of
      2 * N * K bytes, plus room for four fp32 copies of the output when the shape has few output tiles
      (``ops.pooled_workspace``, one per device and stream, reused by every module): problems with few
      output tiles run the large-tile kernel with K split over workgroups, the rest one weight pass into the
      workspace (bf16, the same rounding chain) followed by the library's dense bf16 tile kernel.
    * ``"two_pass"`` (opt-in): one HIP dequantize launch writes a transient bf16 weight and the device library's
      dense GEMM (``torch.matmul``) consumes it: no kernel of this library does the contraction then.  At 4096 rows it
      is about 10 % faster than ``"auto"`` on MI355X.
    * ``"fused"``: the fused dequant-GEMM kernels of the library (``sngguf_linear``), which need
      no transient memory.
    * ``"resident"``: the bf16 weight is written once by the library's weight pass, kept (2 * N * K bytes per module)
      and reused by later calls until the packed bytes move or change; every call is then the library's dense tile
      kernel alone (K split over workgroups for few output tiles).  For towers that see thousands of
      rows many times over (the denoising loop) on a device with memory to spare, it removes the
      weight pass from every call but the first.  Not meant to be combined with layer offloading; after an in-place
      rewrite of the packed bytes through ``weight.data`` call ``weights_changed()``.

    ``decode_layout = "tiled"`` (Q8_0 with ``in_features`` a multiple of 256 only; default ``"native"``) makes the
    decode calls (at most 16 rows) read an operand-order copy of the weight that is built on first use and kept
    beside the GGUF bytes (the same 34 bytes per block again): 8 - 10 % faster on the M = 1 MLP step, for models
    that stay resident on the device.  The copy follows the packed bytes: it is rebuilt when they move, and after
    ``weights_changed()`` when they were rewritten in place through ``weight.data``.

    Other compute dtypes always take dequantize + matmul.
    """

    numerics: int = ops.NUM_UPSTREAM_FP16
    gemm_policy: str = "auto"     # "auto" | "two_pass" | "fused" | "resident", for inputs beyond the fused GEMV's row limit
    _dense_cache = None           # (key, bf16 weight) of the "resident" policy
    decode_layout: str = "native"  # "native" | "tiled": weight layout the decode kernels read
    _tiled_cache = None           # (key, operand-order copy) of the "tiled" decode layout

    def __init__(self, in_features: int, out_features: int, bias: bool = False,
                 compute_dtype: Optional[torch.dtype] = None, device=None) -> None:
        super().__init__(in_features, out_features, bias, device)
        self.compute_dtype = compute_dtype

    def _weight_type(self) -> int:
        w = self.weight
        if not hasattr(w, "quant_type"):
            raise RuntimeError("GGUFLinear.weight is not a GGUFParameter (no quant_type); was the checkpoint loaded?")
        return int(w.quant_type)

    def _checked_rows(self, inputs: torch.Tensor, *others: Optional[torch.Tensor]) -> torch.Tensor:
        """``inputs`` as contiguous bf16 rows ``[M, in_features]`` for a raw library call, after the checks the custom
        ops make: every tensor (inputs, weight, bias, ``others``) on one HIP device, the packed weight a whole
        number of blocks of shape ``[out_features, in_features]``, the input's last dim ``in_features``.  Raises
        ``SnGgufError`` before anything is launched - a host pointer handed to a kernel is a GPU memory fault."""
        ops._require_device(inputs, self.weight, self.bias, *others)
        _, n, k = ops._packed_2d(self.weight, self._weight_type())
        if (n, k) != (self.out_features, self.in_features):
            raise ops.SnGgufError(f"GGUFLinear: packed weight decodes to {(n, k)}, the module is {(self.out_features, self.in_features)}")
        if not self.weight.is_contiguous():
            raise ops.SnGgufError("GGUFLinear: the packed weight must be contiguous")
        return ops._as_bf16_rows(inputs, self.in_features, "GGUFLinear")

    def tiled_weight(self) -> Optional[torch.Tensor]:
        """The operand-order copy of the weight when ``decode_layout == "tiled"`` applies to this module (Q8_0,
        ``in_features`` a multiple of 256, weight on the device), built on first use; else ``None``."""
        if self.decode_layout != "tiled":
            if self.decode_layout != "native":
                raise ValueError(f"GGUFLinear.decode_layout is {self.decode_layout!r}; expected 'native' or 'tiled'")
            return None
        if self._weight_type() != ops.Q8_0 or self.in_features % 256 != 0 or self.weight.device.type != "cuda":
            return None
        key = (self.weight.data_ptr(), self.weight._version)
        if self._tiled_cache is None or self._tiled_cache[0] != key:
            self._tiled_cache = (key, ops.q8_0_tile(self.weight.data))
        return self._tiled_cache[1]

    def _decode_tiled(self, inputs: torch.Tensor, residual: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        rows = inputs.numel() // self.in_features if inputs.numel() else 0
        if not 0 < rows <= 16:
            return None
        tiled = self.tiled_weight()
        if tiled is None:
            return None
        x2d = self._checked_rows(inputs, residual)
        out = torch.empty((*inputs.shape[:-1], self.out_features), dtype=torch.bfloat16, device=inputs.device)
        bias = self.bias.detach().to(torch.bfloat16).contiguous() if self.bias is not None else None
        if residual is not None and (residual.dtype != torch.bfloat16 or tuple(residual.shape) != tuple(out.shape)):
            raise ops.SnGgufError(f"GGUFLinear: residual must be bf16 of shape {tuple(out.shape)}")
        res2d = residual.reshape(-1, self.out_features).contiguous() if residual is not None else None
        ops.linear_tiled_into(x2d, tiled, bias, res2d, out.view(-1, self.out_features), self.numerics)
        return out

    def forward(self, inputs: torch.Tensor) -> torch.Tensor:
        qtype = self._weight_type()
        compute_dtype = self.compute_dtype or inputs.dtype
        if inputs.dtype != compute_dtype:
            raise RuntimeError(f"GGUFLinear: input dtype {inputs.dtype} does not match compute dtype {compute_dtype}")
        if compute_dtype == torch.bfloat16:
            rows = inputs.numel() // self.in_features if inputs.numel() else 0
            stack = self.__dict__.get("_shared_stack")   # modality.SharedInputStack: q / k / v in one decode launch
            if stack is not None:
                out = stack.member_forward(self, inputs)
                if out is not None:
                    return out
            if self.decode_layout != "native":
                out = self._decode_tiled(inputs, None)
                if out is not None:
                    return out
            if rows <= 16 or (rows <= 64 and self.in_features % 256 == 0) or self.gemm_policy == "fused" or qtype == ops.BF16:
                return ops.linear(inputs, self.weight, qtype, self.bias, self.numerics)
            if self.gemm_policy not in ("auto", "two_pass", "resident"):
                raise ValueError(f"GGUFLinear.gemm_policy is {self.gemm_policy!r}; expected 'auto', 'two_pass', 'fused' or 'resident'")
            x2d = self._checked_rows(inputs)
            out = torch.empty((*inputs.shape[:-1], self.out_features), dtype=torch.bfloat16, device=inputs.device)
            if self.gemm_policy == "auto":
                # the library's own kernels: K split over workgroups for few output tiles, else one weight pass into the
                # pooled workspace + the dense tile kernel (sngguf_linear_ws picks)
                workspace = ops.pooled_workspace(inputs.device, self._workspace_bytes(rows))
                bias = self.bias.detach().to(torch.bfloat16).contiguous() if self.bias is not None else None
                ops.linear_ws_into(x2d, self.weight, qtype, bias, out.view(-1, self.out_features), workspace, self.numerics)
            else:
                self.two_pass_into(x2d, out.view(-1, self.out_features))
            return out
        weight = ops.dequantize(self.weight, qtype, torch.float16 if self.numerics == ops.NUM_UPSTREAM_FP16 and qtype != ops.BF16
                                else torch.float32, self.numerics).to(compute_dtype)
        bias = self.bias.to(compute_dtype) if self.bias is not None else None
        return torch.nn.functional.linear(inputs, weight, bias)

    def forward_normed(self, inputs: torch.Tensor, norm_weight: torch.Tensor, eps: float) -> torch.Tensor:
        """``self(RMSNorm(inputs))`` with the norm of the decoder layers (``Qwen3RMSNorm``,
        ``modeling_qwen3.py:192-197``; it feeds q / k / v at ``:919`` and the MLP at ``:938``).  Where the library
        offers it (Q8_0, a decode-sized input: ``ops.rmsnorm_fits``) the norm runs inside the projection kernel on
        the activations staged in LDS; otherwise as torch operations in front of ``forward``."""
        rows = inputs.numel() // self.in_features if inputs.numel() else 0
        fused = (inputs.is_cuda and rows > 0 and inputs.dtype == torch.bfloat16 and norm_weight.dtype == torch.bfloat16
                 and (self.compute_dtype or inputs.dtype) == torch.bfloat16
                 and ops.rmsnorm_fits(int(self.weight.quant_type), rows, self.in_features))
        if not fused:
            return self.forward(rms_norm(inputs, norm_weight, eps))
        x2d = self._checked_rows(inputs, norm_weight)
        if norm_weight.numel() != self.in_features:
            raise ops.SnGgufError(f"GGUFLinear: norm weight has {norm_weight.numel()} elements, in_features is {self.in_features}")
        out = torch.empty((*inputs.shape[:-1], self.out_features), dtype=torch.bfloat16, device=inputs.device)
        bias = self.bias.detach().to(torch.bfloat16).contiguous() if self.bias is not None else None
        tiled = self.tiled_weight() if self.decode_layout != "native" else None
        if tiled is not None:
            ops.rmsnorm_linear_tiled_into(x2d, norm_weight.contiguous(), eps, tiled, bias, out.view(-1, self.out_features),
                                          self.numerics)
        else:
            ops.rmsnorm_linear_into(x2d, norm_weight.contiguous(), eps, self.weight, self._weight_type(), bias,
                                    out.view(-1, self.out_features), self.numerics)
        return out

    def forward_argmax(self, inputs: torch.Tensor) -> torch.Tensor:
        """``torch.argmax(self(inputs), dim=-1)`` - the greedy next-token step on an ``lm_head``
        (``modeling_neo_chat.py:557,586``) - with the arg-max taken in the projection kernel's epilogue at decode, so the
        vocabulary-sized logits row is never written."""
        if inputs.dtype != torch.bfloat16 or (self.compute_dtype or inputs.dtype) != torch.bfloat16:
            return self.forward(inputs).argmax(dim=-1)
        return ops.lm_head_argmax(inputs, self.weight, self._weight_type(), self.bias, self.numerics)

    def forward_residual(self, inputs: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
        """``residual + self(inputs)`` (the decoder layer's ``hidden_states = residual + o_proj(...)`` /
        ``residual + mlp(...)``, modeling_qwen3.py:934,940).  For bf16 inputs within the fused kernels' row
        range the add happens in the projection's epilogue; otherwise it is the plain sum."""
        rows = inputs.numel() // self.in_features if inputs.numel() else 0
        fused_rows = rows <= 16 or (rows <= 64 and self.in_features % 256 == 0) or self.gemm_policy == "fused"
        if inputs.dtype == torch.bfloat16 and (self.compute_dtype or inputs.dtype) == torch.bfloat16 and fused_rows \
                and residual.dtype == torch.bfloat16:
            if self.decode_layout != "native":
                out = self._decode_tiled(inputs, residual)
                if out is not None:
                    return out
            return ops.linear_residual(inputs, self.weight, self._weight_type(), residual, self.bias, self.numerics)
        return residual + self(inputs)

    def _workspace_bytes(self, rows: int) -> int:
        """What the workspace route is given for ``rows`` rows: the decoded weight, and for shapes with few 256 x 256
        output tiles room for four fp32 copies of the output behind it (the library then splits K over workgroups)."""
        n, k = self.out_features, self.in_features
        nbytes = ops.linear_workspace_bytes(n, k)
        if -(-rows // 256) * -(-n // 256) <= 128:
            nbytes += 16 * rows * n
        return nbytes

    def two_pass_into(self, x2d: torch.Tensor, out2d: torch.Tensor) -> None:
        """``out2d[M, N] = x2d[M, K] @ W^T (+ bias)`` for bf16 rows: one dequantize launch to a transient
        bf16 weight, then the dense GEMM writing straight into ``out2d`` (contiguous rows)."""
        # the bf16 the kernel writes is the fp16 chain rounded once more, i.e. `.to(bfloat16)` of the fp16 tensor
        if self.gemm_policy == "resident":
            # the kept bf16 rows through the library's own dense tile kernel (K split over workgroups for few tiles)
            key = (self.weight.data_ptr(), self.weight._version, self._weight_type(), self.numerics)
            if self._dense_cache is None or self._dense_cache[0] != key:
                self._dense_cache = (key, ops.dequantize(self.weight, self._weight_type(), torch.bfloat16, self.numerics))
            weight = self._dense_cache[1]
            rows, n = x2d.shape[0], self.out_features
            few = -(-rows // 256) * -(-n // 256) <= 128
            workspace = ops.pooled_workspace(x2d.device, 16 * rows * n) if few else None
            bias = self.bias.detach().to(torch.bfloat16).contiguous() if self.bias is not None else None
            ops.linear_ws_into(x2d, weight.view(torch.uint8), ops.BF16, bias, out2d, workspace, self.numerics)
            return
        else:
            weight = ops.dequantize(self.weight, self._weight_type(), torch.bfloat16, self.numerics)
        if self.bias is None:
            torch.matmul(x2d, weight.t(), out=out2d)
        else:
            torch.addmm(self.bias.to(torch.bfloat16), x2d, weight.t(), out=out2d)

    def weights_changed(self) -> None:
        """Tell the module that the packed bytes were rewritten in place.  The kept copies (``"resident"`` bf16 weight,
        ``"tiled"`` decode layout) follow ``weight.data_ptr()`` and ``weight._version``: rebinding ``weight.data`` or an
        in-place op on ``weight`` itself is noticed, a write through ``weight.data`` (``weight.data.copy_(...)``, what an
        offloader's upload into a reused buffer amounts to) is not - it leaves both untouched - so call this after one."""
        self._dense_cache = None
        self._tiled_cache = None

    def drop_dense_cache(self) -> None:
        """Release the bf16 weight the "resident" policy keeps."""
        self._dense_cache = None

    def drop_tiled_cache(self) -> None:
        """Release the operand-order copy the "tiled" decode layout keeps."""
        self._tiled_cache = None

    def extra_repr(self) -> str:
        qt = getattr(self.weight, "quant_type", None)
        return (f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, "
                f"quant_type={qt.name if qt is not None else None}, compute_dtype={self.compute_dtype}")


def _replace_with_gguf_linear(model: nn.Module, compute_dtype, state_dict: dict, prefix: str = "",
                              modules_to_not_convert=()) -> nn.Module:
    """Swap every ``nn.Linear`` whose ``<prefix>weight`` entry of ``state_dict`` is a
    :class:`GGUFParameter` for a :class:`GGUFLinear` built on the meta device."""
    for name, module in list(model.named_children()):
        module_prefix = f"{prefix}{name}."
        _replace_with_gguf_linear(module, compute_dtype, state_dict, module_prefix, modules_to_not_convert)
        if isinstance(module, nn.Linear) and not isinstance(module, GGUFLinear) and name not in modules_to_not_convert:
            if isinstance(state_dict.get(module_prefix + "weight"), GGUFParameter):
                with torch.device("meta"):
                    new = GGUFLinear(module.in_features, module.out_features, module.bias is not None,
                                     compute_dtype=compute_dtype)
                new.source_cls = type(module)
                new.requires_grad_(False)
                model._modules[name] = new
    return model
