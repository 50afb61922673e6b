"""Modality-grouped launcher: text rows through the understanding weights, image rows through
the generation (``_mot_gen``) weights, in one pass over the hidden states.

The reference routes a whole forward to one tower (``Qwen3DecoderLayer.forward``,
``src/sensenova_u1/models/neo_unify/modeling_qwen3.py:983-1006``) and spells out the mixed
case only in code below a ``raise`` (``:779-783,802-806,825-829,879-883,1036-1041``):

    out = hidden.new_zeros(...); out[~ind] = proj(hidden[~ind]); out[ind] = proj_mot_gen(hidden[ind])

``grouped_linear`` computes exactly that for a pair of ``GGUFLinear`` modules.  Pairing follows
the naming rule the offloader uses (``src/sensenova_u1/utils/layer_offload.py:195-222``): the
generation twin of ``X`` is ``X_mot_gen`` in the same parent module.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from . import ops
from .quantized_linear import GGUFLinear, rms_norm

MOT_GEN_SUFFIX = "_mot_gen"


def grouped_linear(hidden_states: torch.Tensor, image_gen_indicators: Optional[torch.Tensor], proj: GGUFLinear,
                   proj_mot_gen: GGUFLinear, n_text: Optional[int] = None) -> torch.Tensor:
    """Route rows of ``hidden_states[..., K]`` to ``proj`` (indicator False) or ``proj_mot_gen``
    (indicator True) in one launch.

    ``image_gen_indicators`` is a bool tensor over the leading dims.  When the layout is known
    to be ``[text rows | image rows]`` pass ``image_gen_indicators=None`` and ``n_text`` instead:
    no row map is built and both groups stream contiguous rows.  In that form, with more than 64
    rows, ``proj.gemm_policy`` decides as it does for a single module: ``"auto"`` runs
    ``sngguf_grouped_linear_ws`` on a pooled workspace (each group on the library kernels its row count calls
    for), ``"fused"`` the fused grouped kernel, ``"two_pass"`` / ``"resident"`` a weight pass + the device
    library's GEMM per group.
    """
    for mod in (proj, proj_mot_gen):
        if type(mod).__name__ != "GGUFLinear":
            raise TypeError(f"grouped_linear needs GGUFLinear modules, got {type(mod).__name__}")
    if (proj.in_features, proj.out_features) != (proj_mot_gen.in_features, proj_mot_gen.out_features):
        raise ValueError("understanding and generation projections differ in shape")
    if image_gen_indicators is None:
        if n_text is None:
            raise ValueError("give either image_gen_indicators or n_text")
        ind, split = None, int(n_text)
        x2d = hidden_states.reshape(-1, hidden_states.shape[-1])
        if x2d.shape[0] > 64 and proj.gemm_policy != "fused" and hidden_states.dtype == torch.bfloat16:
            if not 0 <= split <= x2d.shape[0]:
                raise ValueError(f"n_text={split} is outside 0..{x2d.shape[0]}")
            out = torch.empty((x2d.shape[0], proj.out_features), dtype=torch.bfloat16, device=hidden_states.device)
            if proj.gemm_policy == "auto":
                # the library's workspace route: each group takes the kernels its own row count calls for
                x2d = proj._checked_rows(hidden_states)
                proj_mot_gen._checked_rows(hidden_states)
                ws = ops.pooled_workspace(x2d.device, max(proj._workspace_bytes(split), proj._workspace_bytes(x2d.shape[0] - split)))
                bu = proj.bias.detach().to(torch.bfloat16).contiguous() if proj.bias is not None else None
                bg = proj_mot_gen.bias.detach().to(torch.bfloat16).contiguous() if proj_mot_gen.bias is not None else None
                ops.grouped_linear_ws_into(x2d, None, split, proj.weight, int(proj.weight.quant_type), proj_mot_gen.weight,
                                           int(proj_mot_gen.weight.quant_type), bu, bg, out, None, ws, proj.numerics)
                return out.reshape(*hidden_states.shape[:-1], proj.out_features)
            for mod, lo, hi in ((proj, 0, split), (proj_mot_gen, split, x2d.shape[0])):
                if hi - lo > 64:
                    mod.two_pass_into(x2d[lo:hi], out[lo:hi])
                elif hi > lo:
                    out[lo:hi] = mod(x2d[lo:hi])
            return out.reshape(*hidden_states.shape[:-1], proj.out_features)
    else:
        if tuple(image_gen_indicators.shape) != tuple(hidden_states.shape[:-1]):
            raise ValueError("image_gen_indicators must cover the leading dims of hidden_states")
        ind, split = image_gen_indicators, 0
    return ops.grouped_linear(hidden_states, ind, split, proj.weight, int(proj.weight.quant_type),
                              proj_mot_gen.weight, int(proj_mot_gen.weight.quant_type), proj.bias, proj_mot_gen.bias,
                              proj.numerics)


def find_mot_pairs(module: nn.Module) -> dict[str, tuple[GGUFLinear, GGUFLinear]]:
    """``{qualified name of X: (X, X_mot_gen)}`` for every GGUFLinear with a generation twin."""
    pairs = {}
    for parent_name, parent in module.named_modules():
        for name, child in parent.named_children():
            twin = getattr(parent, name + MOT_GEN_SUFFIX, None)
            if isinstance(child, GGUFLinear) and isinstance(twin, GGUFLinear):
                pairs[f"{parent_name}.{name}" if parent_name else name] = (child, twin)
    return pairs


class FusedProjections(nn.Module):
    """Several ``GGUFLinear`` modules that read the same input, evaluated as one projection.

    Packed GGUF rows are independent of each other, so the weights of projections with the same
    ``in_features`` and quant type can simply be stacked row-wise: ``q_proj`` / ``k_proj`` / ``v_proj``
    (``modeling_qwen3.py:444,450,456``) become one ``[N_q + N_k + N_v, row_bytes]`` tensor and one
    launch that reads the hidden states once.  At decode every launch costs a fixed 5-8 us on top of
    its bytes, which for the 4096 -> 1024 k/v projections is more than the bytes themselves.

    ``forward`` returns one tensor per source projection (views into the fused output).  The stacked
    copy is a new device tensor; ``release_sources=True`` empties the sources' own ``weight.data``
    afterwards so the bytes are not held twice.
    """

    def __init__(self, projections, release_sources: bool = False) -> None:
        super().__init__()
        projections = list(projections)
        if not projections:
            raise ValueError("FusedProjections needs at least one projection")
        first = projections[0]
        for mod in projections:
            if type(mod).__name__ != "GGUFLinear":
                raise TypeError(f"FusedProjections needs GGUFLinear modules, got {type(mod).__name__}")
            if mod.in_features != first.in_features or int(mod.weight.quant_type) != int(first.weight.quant_type):
                raise ValueError("fused projections must share in_features and quant type")
            if (mod.bias is None) != (first.bias is None) or mod.numerics != first.numerics \
                    or mod.compute_dtype != first.compute_dtype:
                raise ValueError("fused projections must agree on bias, numerics and compute dtype")
        self.splits = [mod.out_features for mod in projections]
        fused = GGUFLinear(first.in_features, sum(self.splits), bias=first.bias is not None,
                           compute_dtype=first.compute_dtype, device="meta")
        packed = torch.cat([mod.weight.as_tensor() for mod in projections], dim=0)
        fused.weight = type(first.weight)(packed, quant_type=first.weight.quant_type)
        if first.bias is not None:
            fused.bias = nn.Parameter(torch.cat([mod.bias.detach() for mod in projections]), requires_grad=False)
        fused.numerics = first.numerics
        fused.gemm_policy = first.gemm_policy
        self.fused = fused
        if release_sources:
            for mod in projections:
                mod.weight.data = torch.empty((0, mod.weight.shape[-1]), dtype=torch.uint8, device=mod.weight.device)

    def forward(self, x: torch.Tensor, norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6):
        """With ``norm_weight`` the projections read ``RMSNorm(x)`` (``GGUFLinear.forward_normed``): for the q / k / v
        stack that is ``input_layernorm`` (``modeling_qwen3.py:919``), folded into the same launch at decode."""
        y = self.fused(x) if norm_weight is None else self.fused.forward_normed(x, norm_weight, eps)
        return torch.split(y, self.splits, dim=-1)


# Whether ``gated_mlp`` may run the whole MLP as ONE launch where the library offers it (``ops.mlp_decode_fits``: Q8_0,
# hidden 4096, intermediate 12288, one or two rows).  That launch needs every compute unit of the device at once; a
# process that runs kernels on several streams at the same time should switch it off.
ONE_LAUNCH_MLP = True


def _one_launch_mlp(x, rows, gate_proj, up_proj, down_proj, norm_weight, residual) -> bool:
    if not (ONE_LAUNCH_MLP and 0 < rows <= 2 and x.is_cuda and x.dtype == torch.bfloat16):
        return False
    mods = (gate_proj, up_proj, down_proj)
    if any(m.bias is not None or m.decode_layout != "native" or m.numerics != gate_proj.numerics or not m.weight.is_cuda
           or (m.compute_dtype or x.dtype) != torch.bfloat16 for m in mods):
        return False
    if norm_weight is not None and (norm_weight.dtype != torch.bfloat16 or norm_weight.numel() != gate_proj.in_features):
        return False
    if residual is not None and (residual.dtype != torch.bfloat16 or tuple(residual.shape) != (*x.shape[:-1], down_proj.out_features)):
        return False
    if int(gate_proj.weight.quant_type) != int(up_proj.weight.quant_type):
        return False
    if (up_proj.in_features, up_proj.out_features) != (gate_proj.in_features, gate_proj.out_features) \
            or (down_proj.in_features, down_proj.out_features) != (gate_proj.out_features, gate_proj.in_features):
        return False
    return ops.mlp_decode_fits(int(gate_proj.weight.quant_type), int(down_proj.weight.quant_type), rows, gate_proj.in_features,
                               gate_proj.out_features)


def gated_mlp(x: torch.Tensor, gate_proj: GGUFLinear, up_proj: GGUFLinear, down_proj: GGUFLinear,
              norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6,
              residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``down_proj(silu(gate_proj(x)) * up_proj(x))`` (``Qwen3MLP.forward``, modeling_qwen3.py:214-216).

    For decode (at most 16 rows, same quant type on gate and up, no bias) the gate and up
    projections and the SiLU product run as one fused GEMV launch.  With ``norm_weight`` the MLP reads
    ``RMSNorm(x)`` (``post_attention_layernorm``, modeling_qwen3.py:938); where ``ops.rmsnorm_fits`` allows, the norm
    is part of that same launch.  With ``residual`` the result is ``residual + mlp`` (modeling_qwen3.py:940-941), added
    in the down projection's epilogue.  One or two rows of the 8B model's shape in Q8_0 run as ONE launch
    (``sngguf_mlp_decode``; see ``ONE_LAUNCH_MLP``): same values as the separate launches up to the order in which the
    down projection's partial sums are added."""
    rows = x.numel() // x.shape[-1] if x.numel() else 0
    if _one_launch_mlp(x, rows, gate_proj, up_proj, down_proj, norm_weight, residual):
        x2d = gate_proj._checked_rows(x, norm_weight, residual)
        up_proj._checked_rows(x)
        # (the down projection's input never exists as a tensor here: its packed weight is checked by itself)
        ops._require_device(x, down_proj.weight)
        _, dn, dk = ops._packed_2d(down_proj.weight, down_proj._weight_type())
        if (dn, dk) != (down_proj.out_features, down_proj.in_features) or not down_proj.weight.is_contiguous():
            raise ops.SnGgufError("gated_mlp: the down projection's packed weight does not match the module")
        out = torch.empty((*x.shape[:-1], down_proj.out_features), dtype=torch.bfloat16, device=x.device)
        res2d = residual.reshape(-1, down_proj.out_features).contiguous() if residual is not None else None
        ws = ops.mlp_decode_workspace(x.device, rows, gate_proj.in_features, gate_proj.out_features)
        ops.mlp_decode_into(x2d, norm_weight.contiguous() if norm_weight is not None else None, eps, gate_proj.weight, up_proj.weight,
                            int(gate_proj.weight.quant_type), down_proj.weight, int(down_proj.weight.quant_type), res2d,
                            out.view(-1, down_proj.out_features), ws, gate_proj.numerics)
        return out
    if residual is not None:
        return down_proj.forward_residual(_gated_activations(x, rows, gate_proj, up_proj, norm_weight, eps), residual)
    return down_proj(_gated_activations(x, rows, gate_proj, up_proj, norm_weight, eps))


def _gated_activations(x, rows, gate_proj, up_proj, norm_weight, eps) -> torch.Tensor:
    """``silu(gate_proj(n)) * up_proj(n)``, n = RMSNorm(x) if ``norm_weight`` is given else x."""
    same = int(gate_proj.weight.quant_type) == int(up_proj.weight.quant_type)
    decode = 0 < rows <= 16 and same and gate_proj.bias is None and up_proj.bias is None and x.dtype == torch.bfloat16
    if norm_weight is not None:
        if (decode and x.is_cuda and norm_weight.dtype == torch.bfloat16
                and ops.rmsnorm_fits(int(gate_proj.weight.quant_type), rows, gate_proj.in_features)):
            x2d = gate_proj._checked_rows(x, norm_weight)
            up_proj._checked_rows(x)
            if (up_proj.in_features, up_proj.out_features) != (gate_proj.in_features, gate_proj.out_features) \
                    or norm_weight.numel() != gate_proj.in_features:
                raise ops.SnGgufError("gated_mlp: gate, up and the norm weight differ in shape")
            h = torch.empty((*x.shape[:-1], gate_proj.out_features), dtype=torch.bfloat16, device=x.device)
            tg, tu = gate_proj.tiled_weight(), up_proj.tiled_weight()
            if tg is not None and tu is not None:
                ops.rmsnorm_gate_up_silu_tiled_into(x2d, norm_weight.contiguous(), eps, tg, tu,
                                                    h.view(-1, gate_proj.out_features), gate_proj.numerics)
            else:
                ops.rmsnorm_gate_up_silu_into(x2d, norm_weight.contiguous(), eps, gate_proj.weight, up_proj.weight,
                                              int(gate_proj.weight.quant_type), h.view(-1, gate_proj.out_features),
                                              gate_proj.numerics)
            return h
        x = rms_norm(x, norm_weight, eps)
    tg = gate_proj.tiled_weight() if decode else None
    tu = up_proj.tiled_weight() if decode and tg is not None else None
    if tu is not None:
        x2d = gate_proj._checked_rows(x)
        up_proj._checked_rows(x)
        if up_proj.out_features != gate_proj.out_features:
            raise ops.SnGgufError("gated_mlp: gate and up differ in shape")
        h = torch.empty((*x.shape[:-1], gate_proj.out_features), dtype=torch.bfloat16, device=x.device)
        ops.gate_up_silu_tiled_into(x2d, tg, tu, h.view(-1, gate_proj.out_features), gate_proj.numerics)
    elif decode and gate_proj.in_features % 64 == 0:
        h = ops.gate_up_silu(x, gate_proj.weight, up_proj.weight, int(gate_proj.weight.quant_type), gate_proj.numerics)
    elif _gated_tile_route(x, rows, same, gate_proj, up_proj):
        # thousands of rows (the generation tower's image tokens): both weight passes into one interleaved workspace,
        # then one dense GEMM launch whose epilogue applies silu and the product
        x2d = gate_proj._checked_rows(x)
        up_proj._checked_rows(x)
        n, k = gate_proj.out_features, gate_proj.in_features
        h = torch.empty((*x.shape[:-1], n), dtype=torch.bfloat16, device=x.device)
        ws = ops.pooled_workspace(x.device, ops.gate_up_silu_workspace_bytes(n, k))
        ops.gate_up_silu_ws_into(x2d, gate_proj.weight, up_proj.weight, int(gate_proj.weight.quant_type), h.view(-1, n), ws,
                                 gate_proj.numerics)
    else:
        h = torch.nn.functional.silu(gate_proj(x)) * up_proj(x)
    return h


# The gated launch has ceil(rows / 256) x ceil(N / 128) output tiles and no K split, so it pays when those tiles come close
# to whole rounds of the chip's 256 compute units.  Measured on 12288 x 4096 (gated launch / two launches and the product,
# us): 512 rows (0.75 of a round) 183 / 199, 768 (1.125 rounds) 265 / 245, 1024 (1.5) 237 / 246, 1280 (1.875) 287 / 312,
# 1536 (2.25) 368 / 460, 2048 354 / 446, 4096 631 / 706.
GATED_TILE_MIN_ROWS = 512
GATED_TILE_MIN_FILL = 0.7


def gated_tile_fill(rows: int, n: int) -> float:
    """Share of the compute units' tile slots that the gated launch's tiles fill, over its rounds."""
    tiles = -(-rows // 256) * -(-n // 128)
    return tiles / (256 * -(-tiles // 256))


def _gated_tile_route(x, rows, same, gate_proj, up_proj) -> bool:
    """Whether ``gated_mlp`` runs gate / up / SiLU as one dense GEMM launch: enough rows and tiles to fill the chip, both
    weights of one packed type and shape, no bias, default GEMM policy."""
    if not (rows >= GATED_TILE_MIN_ROWS and same and x.is_cuda and x.dtype == torch.bfloat16):
        return False
    if gate_proj.bias is not None or up_proj.bias is not None:
        return False
    if (gate_proj.in_features, gate_proj.out_features) != (up_proj.in_features, up_proj.out_features):
        return False
    if getattr(gate_proj, "gemm_policy", "auto") != "auto" or getattr(up_proj, "gemm_policy", "auto") != "auto":
        return False
    if gate_proj.numerics != up_proj.numerics:
        return False
    if gated_tile_fill(rows, gate_proj.out_features) < GATED_TILE_MIN_FILL:
        return False
    return ops.gate_up_silu_ws_fits(int(gate_proj.weight.quant_type), rows, gate_proj.out_features, gate_proj.in_features)


def _is_silu(fn) -> bool:
    """Whether ``fn`` computes SiLU (``ACT2FN["silu"]`` is an ``nn.SiLU`` or a class of its own, depending on the
    transformers version): decided on three values, bit for bit."""
    if not callable(fn):
        return False
    probe = torch.tensor([-1.5, 0.0, 2.25], dtype=torch.float32)
    try:
        return bool(torch.equal(fn(probe), torch.nn.functional.silu(probe)))
    except Exception:
        return False


def _fused_mlp_forward(self, x):
    return gated_mlp(x, self.gate_proj, self.up_proj, self.down_proj)


def fuse_gated_mlps(model: nn.Module) -> int:
    """Point the forward of every SiLU-gated MLP of ``model`` at ``gated_mlp``; returns how many were found.

    A module qualifies when it looks like ``Qwen3MLP`` (``modeling_qwen3.py:203-216``; the generation tower's
    ``mlp_mot_gen`` is the same class): children ``gate_proj``, ``up_proj``, ``down_proj`` that are all ``GGUFLinear``,
    an ``act_fn`` that computes SiLU, and a forward of one argument.  Its forward then is
    ``down_proj(silu(gate_proj(x)) * up_proj(x))`` with the gate / up pair and the SiLU product in one launch at decode
    row counts, every rounding of the three-launch form kept, and the unchanged three module calls beyond 16 rows.  The
    original forward is kept and ``unfuse_gated_mlps`` puts it back."""
    import inspect
    import types

    n = 0
    for m in model.modules():
        if "_sn_unfused_forward" in m.__dict__:
            n += 1
            continue
        projs = [getattr(m, name, None) for name in ("gate_proj", "up_proj", "down_proj")]
        if not all(isinstance(p, GGUFLinear) for p in projs) or not _is_silu(getattr(m, "act_fn", None)):
            continue
        try:
            params = [p for p in inspect.signature(m.forward).parameters.values()
                      if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD)]
        except (TypeError, ValueError):
            continue
        if len(params) != 1:
            continue
        m.__dict__["_sn_unfused_forward"] = m.forward
        m.forward = types.MethodType(_fused_mlp_forward, m)
        n += 1
    return n


def unfuse_gated_mlps(model: nn.Module) -> int:
    """Undo ``fuse_gated_mlps``; returns how many modules got their own forward back."""
    n = 0
    for m in model.modules():
        if "_sn_unfused_forward" in m.__dict__:
            del m.__dict__["_sn_unfused_forward"]
            m.__dict__.pop("forward", None)   # the class's forward shows through again
            n += 1
    return n


class SharedInputStack:
    """Projections that the model calls one after the other on the same tensor (``q_proj``, ``k_proj``, ``v_proj``:
    ``modeling_qwen3.py:444,450,456`` and the ``_mot_gen`` triple at ``:602,608,614``), with their packed rows stored one
    after another in ONE device tensor and every module's ``weight.data`` a view of its rows.

    The modules stay separate ``GGUFLinear`` objects and the model code stays as it is.  The first member's forward runs
    one launch over all rows - packed GGUF rows are independent, so the stacked rows are a valid weight of
    ``sum(out_features)`` rows - and keeps the result; the following members, called with the same tensor (same
    storage, shape, strides and version counter), return their columns of it.  Anything else - another input, a weight
    that no longer lies where the stack put it (``.to()``, an offloader's rebinding) - falls back to the member's own
    launch.  At decode that is one launch instead of three (the 4096 -> 1024 k / v launches cost more in launch overhead
    than in bytes); over thousands of image rows one launch of 384 large tiles instead of 256 + 64 + 64 (k / v alone have
    too few tiles to fill the chip).  Every output is the same dot product of the same rounded operands as the member's
    own launch computes; beyond 64 rows the order in which the K steps' fp32 sums are added can differ (the narrow
    members' own launches split K over workgroups), i.e. the last place of a bf16 output now and then.
    Outputs of one step are ranges of one buffer: disjoint, every row contiguous, but not separately allocated - with
    several rows they are strided views (see ``member_forward``).  The pending result is recognised by the input's
    address, shape, strides and version counter: a write into the input that bypasses the version counter (through
    ``x.data`` or a raw pointer) between the members' calls is not seen."""

    MULTI_ROW = True   # serve inputs of several rows too (outputs are then column ranges of one buffer)

    def __init__(self, members) -> None:
        members = list(members)
        first = members[0]
        for mod in members:
            if not isinstance(mod, GGUFLinear):
                raise TypeError(f"SharedInputStack needs GGUFLinear modules, got {type(mod).__name__}")
            if mod.in_features != first.in_features or int(mod.weight.quant_type) != int(first.weight.quant_type):
                raise ValueError("stacked projections must share in_features and quant type")
            if mod.bias is not None or mod.numerics != first.numerics or mod.compute_dtype != first.compute_dtype:
                raise ValueError("stacked projections must have no bias and agree on numerics and compute dtype")
            if not mod.weight.is_cuda or mod.weight.device != first.weight.device:
                raise ValueError("stacked projections must live on one HIP device")
        self.members = members
        self.index = {id(mod): i for i, mod in enumerate(members)}
        self.splits = [mod.out_features for mod in members]
        self.offsets = [sum(self.splits[:i]) for i in range(len(members))]
        self.row_bytes = first.weight.as_tensor().reshape(first.out_features, -1).shape[1]
        if any((off * self.row_bytes) % 16 for off in self.offsets):
            raise ValueError("a member's rows would not start 16-byte aligned inside the stack")
        self.stacked = torch.cat([mod.weight.as_tensor().reshape(mod.out_features, -1) for mod in members], dim=0)
        for mod, off in zip(members, self.offsets):
            mod.weight.data = self.stacked[off:off + mod.out_features]
            mod.weights_changed()
            mod.__dict__["_shared_stack"] = self
        self._pending = None

    def intact(self) -> bool:
        if self.stacked is None:
            return False
        base = self.stacked.data_ptr()
        first = self.members[0]
        for mod, off in zip(self.members, self.offsets):
            w = mod.weight
            if (w.data_ptr() != base + off * self.row_bytes or w.device != self.stacked.device or mod.decode_layout != "native"
                    or mod.numerics != first.numerics or int(w.quant_type) != int(first.weight.quant_type) or mod.bias is not None):
                self.release_if_moved()
                return False
        return True

    def release_if_moved(self) -> bool:
        """Drop the stacked device tensor once no member's weight lies in it any more (an offloader has rebound every
        ``weight.data`` to its own arenas, the model went to another device): the stack would otherwise keep a second
        copy of the packed rows alive for nothing.  The members keep whatever storage they have now and are detached;
        returns whether the stack was released."""
        if self.stacked is None:
            return True
        store = self.stacked.untyped_storage().data_ptr()
        for mod in self.members:
            w = mod.weight
            if w.device == self.stacked.device and w.untyped_storage().data_ptr() == store:
                return False
        self.stacked = None
        self._pending = None
        for mod in self.members:
            if mod.__dict__.get("_shared_stack") is self:
                del mod.__dict__["_shared_stack"]
        return True

    def member_forward(self, mod: GGUFLinear, x: torch.Tensor) -> Optional[torch.Tensor]:
        """The member's output if the stack can supply it, else None (the member then runs its own launch)."""
        i = self.index[id(mod)]
        rows = x.numel() // mod.in_features if x.numel() else 0
        # several rows: the members' outputs are column ranges of one [rows, sum(out_features)] buffer - every row
        # contiguous, rows a fixed stride apart.  Splitting the last dimension into heads (`.view(*shape[:-1], -1, head_dim)`,
        # modeling_qwen3.py:444,450,456) works on such a tensor; merging dimensions would need `.reshape`.  One row gives
        # plain contiguous tensors.  MULTI_ROW switches the several-row form off.
        if not (rows >= 1 and (rows == 1 or self.MULTI_ROW) and x.is_cuda and x.dtype == torch.bfloat16):
            if i == 0:
                self._pending = None
            return None
        key = (x.data_ptr(), x._version, tuple(x.shape), tuple(x.stride()))
        if i == 0:
            self._pending = None
            if len(self.members) == 1 or not self.intact():
                return None
            first = self.members[0]
            qt = int(first.weight.quant_type)
            if rows <= 16 or (rows <= 64 and first.in_features % 256 == 0) or first.gemm_policy == "fused" or qt == ops.BF16:
                y = ops.linear(x, self.stacked, qt, None, first.numerics)
            elif first.gemm_policy == "auto" and x.is_contiguous():
                # the workspace route of a single module (quantized_linear.GGUFLinear.forward), on the stacked rows
                n, k = self.stacked.shape[0], first.in_features
                nbytes = ops.linear_workspace_bytes(n, k)
                if -(-rows // 256) * -(-n // 256) <= 128:
                    nbytes += 16 * rows * n
                x2d = first._checked_rows(x)
                y = torch.empty((*x.shape[:-1], n), dtype=torch.bfloat16, device=x.device)
                ops.linear_ws_into(x2d, self.stacked, qt, None, y.view(-1, n), ops.pooled_workspace(x.device, nbytes), first.numerics)
            else:
                return None
            # x itself is kept with the result: while it is alive no other tensor can take its address, so an equal key
            # can only come from a tensor that shares its storage, shape, strides and version - the same values
            self._pending = (key, y, x)
            return y[..., :self.splits[0]]
        pending = self._pending
        if pending is None or pending[0] != key:
            return None
        if i == len(self.members) - 1:
            self._pending = None
        return pending[1][..., self.offsets[i]:self.offsets[i] + self.splits[i]]

    def dissolve(self) -> None:
        """Give every member its own storage back (a copy of its rows) and detach it from the stack."""
        for mod, off in zip(self.members, self.offsets):
            if mod.__dict__.get("_shared_stack") is self:
                del mod.__dict__["_shared_stack"]
                mod.weight.data = mod.weight.data.clone()
                mod.weights_changed()
        self._pending = None


def stack_shared_input_projections(model: nn.Module, names=("q_proj", "k_proj", "v_proj")) -> int:
    """Build a ``SharedInputStack`` for every module of ``model`` that owns the projections ``names`` (and for their
    ``_mot_gen`` twins) as ``GGUFLinear`` modules on a HIP device with one quant type, no bias and the native decode
    layout; returns how many stacks were built.  Groups that do not qualify are left alone."""
    n = 0
    for parent in model.modules():
        for suffix in ("", MOT_GEN_SUFFIX):
            members = [getattr(parent, name + suffix, None) for name in names]
            if not all(isinstance(m, GGUFLinear) for m in members):
                continue
            if any("_shared_stack" in m.__dict__ for m in members):
                n += all(m.__dict__.get("_shared_stack") is members[0].__dict__.get("_shared_stack") for m in members)
                continue
            try:
                if any(m.decode_layout != "native" for m in members):
                    continue
                SharedInputStack(members)
            except (TypeError, ValueError):
                continue
            n += 1
    return n
