"""ctypes binding of libsngguf.so and its registration as torch custom ops ``sn_gguf::*``.

The library is the product: there is no CPU implementation behind these ops.  If the shared
object is missing or a tensor is not on a HIP device the call raises; nothing falls back to
eager PyTorch arithmetic.

Ops (all launch on the current torch stream of the input's device, never synchronise):

* ``sn_gguf::dequantize(packed, quant_type, out_dtype, numerics) -> Tensor``
* ``sn_gguf::linear(x, packed, quant_type, bias, numerics) -> Tensor``
* ``sn_gguf::gate_up_silu(x, gate, up, quant_type, numerics) -> Tensor``
* ``sn_gguf::grouped_linear(x, indicator, n_text, packed_und, qt_und, packed_gen, qt_gen,
  bias_und, bias_gen, numerics) -> Tensor``
"""
from __future__ import annotations

import contextlib
import ctypes
import os
from typing import Optional

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libsngguf.so")

Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 2, 3, 6, 7, 8, 10, 11, 12, 13, 14
BF16 = 30   # plain bfloat16 rows, a GGUF tensor type like the others: blocks of one element, two bytes
NUM_GGML_FP32, NUM_UPSTREAM_FP16 = 0, 1
# type -> (block elements, block bytes)
GGML_QUANT_SIZES = {Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q8_0: (32, 34),
                    Q2_K: (256, 84), Q3_K: (256, 110), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210), BF16: (1, 2)}
_OUT_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}

EXPORTED_SYMBOLS = (
    "sngguf_version", "sngguf_strerror", "sngguf_type_size", "sngguf_block_size", "sngguf_dequantize",
    "sngguf_linear", "sngguf_linear_residual", "sngguf_linear_workspace_bytes", "sngguf_linear_ws", "sngguf_linear_static_max_outputs", "sngguf_linear_static", "sngguf_gate_up_silu", "sngguf_gate_up_silu_workspace_bytes", "sngguf_gate_up_silu_ws_fits", "sngguf_gate_up_silu_ws", "sngguf_lm_head_argmax_workspace_bytes", "sngguf_lm_head_argmax", "sngguf_grouped_workspace_bytes", "sngguf_grouped_linear",
    "sngguf_grouped_linear_ws", "sngguf_q8_0_tiled_bytes", "sngguf_q8_0_tile", "sngguf_linear_tiled", "sngguf_gate_up_silu_tiled",
    "sngguf_rmsnorm_fits", "sngguf_rmsnorm", "sngguf_rmsnorm_linear", "sngguf_rmsnorm_gate_up_silu",
    "sngguf_rmsnorm_linear_tiled", "sngguf_rmsnorm_gate_up_silu_tiled",
    "sngguf_mlp_decode_workspace_bytes", "sngguf_mlp_decode_status_offset", "sngguf_mlp_decode_fits", "sngguf_mlp_decode",
    "sngguf_probe_stream_read_out_bytes", "sngguf_probe_stream_read",
    "sngguf_file_open", "sngguf_file_close", "sngguf_file_version", "sngguf_file_alignment", "sngguf_file_tensor_count",
    "sngguf_file_tensor", "sngguf_file_metadata_count", "sngguf_file_metadata", "sngguf_file_read_tensors",
)

_lib = None


class SnGgufError(RuntimeError):
    """A libsngguf entry point returned a negative status."""


def load_library() -> ctypes.CDLL:
    """Load libsngguf.so (once).  Raises if it has not been built: build it with
    ``python -m sensenova_u1_amd.build`` on a host with hipcc."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise SnGgufError(
            f"{LIB_PATH} is missing: the HIP library has not been built "
            "(run `python -m sensenova_u1_amd.build`); there is no CPU fallback for sn_gguf ops")
    lib = ctypes.CDLL(LIB_PATH)
    vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    lib.sngguf_version.argtypes = []
    lib.sngguf_version.restype = ci
    lib.sngguf_strerror.argtypes = [ci]
    lib.sngguf_strerror.restype = ctypes.c_char_p
    lib.sngguf_type_size.argtypes = [ci]
    lib.sngguf_type_size.restype = i64
    lib.sngguf_block_size.argtypes = [ci]
    lib.sngguf_block_size.restype = i64
    lib.sngguf_dequantize.argtypes = [vp, ci, i64, i64, vp, ci, ci, vp]
    lib.sngguf_dequantize.restype = ci
    lib.sngguf_linear.argtypes = [vp, i64, vp, ci, i64, i64, vp, vp, ci, vp]
    lib.sngguf_linear.restype = ci
    lib.sngguf_linear_residual.argtypes = [vp, i64, vp, ci, i64, i64, vp, vp, vp, ci, vp]
    lib.sngguf_linear_residual.restype = ci
    lib.sngguf_linear_workspace_bytes.argtypes = [i64, i64]
    lib.sngguf_linear_workspace_bytes.restype = i64
    lib.sngguf_linear_ws.argtypes = [vp, i64, vp, ci, i64, i64, vp, vp, vp, i64, ci, vp]
    lib.sngguf_linear_ws.restype = ci
    lib.sngguf_linear_static_max_outputs.argtypes = []
    lib.sngguf_linear_static_max_outputs.restype = i64
    lib.sngguf_linear_static.argtypes = [vp, i64, vp, ci, i64, i64, vp, vp, ci, vp]
    lib.sngguf_linear_static.restype = ci
    lib.sngguf_gate_up_silu.argtypes = [vp, i64, vp, vp, ci, i64, i64, vp, ci, vp]
    lib.sngguf_gate_up_silu.restype = ci
    lib.sngguf_gate_up_silu_workspace_bytes.argtypes = [i64, i64]
    lib.sngguf_gate_up_silu_workspace_bytes.restype = i64
    lib.sngguf_gate_up_silu_ws_fits.argtypes = [ci, i64, i64, i64]
    lib.sngguf_gate_up_silu_ws_fits.restype = ci
    lib.sngguf_gate_up_silu_ws.argtypes = [vp, i64, vp, vp, ci, i64, i64, vp, vp, i64, ci, vp]
    lib.sngguf_gate_up_silu_ws.restype = ci
    lib.sngguf_lm_head_argmax_workspace_bytes.argtypes = [i64, i64]
    lib.sngguf_lm_head_argmax_workspace_bytes.restype = i64
    lib.sngguf_lm_head_argmax.argtypes = [vp, i64, vp, ci, i64, i64, vp, vp, vp, ci, vp]
    lib.sngguf_lm_head_argmax.restype = ci
    lib.sngguf_grouped_workspace_bytes.argtypes = [i64]
    lib.sngguf_grouped_workspace_bytes.restype = i64
    lib.sngguf_grouped_linear.argtypes = [vp, i64, vp, i64, vp, ci, vp, ci, i64, i64, vp, vp, vp, vp, ci, vp]
    lib.sngguf_grouped_linear.restype = ci
    lib.sngguf_grouped_linear_ws.argtypes = [vp, i64, vp, i64, vp, ci, vp, ci, i64, i64, vp, vp, vp, vp, vp, i64, ci, vp]
    lib.sngguf_grouped_linear_ws.restype = ci
    lib.sngguf_q8_0_tiled_bytes.argtypes = [i64, i64]
    lib.sngguf_q8_0_tiled_bytes.restype = i64
    lib.sngguf_q8_0_tile.argtypes = [vp, i64, i64, vp, vp]
    lib.sngguf_q8_0_tile.restype = ci
    lib.sngguf_linear_tiled.argtypes = [vp, i64, vp, i64, i64, vp, vp, vp, ci, vp]
    lib.sngguf_linear_tiled.restype = ci
    lib.sngguf_gate_up_silu_tiled.argtypes = [vp, i64, vp, vp, i64, i64, vp, ci, vp]
    lib.sngguf_gate_up_silu_tiled.restype = ci
    lib.sngguf_mlp_decode_workspace_bytes.argtypes = [i64, i64, i64]
    lib.sngguf_mlp_decode_workspace_bytes.restype = i64
    lib.sngguf_mlp_decode_status_offset.argtypes = []
    lib.sngguf_mlp_decode_status_offset.restype = i64
    lib.sngguf_mlp_decode_fits.argtypes = [ci, ci, i64, i64, i64]
    lib.sngguf_mlp_decode_fits.restype = ci
    lib.sngguf_mlp_decode.argtypes = [vp, i64, vp, ctypes.c_float, vp, vp, ci, vp, ci, i64, i64, vp, vp, vp, i64, ci, ci, vp]
    lib.sngguf_mlp_decode.restype = ci
    lib.sngguf_probe_stream_read_out_bytes.argtypes = []
    lib.sngguf_probe_stream_read_out_bytes.restype = i64
    lib.sngguf_probe_stream_read.argtypes = [vp, i64, vp, ci, ci, vp]
    lib.sngguf_probe_stream_read.restype = ci
    cf = ctypes.c_float
    lib.sngguf_rmsnorm_fits.argtypes = [ci, i64, i64]
    lib.sngguf_rmsnorm_fits.restype = ci
    lib.sngguf_rmsnorm.argtypes = [vp, i64, i64, vp, cf, vp, vp]
    lib.sngguf_rmsnorm.restype = ci
    lib.sngguf_rmsnorm_linear.argtypes = [vp, i64, vp, cf, vp, ci, i64, i64, vp, vp, ci, vp]
    lib.sngguf_rmsnorm_linear.restype = ci
    lib.sngguf_rmsnorm_gate_up_silu.argtypes = [vp, i64, vp, cf, vp, vp, ci, i64, i64, vp, ci, vp]
    lib.sngguf_rmsnorm_gate_up_silu.restype = ci
    lib.sngguf_rmsnorm_linear_tiled.argtypes = [vp, i64, vp, cf, vp, i64, i64, vp, vp, ci, vp]
    lib.sngguf_rmsnorm_linear_tiled.restype = ci
    lib.sngguf_rmsnorm_gate_up_silu_tiled.argtypes = [vp, i64, vp, cf, vp, vp, i64, i64, vp, ci, vp]
    lib.sngguf_rmsnorm_gate_up_silu_tiled.restype = ci
    # host-only GGUF container reader
    cp = ctypes.c_char_p
    lib.sngguf_file_open.argtypes = [cp, ctypes.POINTER(vp), cp, i64]
    lib.sngguf_file_open.restype = ci
    lib.sngguf_file_close.argtypes = [vp]
    lib.sngguf_file_close.restype = None
    lib.sngguf_file_version.argtypes = [vp]
    lib.sngguf_file_version.restype = ci
    lib.sngguf_file_alignment.argtypes = [vp]
    lib.sngguf_file_alignment.restype = i64
    lib.sngguf_file_tensor_count.argtypes = [vp]
    lib.sngguf_file_tensor_count.restype = i64
    lib.sngguf_file_tensor.argtypes = [vp, i64, vp]
    lib.sngguf_file_tensor.restype = ci
    lib.sngguf_file_metadata_count.argtypes = [vp]
    lib.sngguf_file_metadata_count.restype = i64
    lib.sngguf_file_metadata.argtypes = [vp, i64, vp]
    lib.sngguf_file_metadata.restype = ci
    lib.sngguf_file_read_tensors.argtypes = [vp, ctypes.POINTER(i64), ctypes.POINTER(vp), i64, ci]
    lib.sngguf_file_read_tensors.restype = ci
    _lib = lib
    return lib


def _check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load_library().sngguf_strerror(rc).decode()
        raise SnGgufError(f"{what} failed: {msg} (code {rc})")


def _require_device(*tensors: Optional[torch.Tensor]) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if t.device.type != "cuda":
            raise SnGgufError(
                f"sn_gguf ops run on a HIP device only, got a tensor on '{t.device}'; "
                "there is no CPU implementation")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise SnGgufError(f"tensors on different devices: {dev} and {t.device}")
    return dev


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_NO_GUARD = contextlib.nullcontext()


def _stream(dev: torch.device) -> int:
    """The current torch stream of ``dev`` as a raw handle."""
    if _raw_stream is not None:
        return _raw_stream(dev.index if dev.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(dev).cuda_stream


def _on(dev: torch.device):
    """Context in which ``dev`` is the current device (a launch on one of its streams needs that); free of charge when
    it already is, which is every call of a one-GPU process."""
    if dev.index is None or dev.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(dev)


def _ptr(t: Optional[torch.Tensor]):
    """Device address for a ``void*`` argument (ctypes converts the integer)."""
    return None if t is None else t.data_ptr()


def _packed_2d(packed: torch.Tensor, quant_type: int):
    """View the packed weight as uint8 [N, row_bytes]; returns (tensor, N, K)."""
    if quant_type not in GGML_QUANT_SIZES:
        raise SnGgufError(f"quant type {quant_type} is not implemented (have Q4_0=2, Q4_1=3, Q5_0=6, Q5_1=7, Q8_0=8, Q2_K=10, Q3_K=11, Q4_K=12, Q5_K=13, Q6_K=14, BF16=30)")
    bs, ts = GGML_QUANT_SIZES[quant_type]
    if type(packed) is torch.Tensor and packed.dtype == torch.uint8 and packed.dim() == 2 and packed.is_contiguous() \
            and not packed.requires_grad:
        if packed.shape[1] % ts != 0:
            raise SnGgufError(f"packed row of {packed.shape[1]} bytes is not a whole number of {ts}-byte blocks")
        return packed, packed.shape[0], packed.shape[1] // ts * bs
    p = packed.detach()
    if p.dtype != torch.uint8:
        p = p.view(torch.uint8)
    if p.dim() != 2:
        p = p.reshape(-1, p.shape[-1])
    if not p.is_contiguous():
        p = p.contiguous()
    if p.shape[1] % ts != 0:
        raise SnGgufError(f"packed row of {p.shape[1]} bytes is not a whole number of {ts}-byte blocks")
    return p, p.shape[0], p.shape[1] // ts * bs


# ---- raw entry points (tensor in, tensor out; used by the custom ops and by the bench) --------------

def dequantize_into(packed: torch.Tensor, quant_type: int, out: torch.Tensor, numerics: int) -> None:
    dev = _require_device(packed, out)
    p, n, k = _packed_2d(packed, quant_type)
    if out.numel() != n * k or not out.is_contiguous() or out.dtype not in _OUT_CODE:
        raise SnGgufError("dequantize: out must be a contiguous fp32/fp16/bf16 tensor of N*K elements")
    with _on(dev):
        rc = load_library().sngguf_dequantize(_ptr(p), quant_type, n, k, _ptr(out), _OUT_CODE[out.dtype], numerics,
                                              _stream(dev))
    _check(rc, "sngguf_dequantize")


def linear_into(x2d: torch.Tensor, packed: torch.Tensor, quant_type: int, bias: Optional[torch.Tensor],
                y2d: torch.Tensor, numerics: int) -> None:
    """y2d[M, N] = x2d[M, K] @ W^T (+ bias); x2d / y2d contiguous bf16, no checks beyond the library's."""
    dev = x2d.device
    n, k = y2d.shape[1], x2d.shape[1]
    with _on(dev):
        rc = load_library().sngguf_linear(_ptr(x2d), x2d.shape[0], _ptr(packed), quant_type, n, k, _ptr(bias),
                                          _ptr(y2d), numerics, _stream(dev))
    _check(rc, "sngguf_linear")


def grouped_workspace_bytes(m: int) -> int:
    """Bytes of row-map scratch the grouped launcher needs for ``m`` rows when it is given an indicator."""
    return int(load_library().sngguf_grouped_workspace_bytes(m))


_workspaces: dict = {}


def pooled_workspace(dev: torch.device, nbytes: int) -> torch.Tensor:
    """A device scratch tensor of at least ``nbytes`` bytes for the workspace entry points, kept per (device, stream)
    and grown on demand, so that a forward pass over many modules allocates once.  Calls on one stream are ordered, and
    nothing in a workspace outlives the call that filled it.  While a HIP graph is being captured a fresh tensor is
    handed out instead (it then belongs to the graph's own memory pool)."""
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), torch.cuda.current_stream(dev).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
        _workspaces[key] = ws
    return ws


def release_workspaces() -> None:
    """Drop the pooled workspaces (they are reallocated on the next call that needs one)."""
    _workspaces.clear()
    _mlp_workspaces.clear()


_mlp_workspaces: dict = {}
_MLP_CTL_BYTES = 8192


def mlp_decode_fits(qt_gate_up: int, qt_down: int, m: int, hidden: int, inter: int) -> bool:
    """Whether ``mlp_decode_into`` runs this MLP as one launch (else it runs the separate launches, same values)."""
    return bool(load_library().sngguf_mlp_decode_fits(int(qt_gate_up), int(qt_down), m, hidden, inter))


def mlp_decode_workspace_bytes(m: int, hidden: int, inter: int) -> int:
    return int(load_library().sngguf_mlp_decode_workspace_bytes(m, hidden, inter))


def mlp_decode_workspace(dev: torch.device, m: int, hidden: int, inter: int) -> torch.Tensor:
    """The persistent workspace of ``mlp_decode_into`` for ``dev`` (one per device, grown on demand): its first 8 KB are
    zero when it is created and belong to the launches from then on.  Calls that may overlap in time on one device
    (several streams) need workspaces of their own: allocate them with ``torch.zeros``."""
    nbytes = mlp_decode_workspace_bytes(m, hidden, inter)
    if nbytes <= 0:
        raise SnGgufError(f"mlp_decode: no workspace for {m} rows, hidden {hidden}, intermediate {inter}")
    key = dev.index if dev.index is not None else torch.cuda.current_device()
    ws = _mlp_workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        # (created while a graph is being captured, the tensor lives in the graph's pool and is zeroed by every replay:
        # still a valid start state; the reference kept here keeps the pool from handing its memory out again)
        ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        _mlp_workspaces[key] = ws
    return ws


def mlp_decode_gave_up(workspace: torch.Tensor) -> bool:
    """Whether a one-launch call on this workspace ever gave up waiting for the other workgroups (its results are void
    then).  Reads device memory: synchronises."""
    off = int(load_library().sngguf_mlp_decode_status_offset())
    return bool(int(workspace[off:off + 4].view(torch.int32).item()) != 0)


def mlp_decode_into(x2d: torch.Tensor, gamma: Optional[torch.Tensor], eps: float, gate: torch.Tensor, up: torch.Tensor,
                    qt_gate_up: int, down: torch.Tensor, qt_down: int, residual: Optional[torch.Tensor], y2d: torch.Tensor,
                    workspace: torch.Tensor, numerics: int, spin_limit: int = 0) -> None:
    """y2d[M, hidden] = [residual +] down(silu(gate(n)) * up(n)), n = RMSNorm(x2d; gamma, eps) if gamma is given else
    x2d: Qwen3MLP.forward (modeling_qwen3.py:214-216) with the layer's second norm and residual add (:936-941), for up
    to 16 rows; ONE launch where ``mlp_decode_fits`` says so."""
    dev = x2d.device
    m, hidden = x2d.shape
    inter = gate.shape[0]
    with _on(dev):
        rc = load_library().sngguf_mlp_decode(_ptr(x2d), m, _ptr(gamma), float(eps), _ptr(gate), _ptr(up), int(qt_gate_up), _ptr(down),
                                              int(qt_down), hidden, inter, _ptr(residual), _ptr(y2d), _ptr(workspace),
                                              workspace.numel() * workspace.element_size(), numerics, int(spin_limit), _stream(dev))
    _check(rc, "sngguf_mlp_decode")


def linear_workspace_bytes(n: int, k: int) -> int:
    """Bytes of workspace with which ``linear_ws_into`` can take the weight-pass route (2 * n * k)."""
    return int(load_library().sngguf_linear_workspace_bytes(n, k))


def linear_ws_into(x2d: torch.Tensor, packed: torch.Tensor, quant_type: int, bias: Optional[torch.Tensor],
                   y2d: torch.Tensor, workspace: Optional[torch.Tensor], numerics: int) -> None:
    """As ``linear_into``; with a device ``workspace`` of at least ``linear_workspace_bytes(N, K)`` bytes large
    problems run as one weight pass into the workspace (bf16) and the library's dense tile GEMM."""
    dev = x2d.device
    n, k = y2d.shape[1], x2d.shape[1]
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    with _on(dev):
        rc = load_library().sngguf_linear_ws(_ptr(x2d), x2d.shape[0], _ptr(packed), quant_type, n, k, _ptr(bias),
                                             _ptr(y2d), _ptr(workspace), ws_bytes, numerics, _stream(dev))
    _check(rc, "sngguf_linear_ws")


def linear_static_max_outputs() -> int:
    """Largest ``M * N`` that ``linear_static_into`` takes."""
    return int(load_library().sngguf_linear_static_max_outputs())


def linear_static_into(x2d: torch.Tensor, packed: torch.Tensor, quant_type: int, bias: Optional[torch.Tensor],
                       y2d: torch.Tensor, numerics: int) -> None:
    """As ``linear_ws_into`` with the library's own static device area (64 MiB per GPU) as the workspace: the call
    allocates nothing.  ``M * N`` beyond ``linear_static_max_outputs()`` is refused."""
    dev = x2d.device
    n, k = y2d.shape[1], x2d.shape[1]
    with _on(dev):
        rc = load_library().sngguf_linear_static(_ptr(x2d), x2d.shape[0], _ptr(packed), quant_type, n, k, _ptr(bias),
                                                 _ptr(y2d), numerics, _stream(dev))
    _check(rc, "sngguf_linear_static")


def linear_residual_into(x2d: torch.Tensor, packed: torch.Tensor, quant_type: int, bias: Optional[torch.Tensor],
                         residual2d: torch.Tensor, y2d: torch.Tensor, numerics: int) -> None:
    """y2d[M, N] = residual2d + (x2d @ W^T + bias), rounded to bf16 after the projection and after the add."""
    dev = x2d.device
    n, k = y2d.shape[1], x2d.shape[1]
    with _on(dev):
        rc = load_library().sngguf_linear_residual(_ptr(x2d), x2d.shape[0], _ptr(packed), quant_type, n, k, _ptr(bias),
                                                   _ptr(residual2d), _ptr(y2d), numerics, _stream(dev))
    _check(rc, "sngguf_linear_residual")


def gate_up_silu_into(x2d: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, quant_type: int, h2d: torch.Tensor,
                      numerics: int) -> None:
    dev = x2d.device
    with _on(dev):
        rc = load_library().sngguf_gate_up_silu(_ptr(x2d), x2d.shape[0], _ptr(gate), _ptr(up), quant_type,
                                                h2d.shape[1], x2d.shape[1], _ptr(h2d), numerics,
                                                _stream(dev))
    _check(rc, "sngguf_gate_up_silu")


def gate_up_silu_workspace_bytes(n: int, k: int) -> int:
    """Bytes of workspace ``gate_up_silu_ws_into`` needs beyond 16 rows (512 * ceil(n / 128) * k)."""
    return int(load_library().sngguf_gate_up_silu_workspace_bytes(n, k))


def gate_up_silu_ws_fits(quant_type: int, m: int, n: int, k: int) -> bool:
    """Whether the dense tile kernel's gated epilogue takes ``m`` rows of this pair (shape rule of the library)."""
    return bool(load_library().sngguf_gate_up_silu_ws_fits(quant_type, m, n, k))


def gate_up_silu_ws_into(x2d: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, quant_type: int, h2d: torch.Tensor,
                         workspace: torch.Tensor, numerics: int) -> None:
    """h2d[M, N] = silu(x2d @ Wg^T) * (x2d @ Wu^T) beyond decode sizes: one weight pass per matrix into ``workspace``
    (at least ``gate_up_silu_workspace_bytes(N, K)`` bytes) and one launch of the dense tile kernel with the gated
    epilogue; the two projection outputs are never written."""
    dev = x2d.device
    with _on(dev):
        rc = load_library().sngguf_gate_up_silu_ws(_ptr(x2d), x2d.shape[0], _ptr(gate), _ptr(up), quant_type, h2d.shape[1],
                                                   x2d.shape[1], _ptr(h2d), _ptr(workspace),
                                                   workspace.numel() * workspace.element_size(), numerics, _stream(dev))
    _check(rc, "sngguf_gate_up_silu_ws")


def lm_head_argmax_fits(quant_type: int, m: int, k: int) -> bool:
    """Whether ``lm_head_argmax`` has a fused kernel for ``m`` rows of width ``k`` of this weight type."""
    return quant_type in GGML_QUANT_SIZES and quant_type != BF16 and 0 < m <= 16 and k % 256 == 0


def lm_head_argmax(x: torch.Tensor, packed: torch.Tensor, quant_type: int, bias: Optional[torch.Tensor] = None,
                   numerics: int = NUM_UPSTREAM_FP16) -> torch.Tensor:
    """``torch.argmax(linear(x), dim=-1)`` without materialising the logits: int64 indices over the leading dims of
    ``x``.  The greedy-token step of the reference's think loop (``modeling_neo_chat.py:557,586``).  Shapes the fused
    kernels do not take (more than 16 rows, ``K % 256 != 0``, BF16 rows) run as ``linear`` followed by ``argmax``."""
    packed, bias = _plain(packed), _plain(bias)
    _require_device(x, packed, bias)
    p, n, k = _packed_2d(packed, quant_type)
    x2d = _as_bf16_rows(x, k, "lm_head_argmax")
    m = x2d.shape[0]
    if not lm_head_argmax_fits(quant_type, m, k) or n == 0:
        if n == 0:
            raise SnGgufError("lm_head_argmax: the weight has no rows")
        return torch.ops.sn_gguf.linear(x, p, int(quant_type), bias, int(numerics)).argmax(dim=-1)
    lib = load_library()
    ws = torch.empty(int(lib.sngguf_lm_head_argmax_workspace_bytes(m, n)), dtype=torch.uint8, device=x.device)
    out = torch.empty(x.shape[:-1], dtype=torch.int64, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.sngguf_lm_head_argmax(_ptr(x2d), m, _ptr(p), int(quant_type), n, k, _ptr(_bias_bf16(bias, n, "lm_head_argmax")),
                                       _ptr(ws), _ptr(out), int(numerics), ctypes.c_void_p(_stream(x.device)))
    _check(rc, "sngguf_lm_head_argmax")
    return out


def rmsnorm_fits(quant_type: int, m: int, k: int) -> bool:
    """Whether the fused-norm entry points take ``m`` rows of width ``k`` for this weight type."""
    return bool(load_library().sngguf_rmsnorm_fits(quant_type, m, k))


def rms_norm(x: torch.Tensor, gamma: torch.Tensor, eps: float) -> torch.Tensor:
    """``Qwen3RMSNorm.forward`` (``modeling_qwen3.py:192-197``) over the last dim of a bf16 tensor as one library launch."""
    _require_device(x, gamma)
    k = x.shape[-1]
    if x.dtype != torch.bfloat16 or gamma.dtype != torch.bfloat16 or gamma.numel() != k or k % 8 != 0:
        raise SnGgufError("rms_norm: bf16 rows with a bf16 weight of the same width (a multiple of 8) are needed")
    x2d = x.reshape(-1, k)
    x2d = x2d if x2d.is_contiguous() else x2d.contiguous()
    y = torch.empty_like(x2d)
    if x2d.shape[0]:
        with torch.cuda.device(x.device):
            rc = load_library().sngguf_rmsnorm(_ptr(x2d), x2d.shape[0], k, _ptr(gamma.contiguous()), float(eps), _ptr(y),
                                               ctypes.c_void_p(_stream(x.device)))
        _check(rc, "sngguf_rmsnorm")
    return y.reshape(x.shape)


def rmsnorm_linear_into(x2d: torch.Tensor, gamma: torch.Tensor, eps: float, packed: torch.Tensor, quant_type: int,
                        bias: Optional[torch.Tensor], y2d: torch.Tensor, numerics: int) -> None:
    """y2d[M, N] = RMSNorm(x2d; gamma, eps) @ W^T (+ bias), the norm of Qwen3RMSNorm
    (modeling_qwen3.py:192-197) applied inside the projection kernel; shapes as ``rmsnorm_fits`` allows."""
    dev = x2d.device
    with _on(dev):
        rc = load_library().sngguf_rmsnorm_linear(_ptr(x2d), x2d.shape[0], _ptr(gamma), float(eps), _ptr(packed), quant_type,
                                                  y2d.shape[1], x2d.shape[1], _ptr(bias), _ptr(y2d), numerics,
                                                  _stream(dev))
    _check(rc, "sngguf_rmsnorm_linear")


def rmsnorm_gate_up_silu_into(x2d: torch.Tensor, gamma: torch.Tensor, eps: float, gate: torch.Tensor, up: torch.Tensor,
                              quant_type: int, h2d: torch.Tensor, numerics: int) -> None:
    """h2d = silu(n @ Wg^T) * (n @ Wu^T) with n = RMSNorm(x2d; gamma, eps), in one launch."""
    dev = x2d.device
    with _on(dev):
        rc = load_library().sngguf_rmsnorm_gate_up_silu(_ptr(x2d), x2d.shape[0], _ptr(gamma), float(eps), _ptr(gate), _ptr(up),
                                                        quant_type, h2d.shape[1], x2d.shape[1], _ptr(h2d), numerics,
                                                        _stream(dev))
    _check(rc, "sngguf_rmsnorm_gate_up_silu")


def rmsnorm_linear_tiled_into(x2d: torch.Tensor, gamma: torch.Tensor, eps: float, tiled: torch.Tensor,
                              bias: Optional[torch.Tensor], y2d: torch.Tensor, numerics: int) -> None:
    """``rmsnorm_linear_into`` with W given as its tiled copy."""
    dev = x2d.device
    with _on(dev):
        rc = load_library().sngguf_rmsnorm_linear_tiled(_ptr(x2d), x2d.shape[0], _ptr(gamma), float(eps), _ptr(tiled),
                                                        y2d.shape[1], x2d.shape[1], _ptr(bias), _ptr(y2d), numerics,
                                                        _stream(dev))
    _check(rc, "sngguf_rmsnorm_linear_tiled")


def rmsnorm_gate_up_silu_tiled_into(x2d: torch.Tensor, gamma: torch.Tensor, eps: float, tiled_gate: torch.Tensor,
                                    tiled_up: torch.Tensor, h2d: torch.Tensor, numerics: int) -> None:
    """``rmsnorm_gate_up_silu_into`` on two tiled matrices."""
    dev = x2d.device
    with _on(dev):
        rc = load_library().sngguf_rmsnorm_gate_up_silu_tiled(_ptr(x2d), x2d.shape[0], _ptr(gamma), float(eps), _ptr(tiled_gate),
                                                              _ptr(tiled_up), h2d.shape[1], x2d.shape[1], _ptr(h2d), numerics,
                                                              _stream(dev))
    _check(rc, "sngguf_rmsnorm_gate_up_silu_tiled")


def grouped_linear_into(x2d, indicator, n_text, packed_und, qt_und, packed_gen, qt_gen, bias_und, bias_gen, y2d,
                        workspace, numerics) -> None:
    dev = x2d.device
    with _on(dev):
        rc = load_library().sngguf_grouped_linear(
            _ptr(x2d), x2d.shape[0], _ptr(indicator), n_text, _ptr(packed_und), qt_und, _ptr(packed_gen), qt_gen,
            y2d.shape[1], x2d.shape[1], _ptr(bias_und), _ptr(bias_gen), _ptr(y2d), _ptr(workspace), numerics,
            _stream(dev))
    _check(rc, "sngguf_grouped_linear")


def grouped_linear_ws_into(x2d, indicator, n_text, packed_und, qt_und, packed_gen, qt_gen, bias_und, bias_gen, y2d,
                           workspace, dense_workspace, numerics) -> None:
    """As ``grouped_linear_into``; with a device ``dense_workspace`` of at least ``2 * linear_workspace_bytes(N, K)``
    bytes large problems decode both weight sets once and run one dense tile-GEMM launch over both row groups."""
    dev = x2d.device
    dw_bytes = dense_workspace.numel() * dense_workspace.element_size() if dense_workspace is not None else 0
    with _on(dev):
        rc = load_library().sngguf_grouped_linear_ws(
            _ptr(x2d), x2d.shape[0], _ptr(indicator), n_text, _ptr(packed_und), qt_und, _ptr(packed_gen), qt_gen,
            y2d.shape[1], x2d.shape[1], _ptr(bias_und), _ptr(bias_gen), _ptr(y2d), _ptr(workspace), _ptr(dense_workspace),
            dw_bytes, numerics, _stream(dev))
    _check(rc, "sngguf_grouped_linear_ws")


def q8_0_tile(packed: torch.Tensor) -> torch.Tensor:
    """Operand-order copy of a Q8_0 weight ``[N, K / 32 * 34]`` (device tensor, K a multiple of 256) for the tiled decode
    entry points; a flat uint8 tensor of ``sngguf_q8_0_tiled_bytes(N, K)`` bytes."""
    n, k = packed.shape[0], packed.shape[1] // 34 * 32
    nbytes = int(load_library().sngguf_q8_0_tiled_bytes(n, k))
    if nbytes == 0 and n > 0:
        raise SnGgufError(f"q8_0_tile: in_features = {k} is not a multiple of 256")
    out = torch.empty(nbytes, dtype=torch.uint8, device=packed.device)
    with torch.cuda.device(packed.device):
        rc = load_library().sngguf_q8_0_tile(_ptr(packed), n, k, _ptr(out), ctypes.c_void_p(_stream(packed.device)))
    _check(rc, "sngguf_q8_0_tile")
    return out


def linear_tiled_into(x2d: torch.Tensor, tiled: torch.Tensor, bias: Optional[torch.Tensor], residual: Optional[torch.Tensor],
                      y2d: torch.Tensor, numerics: int) -> None:
    """y2d[M, N] = x2d[M, K] @ W^T (+ bias) (+ residual) with W given as its tiled copy; M <= 16."""
    dev = x2d.device
    with _on(dev):
        rc = load_library().sngguf_linear_tiled(_ptr(x2d), x2d.shape[0], _ptr(tiled), y2d.shape[1], x2d.shape[1], _ptr(bias),
                                                _ptr(residual), _ptr(y2d), numerics, _stream(dev))
    _check(rc, "sngguf_linear_tiled")


def gate_up_silu_tiled_into(x2d: torch.Tensor, tiled_gate: torch.Tensor, tiled_up: torch.Tensor, h2d: torch.Tensor,
                            numerics: int) -> None:
    dev = x2d.device
    with _on(dev):
        rc = load_library().sngguf_gate_up_silu_tiled(_ptr(x2d), x2d.shape[0], _ptr(tiled_gate), _ptr(tiled_up), h2d.shape[1],
                                                      x2d.shape[1], _ptr(h2d), numerics, _stream(dev))
    _check(rc, "sngguf_gate_up_silu_tiled")


def _as_bf16_rows(x: torch.Tensor, k: int, what: str) -> torch.Tensor:
    if x.dtype != torch.bfloat16:
        raise SnGgufError(f"{what}: activations must be torch.bfloat16, got {x.dtype}")
    if x.shape[-1] != k:
        raise SnGgufError(f"{what}: last dim of the input is {x.shape[-1]}, the weight has in_features={k}")
    x2d = x.reshape(-1, k)
    return x2d if x2d.is_contiguous() else x2d.contiguous()


def _bf16_rows_flat(x: torch.Tensor, k: int, what: str):
    """``x`` as contiguous bf16 rows of width ``k`` without making a view: (tensor whose memory is [M, K], M)."""
    if x.dtype != torch.bfloat16:
        raise SnGgufError(f"{what}: activations must be torch.bfloat16, got {x.dtype}")
    if x.shape[-1] != k:
        raise SnGgufError(f"{what}: last dim of the input is {x.shape[-1]}, the weight has in_features={k}")
    xc = x if x.is_contiguous() else x.contiguous()
    return xc, (xc.numel() // k if k else 0)


def _bias_bf16(bias: Optional[torch.Tensor], n: int, what: str) -> Optional[torch.Tensor]:
    if bias is None:
        return None
    if bias.numel() != n:
        raise SnGgufError(f"{what}: bias has {bias.numel()} elements, expected {n}")
    b = bias.detach()
    if b.dtype != torch.bfloat16:
        b = b.to(torch.bfloat16)
    return b.contiguous()


# ---- torch custom ops ----------------------------------------------------------------------------------

_torch_lib = torch.library.Library("sn_gguf", "DEF")
_torch_lib.define("dequantize(Tensor packed, int quant_type, ScalarType out_dtype, int numerics) -> Tensor")
_torch_lib.define("linear(Tensor x, Tensor packed, int quant_type, Tensor? bias, int numerics) -> Tensor")
_torch_lib.define("linear_residual(Tensor x, Tensor packed, int quant_type, Tensor? bias, Tensor residual, int numerics) -> Tensor")
_torch_lib.define("gate_up_silu(Tensor x, Tensor gate, Tensor up, int quant_type, int numerics) -> Tensor")
_torch_lib.define(
    "grouped_linear(Tensor x, Tensor? indicator, int n_text, Tensor packed_und, int quant_type_und, "
    "Tensor packed_gen, int quant_type_gen, Tensor? bias_und, Tensor? bias_gen, int numerics) -> Tensor")


def _dequantize_hip(packed, quant_type, out_dtype, numerics):
    _require_device(packed)
    p, n, k = _packed_2d(packed, quant_type)
    out = torch.empty((*packed.shape[:-1], k), dtype=out_dtype, device=packed.device)
    dequantize_into(p, quant_type, out, numerics)
    return out


def _linear_hip(x, packed, quant_type, bias, numerics):
    dev = _require_device(x, packed, bias)
    p, n, k = _packed_2d(packed, quant_type)
    xc, m = _bf16_rows_flat(x, k, "linear")
    y = torch.empty((*x.shape[:-1], n), dtype=torch.bfloat16, device=dev)
    if m and n:
        b = _bias_bf16(bias, n, "linear")   # (held until the launch is enqueued)
        with _on(dev):
            rc = load_library().sngguf_linear(xc.data_ptr(), m, p.data_ptr(), quant_type, n, k, _ptr(b), y.data_ptr(),
                                              numerics, _stream(dev))
        _check(rc, "sngguf_linear")
    return y


def _linear_residual_hip(x, packed, quant_type, bias, residual, numerics):
    _require_device(x, packed, bias, residual)
    p, n, k = _packed_2d(packed, quant_type)
    x2d = _as_bf16_rows(x, k, "linear_residual")
    if residual.dtype != torch.bfloat16 or tuple(residual.shape) != (*x.shape[:-1], n):
        raise SnGgufError(f"linear_residual: residual must be bf16 of shape {(*x.shape[:-1], n)}")
    r2d = residual.reshape(-1, n)
    r2d = r2d if r2d.is_contiguous() else r2d.contiguous()
    y = torch.empty((*x.shape[:-1], n), dtype=torch.bfloat16, device=x.device)
    if y.numel():
        linear_residual_into(x2d, p, quant_type, _bias_bf16(bias, n, "linear_residual"), r2d, y.view(-1, n), numerics)
    return y


def _gate_up_silu_hip(x, gate, up, quant_type, numerics):
    _require_device(x, gate, up)
    pg, n, k = _packed_2d(gate, quant_type)
    pu, n2, k2 = _packed_2d(up, quant_type)
    if (n, k) != (n2, k2):
        raise SnGgufError("gate_up_silu: gate and up weights differ in shape")
    xc, m = _bf16_rows_flat(x, k, "gate_up_silu")
    h = torch.empty((*x.shape[:-1], n), dtype=torch.bfloat16, device=x.device)
    if m and n:
        dev = x.device
        with _on(dev):
            rc = load_library().sngguf_gate_up_silu(xc.data_ptr(), m, pg.data_ptr(), pu.data_ptr(), quant_type, n, k,
                                                    h.data_ptr(), numerics, _stream(dev))
        _check(rc, "sngguf_gate_up_silu")
    return h


def _grouped_linear_hip(x, indicator, n_text, packed_und, qt_und, packed_gen, qt_gen, bias_und, bias_gen, numerics):
    _require_device(x, indicator, packed_und, packed_gen, bias_und, bias_gen)
    pu, n, k = _packed_2d(packed_und, qt_und)
    pg, n2, k2 = _packed_2d(packed_gen, qt_gen)
    if (n, k) != (n2, k2):
        raise SnGgufError("grouped_linear: the two weight sets differ in shape")
    x2d = _as_bf16_rows(x, k, "grouped_linear")
    m = x2d.shape[0]
    y = torch.empty((*x.shape[:-1], n), dtype=torch.bfloat16, device=x.device)
    if not y.numel():
        return y
    ind = ws = None
    if indicator is not None:
        if indicator.numel() != m:
            raise SnGgufError(f"grouped_linear: indicator has {indicator.numel()} entries for {m} rows")
        ind = indicator.detach().reshape(-1)
        ind = (ind != 0).to(torch.uint8) if ind.dtype != torch.uint8 else ind.contiguous()
        ws = torch.empty(grouped_workspace_bytes(m), dtype=torch.uint8, device=x.device)
    grouped_linear_into(x2d, ind, n_text, pu, qt_und, pg, qt_gen, _bias_bf16(bias_und, n, "grouped_linear"),
                        _bias_bf16(bias_gen, n, "grouped_linear"), y.view(-1, n), ws, numerics)
    return y


def _no_cpu(*args, **kwargs):
    raise SnGgufError("sn_gguf ops have no CPU implementation: move the tensors to the MI355X (HIP) device")


for _name, _fn in (("dequantize", _dequantize_hip), ("linear", _linear_hip), ("linear_residual", _linear_residual_hip),
                   ("gate_up_silu", _gate_up_silu_hip),
                   ("grouped_linear", _grouped_linear_hip)):
    _torch_lib.impl(_name, _fn, "CUDA")  # torch's dispatch key for HIP devices
    _torch_lib.impl(_name, _no_cpu, "CPU")


def _packed_shape(packed, quant_type):
    bs, ts = GGML_QUANT_SIZES[quant_type]
    return packed.shape[-1] // ts * bs


def _dequantize_meta(packed, quant_type, out_dtype, numerics):
    return packed.new_empty((*packed.shape[:-1], _packed_shape(packed, quant_type)), dtype=out_dtype)


def _linear_meta(x, packed, quant_type, bias, numerics):
    return x.new_empty((*x.shape[:-1], packed.shape[0]), dtype=torch.bfloat16)


def _linear_residual_meta(x, packed, quant_type, bias, residual, numerics):
    return x.new_empty((*x.shape[:-1], packed.shape[0]), dtype=torch.bfloat16)


def _gate_up_silu_meta(x, gate, up, quant_type, numerics):
    return x.new_empty((*x.shape[:-1], gate.shape[0]), dtype=torch.bfloat16)


def _grouped_linear_meta(x, indicator, n_text, packed_und, qt_und, packed_gen, qt_gen, bias_und, bias_gen, numerics):
    return x.new_empty((*x.shape[:-1], packed_und.shape[0]), dtype=torch.bfloat16)


_torch_lib.impl("dequantize", _dequantize_meta, "Meta")
_torch_lib.impl("linear", _linear_meta, "Meta")
_torch_lib.impl("linear_residual", _linear_residual_meta, "Meta")
_torch_lib.impl("gate_up_silu", _gate_up_silu_meta, "Meta")
_torch_lib.impl("grouped_linear", _grouped_linear_meta, "Meta")


# ---- Python-facing wrappers ----------------------------------------------------------------------------------

def _plain(t):
    """Strip Parameter subclasses so the dispatcher sees an ordinary tensor."""
    if t is None:
        return None
    if type(t) is torch.Tensor:
        return t if not t.requires_grad else t.detach()
    with torch._C.DisableTorchFunctionSubclass():   # (attribute reads of a tagged Parameter cost microseconds each otherwise)
        return torch.Tensor._make_subclass(torch.Tensor, t, False)


def _eager(x: torch.Tensor) -> bool:
    """Whether a call can go straight to the HIP implementation: a real device tensor, nothing tracing or intercepting.
    (The registered ops stay the route of torch.compile / export / dispatch modes; in plain eager inference the dispatcher
    hop costs about as much host time as the launch itself.)"""
    return (type(x) is torch.Tensor and x.is_cuda and not torch.compiler.is_compiling()
            and torch._C._len_torch_dispatch_stack() == 0)


def dequantize(packed: torch.Tensor, quant_type: int, out_dtype: torch.dtype = torch.float32,
               numerics: int = NUM_GGML_FP32) -> torch.Tensor:
    return torch.ops.sn_gguf.dequantize(_plain(packed), int(quant_type), out_dtype, int(numerics))


def linear(x: torch.Tensor, packed: torch.Tensor, quant_type: int, bias: Optional[torch.Tensor] = None,
           numerics: int = NUM_UPSTREAM_FP16) -> torch.Tensor:
    if _eager(x):
        return _linear_hip(x, _plain(packed), int(quant_type), _plain(bias), int(numerics))
    return torch.ops.sn_gguf.linear(x, _plain(packed), int(quant_type), _plain(bias), int(numerics))


def linear_residual(x: torch.Tensor, packed: torch.Tensor, quant_type: int, residual: torch.Tensor,
                    bias: Optional[torch.Tensor] = None, numerics: int = NUM_UPSTREAM_FP16) -> torch.Tensor:
    """``residual + linear(x)`` in one launch (bf16 rounding after the projection and after the add)."""
    if _eager(x):
        return _linear_residual_hip(x, _plain(packed), int(quant_type), _plain(bias), residual, int(numerics))
    return torch.ops.sn_gguf.linear_residual(x, _plain(packed), int(quant_type), _plain(bias), residual, int(numerics))


def gate_up_silu(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, quant_type: int,
                 numerics: int = NUM_UPSTREAM_FP16) -> torch.Tensor:
    if _eager(x):
        return _gate_up_silu_hip(x, _plain(gate), _plain(up), int(quant_type), int(numerics))
    return torch.ops.sn_gguf.gate_up_silu(x, _plain(gate), _plain(up), int(quant_type), int(numerics))


def grouped_linear(x: torch.Tensor, indicator: Optional[torch.Tensor], n_text: int, packed_und: torch.Tensor,
                   quant_type_und: int, packed_gen: torch.Tensor, quant_type_gen: int,
                   bias_und: Optional[torch.Tensor] = None, bias_gen: Optional[torch.Tensor] = None,
                   numerics: int = NUM_UPSTREAM_FP16) -> torch.Tensor:
    return torch.ops.sn_gguf.grouped_linear(x, _plain(indicator), int(n_text), _plain(packed_und), int(quant_type_und),
                                            _plain(packed_gen), int(quant_type_gen), _plain(bias_und),
                                            _plain(bias_gen), int(numerics))
