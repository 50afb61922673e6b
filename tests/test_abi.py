"""The C-ABI library loads on a CPU-only host and exports every symbol include/sngguf.h declares.
No compute call is made here (that needs a GPU)."""
import ctypes
import os
import re

from sensenova_u1_amd import ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "sngguf.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sngguf_\w+)\s*\(", text)))


def test_header_symbols_exported():
    lib = ops.load_library()
    names = _declared_symbols()
    assert len(names) >= 9
    for name in names:
        assert hasattr(lib, name), f"libsngguf.so does not export {name}"
    assert set(names) == set(ops.EXPORTED_SYMBOLS)


def test_host_only_entry_points():
    lib = ops.load_library()
    assert lib.sngguf_version() >= 100
    assert (lib.sngguf_block_size(8), lib.sngguf_type_size(8)) == (32, 34)
    assert (lib.sngguf_block_size(12), lib.sngguf_type_size(12)) == (256, 144)
    assert (lib.sngguf_block_size(14), lib.sngguf_type_size(14)) == (256, 210)
    assert (lib.sngguf_block_size(13), lib.sngguf_type_size(13)) == (256, 176)
    assert (lib.sngguf_block_size(11), lib.sngguf_type_size(11)) == (256, 110)
    assert [lib.sngguf_type_size(t) for t in (2, 3, 6, 7, 10)] == [18, 20, 22, 24, 84]
    assert [lib.sngguf_block_size(t) for t in (2, 3, 6, 7, 10)] == [32, 32, 32, 32, 256]
    assert lib.sngguf_block_size(9) == 0 and lib.sngguf_type_size(16) == 0 and lib.sngguf_type_size(0) == 0
    assert lib.sngguf_grouped_workspace_bytes(1000) >= 4 * 1000 + 4
    assert lib.sngguf_strerror(0) == b"ok"
    for code in range(-8, 0):
        assert lib.sngguf_strerror(code) not in (b"ok", b"unknown error")


def test_argument_validation_needs_no_device():
    """Bad arguments are rejected before anything touches the GPU, so this runs on a CPU host."""
    lib = ops.load_library()
    buf = ctypes.create_string_buffer(4096 + 64)
    p = ctypes.c_void_p((ctypes.addressof(buf) + 63) // 64 * 64)
    odd = ctypes.c_void_p(p.value + 2)
    E_TYPE, E_SHAPE, E_NULL, E_ALIGN = -1, -2, -3, -4
    assert lib.sngguf_dequantize(p, 16, 1, 256, p, 0, 0, None) == E_TYPE        # IQ2_XXS not implemented
    assert lib.sngguf_dequantize(p, 8, 1, 32, p, 7, 0, None) == E_TYPE          # bad out dtype
    assert lib.sngguf_dequantize(p, 8, 1, 32, p, 0, 5, None) == E_TYPE          # bad numerics
    assert lib.sngguf_dequantize(p, 8, 1, 33, p, 0, 0, None) == E_SHAPE         # cols % 32
    assert lib.sngguf_dequantize(p, 12, 1, 128, p, 0, 0, None) == E_SHAPE       # cols % 256
    assert lib.sngguf_dequantize(p, 8, -1, 32, p, 0, 0, None) == E_SHAPE
    assert lib.sngguf_dequantize(None, 8, 1, 32, p, 0, 0, None) == E_NULL
    assert lib.sngguf_dequantize(odd, 8, 1, 32, p, 0, 0, None) == E_ALIGN
    assert lib.sngguf_dequantize(p, 8, 0, 32, None, 0, 0, None) == 0            # empty: nothing to do
    assert lib.sngguf_linear(p, 1, p, 8, 4, 48, None, p, 1, None) == E_SHAPE    # K % 32
    assert lib.sngguf_linear(p, 1, p, 14, 4, 64, None, p, 1, None) == E_SHAPE   # K % 256
    assert lib.sngguf_linear(None, 1, p, 8, 4, 64, None, p, 1, None) == E_NULL
    assert lib.sngguf_linear(p, 1, p, 8, 4, 64, None, odd, 1, None) == E_ALIGN
    assert lib.sngguf_linear(p, 0, p, 8, 4, 64, None, p, 1, None) == 0
    assert lib.sngguf_linear_residual(p, 1, p, 8, 4, 64, None, None, p, 1, None) == E_NULL   # residual is required
    assert lib.sngguf_linear_residual(p, 1, p, 8, 4, 64, None, odd, p, 1, None) == E_ALIGN
    assert lib.sngguf_linear_residual(p, 0, p, 8, 4, 64, None, None, p, 1, None) == 0
    assert lib.sngguf_linear_workspace_bytes(12288, 4096) == 2 * 12288 * 4096 and lib.sngguf_linear_workspace_bytes(0, 5) == 0
    assert lib.sngguf_linear_ws(p, 1, p, 8, 4, 48, None, p, None, 0, 1, None) == E_SHAPE      # same checks as sngguf_linear
    assert lib.sngguf_linear_ws(p, 1, p, 8, 4, 64, None, p, odd, 64, 1, None) == E_ALIGN       # workspace alignment
    assert lib.sngguf_linear_ws(p, 0, p, 8, 4, 64, None, p, None, 0, 1, None) == 0
    assert lib.sngguf_gate_up_silu(p, 17, p, p, 8, 4, 64, p, 1, None) == E_SHAPE  # decode only
    assert lib.sngguf_linear(p, 1, p, 2, 4, 48, None, p, 1, None) == E_SHAPE    # Q4_0: K % 32
    assert lib.sngguf_gate_up_silu(p, 1, p, None, 8, 4, 64, p, 1, None) == E_NULL
    assert lib.sngguf_grouped_linear(p, 4, p, 0, p, 8, p, 8, 4, 64, None, None, p, None, 1, None) == E_NULL  # no workspace
    assert lib.sngguf_grouped_linear(p, 4, None, 9, p, 8, p, 8, 4, 64, None, None, p, None, 1, None) == E_SHAPE  # n_text > M
    assert lib.sngguf_q8_0_tiled_bytes(4096, 4096) == 4096 * 4096 // 32 * 34 and lib.sngguf_q8_0_tiled_bytes(17, 256) == 32 * 8 * 34
    assert lib.sngguf_q8_0_tiled_bytes(16, 288) == 0                                          # K % 256
    assert lib.sngguf_q8_0_tile(p, 16, 288, p, None) == E_SHAPE
    assert lib.sngguf_q8_0_tile(None, 16, 256, p, None) == E_NULL
    assert lib.sngguf_linear_tiled(p, 17, p, 16, 256, None, None, p, 1, None) == E_SHAPE      # decode rows only
    assert lib.sngguf_linear_tiled(p, 1, p, 16, 256, None, None, odd, 1, None) == E_ALIGN
    assert lib.sngguf_linear_tiled(p, 1, p, 16, 256, None, None, p, 5, None) == E_TYPE
    assert lib.sngguf_gate_up_silu_tiled(p, 1, p, None, 16, 256, p, 1, None) == E_NULL
    assert lib.sngguf_linear_tiled(p, 0, p, 16, 256, None, None, p, 1, None) == 0
    # without a dense workspace the _ws form is the plain one, with the same checks
    assert lib.sngguf_grouped_linear_ws(p, 4, None, 9, p, 8, p, 8, 4, 64, None, None, p, None, None, 0, 1, None) == E_SHAPE
    assert lib.sngguf_grouped_linear_ws(p, 4, p, 0, p, 8, p, 8, 4, 64, None, None, p, None, None, 0, 1, None) == E_NULL
    assert lib.sngguf_grouped_linear_ws(p, 0, None, 0, p, 8, p, 8, 4, 64, None, None, p, None, None, 0, 1, None) == 0
    # RMSNorm fused in front of a decode projection: rows of whole 256-element runs, M (2 K + 64) <= 36 KB
    assert lib.sngguf_rmsnorm_fits(8, 1, 4096) == 1 and lib.sngguf_rmsnorm_fits(8, 4, 4096) == 1 and lib.sngguf_rmsnorm_fits(8, 5, 4096) == 0
    assert lib.sngguf_rmsnorm_fits(8, 8, 2048) == 1 and lib.sngguf_rmsnorm_fits(8, 1, 4128) == 0   # K % 256
    assert lib.sngguf_rmsnorm_fits(12, 1, 4096) == 1 and lib.sngguf_rmsnorm_fits(8, 0, 4096) == 0
    assert lib.sngguf_rmsnorm_fits(16, 1, 4096) == 0 and lib.sngguf_rmsnorm_fits(2, 1, 4128) == 0   # unknown type; Q4_0 rows of 129 blocks
    eps = ctypes.c_float(1e-6)
    assert lib.sngguf_rmsnorm_linear(p, 1, p, eps, p, 16, 16, 256, None, p, 1, None) == E_TYPE       # unknown type
    assert lib.sngguf_rmsnorm_linear(p, 1, p, eps, p, 2, 16, 288, None, p, 1, None) == E_SHAPE       # Q4_0, K % 256
    assert lib.sngguf_rmsnorm_linear(p, 5, p, eps, p, 8, 16, 4096, None, p, 1, None) == E_SHAPE      # rows do not fit
    assert lib.sngguf_rmsnorm_linear(p, 1, None, eps, p, 8, 16, 256, None, p, 1, None) == E_NULL     # gamma
    assert lib.sngguf_rmsnorm_linear(p, 1, odd, eps, p, 8, 16, 256, None, p, 1, None) == E_ALIGN
    assert lib.sngguf_rmsnorm_linear(p, 1, p, ctypes.c_float(-1.0), p, 8, 16, 256, None, p, 1, None) == E_SHAPE
    assert lib.sngguf_rmsnorm_linear(p, 1, p, ctypes.c_float(float("nan")), p, 8, 16, 256, None, p, 1, None) == E_SHAPE
    assert lib.sngguf_rmsnorm_linear(p, 0, p, eps, p, 8, 16, 256, None, p, 1, None) == 0
    assert lib.sngguf_rmsnorm_gate_up_silu(p, 1, p, eps, p, None, 8, 16, 256, p, 1, None) == E_NULL
    assert lib.sngguf_rmsnorm_gate_up_silu(p, 1, p, eps, p, p, 8, 16, 256, p, 7, None) == E_TYPE
    assert lib.sngguf_rmsnorm_linear_tiled(p, 5, p, eps, p, 16, 4096, None, p, 1, None) == E_SHAPE
    assert lib.sngguf_rmsnorm_linear_tiled(p, 1, None, eps, p, 16, 256, None, p, 1, None) == E_NULL
    assert lib.sngguf_rmsnorm_linear_tiled(p, 0, p, eps, p, 16, 256, None, p, 1, None) == 0
    assert lib.sngguf_rmsnorm_gate_up_silu_tiled(p, 1, p, eps, p, None, 16, 256, p, 1, None) == E_NULL
    assert lib.sngguf_rmsnorm_gate_up_silu_tiled(p, 1, odd, eps, p, p, 16, 256, p, 1, None) == E_ALIGN
