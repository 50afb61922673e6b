"""MI355X (gfx950) GGUF quantized-linear path for SenseNova-U1: drop-in ``GGUFLinear`` module and
GGUF loader over hand-written HIP kernels (libsngguf.so, C ABI in include/sngguf.h)."""
from .gguf_file import GGML_QUANT_SIZES, GGMLQuantizationType, GGUFReader, GGUFWriter, NativeGGUFReader
from .gguf_loader import count_gguf_linear, load_gguf_checkpoint, load_gguf_model, match_state_dict, set_gguf2meta_model
from .layer_offload import LayerOffloadWrapper, LayerStreamer, PackedLayerStore
from .modality import FusedProjections, SharedInputStack, find_mot_pairs, stack_shared_input_projections, fuse_gated_mlps, gated_mlp, grouped_linear, unfuse_gated_mlps
from .quantized_linear import (
    SUPPORTED_GGUF_QUANT_TYPES,
    GGUFLinear,
    GGUFParameter,
    dequantize_gguf_tensor,
    set_decode_layout,
)

__all__ = [
    "GGML_QUANT_SIZES", "GGMLQuantizationType", "GGUFReader", "GGUFWriter",
    "load_gguf_checkpoint", "load_gguf_model", "set_gguf2meta_model", "match_state_dict", "count_gguf_linear",
    "GGUFLinear", "GGUFParameter", "SUPPORTED_GGUF_QUANT_TYPES", "dequantize_gguf_tensor",
    "grouped_linear", "find_mot_pairs", "gated_mlp", "fuse_gated_mlps", "unfuse_gated_mlps", "FusedProjections", "SharedInputStack", "stack_shared_input_projections", "NativeGGUFReader",
    "LayerOffloadWrapper", "PackedLayerStore", "LayerStreamer", "set_decode_layout",
]
