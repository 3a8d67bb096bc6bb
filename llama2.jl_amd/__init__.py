"""MI355X (gfx950) implementation of Llama2.jl's per-token decode path.

The package keeps the reference's surface (ModelConfig, LanguageModel, load_gguf_model,
load_karpathy_model, encode, sample, CharTokenizer) over a C-ABI HIP library, libl2hip.so.
The directory name contains a dot, so it is imported through importlib (see
__graft_entry__.load_package) under the module name `llama2_jl_amd`.
"""
from ._lib import Context, L2HError, default_context, lib  # noqa: F401
from .gguf import load_gguf_model, read_gguf, save_gguf_model, write_gguf  # noqa: F401
from .inference import (DeviceModel, LanguageModel, ModelConfig, RunState, TransformerLayerWeights,  # noqa: F401
                        TransformerWeights, generate, sample, transformer_)
from .karpathy import load_karpathy_model, save_karpathy_model  # noqa: F401
from .kquants import QuantMatrix, dequantize, matmul, quantize_q8_K, quantize_weights  # noqa: F401
from .tokenizer import BPETokenizer, CharTokenizer, encode  # noqa: F401

__all__ = ["ModelConfig", "CharTokenizer", "LanguageModel", "load_gguf_model", "load_karpathy_model", "encode",
           "sample"]  # the reference's exports minus `train` (src/Llama2.jl:12-14)
