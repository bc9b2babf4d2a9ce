"""lighterpp_amd -- MI355X (gfx950) implementation of the Lighter++ batch-1 decode
path.  The product is liblpp_hip.so (C ABI in include/lpp.h, sources in csrc/);
this package only binds it for the tests and the benchmark."""
from . import capi  # noqa: F401
from .model import CONFIGS, Checkpoint, Gguf, Model, Shape, Tokenizer, synth_tensor, write_checkpoint  # noqa: F401

__all__ = ["capi", "CONFIGS", "Checkpoint", "Gguf", "Model", "Shape", "Tokenizer", "synth_tensor", "write_checkpoint"]
