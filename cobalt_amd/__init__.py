"""cobalt_amd: the CoBALT sparse low-bit linear layer (CBK1 packed weights x fp16/bf16
activations) on MI355X, as a C-ABI HIP library behind a drop-in nn.Module."""
from . import format  # noqa: F401
from .format import PackedMatrix, pack_raw, synth_packed  # noqa: F401
from .linear import CobaltLinear, patch_model  # noqa: F401
from . import ops  # noqa: F401

__all__ = ["format", "ops", "PackedMatrix", "pack_raw", "synth_packed", "CobaltLinear", "patch_model"]
