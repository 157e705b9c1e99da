"""MI355X-native FP8 grouped-expert path for PithTrain.

Same Python operator surface as ``pithtrain.operators`` for the hot path (FP8 quantisation,
grouped / dense FP8 linears, token permute with dedup, SwiGLU / bias epilogues); every kernel is
hand-written HIP for gfx950 behind the C-ABI in ``include/pithtrain_hip.h``.
"""

from . import _lib  # noqa: F401

__version__ = "0.1.0"
