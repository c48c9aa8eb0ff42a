"""EXL3 (ExLlamaV3 trellis quantization) linear layers on MI355X: ``format`` (host-side facts of the format) and
``linear`` (the GPU layer)."""

from . import format  # noqa: F401
