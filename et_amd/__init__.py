"""et_amd — MI355X (gfx950) implementation of the E.T. encoder hot path.

Layers, mirroring the reference tree:
  et_amd.kernels  — the launchers of kernels/kernels.h over device tensors
  et_amd.formats  — tile_mat / row_mat pruned-weight formats (host side)
  et_amd.encoder  — Linear_tile / Linear_row / Encoder_* objects
Everything computes through libet_amd.so (hand-written HIP); torch is used only
to own device memory and streams.
"""
from . import _lib  # noqa: F401
from ._lib import EtError, lib  # noqa: F401

__all__ = ["EtError", "lib", "kernels", "formats", "encoder"]
