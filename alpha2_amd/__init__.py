"""alpha2_amd: MI355X (gfx950) compute backend for alpha2's GPT training step.

    from alpha2_amd import HipBackend          # the reference's `Backend` interface over libalpha_hip.so
"""
from .backend import HipBackend, TensorData, shapeSize, shapeStrides  # noqa: F401
from .rng import SeededRng  # noqa: F401

__all__ = ["HipBackend", "TensorData", "SeededRng", "shapeSize", "shapeStrides"]
