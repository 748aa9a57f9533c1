"""alpha2_amd: MI355X (gfx950) compute backend for alpha2's GPT training step.

    from alpha2_amd import HipBackend          # the reference's `Backend` interface over libalpha_hip.so
    from alpha2_amd import FastHipBackend      # the same interface with bf16 storage and fused epilogues behind it
"""
from .backend import HipBackend, TensorData, shapeSize, shapeStrides  # noqa: F401
from .backend_fast import FastHipBackend  # noqa: F401
from .rng import SeededRng  # noqa: F401

__all__ = ["HipBackend", "FastHipBackend", "TensorData", "SeededRng", "shapeSize", "shapeStrides"]
