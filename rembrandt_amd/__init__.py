"""rembrandt_amd -- MI355X-native operator hot path for rembrandt, behind a C ABI.

`rembrandt_amd._lib` binds the C ABI; `rembrandt_amd.ops` wraps each entry point for torch
device tensors (torch supplies device memory and the stream only); `rembrandt_amd.synth` is the
seeded synthetic-data generator.
"""
from . import _lib  # noqa: F401

__all__ = ["_lib"]
