"""MI355X (gfx950) dense-compute backend behind SpiralTorch's st-tensor / st-backend-hip operator API.

  spiraltorch_amd.hip     mirror of the `st_backend_hip` crate (host-slice GEMM family, conv2d, attention)
                          plus device-resident handles for benchmarks
  spiraltorch_amd.tensor  mirror of the `st-tensor` methods whose HIP arm this build implements
  spiraltorch_amd.inputs  deterministic synthetic input generator

The compute lives in spiraltorch_amd/libsthip.so (C ABI declared in include/st_hip.h), built from
spiraltorch_amd/csrc with hipcc for gfx950.  Importing this package does not load the library; the
first operator call does, and raises if it is missing.
"""
from . import hip, inputs, tensor  # noqa: F401
from .tensor import Conv2d, LayerNorm, Linear, PackedB, Tensor, TensorError  # noqa: F401

__all__ = ["hip", "inputs", "tensor", "Tensor", "TensorError", "Conv2d", "Linear", "LayerNorm", "PackedB"]
