"""deepj_amd: MI355X (gfx950) backend for DeepJ behind its TensorBackend / ComputeGraph /
GpuRuntime boundary.  The compute lives in libdeepj_hip.so (hand-written HIP kernels
reached through the C ABI in include/deepj_hip.h); this package is the host-side twin of
the reference's Java classes around that boundary."""
from . import opcodes
from ._native import HipNative, LIB_PATH
from .compute_graph import ComputeGraph, GpuBuffer
from .hip_backend import HipBackend, HipGpuRuntime
from .tensor import Tensor
from .models import (DeepSeekConfig, DeepSeekModel, GPTConfig, GPTModel, JavaRandom, LlamaConfig, LlamaModel,
                     TextGenerator)
from .persistence import ModelSerializer, parameter_names, parameter_shapes

__all__ = ["ModelSerializer", "parameter_names", "parameter_shapes", "opcodes", "HipNative", "LIB_PATH", "ComputeGraph", "GpuBuffer", "HipBackend", "HipGpuRuntime", "Tensor",
           "LlamaConfig", "LlamaModel", "GPTConfig", "GPTModel", "DeepSeekConfig", "DeepSeekModel", "TextGenerator", "JavaRandom"]
