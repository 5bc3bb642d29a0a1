"""homura_amd — MI355X-native kernels for Homura's batch-1 decode hot path.

Python here is a thin harness over the C boundary (include/homura_amd.h): device buffers,
a context, and handles onto the C++ host classes that mirror the reference's
HfModel / ExecutionPlan / KvCache. There is no CPU fallback: without the built library,
or without a GPU, the calls raise.
"""
from .runtime import (Context, DeviceBuffer, HfModel, HomuraError, TransformerConfig,  # noqa: F401
                      DTYPE_BF16, DTYPE_F32, DTYPE_Q4_0, DTYPE_Q8_0, DTYPE_Q4_K, DTYPE_Q6_K)
from . import synth  # noqa: F401

__all__ = ["Context", "DeviceBuffer", "HfModel", "HomuraError", "TransformerConfig", "synth",
           "DTYPE_F32", "DTYPE_BF16", "DTYPE_Q8_0", "DTYPE_Q4_0", "DTYPE_Q4_K", "DTYPE_Q6_K"]
