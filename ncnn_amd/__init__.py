"""MI355X-native int8 / block-quant hot path of ncnn: Python binding over the C ABI (include/ncnnhip.h).

The compute lives in ncnn_amd/lib/libncnnhip.so (hand-written gfx950 kernels).  There is no CPU
fallback: loading fails loudly when the library has not been built, and every call fails when no
gfx950 device is present.
"""
from .hip import (Activation, ConvDesc, DeviceBuffer, NcnnHipError, Runtime, lib, library_path)  # noqa: F401
