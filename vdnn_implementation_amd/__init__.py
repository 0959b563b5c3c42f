"""MI355X-native vDNN training engine: host-side Python binding.

The product is the native library (HIP kernels behind include/vdnn_backend.h, the C++ Layer/Network
classes behind include/vdnn_capi.h). This package loads it with ctypes and mirrors the reference's
host interface (Network, the policy and algorithm enums). There is no fallback path: if the library
has not been built, importing `vdnn_implementation_amd.backend` raises.
"""
from .enums import (ALEXNET, ALEXNET_LRN, BASELINE, OVERFEAT, VDNN_ALL, VDNN_CONV, VDNN_DYNAMIC_ALGO,  # noqa: F401
                    VDNN_MEMORY_OPT_ALGO, VDNN_NONE, VDNN_PERF_OPT_ALGO, VGG16_64, VGG16_128, VGG16_256, VGG16_512)
