"""portdnn_amd: MI355X (gfx950) implementation of portDNN's convolution,
depthwise-convolution and pooling hot path.

The product is the C-ABI shared library ``libsnn_hip.so`` (declared in
``include/snn_hip.h``) and the C++ drop-in headers under ``include/portdnn``.
This Python package only loads that library for the test-suite and the
benchmark; it contains no compute of its own and no CPU fallback: if the
library has not been built, importing :mod:`portdnn_amd.capi` raises.
"""
from .capi import (  # noqa: F401
    ALGO, DIRECTION, POOL_OP, STATUS, ConvParams, DepthwiseParams,
    PoolParams, SnnHipError, lib, lib_path,
)

__version__ = "0.1.0"
