"""zllm_amd: zllm's quantized linear-layer hot path as a HIP backend for MI355X.

The product is libzllm_hip.so (include/zllm_hip.h): a command-stream host with
hand-written gfx950 kernels. This package holds its sources (csrc/), the build
step, and a host-side twin of the reference's recorder / kernel interface used
to drive the library exactly as zllm would.
"""
from . import cmd, kernels  # noqa: F401
from .backend import Backend  # noqa: F401
from .host import Device, Host  # noqa: F401
