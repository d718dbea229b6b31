"""cosmos_amd - MI355X-native Cosmos 3 generator (DM) block forward.

Python host code (PyTorch-ROCm for device memory and streams) over hand-written HIP kernels reached
through the C ABI in include/cosmos_dm.h.
"""
from . import _lib, ops, rotary  # noqa: F401
from .config import DMConfig, CONFIGS  # noqa: F401
from .sampler import FlowEulerStepper, UniPCStepper, flow_sigmas  # noqa: F401
from .modules import (AdoptedAttention, DMAttention, DMAttnProcessor, DMBlock, DMStack, DMTransformer,  # noqa: F401
                      GraphedStack, TimestepEmbedder, Workspace, adopt_attention)
from .checkpoint import export_generator_weights, load_generator_weights  # noqa: F401

__version__ = "0.1.0"
