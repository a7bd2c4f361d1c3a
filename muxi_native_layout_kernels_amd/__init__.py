"""MI355X (gfx950) native-layout GeMV / narrow-GeMM / fused-MoE kernels.

Python host code over a C-ABI HIP library (`libmlk.so`, declared in
`include/mlk.h`).  The operator names mirror the reference's extension module;
`import muxi_layout_kernels` gives the same names under the reference's own
import path.
"""
from .ops import *  # noqa: F401,F403
from . import ops, arg_selector  # noqa: F401

__version__ = "0.1.0"
