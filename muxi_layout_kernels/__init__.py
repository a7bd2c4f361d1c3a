"""Drop-in import path of the reference package (muxi_layout_kernels/__init__.py:1 re-exports
its extension module); here the names come from the gfx950 implementation."""
from muxi_native_layout_kernels_amd.ops import *  # noqa: F401,F403
