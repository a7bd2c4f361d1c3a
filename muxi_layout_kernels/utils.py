"""Import path of the reference's torch helpers (muxi_layout_kernels/utils.py)."""
from muxi_native_layout_kernels_amd.utils import *  # noqa: F401,F403
