"""Import path of the reference's fused-MoE entry (muxi_layout_kernels/muxi_moe_planC.py)."""
from muxi_native_layout_kernels_amd.moe_planC import fused_moe  # noqa: F401
