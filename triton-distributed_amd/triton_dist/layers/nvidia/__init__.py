"""Import-path compatibility with the reference's triton_dist.layers.nvidia (layers/nvidia/__init__.py)."""
from triton_dist.layers.amd.sp_flash_decode_layer import SpGQAFlashDecodeAttention

__all__ = ["SpGQAFlashDecodeAttention"]
