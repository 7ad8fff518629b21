from .sp_flash_decode_layer import SpGQAFlashDecodeAttention

__all__ = ["SpGQAFlashDecodeAttention"]
