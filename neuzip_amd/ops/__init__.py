from neuzip_amd.ops.linear import CompressedLinear

__all__ = ["CompressedLinear"]
