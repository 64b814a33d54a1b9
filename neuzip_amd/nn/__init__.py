from neuzip_amd.nn.embedding import Embedding
from neuzip_amd.nn.linear import Linear
from neuzip_amd.nn.module import Parameter

__all__ = ["Parameter", "Linear", "Embedding"]
