from .group_quantize_decompress import *
