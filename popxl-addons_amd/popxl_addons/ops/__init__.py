"""Custom ops.  The reference keeps the group-quantization ops out of this namespace to avoid a
compile on import (popxl_addons/ops/__init__.py:2); nothing is compiled on import here (the HIP
library is prebuilt and loaded on first use), so the three public names are available from
`popxl_addons.ops` as well as from `popxl_addons.ops.group_quantize_decompress`."""
from .group_quantize_decompress import (  # noqa: F401
    group_quantize_compress,
    group_quantize_compress_numpy,
    group_quantize_decompress,
    group_quantize_decompress_numpy,
)
