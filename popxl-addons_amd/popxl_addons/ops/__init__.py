"""Custom ops.  As in the reference (popxl_addons/ops/__init__.py), the group-quantization ops are
imported from their own sub-package: `from popxl_addons.ops.group_quantize_decompress import ...`."""
