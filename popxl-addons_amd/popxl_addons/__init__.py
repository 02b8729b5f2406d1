"""MI355X-native group-quantization path of popxl-addons.

Only the 4-bit group-quantization decompress path is provided: the op wrappers under
`popxl_addons.ops.group_quantize_decompress` and the `LinearGQ` layer under
`popxl_addons.layers.linear_gq`, at the reference's import paths.  Importing this package loads
neither torch nor the HIP library; both are loaded on first use of a device op.
"""
__version__ = "0.1.0"
