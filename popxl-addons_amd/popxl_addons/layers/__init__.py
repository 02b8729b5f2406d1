"""Layers.  As in the reference (popxl_addons/layers/__init__.py), `LinearGQ` is imported from its
own module: `from popxl_addons.layers.linear_gq import LinearGQ`."""
