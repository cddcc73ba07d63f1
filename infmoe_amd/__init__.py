"""MI355X (gfx950) implementation of the InfMoE MoELayerPlugin hot path.

The product is the C-ABI library infmoe_amd/lib/libinfmoe.so (include/infmoe.h); this package
is its Python binding, mirroring python/infmoe of the reference.
"""
from .config import MoELayerConfig  # noqa: F401
from .plugin import MoELayerPlugin, Plugin  # noqa: F401
