"""mhc - MI355X-native fused mHC layer; same public names as the reference's mhc package
(src/python/mhc/__init__.py:1-15)."""
from .layer import MHCLayer
from .ops import (
    sinkhorn_knopp,
    rmsnorm,
    mhc_layer_fused,
    mhc_layer_fused_dynamic,
    mhc_layer_fused_inference,
)

__all__ = [
    "MHCLayer",
    "sinkhorn_knopp",
    "rmsnorm",
    "mhc_layer_fused",
    "mhc_layer_fused_dynamic",
    "mhc_layer_fused_inference",
]
