"""MI355X-native 3D Gaussian Splatting rasterizer with the ds_splat API."""
from .rasterizer import DsRasterizerFunction, GaussianRasterizationSettings, GaussianRasterizer

__all__ = ["GaussianRasterizationSettings", "GaussianRasterizer", "DsRasterizerFunction"]
