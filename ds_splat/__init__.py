#!/usr/bin/env python3
# Drop-in import name: ``from ds_splat import GaussianRasterizationSettings, GaussianRasterizer``
from ds_splat_amd.rasterizer import GaussianRasterizationSettings, GaussianRasterizer  # noqa: F401
