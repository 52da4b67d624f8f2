"""Adaptor with the calling convention of the original 3DGS rasterizer
(graphdeco-inria/diff-gaussian-rasterization), for trainers written against it:

    from ds_splat_amd.inria_compat import GaussianRasterizationSettings, GaussianRasterizer
    color, radii = GaussianRasterizer(settings)(means3D=..., means2D=..., opacities=..., shs=...,
                                                scales=..., rotations=...)

Differences from ``ds_splat.GaussianRasterizer`` (ds_splat/rasterizer.py:132-194 of the
reference), which this wraps:
  * keyword arguments in the original order (``opacities`` third, everything after optional);
  * the image comes back channel-first, ``[3, H, W]``, with the background composited:
    ``color = image + final_T * bg``.  The backward of the wrapped rasterizer already contains
    the gradient of exactly that term (cpp/gsplat/backward.cu:156-168 of the reference carries
    ``-T_final * ra * bg . v_out`` although its forward never adds the background), so the
    composited forward and the unchanged backward are consistent;
  * the settings tuple has no ``max_sh_degree`` (it is 3).
"""
from typing import NamedTuple

import torch

from . import _native
from .rasterizer import DsRasterizerFunction, _NativeSettings


class GaussianRasterizationSettings(NamedTuple):
    image_height: int
    image_width: int
    tanfovx: float
    tanfovy: float
    bg: torch.Tensor
    scale_modifier: float
    viewmatrix: torch.Tensor
    projmatrix: torch.Tensor
    sh_degree: int
    campos: torch.Tensor
    prefiltered: bool = False
    debug: bool = False


class _CompositedFunction(DsRasterizerFunction):
    """Same forward and backward as DsRasterizerFunction; the returned image has the background
    composited.  final_T reaches the image only through that product, whose gradient the
    backward kernel already accounts for."""

    @staticmethod
    def forward(ctx, means_3d, means_2d, shs, colors_precomp, opacities, scales, rotations, cov_3d_precomp,
                raster_settings):
        image, radii, final_T = DsRasterizerFunction.run_forward(ctx, means_3d, means_2d, shs, colors_precomp,
                                                                 opacities, scales, rotations, cov_3d_precomp,
                                                                 raster_settings)
        bg = raster_settings.bg.to(device=image.device, dtype=image.dtype).reshape(1, 1, 3)
        return image + final_T.unsqueeze(-1) * bg, radii

    @staticmethod
    def backward(ctx, rendered_img_grad, _):
        return DsRasterizerFunction.backward(ctx, rendered_img_grad, _)


class GaussianRasterizer(torch.nn.Module):
    def __init__(self, raster_settings):
        super().__init__()
        self.raster_settings = raster_settings

    def _native_settings(self):
        rs = self.raster_settings
        s = _NativeSettings()
        s.image_height, s.image_width = int(rs.image_height), int(rs.image_width)
        s.tanfovx, s.tanfovy = float(rs.tanfovx), float(rs.tanfovy)
        s.bg = rs.bg
        s.scale_modifier = float(rs.scale_modifier)
        s.view_matrix = rs.viewmatrix.t().contiguous()
        s.proj_matrix = rs.projmatrix.t().contiguous()
        s.sh_degree, s.max_sh_degree = int(rs.sh_degree), 3
        s.campos = rs.campos
        s.prefiltered, s.debug = bool(rs.prefiltered), bool(rs.debug)
        return s

    def forward(self, means3D, means2D, opacities, shs=None, colors_precomp=None, scales=None, rotations=None,
                cov3D_precomp=None):
        if (shs is None) == (colors_precomp is None):
            raise Exception("Please provide excatly one of either SHs or precomputed colors!")
        if ((scales is None or rotations is None) and cov3D_precomp is None) or \
                ((scales is not None or rotations is not None) and cov3D_precomp is not None):
            raise Exception("Please provide exactly one of either scale/rotation pair or precomputed 3D covariance!")
        _native.load_torch_ext()
        dev = means3D.device
        empty = lambda: torch.empty(0, dtype=torch.float32, device=dev)
        args = [empty() if t is None else t for t in (shs, colors_precomp, scales, rotations, cov3D_precomp)]
        shs, colors_precomp, scales, rotations, cov3D_precomp = args
        image, radii = _CompositedFunction.apply(means3D, means2D, shs, colors_precomp, opacities, scales, rotations,
                                                 cov3D_precomp, self._native_settings())
        return image.permute(2, 0, 1), radii
