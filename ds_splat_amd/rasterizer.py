"""Python surface of the rasterizer: the same names, field order, argument order, returned
tensors and error behaviour as the reference's ``ds_splat/rasterizer.py`` (:7-194), on top of
the gfx950 library.

    from ds_splat import GaussianRasterizationSettings, GaussianRasterizer

``GaussianRasterizer(settings)(means_3d, means_2d, shs, colors_precomp, opacities, scales,
rotations, cov_3d_precomp)`` returns ``(image[H, W, 3], radii[N] int32)``; the image is HWC and
the background is not composited.  Backward returns gradients for the eight tensor inputs in
that order: v_means3d[N,3], v_means2d[N,3] (pixel units, third column zero), v_shs[N,B,3],
v_colors[N,3], v_opacity[N,1], v_scales[N,3], v_rotations[N,4], v_cov3d[N,6].
"""
from dataclasses import dataclass

import torch

from . import stages


def _check_input(t, name):
    # CHECK_INPUT, cpp/gsplat/bindings.h:9-16
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)


def _ok_or_empty(t):
    return t.numel() == 0 or (t.is_contiguous() and t.is_cuda)


def _validate(means_3d, means_2d, shs, colors_precomp, opacities, scales, rotations, cov3d_precomp, settings):
    """The checks of rasterizer_forward_deepsense, cpp/rasterizer_torch.cu:176-190 and :124-129."""
    _check_input(means_3d, "means_3d")
    _check_input(means_2d, "means_2d")
    _check_input(opacities, "opacities")
    if not _ok_or_empty(shs):
        raise RuntimeError("shs error")
    if not _ok_or_empty(scales):
        raise RuntimeError("scales error")
    if not _ok_or_empty(rotations):
        raise RuntimeError("rotations error")
    if not ((cov3d_precomp.numel() > 0 and cov3d_precomp.is_contiguous() and cov3d_precomp.is_cuda) or
            (cov3d_precomp.numel() == 0 and scales.numel() > 0 and scales.shape[0] == rotations.shape[0])):
        raise RuntimeError("cov3D error")
    if not ((colors_precomp.numel() > 0 and colors_precomp.is_contiguous() and colors_precomp.is_cuda) or
            (colors_precomp.numel() == 0 and shs.numel() > 0)):
        raise RuntimeError("SHS error")
    for t, name in ((means_3d, "means_3d"), (opacities, "opacities"), (shs, "shs"), (scales, "scales"),
                    (rotations, "rotations"), (cov3d_precomp, "cov3D_precomp"), (colors_precomp, "colors_precomp")):
        if t.numel() > 0 and t.dtype != torch.float32:
            raise RuntimeError("%s must be float32" % name)
    n = means_3d.numel() // 3
    if opacities.numel() != n:
        raise RuntimeError("opacities must have one entry per Gaussian")
    if shs.numel() > 0:
        coeff = (settings.sh_degree + 1) ** 2
        max_coeff = (settings.max_sh_degree + 1) ** 2
        if not (0 <= settings.sh_degree <= 3) or settings.max_sh_degree != 3:
            raise RuntimeError("sh_degree must be in [0, 3] and max_sh_degree must be 3")
        if shs.dim() != 3 or shs.shape[0] != n or shs.shape[1] < coeff or shs.shape[1] != max_coeff \
                or shs.shape[2] != 3:
            raise RuntimeError("shs must have shape [N, (max_sh_degree+1)^2, 3]")
    if scales.numel() > 0 and (scales.numel() != 3 * n or rotations.numel() != 4 * n):
        raise RuntimeError("scales must be [N,3] and rotations [N,4]")
    if cov3d_precomp.numel() > 0 and cov3d_precomp.numel() != 6 * n:
        raise RuntimeError("cov3D_precomp must be [N,6]")
    if colors_precomp.numel() > 0 and colors_precomp.numel() != 3 * n:
        raise RuntimeError("colors_precomp must be [N,3]")


def _num_bases(shs):
    # rasterizer_torch.cu:224-239 maps shs.size(-2) in {1,4,9,16} to a degree (anything else
    # to 3) and gsplat/sh.cuh:18-29 maps the degree back to the number of bases
    b = shs.shape[-2] if shs.dim() >= 2 else 0
    return b if b in (1, 4, 9, 16) else 16


class DsRasterizerFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means_3d, means_2d, shs, colors_precomp, opacities, scales, rotations, cov_3d_precomp,
                raster_settings):
        s = raster_settings
        _validate(means_3d, means_2d, shs, colors_precomp, opacities, scales, rotations, cov_3d_precomp, s)
        with torch.cuda.device(means_3d.device):
            cam = stages.CameraArgs(s.image_height, s.image_width, s.tanfovx, s.tanfovy, s.bg, s.scale_modifier,
                                    s.view_matrix, s.proj_matrix, s.sh_degree, s.max_sh_degree, s.campos)
            opt = lambda t: t if t.numel() > 0 else None
            image, st = stages.forward(cam, means_3d, opt(scales), opt(rotations), opacities, opt(shs),
                                       opt(cov_3d_precomp), opt(colors_precomp))
        ctx.cam = cam
        ctx.state = st
        ctx.num_bases = _num_bases(shs) if shs.numel() > 0 else 0
        ctx.opacity_shape = opacities.shape
        ctx.save_for_backward(means_3d, scales, rotations)
        ctx.mark_non_differentiable(st.radii)
        return image, st.radii

    @staticmethod
    def backward(ctx, rendered_img_grad, _):
        means_3d, scales, rotations = ctx.saved_tensors
        st, cam = ctx.state, ctx.cam
        opt = lambda t: t if t.numel() > 0 else None
        with torch.cuda.device(means_3d.device):
            g = stages.backward(cam, st, ctx.num_bases, means_3d, opt(scales), opt(rotations),
                                rendered_img_grad.contiguous())
        v_opacity = g["v_opacity"]
        if tuple(ctx.opacity_shape) != tuple(v_opacity.shape):
            v_opacity = v_opacity.reshape(ctx.opacity_shape)
        needs = ctx.needs_input_grad
        pick = lambda i, t: t if needs[i] else None
        return (pick(0, g["v_mean3d"]), pick(1, g["v_means2d"]), pick(2, g["v_shs"]), pick(3, g["v_colors"]),
                pick(4, v_opacity), pick(5, g["v_scale"]), pick(6, g["v_quat"]), pick(7, g["v_cov3d"]), None)


@dataclass
class GaussianRasterizationSettings:
    image_height: int
    image_width: int
    tanfovx: float
    tanfovy: float
    bg: torch.Tensor
    scale_modifier: float
    viewmatrix: torch.Tensor
    projmatrix: torch.Tensor
    sh_degree: int
    max_sh_degree: int
    campos: torch.Tensor
    prefiltered: bool
    debug: bool


class _NativeSettings:
    """Plays the role of ``ds_splat_cuda.RasterizationSettings`` (cpp/rasterizer_python.cpp:5-19):
    the thirteen fields, with the two matrices already transposed to row-major."""
    __slots__ = ("image_height", "image_width", "tanfovx", "tanfovy", "bg", "scale_modifier", "view_matrix",
                 "proj_matrix", "sh_degree", "max_sh_degree", "campos", "prefiltered", "debug")


class GaussianRasterizer(torch.nn.Module):
    def __init__(self, raster_settings: GaussianRasterizationSettings):
        super().__init__()
        self._settings = raster_settings

    @property
    def settings_for_cpp_code(self):
        s = _NativeSettings()
        s.image_height = self._settings.image_height
        s.image_width = self._settings.image_width
        s.tanfovx = self._settings.tanfovx
        s.tanfovy = self._settings.tanfovy
        s.bg = self._settings.bg
        s.scale_modifier = self._settings.scale_modifier
        s.view_matrix = self._settings.viewmatrix.t().contiguous()
        s.proj_matrix = self._settings.projmatrix.t().contiguous()
        s.sh_degree = self._settings.sh_degree
        s.max_sh_degree = self._settings.max_sh_degree
        s.campos = self._settings.campos
        s.prefiltered = self._settings.prefiltered
        s.debug = self._settings.debug
        return s

    def forward(self, means_3d, means_2d, shs, colors_precomp, opacities, scales, rotations, cov_3d_precomp):
        dev = means_3d.device
        empty = lambda: torch.empty(0, dtype=torch.float32, device=dev)
        if cov_3d_precomp is None:
            cov_3d_precomp = empty()
        if colors_precomp is None:
            colors_precomp = empty()
        if scales is None:
            scales = empty()
        if rotations is None:
            rotations = empty()
        if shs is None:
            shs = empty()
        return DsRasterizerFunction.apply(means_3d, means_2d, shs, colors_precomp, opacities, scales, rotations,
                                          cov_3d_precomp, self.settings_for_cpp_code)
