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

from . import _native


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
    """Forward and backward through the C++ torch binding (csrc/torch_ext.cpp), which allocates the
    outputs and calls the C ABI of libdsx.so on the current stream."""

    @staticmethod
    def forward(ctx, means_3d, means_2d, shs, colors_precomp, opacities, scales, rotations, cov_3d_precomp,
                raster_settings):
        image, radii, _ = DsRasterizerFunction.run_forward(ctx, means_3d, means_2d, shs, colors_precomp, opacities,
                                                           scales, rotations, cov_3d_precomp, raster_settings)
        return image, radii

    @staticmethod
    def run_forward(ctx, means_3d, means_2d, shs, colors_precomp, opacities, scales, rotations, cov_3d_precomp,
                    raster_settings):
        """The forward proper; also returns final_T (for wrappers that composite a background)."""
        s = raster_settings
        _validate(means_3d, means_2d, shs, colors_precomp, opacities, scales, rotations, cov_3d_precomp, s)
        ext = _native.load_torch_ext()
        opt = lambda t: t if t.numel() > 0 else None
        stream = torch.cuda.current_stream(means_3d.device).cuda_stream
        # (the last entry: tiles per side of the bins of the tile lists; the backward is given the same)
        cam = (int(s.image_height), int(s.image_width), float(s.tanfovx), float(s.tanfovy), float(s.scale_modifier),
               int(s.sh_degree), int(s.max_sh_degree), s.view_matrix, s.proj_matrix, s.campos, s.bg,
               _native.default_list_bin())
        # a backward will follow: the forward's blend kernel, which leaves the memory system idle,
        # prepares the gradient accumulator on the side (sums zeroed, conics beside them), and the
        # first backward needs no fill and no second look at the splat records
        prepare_backward = any(ctx.needs_input_grad[:8])
        image, radii, splats, sorted_ids, ranges, final_T, final_idx, ctx.prepared_grads = ext.forward(
            *cam, means_3d, opt(scales), opt(rotations), opacities, opt(shs), opt(cov_3d_precomp), opt(colors_precomp),
            prepare_backward, stream)
        ctx.cam = cam
        ctx.num_bases = _num_bases(shs) if shs.numel() > 0 else 0
        ctx.opacity_shape = opacities.shape
        ctx.num_keys = sorted_ids.numel()
        # the reference also keeps the 3-D covariances (cpp/rasterizer_torch.cu:207); the backward here
        # rebuilds them from scales and rotations, or reads the ones that were passed in
        ctx.save_for_backward(means_3d, scales, rotations, splats, cov_3d_precomp, radii, ranges, sorted_ids, final_T,
                              final_idx)
        ctx.mark_non_differentiable(radii)
        # no zero tensors for outputs that take no gradient (autograd would fill an int32[N] of zeros
        # for radii before every backward: a kernel launch in the middle of the step)
        ctx.set_materialize_grads(False)
        return image, radii, final_T

    @staticmethod
    def backward(ctx, rendered_img_grad, _):
        if rendered_img_grad is None:   # nothing flows into the image (gradients are not materialised)
            return (None,) * 9
        means_3d, scales, rotations, splats, cov3d_precomp, radii, ranges, sorted_ids, final_T, final_idx = \
            ctx.saved_tensors
        ext = _native.load_torch_ext()
        opt = lambda t: t if t.numel() > 0 else None
        stream = torch.cuda.current_stream(means_3d.device).cuda_stream
        # the reference computes all eight gradients and autograd drops those of inputs that take
        # none (cpp/rasterizer_torch.cu:315, ds_splat/rasterizer.py:112); here the kernel is told
        # which ones are wanted and writes no others (v_colors and v_cov3d in the usual training
        # set-up with SH colours, scales and rotations: 36 of 320 bytes per Gaussian)
        needs = ctx.needs_input_grad
        wanted = sum(1 << i for i in range(8) if needs[i])
        prepared_grads, ctx.prepared_grads = ctx.prepared_grads, None   # good for one backward: it leaves sums behind
        v_mean3d, v_means2d, v_shs, v_colors, v_opacity, v_scale, v_quat, v_cov3d = ext.backward(
            *ctx.cam, ctx.num_bases, means_3d, opt(scales), opt(rotations), splats, opt(cov3d_precomp), radii, ranges,
            sorted_ids, final_T, final_idx, rendered_img_grad.contiguous(), prepared_grads, wanted, stream)
        if v_opacity is not None and tuple(ctx.opacity_shape) != tuple(v_opacity.shape):
            v_opacity = v_opacity.reshape(ctx.opacity_shape)
        return (v_mean3d, v_means2d, v_shs, v_colors, v_opacity, v_scale, v_quat, v_cov3d, None)


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
        self._native_cache = None

    @property
    def settings_for_cpp_code(self):
        # the reference transposes both matrices on every call (ds_splat/rasterizer.py:147-148);
        # the result is kept here for as long as the settings hold the same, unmodified tensors.
        # The cache entry keeps the tensors themselves (compared with `is`: an address alone could
        # be a new tensor in a freed one's place) and their version counters; tensors without one
        # (created under torch.inference_mode) are transposed on every call.
        rs = self._settings
        try:
            versions = (rs.viewmatrix._version, rs.projmatrix._version)
        except RuntimeError:
            return self._build_native_settings()
        scalars = (rs.image_height, rs.image_width, rs.tanfovx, rs.tanfovy, rs.scale_modifier, rs.sh_degree,
                   rs.max_sh_degree, rs.prefiltered, rs.debug)
        c = self._native_cache
        if (c is not None and c[0] is rs and c[1] is rs.viewmatrix and c[2] is rs.projmatrix and c[3] is rs.bg
                and c[4] is rs.campos and c[5] == versions and c[6] == scalars):
            return c[7]
        s = self._build_native_settings()
        self._native_cache = (rs, rs.viewmatrix, rs.projmatrix, rs.bg, rs.campos, versions, scalars, s)
        return s

    def _build_native_settings(self):
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
