"""Deterministic synthetic scenes for tests and benchmarks.

The five named workloads are the synthetic configurations the benchmark is quoted on:
a pinhole camera at the origin looking down +z (identity view matrix, 60 degree horizontal
field of view, square pixels, znear 0.01, zfar 100), Gaussians drawn from the stated
distributions with ``torch.Generator('cpu')`` seeded with ``1234 + index``.

Everything is generated on the CPU as float32 and moved by the caller, so the GPU path and
a CPU checker can be fed bit-identical inputs.
"""
import math
from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class SceneSpec:
    name: str
    n: int
    width: int
    height: int
    sh_degree: int
    xy_half: float          # means uniform in [-xy_half, xy_half]^2
    z_range: tuple          # ... x [z0, z1]
    scale_mu: float         # per-axis scale = exp(N(mu, sigma))
    scale_sigma: float
    opacity_mu: float       # opacity = sigmoid(N(mu, opacity_sigma))
    backward: bool
    seed: int
    opacity_sigma: float = 1.0


WORKLOADS = {
    "cfg0": SceneSpec("cfg0", 16_384, 256, 256, 0, 2.0, (2.0, 10.0), -3.0, 0.5, 0.0, False, 1234),
    "cfg1": SceneSpec("cfg1", 500_000, 1920, 1080, 3, 5.0, (2.0, 20.0), -3.0, 0.5, 0.0, True, 1235),
    "cfg2": SceneSpec("cfg2", 3_000_000, 1920, 1080, 3, 5.0, (2.0, 20.0), -3.5, 0.6, 0.0, True, 1236),
    "cfg3": SceneSpec("cfg3", 6_000_000, 3840, 2160, 3, 8.0, (1.0, 30.0), -4.0, 0.5, 0.0, False, 1237),
    "cfg4": SceneSpec("cfg4", 1_000_000, 1920, 1080, 3, 3.0, (2.0, 12.0), -1.5, 0.7, -1.0, True, 1238),
    # The regime of a scene in training, which the five above do not reach (their opaque Gaussians
    # saturate a pixel after a few percent of its tile's list, and almost no Gaussian behind the first
    # layer receives a gradient): faint Gaussians, opacity about 0.02 to 0.08, so that no pixel's
    # transmittance falls to 1e-4.  Every pixel walks its whole list (about 300 blended Gaussians per
    # pixel) and every visible Gaussian receives a gradient.
    "dense": SceneSpec("dense", 2_000_000, 1920, 1080, 3, 5.0, (2.0, 20.0), -3.5, 0.6, -3.3, True, 1239, 0.4),
}


def camera(width, height, fovx_deg=60.0, znear=0.01, zfar=100.0):
    """Returns (tanfovx, tanfovy, viewmatrix, projmatrix, campos) in the convention the
    rasterizer's Python API expects: both matrices TRANSPOSED (translation in the last row),
    projmatrix = (P @ V).T."""
    tanfovx = math.tan(math.radians(fovx_deg) / 2.0)
    tanfovy = tanfovx * height / width
    V = torch.eye(4, dtype=torch.float32)
    P = torch.zeros(4, 4, dtype=torch.float32)
    P[0, 0] = 1.0 / tanfovx
    P[1, 1] = 1.0 / tanfovy
    P[2, 2] = zfar / (zfar - znear)
    P[2, 3] = -zfar * znear / (zfar - znear)
    P[3, 2] = 1.0
    full = P @ V
    return tanfovx, tanfovy, V.t().contiguous(), full.t().contiguous(), torch.zeros(3, dtype=torch.float32)


def make_scene(spec, n=None, width=None, height=None, sh_degree=None, seed=None):
    """Draws a scene.  ``n``/``width``/``height``/``sh_degree``/``seed`` override the spec
    (used by tests to shrink a workload while keeping its distributions)."""
    if isinstance(spec, str):
        spec = WORKLOADS[spec]
    n = spec.n if n is None else n
    width = spec.width if width is None else width
    height = spec.height if height is None else height
    sh_degree = spec.sh_degree if sh_degree is None else sh_degree
    g = torch.Generator(device="cpu")
    g.manual_seed(spec.seed if seed is None else seed)

    def uni(lo, hi):
        return torch.rand(n, generator=g, dtype=torch.float32) * (hi - lo) + lo

    means = torch.stack([uni(-spec.xy_half, spec.xy_half), uni(-spec.xy_half, spec.xy_half),
                         uni(spec.z_range[0], spec.z_range[1])], dim=1).contiguous()
    scales = torch.exp(torch.randn(n, 3, generator=g, dtype=torch.float32) * spec.scale_sigma + spec.scale_mu)
    quats = torch.randn(n, 4, generator=g, dtype=torch.float32)
    quats = (quats / quats.norm(dim=1, keepdim=True)).contiguous()
    opacities = torch.sigmoid(torch.randn(n, 1, generator=g, dtype=torch.float32) * spec.opacity_sigma + spec.opacity_mu)
    shs = torch.zeros(n, 16, 3, dtype=torch.float32)
    shs[:, 0, :] = torch.randn(n, 3, generator=g, dtype=torch.float32) * 0.5
    if sh_degree > 0:
        nb = (sh_degree + 1) ** 2
        shs[:, 1:nb, :] = torch.randn(n, nb - 1, 3, generator=g, dtype=torch.float32) * 0.05
    v_image = torch.randn(height, width, 3, generator=g, dtype=torch.float32)
    tanfovx, tanfovy, viewmatrix, projmatrix, campos = camera(width, height)
    return dict(
        name=spec.name, n=n, width=width, height=height, sh_degree=sh_degree,
        means_3d=means, scales=scales.contiguous(), rotations=quats, opacities=opacities.contiguous(),
        shs=shs.contiguous(), v_image=v_image, tanfovx=tanfovx, tanfovy=tanfovy,
        viewmatrix=viewmatrix, projmatrix=projmatrix, campos=campos,
        bg=torch.zeros(3, dtype=torch.float32), scale_modifier=1.0, backward=spec.backward)
