"""Shared helpers for the tests: oracle settings from a synthetic scene, numpy views."""
import numpy as np
import torch

from oracle.binding import make_settings


def scene_settings(sc, bg=None, sh_degree=None, scale_modifier=None):
    """Oracle settings for a scene from ds_splat_amd.synthetic.make_scene (matrices are
    transposed back to row-major math convention, as ds_splat/rasterizer.py:147-148 does)."""
    return make_settings(
        sc["height"], sc["width"], sc["tanfovx"], sc["tanfovy"],
        sc["bg"].numpy() if bg is None else bg,
        sc["scale_modifier"] if scale_modifier is None else scale_modifier,
        sc["viewmatrix"].t().contiguous().numpy(), sc["projmatrix"].t().contiguous().numpy(),
        sc["sh_degree"] if sh_degree is None else sh_degree, sc["campos"].numpy())


def arrays(sc):
    return {k: v.numpy() for k, v in sc.items() if isinstance(v, torch.Tensor)}


def look_at_view(eye, target, up=(0.0, 1.0, 0.0)):
    """Row-major world->view matrix with +z forward (float64)."""
    eye = np.asarray(eye, np.float64)
    f = np.asarray(target, np.float64) - eye
    f /= np.linalg.norm(f)
    r = np.cross(np.asarray(up, np.float64), f)
    r /= np.linalg.norm(r)
    u = np.cross(f, r)
    V = np.eye(4)
    V[0, :3], V[1, :3], V[2, :3] = r, u, f
    V[:3, 3] = -V[:3, :3] @ eye
    return V


def perspective(tanfovx, tanfovy, znear=0.01, zfar=100.0):
    P = np.zeros((4, 4))
    P[0, 0] = 1.0 / tanfovx
    P[1, 1] = 1.0 / tanfovy
    P[2, 2] = zfar / (zfar - znear)
    P[2, 3] = -zfar * znear / (zfar - znear)
    P[3, 2] = 1.0
    return P
