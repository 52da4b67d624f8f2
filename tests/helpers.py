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


# Cameras for the GPU parity tests.  "identity" is the benchmark's (view = I, campos = 0, square
# pixels); the others exercise what the identity hides: the layout of the view matrix in the
# EWA projection and its backward, campos in the SH view direction, the scale modifier in the
# covariance and its gradient, fx != fy, and Gaussians behind a rotated camera.
CAMERAS = {
    "identity": None,
    # outside the cloud, rotated about all three axes and translated
    "rotated": dict(eye=(3.0, 1.5, -2.0), target=(0.2, -0.1, 6.0), up=(0.1, 1.0, 0.05)),
    # inside the cloud: about half of the Gaussians lie behind the camera
    "inside": dict(eye=(0.5, -0.3, 5.0), target=(-1.0, 0.5, 9.0), up=(0.0, 1.0, 0.2), scale_modifier=1.3),
    # non-square pixels (fx != fy) and a shrinking scale modifier
    "anisotropic": dict(eye=(-2.5, 2.0, -1.0), target=(0.5, 0.0, 7.0), up=(-0.2, 1.0, 0.0), tanfovx=0.62,
                        tanfovy=0.41, scale_modifier=0.7),
}


def set_camera(sc, camera):
    """Replaces the camera of a ds_splat_amd.synthetic scene (in place) by CAMERAS[camera]:
    viewmatrix / projmatrix in the API's transposed convention, campos, tan(fov), scale modifier."""
    spec = CAMERAS[camera] if isinstance(camera, str) else camera
    if spec is None:
        return sc
    tanfovx = float(spec.get("tanfovx", sc["tanfovx"]))
    tanfovy = float(spec.get("tanfovy", sc["tanfovy"]))
    V = look_at_view(spec["eye"], spec["target"], spec.get("up", (0.0, 1.0, 0.0)))
    full = perspective(tanfovx, tanfovy) @ V
    sc["tanfovx"], sc["tanfovy"] = tanfovx, tanfovy
    sc["viewmatrix"] = torch.from_numpy(V.astype(np.float32)).t().contiguous()
    sc["projmatrix"] = torch.from_numpy(full.astype(np.float32)).t().contiguous()
    sc["campos"] = torch.tensor(spec["eye"], dtype=torch.float32)
    sc["scale_modifier"] = float(spec.get("scale_modifier", 1.0))
    return sc


def comparable_gaussians(S, B, width, final_T=None, final_idx=None, slack=8):
    """Mask of the Gaussians whose gradients two correct implementations must agree on.

    Left out: a Gaussian with a borderline backward decision of its own (g_margin), and every
    Gaussian in front of a pixel whose FORWARD walk differs between the two: a decision that falls
    inside the rounding differences of exp (alpha against 1/255, T against 1e-4) may go the other
    way, the pixel then blends one entry more or less, and the terms of everything in front of it
    at that pixel shift.  With the GPU's final_T / final_idx (numpy, [H, W]) those pixels are the
    ones where the two forwards disagree (final_T beyond rtol 1e-4, or another last entry) — the
    caller asserts separately that this happens only at pixels with a small decision margin;
    without them, every pixel whose margin is below 1e-5 counts.  The Gaussians left out are the
    entries of such a pixel's tile list up to the tile's last blended entry (plus `slack`)."""
    gok = B["g_margin"] > 1e-5
    ntx = (width + 15) // 16
    if final_T is None:
        differs = S["margin"] < 1e-5
        last_idx = S["final_idx"]
    else:
        differs = (np.abs(final_T - S["final_T"]) > 1e-4 * np.abs(S["final_T"])) | (final_idx != S["final_idx"])
        last_idx = np.maximum(final_idx, S["final_idx"])
    ys, xs = np.nonzero(differs)
    tiles = np.unique((ys // 16) * ntx + (xs // 16))
    if len(tiles):
        H, W = last_idx.shape
        nty = (H + 15) // 16
        pad = np.zeros((nty * 16, ntx * 16), last_idx.dtype)
        pad[:H, :W] = last_idx
        last = pad.reshape(nty, 16, ntx, 16).max(axis=(1, 3)).reshape(-1)     # last blended entry per tile
        r = S["ranges"]
        for t in tiles.tolist():
            end = min(int(r[t + 1]), int(last[t]) + 1 + slack)
            gok[S["sorted_ids"][int(r[t]):end]] = False
    return gok


GRAD_KEYS = (("means", "v_mean3d"), ("means2d", "v_means2d"), ("shs", "v_shs"), ("opac", "v_opacity"),
             ("scales", "v_scale"), ("rots", "v_quat"))


def check_grads_against_bounds(got, B, bounds, mask, what=""):
    """got: dict key -> numpy array (keys of the oracle's backward()).  Every element of a compared
    Gaussian must lie within its own bound (Oracle.gradient_bounds: 1e-3 of the summed magnitude of
    the terms it is made of).  Returns the largest error / bound ratio seen."""
    worst = 0.0
    for key, g in got.items():
        want = B[key][mask].astype(np.float64)
        err = np.abs(g.reshape(B[key].shape)[mask].astype(np.float64) - want)
        bound = bounds[key].reshape(B[key].shape)[mask]
        ratio = err / np.maximum(bound, 1e-300)
        if ratio.size:
            i = np.unravel_index(np.argmax(ratio), ratio.shape)
            worst = max(worst, float(ratio[i]))
            assert ratio[i] <= 1.0, "%s %s: error %.3e exceeds bound %.3e (want %.6e) at %s" % (
                what, key, err[i], bound[i], want[i], i)
    return worst


def tile_rects(S, radii, width, height):
    """Tile rectangles [sx, ex) x [sy, ey) of every Gaussian from the oracle's pixel means and radii,
    in float32 as cpp/rasterizer_kernels.cu:233-250 computes them (truncation, +1 on the upper
    bound, clamped to the grid).  Checked by the caller against the oracle's own tile counts."""
    ntx, nty = (width + 15) // 16, (height + 15) // 16
    f = np.float32
    cx, cy = S["means2d"][:, 0].astype(f) / f(16), S["means2d"][:, 1].astype(f) / f(16)
    d = radii.astype(f) / f(16)
    trunc = lambda v: np.clip(np.nan_to_num(v, nan=0.0, posinf=2.0e9, neginf=-2.0e9), -2.0e9, 2.0e9).astype(np.int64)
    sx = np.clip(trunc(cx - d), 0, ntx)
    ex = np.clip(trunc((cx + d) + f(1)), 0, ntx)
    sy = np.clip(trunc(cy - d), 0, nty)
    ey = np.clip(trunc((cy + d) + f(1)), 0, nty)
    return sx, ex, sy, ey


def expected_bin_lists(S, radii, width, height, bin_side):
    """What binned tile lists must hold, from the oracle's stage-1 results: (ids, bin_ranges,
    last_tile, masks).  Slot 0 (positions [0, bin_ranges[0])) is the oracle's own list of pairs with a
    negative depth; the list of a bin holds every Gaussian of non-negative depth (the last Gaussian
    excepted: it never emits) whose tile rectangle touches the bin, once, by (depth bits, index).
    masks: per pair, which tiles of the bin the Gaussian's rectangle covers: bit x for the bin's columns,
    bit 8 + y for its rows; all sixteen bits for the pairs of slot 0."""
    n = len(radii)
    ntx, nty = (width + 15) // 16, (height + 15) // 16
    nbx, nby = (ntx + bin_side - 1) // bin_side, (nty + bin_side - 1) // bin_side
    sx, ex, sy, ey = tile_rects(S, radii, width, height)
    counts = (ex - sx) * (ey - sy) * (radii > 0)
    assert (counts == S["tiles_touched"]).all()            # the helper agrees with the oracle's rectangles
    bits = S["means2d"][:, 2].copy().view(np.uint32)
    emits = (counts > 0)
    emits[n - 1] = False
    pos = emits & ((bits >> 31) == 0)
    negatives = int(counts[emits & ~pos].sum())        # pairs of negative depth: they sort first
    order = np.lexsort((np.arange(n), bits))                # by depth bits, then index
    order = order[pos[order]]
    per_bin = [[] for _ in range(nbx * nby)]
    per_bin_masks = [[] for _ in range(nbx * nby)]
    for g in order.tolist():
        for by in range(sy[g] // bin_side, (ey[g] - 1) // bin_side + 1):
            for bx in range(sx[g] // bin_side, (ex[g] - 1) // bin_side + 1):
                per_bin[by * nbx + bx].append(g)
                xm = sum(1 << (x - bx * bin_side) for x in range(max(sx[g], bx * bin_side), min(ex[g], (bx + 1) * bin_side)))
                ym = sum(1 << (y - by * bin_side) for y in range(max(sy[g], by * bin_side), min(ey[g], (by + 1) * bin_side)))
                per_bin_masks[by * nbx + bx].append(xm | (ym << 8))
    ids = [S["sorted_ids"][:negatives].astype(np.int64)]
    masks = [np.full(negatives, 0xffff, np.int64)]
    ranges = [negatives]
    for lst, ms in zip(per_bin, per_bin_masks):
        ids.append(np.asarray(lst, np.int64))
        masks.append(np.asarray(ms, np.int64))
        ranges.append(ranges[-1] + len(lst))
    last_rows = np.where(pos, (ey - 1) * ntx + (ex - 1), -1)
    return (np.concatenate(ids), np.asarray(ranges, np.int64), int(last_rows.max()) if n else -1,
            np.concatenate(masks))
