"""Pins the oracle's forward stages with facts that do not come from the oracle's own
formulas: closed forms in float64 linear algebra, library routines (eigvalsh, inv,
scipy spherical harmonics, stable argsort, cumsum), invariants, hand cases on the decision
boundaries and a brute-force renderer that knows nothing about tiles."""
import math

import numpy as np
import pytest
from scipy.special import sph_harm_y

from ds_splat_amd.synthetic import make_scene
from helpers import arrays, look_at_view, perspective, scene_settings
from oracle.binding import make_settings

RNG = np.random.default_rng(7)


def quat_R(q):
    w, x, y, z = q / np.linalg.norm(q)
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                     [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                     [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])


def sym6(c):
    return np.array([[c[0], c[1], c[2]], [c[1], c[3], c[4]], [c[2], c[4], c[5]]], np.float64)


def general_camera(W=200, H=120, tanfovx=0.7):
    tanfovy = tanfovx * H / W
    V = look_at_view([0.3, -0.2, -1.0], [0.1, 0.2, 4.0], up=(0.1, 1.0, 0.05))
    P = perspective(tanfovx, tanfovy) @ V
    return W, H, tanfovx, tanfovy, V, P


def project(oracle, n=400, mod=1.3, cam=None, sh_degree=3, means=None, scales=None, quats=None, shs=None):
    W, H, tfx, tfy, V, P = cam or general_camera()
    campos = -V[:3, :3].T @ V[:3, 3]
    s = make_settings(H, W, tfx, tfy, [0, 0, 0], mod, V, P, sh_degree, campos)
    if means is None:
        means = np.stack([RNG.uniform(-3, 3, n), RNG.uniform(-2, 2, n), RNG.uniform(-2, 9, n)], 1)
    n = len(means)
    scales = np.exp(RNG.normal(-2.0, 0.7, (n, 3))) if scales is None else scales
    quats = RNG.normal(size=(n, 4)) * RNG.uniform(0.3, 3.0, (n, 1)) if quats is None else quats
    shs = RNG.normal(0, 0.3, (n, 16, 3)) if shs is None else shs
    out = oracle.project_fwd(s, means, scales, quats, shs)
    f32 = lambda a: np.asarray(a, np.float32).astype(np.float64)
    return s, dict(means=f32(means), scales=f32(scales), quats=f32(quats), shs=f32(shs), V=f32(V), P=f32(P),
                   campos=f32(campos), W=W, H=H, tfx=float(np.float32(tfx)), tfy=float(np.float32(tfy)),
                   mod=float(np.float32(mod))), out


# ------------------------------------------------------------------------- cov3d
def test_cov3d_closed_form_and_invariants(oracle):
    _, I, o = project(oracle)
    for i in range(len(I["means"])):
        R = quat_R(I["quats"][i])
        S = np.diag(I["scales"][i] * I["mod"])
        ref = R @ S @ S @ R.T
        got = sym6(o["cov3d"][i])
        np.testing.assert_allclose(got, ref, rtol=2e-5, atol=2e-6 * np.abs(ref).max())
        assert math.isclose(np.trace(got), np.sum((I["scales"][i] * I["mod"]) ** 2), rel_tol=1e-5)
        assert math.isclose(np.linalg.det(got), np.prod((I["scales"][i] * I["mod"]) ** 2), rel_tol=2e-3)


def test_cov3d_identity_quaternion(oracle):
    n = 5
    sc = np.exp(RNG.normal(-1, 0.5, (n, 3)))
    q = np.tile([2.5, 0, 0, 0], (n, 1))      # un-normalised identity rotation
    _, I, o = project(oracle, n=n, mod=2.0, scales=sc, quats=q,
                      means=np.tile([0, 0, 4.0], (n, 1)))
    for i in range(n):
        d = (I["scales"][i] * 2.0) ** 2
        np.testing.assert_allclose(o["cov3d"][i], [d[0], 0, 0, d[1], 0, d[2]], rtol=1e-6, atol=0)


# ------------------------------------------------------------------------- cov2d / conic / radius
def ewa_cov2d(I, i):
    """J W Sigma W^T J^T + 0.3 I with the 1.3*tanfov clamp on t (textbook EWA, float64)."""
    fx, fy = I["W"] / (2 * I["tfx"]), I["H"] / (2 * I["tfy"])
    t = I["V"][:3, :3] @ I["means"][i] + I["V"][:3, 3]
    lx, ly = 1.3 * I["tfx"], 1.3 * I["tfy"]
    tx = min(lx, max(-lx, t[0] / t[2])) * t[2]
    ty = min(ly, max(-ly, t[1] / t[2])) * t[2]
    J = np.array([[fx / t[2], 0, -fx * tx / t[2] ** 2], [0, fy / t[2], -fy * ty / t[2] ** 2]])
    R = quat_R(I["quats"][i])
    S = np.diag(I["scales"][i] * I["mod"])
    Sigma = R @ S @ S @ R.T
    A = J @ I["V"][:3, :3]
    return A @ Sigma @ A.T + 0.3 * np.eye(2), t


def test_conic_radius_pixel_mean_vs_float64(oracle):
    s, I, o = project(oracle, n=600)
    fx, fy = I["W"] / (2 * I["tfx"]), I["H"] / (2 * I["tfy"])
    checked = 0
    for i in range(len(I["means"])):
        cov, t = ewa_cov2d(I, i)
        if t[2] < 0.2:
            continue
        checked += 1
        det = np.linalg.det(cov)
        # conic = inverse of cov2d (the +1e-6 on det is far below float32 resolution here)
        inv = np.linalg.inv(cov)
        np.testing.assert_allclose([o["conic"][i][0], o["conic"][i][1], o["conic"][i][2]],
                                   [inv[0, 0], inv[0, 1], inv[1, 1]], rtol=3e-3, atol=1e-6 / max(det, 1e-6))
        # pixel mean: textbook pinhole
        np.testing.assert_allclose(o["means2d"][i], [fx * t[0] / t[2] + I["W"] / 2, fy * t[1] / t[2] + I["H"] / 2,
                                                     t[2]], rtol=1e-4, atol=1e-3)
        # radius: 3 sigma of the larger eigenvalue (library eigenvalues), when not culled
        if o["radii"][i] > 0:
            lam = np.linalg.eigvalsh(cov)[-1]
            mid, d = 0.5 * np.trace(cov), np.linalg.det(cov)
            if mid * mid - d >= 0.1:
                want = 3 * math.sqrt(lam)
            else:
                want = 3 * math.sqrt(mid + math.sqrt(0.1))     # the floor case, by hand
            assert abs(o["radii"][i] - math.ceil(want)) <= (1 if abs(want - round(want)) < 1e-3 else 0)
    assert checked > 300


def test_cov2d_special_case_on_axis_isotropic(oracle):
    """Identity view, Gaussian on the optical axis, isotropic scale s at depth z:
    cov2d = ((f s / z)^2 + 0.3) I, so conic = I / that and radius = ceil(3 sqrt(.))."""
    W, H, tfx = 640, 480, 0.5
    tfy = tfx * H / W
    V = np.eye(4)
    cam = (W, H, tfx, tfy, V, perspective(tfx, tfy) @ V)
    z = np.array([2.0, 5.0, 9.0])
    sc = np.array([0.05, 0.2, 0.01])
    _, I, o = project(oracle, mod=1.0, cam=cam, means=np.stack([0 * z, 0 * z, z], 1),
                      scales=np.repeat(sc[:, None], 3, 1), quats=RNG.normal(size=(3, 4)))
    f = W / (2 * tfx)
    for i in range(3):
        v = (f * sc[i] / z[i]) ** 2 + 0.3
        np.testing.assert_allclose(o["conic"][i], [1 / v, 0, 1 / v], rtol=1e-4, atol=1e-6)
        # mid^2 - det = 0 < 0.1 -> floor case
        assert o["radii"][i] == math.ceil(3 * math.sqrt(v + math.sqrt(0.1)))
        np.testing.assert_allclose(o["means2d"][i], [W / 2, H / 2, z[i]], rtol=1e-6)


def test_cov2d_clamp_case(oracle):
    """|x/z| > 1.3 tanfov: the Jacobian uses the clamped position (checked via ewa_cov2d,
    which implements the clamp independently) and the Gaussian is outside the frustum."""
    W, H, tfx, tfy, V, P = general_camera()
    Vi = np.linalg.inv(V)
    pts_view = np.array([[4.0, 0.1, 2.0, 1], [-5.0, 0.3, 3.0, 1], [0.2, 3.5, 2.5, 1]])
    means = (Vi @ pts_view.T).T[:, :3]
    _, I, o = project(oracle, cam=(W, H, tfx, tfy, V, P), means=means)
    for i in range(3):
        cov, t = ewa_cov2d(I, i)
        assert abs(t[0] / t[2]) > 1.3 * tfx or abs(t[1] / t[2]) > 1.3 * tfy
        inv = np.linalg.inv(cov)
        np.testing.assert_allclose(o["conic"][i], [inv[0, 0], inv[0, 1], inv[1, 1]], rtol=3e-3, atol=1e-7)
        assert o["radii"][i] == 0 and o["tiles_touched"][i] == 0


# ------------------------------------------------------------------------- frustum
def test_frustum_boundaries(oracle):
    """Strict NDC box on the centre: x,y in (-1,1), z_ndc > 0.1."""
    W, H, tfx = 320, 320, 1.0
    V = np.eye(4)
    P = perspective(tfx, tfx, znear=0.01, zfar=100.0)
    z = 4.0
    # z_ndc = zf/(zf-zn) * (1 - zn/z); solve z_ndc = 0.1 -> z*
    zf, zn = 100.0, 0.01
    zstar = zn / (1 - 0.1 * (zf - zn) / zf)
    means = np.array([
        [0.0, 0.0, z],                 # inside
        [z * 0.999, 0.0, z],           # just inside x
        [z * 1.0, 0.0, z],             # on the boundary: strict -> out
        [z * 1.001, 0.0, z],           # outside x
        [0.0, -z * 0.999, z],          # just inside y
        [0.0, -z * 1.001, z],          # outside y
        [0.0, 0.0, zstar * 1.01],      # just beyond the near cut
        [0.0, 0.0, zstar * 0.99],      # before the near cut
        [0.0, 0.0, -3.0],              # behind the camera, on the axis: w < 0 flips both signs,
                                       # x/w = 0 and z/w = 1.0034 -> PASSES (there is no w > 0 test)
        [2.0, 0.0, -3.0],              # behind the camera inside the mirrored frustum -> passes
        [3.5, 0.0, -3.0],              # behind the camera outside the mirrored frustum -> culled
    ])
    _, I, o = project(oracle, cam=(W, H, tfx, tfx, V, P), means=means,
                      scales=np.full((len(means), 3), 0.05))
    vis = (o["radii"] > 0).tolist()
    assert vis == [True, True, False, False, True, False, True, False, True, True, False]


# ------------------------------------------------------------------------- tile rect
def test_tiles_touched_brute_force(oracle):
    s, I, o = project(oracle, n=800)
    tx, ty = (I["W"] + 15) // 16, (I["H"] + 15) // 16
    f = np.float32
    seen_multi = 0
    for i in range(len(I["means"])):
        r = int(o["radii"][i])
        if r <= 0:
            assert o["tiles_touched"][i] == 0
            continue
        px, py = f(o["means2d"][i][0]), f(o["means2d"][i][1])
        cx, cy, d = px / f(16), py / f(16), f(r) / f(16)
        lo_x, hi_x = int(cx - d), int((cx + d) + f(1))
        lo_y, hi_y = int(cy - d), int((cy + d) + f(1))
        n = sum(1 for b in range(ty) for a in range(tx) if lo_x <= a < hi_x and lo_y <= b < hi_y)
        assert o["tiles_touched"][i] == n
        seen_multi += n > 1
    assert seen_multi > 50


# ------------------------------------------------------------------------- SH
def real_sh(l, m, d):
    theta = np.arccos(d[2])
    phi = np.arctan2(d[1], d[0])
    if m == 0:
        return sph_harm_y(l, 0, theta, phi).real
    if m > 0:
        return math.sqrt(2) * (-1) ** m * sph_harm_y(l, m, theta, phi).real
    return math.sqrt(2) * (-1) ** m * sph_harm_y(l, -m, theta, phi).imag


def test_sh_basis_is_the_real_spherical_harmonics(oracle):
    """rgb - 0.5 for a one-hot coefficient vector is the basis function; it must equal the
    library's real spherical harmonic Y_l^m of the view direction up to a fixed sign per
    basis function (the 3DGS sign convention)."""
    n = 64
    W, H, tfx, tfy, V, P = general_camera()
    campos = -V[:3, :3].T @ V[:3, 3]
    means = RNG.normal(size=(n, 3)) * 3
    signs = {}
    for b in range(16):
        l = int(math.isqrt(b))
        m = b - l * l - l
        shs = np.zeros((n, 16, 3))
        shs[:, b, :] = [0.25, -0.25, 0.125]
        _, I, o = project(oracle, cam=(W, H, tfx, tfy, V, P), means=means, shs=shs, sh_degree=3)
        d = I["means"] - I["campos"]
        d /= np.linalg.norm(d, axis=1, keepdims=True)
        want = np.array([real_sh(l, m, di) for di in d])
        got = (o["rgb"][:, 0].astype(np.float64) - 0.5) / 0.25
        sgn = np.sign(got[np.argmax(np.abs(want))] * want[np.argmax(np.abs(want))])
        signs[b] = sgn
        np.testing.assert_allclose(got, sgn * want, rtol=2e-4, atol=2e-6)
        np.testing.assert_allclose((o["rgb"][:, 1] - 0.5) / -0.25, sgn * want, rtol=2e-4, atol=2e-6)
        np.testing.assert_allclose((o["rgb"][:, 2] - 0.5) / 0.125, sgn * want, rtol=4e-4, atol=4e-6)
    # the 3DGS convention: Condon-Shortley-free basis differs from the library by (-1)^m
    assert all(signs[b] == (-1) ** (b - int(math.isqrt(b)) ** 2 - int(math.isqrt(b))) for b in range(16))


def test_sh_degree_truncation_and_clamp(oracle):
    n = 50
    means = RNG.normal(size=(n, 3)) * 3 + [0, 0, 5]
    shs = RNG.normal(0, 0.6, (n, 16, 3))
    full = {}
    for deg in range(4):
        _, _, o = project(oracle, means=means, shs=shs, sh_degree=deg)
        full[deg] = o["rgb"].copy()
        cut = shs.copy()
        cut[:, (deg + 1) ** 2:, :] = 0
        _, _, o2 = project(oracle, means=means, shs=cut, sh_degree=3)
        np.testing.assert_allclose(o["rgb"], o2["rgb"], rtol=1e-6, atol=1e-7)
        assert (o["rgb"] >= 0).all()
    np.testing.assert_allclose(full[0], np.maximum(0.28209479177387814 * shs[:, 0, :] + 0.5, 0), rtol=1e-6,
                               atol=1e-7)
    assert (full[3] == 0).any() or (0.28209479177387814 * shs[:, 0, :] + 0.5 > -1).all()


def test_precomputed_inputs(oracle):
    n = 40
    W, H, tfx, tfy, V, P = general_camera()
    campos = -V[:3, :3].T @ V[:3, 3]
    s = make_settings(H, W, tfx, tfy, [0, 0, 0], 1.0, V, P, 3, campos)
    means = np.stack([RNG.uniform(-1, 1, n), RNG.uniform(-1, 1, n), RNG.uniform(2, 6, n)], 1)
    scales = np.exp(RNG.normal(-2, 0.5, (n, 3)))
    quats = RNG.normal(size=(n, 4))
    shs = RNG.normal(0, 0.3, (n, 16, 3))
    base = oracle.project_fwd(s, means, scales, quats, shs)
    cols = RNG.uniform(0, 1, (n, 3)).astype(np.float32)
    pre = oracle.project_fwd(s, means, scales, quats, shs, cov3d_precomp=base["cov3d"], colors_precomp=cols)
    assert (pre["rgb"] == cols).all()
    for k in ("means2d", "conic", "radii", "tiles_touched", "cov3d"):
        assert (pre[k] == base[k]).all()


# ------------------------------------------------------------------------- offsets / sort
def test_offsets_is_exclusive_cumsum_and_k_skips_last(oracle):
    c = RNG.integers(0, 9, 1000).astype(np.int32)
    off, k = oracle.offsets(c)
    assert (off == np.concatenate([[0], np.cumsum(c)[:-1]])).all()
    assert k == int(c[:-1].sum())
    assert oracle.offsets(np.zeros(0, np.int32))[1] == 0
    assert oracle.offsets(np.array([7], np.int32))[1] == 0


def test_sort_is_stable_ascending(oracle):
    k = 20000
    keys = (RNG.integers(0, 50, k).astype(np.int64) << 32) | RNG.integers(0, 40, k).astype(np.int64)
    vals = np.arange(k, dtype=np.int32)
    sk, sv = oracle.sort_pairs(keys, vals)
    order = np.argsort(keys, kind="stable")
    assert (sk == keys[order]).all() and (sv == vals[order]).all()


def test_tile_ranges_brute_force_and_unclosed_last_run(oracle):
    T = 12
    tiles = np.sort(RNG.choice([0, 1, 4, 5, 6, 9], 300)).astype(np.int64)      # highest tile 9 < T-1
    keys = (tiles << 32) | RNG.integers(1, 1000, 300).astype(np.int64)
    got = oracle.tile_ranges(keys, T)
    # brute force from the definition: scatter at run ends (never after the final run), max-scan
    want = np.zeros(T + 1, np.int64)
    want[T] = len(keys)
    for i in range(len(keys) - 1):
        if tiles[i] != tiles[i + 1]:
            want[tiles[i] + 1] = i + 1
    want = np.maximum.accumulate(want)
    assert (got == want).all()
    # consequence: the last non-empty tile (9) is empty, its run is credited to tile T-1
    assert got[9] == got[10] and got[T - 1] == got[9] and got[T] == len(keys)
    assert oracle.tile_ranges(np.zeros(0, np.int64), T).tolist() == [0] * (T + 1)


# ------------------------------------------------------------------------- blend forward
def small_scene(n=300, W=64, H=48, seed=3, sh_degree=1):
    sc = make_scene("cfg0", n=n, width=W, height=H, sh_degree=sh_degree, seed=seed)
    return sc


def run_forward(oracle, sc, **kw):
    s = scene_settings(sc)
    A = arrays(sc)
    img, radii, st = oracle.forward(s, A["means_3d"], A["scales"] * kw.get("scale_mul", 1.0), A["rotations"],
                                    A["opacities"], A["shs"], colors_precomp=kw.get("colors"), keep_emitted=True)
    S = oracle.state(s, st, sc["n"], emitted=True)
    oracle.free(st)
    return s, A, img, radii, S


def brute_force_render(S, opac, W, H, n_tiles_x, n_emit):
    """Per pixel: every Gaussian that emitted a key for the pixel's tile, ordered by
    (depth bits, id); float64; knows nothing about sorting or ranges."""
    img = np.zeros((H, W, 3))
    Tf = np.ones((H, W))
    m, con, rgb = S["means2d"].astype(np.float64), S["conic"].astype(np.float64), S["rgb"].astype(np.float64)
    per_tile = {}
    for key, g in zip(S["emitted_keys"], S["emitted_values"]):
        per_tile.setdefault(int(key) >> 32, []).append((int(key) & 0xFFFFFFFF, int(g)))
    for y in range(H):
        for x in range(W):
            lst = sorted(per_tile.get((y // 16) * n_tiles_x + x // 16, []))
            C, T = np.zeros(3), 1.0
            for _, g in lst:
                dx, dy = x + 0.5 - m[g, 0], y + 0.5 - m[g, 1]
                power = -0.5 * (con[g, 0] * dx * dx + con[g, 2] * dy * dy) - con[g, 1] * dx * dy
                alpha = min(0.999, float(opac[g]) * math.exp(power))
                if power >= 0 or alpha < 1 / 255:
                    continue
                if (1 - alpha) * T < 1e-4:
                    break
                C += alpha * T * rgb[g]
                T *= 1 - alpha
            img[y, x], Tf[y, x] = C, T
    return img, Tf


def test_blend_forward_vs_brute_force(oracle):
    sc = small_scene(400)
    s, A, img, radii, S = run_forward(oracle, sc, scale_mul=3.0)
    assert S["num_keys"] > 1000
    ref, Tref = brute_force_render(S, A["opacities"].reshape(-1), sc["width"], sc["height"], 4, S["num_keys"])
    ok = S["margin"] > 1e-4
    assert ok.mean() > 0.98
    np.testing.assert_allclose(img[ok], ref[ok], rtol=1e-4, atol=2e-5)
    np.testing.assert_allclose(S["final_T"][ok], Tref[ok], rtol=1e-4, atol=1e-6)


def test_blend_forward_white_scene_telescopes(oracle):
    """All colours 1 => image = 1 - final_T in every channel."""
    sc = small_scene(500)
    cols = np.ones((sc["n"], 3), np.float32)
    s, A, img, radii, S = run_forward(oracle, sc, scale_mul=3.0, colors=cols)
    for c in range(3):
        np.testing.assert_allclose(img[..., c], 1 - S["final_T"], rtol=0, atol=3e-6)
    assert (S["final_T"] <= 1).all() and (S["final_T"] >= 1e-4 * 0.99).all() and (img >= 0).all()


def test_blend_forward_single_gaussian_closed_form(oracle):
    W, H = 48, 32
    s = make_settings(H, W, 1, 1, [0, 0, 0], 1, np.eye(4), np.eye(4), 0, [0, 0, 0])
    means2d = np.array([[20.3, 13.7, 5.0]], np.float32)
    conic = np.array([[0.05, 0.01, 0.08]], np.float32)
    rgb = np.array([[0.2, 0.5, 0.9]], np.float32)
    opac = np.array([0.8], np.float32)
    ranges = np.zeros(7, np.int32)
    ranges[1:] = 1                               # the only entry belongs to tile 0
    o = oracle.blend_fwd(s, ranges, np.array([0], np.int32), means2d, conic, rgb, opac)
    for y in range(H):
        for x in range(W):
            if x < 16 and y < 16:
                dx, dy = x + 0.5 - 20.3, y + 0.5 - 13.7
                a = 0.8 * math.exp(-0.5 * (0.05 * dx * dx + 0.08 * dy * dy) - 0.01 * dx * dy)
                a = 0.0 if a < 1 / 255 else min(a, 0.999)
            else:
                a = 0.0
            np.testing.assert_allclose(o["image"][y, x], a * rgb[0], rtol=2e-5, atol=1e-7)
            assert math.isclose(o["final_T"][y, x], 1 - a, rel_tol=2e-5, abs_tol=1e-7)


def test_behind_camera_keys_sort_first_and_are_skipped(oracle):
    """A Gaussian behind the camera that passes the frustum test gets a negative depth; the
    sign-extended depth turns its whole key negative (tile field -1), the signed sort puts
    those keys first and the boundary scatter writes their count into ranges[0], so no tile
    ever blends them."""
    sc = small_scene(200)
    A = arrays(sc)
    means = A["means_3d"].copy()
    means[:60, 2] *= -1.0
    s = scene_settings(sc)
    img, radii, st = oracle.forward(s, means, A["scales"] * 3.0, A["rotations"], A["opacities"], A["shs"])
    S = oracle.state(s, st, sc["n"])
    oracle.free(st)
    behind = (means[:, 2] < 0) & (radii > 0)
    nneg = int(S["tiles_touched"][:-1][behind[:-1]].sum())
    assert behind.sum() > 10 and nneg > 10
    assert (S["sorted_keys"][:nneg] < 0).all() and (S["sorted_keys"][nneg:] >= 0).all()
    assert (np.diff(S["sorted_keys"]) >= 0).all()
    assert S["ranges"][0] == nneg
    assert not np.isin(S["sorted_ids"][S["ranges"][0]:], np.nonzero(behind)[0]).any()
    assert np.isfinite(img).all()


def test_last_gaussian_is_never_rendered(oracle):
    sc = small_scene(50)
    s, A, img, radii, S = run_forward(oracle, sc, scale_mul=3.0)
    assert (S["sorted_ids"] != sc["n"] - 1).all()
    assert S["num_keys"] == int(S["tiles_touched"][:-1].sum())
