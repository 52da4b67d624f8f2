"""Pins the oracle's backward stages: central finite differences of float64 forwards
(the blend through the oracle's double instance of the tile walker, the projection through
a textbook EWA written here in numpy), closed forms, the adjoint identity for the SH basis,
and hand cases for the alpha-clamp mismatch between forward (0.999) and backward (0.99)."""
import math

import numpy as np

from ds_splat_amd.synthetic import make_scene
from helpers import arrays, look_at_view, perspective, scene_settings
from oracle.binding import make_settings

RNG = np.random.default_rng(11)


def forward_state(oracle, n=60, W=48, H=32, seed=5, scale_mul=4.0, opac_max=0.95, bg=None):
    sc = make_scene("cfg0", n=n, width=W, height=H, sh_degree=2, seed=seed)
    A = arrays(sc)
    A["opacities"] = np.minimum(A["opacities"], opac_max).astype(np.float32)
    s = scene_settings(sc, bg=bg)
    img, radii, st = oracle.forward(s, A["means_3d"], A["scales"] * scale_mul, A["rotations"], A["opacities"],
                                    A["shs"])
    S = oracle.state(s, st, n)
    oracle.free(st)
    return sc, s, A, S, radii


def rel_err(got, want):
    scale = np.abs(want).max() + 1e-12
    return np.abs(got - want).max() / scale


def fd_blend(oracle, sc, S, opac, w, bg, clamp, eps=1e-6):
    xy = S["means2d"][:, :2].astype(np.float64)
    params = dict(xy=xy, conic=S["conic"].astype(np.float64), rgb=S["rgb"].astype(np.float64),
                  opac=opac.astype(np.float64).reshape(-1))

    def loss(p):
        return oracle.blend_loss_f64(sc["width"], sc["height"], S["ranges"], S["sorted_ids"], p["xy"], p["conic"],
                                     p["rgb"], p["opac"], w, clamp, bg=bg)

    grads = {}
    used = np.unique(S["sorted_ids"])
    for name, arr in params.items():
        g = np.zeros_like(arr)
        flat, gf = arr.reshape(len(arr), -1), g.reshape(len(arr), -1)
        for i in used:
            for j in range(flat.shape[1]):
                old = flat[i, j]
                flat[i, j] = old + eps
                lp = loss(params)
                flat[i, j] = old - eps
                lm = loss(params)
                flat[i, j] = old
                gf[i, j] = (lp - lm) / (2 * eps)
        grads[name] = g
    return grads


def test_blend_backward_matches_finite_differences(oracle):
    sc, s, A, S, radii = forward_state(oracle)
    assert S["num_keys"] > 100
    assert S["final_T"].min() > 2e-4          # nobody terminated: FD sees a smooth function
    w = RNG.normal(size=(sc["height"], sc["width"], 3))
    B = oracle.blend_bwd(s, S["ranges"], S["sorted_ids"], S["means2d"], S["conic"], S["rgb"], A["opacities"],
                         S["final_T"], S["final_idx"], w.astype(np.float32))
    G = fd_blend(oracle, sc, S, A["opacities"], w.astype(np.float32).astype(np.float64), None, 0.999)
    assert rel_err(B["v_rgb"], G["rgb"]) < 1e-4
    assert rel_err(B["v_opacity"].reshape(-1), G["opac"]) < 1e-4
    assert rel_err(B["v_conic"], G["conic"]) < 1e-4
    # the reference differentiates w.r.t. the mean with delta = mean - pixel: same sign as d/d(mean)
    assert rel_err(B["v_xy"], G["xy"]) < 1e-4


def test_blend_backward_background_term(oracle):
    """Backward carries -T_final*ra*bg*v_out although forward never composites bg: it is the
    gradient of image + final_T*bg."""
    bg = np.array([0.3, 0.7, 0.1], np.float32)
    sc, s, A, S, radii = forward_state(oracle, n=40, seed=9, bg=bg)
    w = RNG.normal(size=(sc["height"], sc["width"], 3)).astype(np.float32)
    B = oracle.blend_bwd(s, S["ranges"], S["sorted_ids"], S["means2d"], S["conic"], S["rgb"], A["opacities"],
                         S["final_T"], S["final_idx"], w)
    G = fd_blend(oracle, sc, S, A["opacities"], w.astype(np.float64), bg.astype(np.float64), 0.999)
    assert rel_err(B["v_opacity"].reshape(-1), G["opac"]) < 1e-4
    assert rel_err(B["v_xy"], G["xy"]) < 1e-4
    G0 = fd_blend(oracle, sc, S, A["opacities"], w.astype(np.float64), None, 0.999)
    assert rel_err(G0["opac"], G["opac"]) > 1e-2      # the term is not negligible


def test_v_rgb_closed_form(oracle):
    """v_rgb[g] = sum over pixels of alpha*T_before*v_out, from an independent float64 walk."""
    sc, s, A, S, radii = forward_state(oracle, n=80, seed=21)
    w = RNG.normal(size=(sc["height"], sc["width"], 3)).astype(np.float32)
    B = oracle.blend_bwd(s, S["ranges"], S["sorted_ids"], S["means2d"], S["conic"], S["rgb"], A["opacities"],
                         S["final_T"], S["final_idx"], w)
    want = np.zeros((sc["n"], 3))
    m, con, op = S["means2d"].astype(np.float64), S["conic"].astype(np.float64), A["opacities"].reshape(-1)
    ntx = (sc["width"] + 15) // 16
    for y in range(sc["height"]):
        for x in range(sc["width"]):
            t = (y // 16) * ntx + x // 16
            T = 1.0
            for e in range(S["ranges"][t], S["ranges"][t + 1]):
                g = S["sorted_ids"][e]
                dx, dy = x + 0.5 - m[g, 0], y + 0.5 - m[g, 1]
                power = -0.5 * (con[g, 0] * dx * dx + con[g, 2] * dy * dy) - con[g, 1] * dx * dy
                a = min(0.99, op[g] * math.exp(power))
                if power >= 0 or a < 1 / 255:
                    continue
                want[g] += a * T * w[y, x]
                T *= 1 - a
    assert rel_err(B["v_rgb"], want) < 2e-5


def test_alpha_clamp_mismatch_hand_case(oracle):
    """Opacity 0.995 next to a pixel centre: forward blends alpha ~0.995 (T_final ~0.005);
    backward clamps alpha to 0.99, so ra = 100, T = T_final*100, fac = 0.99*T — worked by
    hand from backward.cu:127-176."""
    W = H = 16
    s = make_settings(H, W, 1, 1, [0, 0, 0], 1, np.eye(4), np.eye(4), 0, [0, 0, 0])
    means2d = np.array([[5.51, 7.5, 3.0]], np.float32)        # 0.01 px right of the centre of pixel (5,7)
    conic = np.array([[0.02, 0.0, 0.02]], np.float32)
    rgb = np.array([[0.25, 0.5, 1.0]], np.float32)
    opac = np.array([0.995], np.float32)
    ranges = np.array([0, 1], np.int32)
    ids = np.array([0], np.int32)
    F = oracle.blend_fwd(s, ranges, ids, means2d, conic, rgb, opac)
    dx = float(np.float32(5.51)) - 5.5
    vis = math.exp(-0.5 * 0.02 * dx * dx)
    assert math.isclose(F["final_T"][7, 5], 1 - 0.995 * vis, rel_tol=1e-3)       # forward: no 0.99 clamp
    assert F["final_idx"][7, 5] == 0
    v_out = np.zeros((H, W, 3), np.float32)
    v_out[7, 5] = [1.0, 2.0, -1.0]
    B = oracle.blend_bwd(s, ranges, ids, means2d, conic, rgb, opac, F["final_T"], F["final_idx"], v_out)
    Tf = float(F["final_T"][7, 5])
    ra = 1 / (1 - 0.99)                                        # backward: alpha = min(0.99, 0.995*vis)
    T = Tf * ra
    fac = 0.99 * T
    np.testing.assert_allclose(B["v_rgb"][0], fac * v_out[7, 5], rtol=1e-4)
    v_alpha = float((rgb[0] * T * v_out[7, 5]).sum())
    np.testing.assert_allclose(B["v_opacity"][0, 0], vis * v_alpha, rtol=1e-4)
    v_sigma = -0.995 * vis * v_alpha
    np.testing.assert_allclose(B["v_xy"][0], [v_sigma * 0.02 * dx, 0.0], rtol=1e-3, atol=1e-9)
    np.testing.assert_allclose(B["v_conic"][0], [0.5 * v_sigma * dx * dx, 0.0, 0.0], rtol=1e-3, atol=1e-12)


def test_forward_skips_zero_power_backward_does_not(oracle):
    """Pixel centre exactly on the mean: power == 0 is skipped by forward (power >= 0,
    rasterizer_kernels.cu:394) so nothing is blended and final_idx stays 0."""
    W = H = 16
    s = make_settings(H, W, 1, 1, [0, 0, 0], 1, np.eye(4), np.eye(4), 0, [0, 0, 0])
    means2d = np.array([[5.5, 7.5, 3.0]], np.float32)
    F = oracle.blend_fwd(s, np.array([0, 1], np.int32), np.array([0], np.int32), means2d,
                         np.array([[2.0, 0.0, 2.0]], np.float32), np.ones((1, 3), np.float32),
                         np.array([0.9], np.float32))
    assert F["final_T"][7, 5] == 1.0 and (F["image"][7, 5] == 0).all()
    assert F["final_T"][7, 6] < 1.0


def test_sh_backward_is_the_adjoint_of_sh_forward(oracle):
    n = 200
    V = look_at_view([0.5, 0.1, -2.0], [0, 0, 3.0])
    tf = 0.8
    P = perspective(tf, tf) @ V
    campos = -V[:3, :3].T @ V[:3, 3]
    means = RNG.normal(size=(n, 3)) * 2 + [0, 0, 3]
    for deg in range(4):
        s = make_settings(64, 64, tf, tf, [0, 0, 0], 1.0, V, P, deg, campos)
        c = RNG.normal(0, 0.1, (n, 16, 3))                       # small: rgb stays unclamped
        v = RNG.normal(size=(n, 3))
        fwd = oracle.project_fwd(s, means, np.full((n, 3), 0.1), np.tile([1.0, 0, 0, 0], (n, 1)), c)
        assert (fwd["rgb"] > 0).all()
        lhs = ((fwd["rgb"].astype(np.float64) - 0.5) * np.float32(v).astype(np.float64)).sum()
        vs = oracle.sh_bwd(s, 16, means, v)
        rhs = (np.float32(c).astype(np.float64) * vs).sum()
        assert math.isclose(lhs, rhs, rel_tol=2e-5)
        nb = (deg + 1) ** 2
        assert (vs[:, nb:, :] == 0).all() and (np.abs(vs[:, :nb, :]).sum(axis=(0, 2)) > 0).all()
    # num_bases below 16 (shs tensor with 4 bases): output shape follows it
    s = make_settings(64, 64, tf, tf, [0, 0, 0], 1.0, V, P, 1, campos)
    assert oracle.sh_bwd(s, 4, means, v).shape == (n, 4, 3)


# ------------------------------------------------------------------------- projection backward
def raw_quat_R(q):
    w, x, y, z = q
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                     [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                     [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])


def ewa_outputs(V, fx, fy, cx, cy, mod, mean, scale=None, quat=None, cov3d=None):
    """(pixel xy, conic) as the function the backward differentiates: rotation from the raw
    quaternion polynomial, no clamp on t, inverse of (J W Sigma W^T J^T + 0.3 I)."""
    if cov3d is None:
        R = raw_quat_R(quat)
        S = np.diag(scale * mod)
        Sigma = R @ S @ S @ R.T
    else:
        c = cov3d
        Sigma = np.array([[c[0], c[1], c[2]], [c[1], c[3], c[4]], [c[2], c[4], c[5]]])
    t = V[:3, :3] @ mean + V[:3, 3]
    J = np.array([[fx / t[2], 0, -fx * t[0] / t[2] ** 2], [0, fy / t[2], -fy * t[1] / t[2] ** 2]])
    A = J @ V[:3, :3]
    cov = A @ Sigma @ A.T + 0.3 * np.eye(2)
    inv = np.linalg.inv(cov)
    zi = 1 / (t[2] + 1e-6)
    return np.array([fx * t[0] * zi + cx, fy * t[1] * zi + cy]), np.array([inv[0, 0], inv[0, 1], inv[1, 1]])


def test_projection_backward_matches_finite_differences(oracle):
    n = 40
    W, H, tfx = 200, 120, 0.7
    tfy = tfx * H / W
    V = look_at_view([0.3, -0.2, -1.0], [0.1, 0.2, 4.0], up=(0.1, 1.0, 0.05))
    P = perspective(tfx, tfy) @ V
    campos = -V[:3, :3].T @ V[:3, 3]
    mod = 1.3
    s = make_settings(H, W, tfx, tfy, [0, 0, 0], mod, V, P, 0, campos)
    Vi = np.linalg.inv(V)
    z = RNG.uniform(2, 8, n)
    pv = np.stack([RNG.uniform(-0.6, 0.6, n) * tfx * z, RNG.uniform(-0.6, 0.6, n) * tfy * z, z, np.ones(n)], 1)
    means = np.float32((Vi @ pv.T).T[:, :3])
    scales = np.float32(np.exp(RNG.normal(-1.5, 0.5, (n, 3))))
    quats = RNG.normal(size=(n, 4))
    quats = np.float32(quats / np.linalg.norm(quats, axis=1, keepdims=True))     # unit, as trained models have
    fwd = oracle.project_fwd(s, means, scales, quats, np.zeros((n, 16, 3)))
    assert (fwd["radii"] > 0).all()
    v_xy = np.float32(RNG.normal(size=(n, 2)))
    v_conic = np.float32(RNG.normal(size=(n, 3)))
    B = oracle.project_bwd(s, means, scales, quats, fwd["conic"], fwd["cov3d"], fwd["radii"], v_xy, v_conic)

    V64 = np.float32(V).astype(np.float64)
    fx, fy = W / (2 * float(np.float32(tfx))), H / (2 * float(np.float32(tfy)))

    def f(i, mean, scale, quat, cov3d=None):
        xy, con = ewa_outputs(V64, fx, fy, W / 2, H / 2, float(np.float32(mod)), mean, scale, quat, cov3d)
        return float(v_xy[i].astype(np.float64) @ xy + v_conic[i].astype(np.float64) @ con)

    def fd(fun, x, eps):
        g = np.zeros_like(x)
        for j in range(len(x)):
            xp, xm = x.copy(), x.copy()
            xp[j] += eps
            xm[j] -= eps
            g[j] = (fun(xp) - fun(xm)) / (2 * eps)
        return g

    for i in range(n):
        m, sc, q = means[i].astype(np.float64), scales[i].astype(np.float64), quats[i].astype(np.float64)
        gm = fd(lambda x: f(i, x, sc, q), m, 1e-6)
        gs = fd(lambda x: f(i, m, x, q), sc, 1e-7)
        gq = fd(lambda x: f(i, m, sc, x), q, 1e-6)
        c3 = fwd["cov3d"][i].astype(np.float64)
        gc = fd(lambda x: f(i, m, None, None, cov3d=x), c3, 1e-8)
        for got, want, name in ((B["v_mean3d"][i], gm, "mean"), (B["v_scale"][i], gs, "scale"),
                                (B["v_quat"][i], gq, "quat"), (B["v_cov3d"][i], gc, "cov3d")):
            assert rel_err(got, want) < 3e-3, (i, name, got, want)


def test_projection_backward_skips_culled(oracle):
    n = 30
    sc = make_scene("cfg0", n=n, width=64, height=64, seed=2)
    A = arrays(sc)
    A["means_3d"][::3, 0] += 50.0                       # far outside the frustum
    s = scene_settings(sc)
    fwd = oracle.project_fwd(s, A["means_3d"], A["scales"], A["rotations"], A["shs"])
    culled = fwd["radii"] <= 0
    assert culled.sum() >= n // 3
    B = oracle.project_bwd(s, A["means_3d"], A["scales"], A["rotations"], fwd["conic"], fwd["cov3d"], fwd["radii"],
                           np.ones((n, 2), np.float32), np.ones((n, 3), np.float32))
    for k in ("v_mean3d", "v_scale", "v_quat", "v_cov3d"):
        assert (B[k][culled] == 0).all() and (np.abs(B[k][~culled]).sum(axis=1) > 0).all()


def test_full_backward_shapes_and_zero_column(oracle):
    sc, s, A, S, radii = forward_state(oracle, n=50, seed=4)
    img, radii, st = oracle.forward(s, A["means_3d"], A["scales"] * 4.0, A["rotations"], A["opacities"], A["shs"])
    v = RNG.normal(size=(sc["height"], sc["width"], 3)).astype(np.float32)
    B = oracle.backward(s, st, 16, A["means_3d"], A["scales"] * 4.0, A["rotations"], A["opacities"], v)
    oracle.free(st)
    assert B["v_means2d"].shape == (50, 3) and (B["v_means2d"][:, 2] == 0).all()
    assert B["v_opacity"].shape == (50, 1) and B["v_shs"].shape == (50, 16, 3)
    assert np.abs(B["v_mean3d"]).max() > 0 and np.isfinite(B["v_quat"]).all()


def test_abs_sums_bound_the_sums_and_equal_them_where_no_term_cancels(oracle):
    """abs_sums (the scale of the gradient tolerances): never below |sum|; equal to the sum where
    every term has one sign (v_rgb under a positive upstream gradient); strictly larger where terms
    cancel (a sign-mixed upstream gradient)."""
    sc, s, A, S, radii = forward_state(oracle, n=80, W=64, H=48, seed=3)
    pos = np.abs(RNG.normal(size=(sc["height"], sc["width"], 3))).astype(np.float32)
    B = oracle.blend_bwd(s, S["ranges"], S["sorted_ids"], S["means2d"], S["conic"], S["rgb"], A["opacities"],
                         S["final_T"], S["final_idx"], pos)
    got = np.concatenate([B["v_xy"], B["v_conic"], B["v_opacity"], B["v_rgb"]], axis=1)
    assert (B["abs_sums"] * (1 + 1e-5) + 1e-30 >= np.abs(got)).all()
    touched = np.abs(B["v_rgb"]).sum(1) > 0
    assert touched.sum() > 20
    np.testing.assert_allclose(B["abs_sums"][:, 6:9], B["v_rgb"], rtol=1e-5, atol=1e-12)
    mixed = RNG.normal(size=(sc["height"], sc["width"], 3)).astype(np.float32)
    B2 = oracle.blend_bwd(s, S["ranges"], S["sorted_ids"], S["means2d"], S["conic"], S["rgb"], A["opacities"],
                          S["final_T"], S["final_idx"], mixed)
    got2 = np.concatenate([B2["v_xy"], B2["v_conic"], B2["v_opacity"], B2["v_rgb"]], axis=1)
    assert (B2["abs_sums"] * (1 + 1e-5) + 1e-30 >= np.abs(got2)).all()
    assert (B2["abs_sums"][touched, 6:9] > 1.05 * np.abs(B2["v_rgb"][touched])).mean() > 0.5
    # |v_image| as the upstream gradient bounds every channel sum of the sign-mixed run
    B3 = oracle.blend_bwd(s, S["ranges"], S["sorted_ids"], S["means2d"], S["conic"], S["rgb"], A["opacities"],
                          S["final_T"], S["final_idx"], np.abs(mixed))
    np.testing.assert_allclose(B2["abs_sums"][:, 6:9], B3["v_rgb"], rtol=1e-5, atol=1e-12)


def test_gradient_bounds_hold_for_perturbed_screen_space_sums(oracle):
    """gradient_bounds propagates a tolerance on the nine screen-space sums through the (linear)
    per-Gaussian backward: outputs of inputs perturbed inside the tolerance stay inside the bounds,
    and a perturbation ten times larger leaves them."""
    sc = make_scene("cfg0", n=300, width=96, height=64, sh_degree=3, seed=8)
    A = arrays(sc)
    V = look_at_view((1.0, 0.5, -1.0), (0.0, 0.0, 6.0))
    s = make_settings(64, 96, 0.6, 0.45, np.zeros(3), 1.3, V, perspective(0.6, 0.45) @ V, 3, (1.0, 0.5, -1.0))
    P = oracle.project_fwd(s, A["means_3d"], A["scales"] * 3, A["rotations"], A["shs"])
    n = 300
    v = RNG.normal(size=(n, 9)).astype(np.float32)
    scale = np.abs(v) * 3.0 + 0.1                                          # plays the abs_sums
    run = lambda u: (oracle.project_bwd(s, A["means_3d"], A["scales"] * 3, A["rotations"], P["conic"], P["cov3d"],
                                        P["radii"], u[:, 0:2], u[:, 2:5]),
                     oracle.sh_bwd(s, 16, A["means_3d"], u[:, 6:9]))
    base, base_sh = run(v)
    bounds = oracle.gradient_bounds(s, 16, A["means_3d"], A["scales"] * 3, A["rotations"], P["conic"], P["cov3d"],
                                    P["radii"], scale, rel=1e-3, floor=0.0)
    sign = np.sign(RNG.normal(size=(n, 9))).astype(np.float32)
    inside, inside_sh = run(v + 0.9e-3 * scale * sign)
    outside, _ = run(v + 1e-2 * scale * sign)
    vis = P["radii"] > 0
    assert vis.sum() > 50
    slack = 1e-6   # float rounding of the two runs themselves, relative to the bound's own scale
    for key in ("v_mean3d", "v_scale", "v_quat", "v_cov3d"):
        err = np.abs(inside[key].astype(np.float64) - base[key])
        assert (err <= bounds[key] * (1 + 1e-3) + slack * np.abs(base[key])).all(), key
        far = np.abs(outside[key].astype(np.float64) - base[key])
        assert (far[vis] > bounds[key][vis]).mean() > 0.3, key
    err = np.abs(inside_sh.astype(np.float64) - base_sh)
    assert (err <= bounds["v_shs"] * (1 + 1e-3) + slack * np.abs(base_sh)).all()
