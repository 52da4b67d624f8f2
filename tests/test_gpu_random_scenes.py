"""GPU parity on randomly drawn scenes (seeded): odd image shapes, 1 to 60000 Gaussians, every SH
degree, tiny to screen-filling footprints, Gaussians behind the camera: whole forward and
backward through the C ABI against the serial oracle."""
import numpy as np
import pytest
import torch

from ds_splat_amd.synthetic import make_scene
from helpers import arrays, check_grads_against_bounds, comparable_gaussians, scene_settings, set_camera

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def draw(rng):
    n = int(rng.choice([1, 2, 3, 255, 256, 257, 1000, 5000, 20000, 60000]))
    c = dict(n=n, W=int(rng.integers(16, 2200)), H=int(rng.integers(16, 1300)),
             name=str(rng.choice(["cfg0", "cfg1", "cfg2", "cfg4"])), deg=int(rng.integers(0, 4)),
             scale_mul=float(rng.choice([0.3, 1.0, 2.0, 6.0, 20.0])), flip=int(rng.integers(0, max(1, n // 10))),
             giants=int(rng.integers(0, 4)) if n >= 1000 else 0, seed=int(rng.integers(1, 1 << 30)))
    c["pick"] = rng.integers(0, n, c["giants"])
    # half of the scenes through a camera drawn at random: anywhere around (or inside) the cloud,
    # rolled, non-square pixels, a scale modifier
    c["bins"] = int(rng.choice([1, 2, 4, 8]))      # tiles per side of the bins the lists are built for
    c["camera"] = None
    if rng.random() < 0.5:
        eye = rng.uniform([-4.0, -3.0, -3.0], [4.0, 3.0, 8.0])
        target = rng.uniform([-1.5, -1.5, 4.0], [1.5, 1.5, 12.0])
        up = np.array([rng.uniform(-0.4, 0.4), 1.0, rng.uniform(-0.4, 0.4)])
        c["camera"] = dict(eye=tuple(float(v) for v in eye), target=tuple(float(v) for v in target),
                           up=tuple(float(v) for v in up), tanfovx=float(rng.uniform(0.3, 0.9)),
                           tanfovy=float(rng.uniform(0.25, 0.8)), scale_modifier=float(rng.choice([0.7, 1.0, 1.3])))
    return c


@pytest.mark.parametrize("sweep_seed", [11, 12, 13])
def test_random_scenes_forward_and_backward(oracle, list_bin, sweep_seed):
    from ds_splat_amd import stages
    rng = np.random.default_rng(sweep_seed)
    done = 0
    compared = 0        # Gaussians whose gradients were compared, over the whole sweep
    worst = 0.0
    for _ in range(14):
        c = draw(rng)
        sc = set_camera(make_scene(c["name"], n=c["n"], width=c["W"], height=c["H"], sh_degree=c["deg"],
                                   seed=c["seed"]), c["camera"])
        A = arrays(sc)
        A["scales"] = (A["scales"] * c["scale_mul"]).astype(np.float32)
        if c["flip"]:
            A["means_3d"][:c["flip"], 2] *= -1.0
        if c["giants"]:
            A["scales"][c["pick"]] *= 100.0
        s = scene_settings(sc)
        img, radii, st = oracle.forward(s, A["means_3d"], A["scales"], A["rotations"], A["opacities"], A["shs"])
        S = oracle.state(s, st, c["n"])
        if S["num_keys"] > 6_000_000:          # keeps the serial oracle's share of the test short
            oracle.free(st)
            continue
        B = oracle.backward(s, st, 16, A["means_3d"], A["scales"], A["rotations"], A["opacities"], A["v_image"])
        oracle.free(st)
        list_bin(c["bins"])
        cam = stages.camera_from_scene(sc, DEV)
        d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
        image, g = stages.forward(cam, d(A["means_3d"]), d(A["scales"]), d(A["rotations"]), d(A["opacities"]),
                                  d(A["shs"]))
        torch.cuda.synchronize()
        what = str({k: v for k, v in c.items() if k != "pick"})
        assert (g.radii.cpu().numpy() == radii).all(), what
        assert (g.ranges.cpu().numpy() == S["ranges"]).all(), what
        if c["bins"] == 1:
            assert g.num_keys == S["num_keys"], what
            assert (g.sorted_ids.cpu().numpy() == S["sorted_ids"]).all(), what
        ok = S["margin"] > 1e-4
        assert (g.final_idx.cpu().numpy()[ok] == S["final_idx"][ok]).all(), what
        np.testing.assert_allclose(image.cpu().numpy()[ok], img[ok], rtol=1e-4, atol=1e-5, err_msg=what)
        o = stages.backward(cam, g, 16, d(A["means_3d"]), d(A["scales"]), d(A["rotations"]), d(A["v_image"]))
        torch.cuda.synchronize()
        # Gaussians that a pixel with a borderline forward decision can reach are not compared
        gok = comparable_gaussians(S, B, c["W"], g.final_T.cpu().numpy(), g.final_idx.cpu().numpy())
        compared += int(gok.sum())
        bounds = oracle.gradient_bounds(s, 16, A["means_3d"], A["scales"], A["rotations"], S["conic"], S["cov3d"],
                                        radii, B["abs_sums"], rel=1e-4)
        got = {key: o[key].cpu().numpy() for key in ("v_mean3d", "v_means2d", "v_shs", "v_opacity", "v_scale",
                                                     "v_quat")}
        worst = max(worst, check_grads_against_bounds(got, B, bounds, gok, what))
        done += 1
    print("sweep %d: %d scenes, gradients of %d Gaussians compared, largest error / bound = %.3f" % (
        sweep_seed, done, compared, worst))
    assert done >= 8 and compared > 20000


def test_image_tolerance_where_the_exponents_terms_cancel(oracle, list_bin):
    """256 thin, long splats over a 795 x 1287 image: far from a splat's centre the three terms of its
    exponent are large and cancel, so every rounding in them shows in alpha.  This scene (drawn by the
    sweep above under another seed) is where a build that folded log2(e) into the conic coefficients
    left the image tolerance by 2 %; the committed exponent keeps it at about two thirds of it."""
    from ds_splat_amd import stages
    c = dict(n=256, W=795, H=1287, name="cfg4", deg=2, scale_mul=0.3, flip=1, seed=493649661)
    sc = make_scene(c["name"], n=c["n"], width=c["W"], height=c["H"], sh_degree=c["deg"], seed=c["seed"])
    A = arrays(sc)
    A["scales"] = (A["scales"] * c["scale_mul"]).astype(np.float32)
    A["means_3d"][:c["flip"], 2] *= -1.0
    s = scene_settings(sc)
    img, radii, st = oracle.forward(s, A["means_3d"], A["scales"], A["rotations"], A["opacities"], A["shs"])
    S = oracle.state(s, st, c["n"])
    oracle.free(st)
    list_bin(1)
    cam = stages.camera_from_scene(sc, DEV)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    image, g = stages.forward(cam, d(A["means_3d"]), d(A["scales"]), d(A["rotations"]), d(A["opacities"]), d(A["shs"]))
    torch.cuda.synchronize()
    ok = S["margin"] > 1e-4
    assert ok.mean() > 0.9
    assert (g.final_idx.cpu().numpy()[ok] == S["final_idx"][ok]).all()
    got, want = image.cpu().numpy()[ok], img[ok]
    worst = float((np.abs(got - want) / (1e-5 + 1e-4 * np.abs(want))).max())
    print("largest image error / tolerance = %.3f" % worst)
    assert worst < 1.0
