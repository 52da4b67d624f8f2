"""GPU parity of the whole path through the public Python API (GaussianRasterizer + autograd)
against the CPU oracle, and size-independent properties at the benchmark's full sizes."""
import numpy as np
import pytest
import torch

from ds_splat_amd.synthetic import make_scene
from helpers import (GRAD_KEYS, arrays, check_grads_against_bounds, comparable_gaussians, scene_settings,
                     set_camera)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def api_run(sc, scale_mul=1.0, backward=True, bg=None, opac_shape=None, colors=None, cov3d=None, wants=None):
    from ds_splat import GaussianRasterizationSettings, GaussianRasterizer
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    settings = GaussianRasterizationSettings(
        image_height=sc["height"], image_width=sc["width"], tanfovx=sc["tanfovx"], tanfovy=sc["tanfovy"],
        bg=t["bg"] if bg is None else torch.tensor(bg, dtype=torch.float32, device=DEV),
        scale_modifier=sc["scale_modifier"], viewmatrix=t["viewmatrix"], projmatrix=t["projmatrix"],
        sh_degree=sc["sh_degree"], max_sh_degree=3, campos=t["campos"], prefiltered=False, debug=False)
    opac = t["opacities"] if opac_shape is None else t["opacities"].reshape(opac_shape)
    leaves = dict(means=t["means_3d"].clone(), means2d=torch.zeros_like(t["means_3d"]), shs=t["shs"].clone(),
                  opac=opac.clone(), scales=(t["scales"] * scale_mul).clone(), rots=t["rotations"].clone())
    if backward:
        for k, v in leaves.items():
            v.requires_grad_(wants is None or k in wants)
    r = GaussianRasterizer(settings)
    if colors is not None:
        image, radii = r(leaves["means"], leaves["means2d"], None, colors, leaves["opac"], leaves["scales"],
                         leaves["rots"], None)
    elif cov3d is not None:
        image, radii = r(leaves["means"], leaves["means2d"], leaves["shs"], None, leaves["opac"], None, None, cov3d)
    else:
        image, radii = r(leaves["means"], leaves["means2d"], leaves["shs"], None, leaves["opac"], leaves["scales"],
                         leaves["rots"], None)
    if backward:
        image.backward(t["v_image"])
    torch.cuda.synchronize()
    return image, radii, leaves


def oracle_run(oracle, sc, scale_mul=1.0, bg=None, backward=True):
    A = arrays(sc)
    A["scales"] = (A["scales"] * scale_mul).astype(np.float32)
    s = scene_settings(sc, bg=bg)
    img, radii, st = oracle.forward(s, A["means_3d"], A["scales"], A["rotations"], A["opacities"], A["shs"])
    S = oracle.state(s, st, sc["n"])
    B = None
    if backward:
        B = oracle.backward(s, st, 16, A["means_3d"], A["scales"], A["rotations"], A["opacities"], A["v_image"])
        # atomics reorder the per-Gaussian sums: every gradient element gets its own tolerance, 1e-4 of
        # the summed magnitudes of the terms it is made of (no tensor-wide floor; measured errors stay
        # below 1e-5 of that figure)
        B["bounds"] = oracle.gradient_bounds(s, 16, A["means_3d"], A["scales"], A["rotations"], S["conic"],
                                             S["cov3d"], radii, B["abs_sums"], rel=1e-4)
    oracle.free(st)
    return img, radii, S, B


def gpu_forward_state(sc, scale_mul=1.0):
    """final_T and final_idx of the GPU's forward (numpy): where they differ from the oracle's, a
    borderline decision went the other way and the pixel's tile list is not compared."""
    from ds_splat_amd import stages
    cam = stages.camera_from_scene(sc, DEV)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    _, st = stages.forward(cam, t["means_3d"], t["scales"] * scale_mul, t["rotations"], t["opacities"], t["shs"])
    torch.cuda.synchronize()
    return st.final_T.cpu().numpy(), st.final_idx.cpu().numpy(), st


def check_grads(leaves, B, ok, what=""):
    got = {key: leaves[leaf].grad.cpu().numpy() for leaf, key in GRAD_KEYS}
    worst = check_grads_against_bounds(got, B, B["bounds"], ok, what)
    moved = B["abs_sums"].sum(axis=1) > 0      # Gaussians that receive any gradient term
    print("%s: gradients of %d of %d Gaussians compared (%.1f %%), of the %d that receive a term %d (%.1f %%); "
          "largest error / bound = %.3f" % (what, int(ok.sum()), ok.size, 100.0 * ok.mean(), int(moved.sum()),
                                            int((ok & moved).sum()), 100.0 * (ok & moved).sum() / max(1, moved.sum()),
                                            worst))
    return worst


# (bins: tiles per side of the bins the tile lists are built for; 0 = the library's choice by image size)
@pytest.mark.parametrize("name,n,W,H,deg,scale_mul,bg,camera,bins", [
    ("cfg0", 16384, 256, 256, 0, 1.0, None, "identity", 0),            # workload cfg0 at full size
    ("cfg0", 16384, 256, 256, 3, 2.0, (0.2, 0.4, 0.9), "identity", 1),
    ("cfg1", 40000, 480, 270, 3, 1.0, None, "identity", 4),            # config 1 distributions, reduced size
    ("cfg4", 3000, 320, 180, 3, 0.5, None, "identity", 2),             # heavy-overlap distributions, reduced size
    ("cfg2", 30000, 333, 177, 2, 1.5, None, "identity", 4),            # ragged image (not a multiple of 16)
    # general cameras: rotated + translated (campos != 0 matters at SH degree 3), a camera inside the
    # cloud (Gaussians behind it) with scale modifier 1.3, non-square pixels with scale modifier 0.7
    ("cfg0", 16384, 256, 256, 3, 2.0, (0.2, 0.4, 0.9), "rotated", 2),
    ("cfg0", 20000, 320, 200, 3, 2.0, None, "inside", 4),
    ("cfg1", 40000, 480, 270, 3, 1.5, (0.5, 0.1, 0.3), "anisotropic", 1),
    ("cfg4", 3000, 320, 180, 2, 0.5, None, "rotated", 8),
    ("cfg1", 40000, 640, 360, 3, 2.0, (0.3, 0.3, 0.3), "inside", 8),
    ("cfg1", 40000, 1000, 520, 3, 2.0, (0.1, 0.2, 0.3), "rotated", 0),  # 63 x 33 tiles: ragged against the bins
])
@pytest.mark.parametrize("pixels_per_lane", ["1", "4"])
def test_api_forward_backward_vs_oracle(oracle, name, n, W, H, deg, scale_mul, bg, camera, bins, pixels_per_lane,
                                        blend_form, list_bin):
    # both forms of the blend kernels, whatever the image size would pick
    blend_form(pixels_per_lane)
    list_bin(bins)
    sc = set_camera(make_scene(name, n=n, width=W, height=H, sh_degree=deg), camera)
    image, radii, leaves = api_run(sc, scale_mul, bg=bg)
    img_o, radii_o, S, B = oracle_run(oracle, sc, scale_mul, bg=bg)
    assert image.shape == (H, W, 3) and radii.dtype == torch.int32 and radii.shape == (n,)
    assert (radii.cpu().numpy() == radii_o).all()
    assert (radii_o > 0).sum() > n // 20
    ok = S["margin"] > 1e-4
    assert ok.mean() > 0.98, ok.mean()
    np.testing.assert_allclose(image.detach().cpu().numpy()[ok], img_o[ok], rtol=1e-4, atol=1e-5)
    T_gpu, idx_gpu, _ = gpu_forward_state(sc, scale_mul)
    # final_idx holds the reference's indices whatever the bin size of the lists
    assert (idx_gpu[ok] == S["final_idx"][ok]).all()
    # the two forwards disagree on a pixel's walk only where a decision was borderline
    assert (S["margin"][(T_gpu != S["final_T"]) & ~np.isclose(T_gpu, S["final_T"], rtol=1e-4, atol=0)] < 1e-4).all()
    gok = comparable_gaussians(S, B, W, T_gpu, idx_gpu)
    assert gok.mean() > 0.9, gok.mean()
    check_grads(leaves, B, gok, "%s %s" % (name, camera))
    assert leaves["opac"].grad.shape == leaves["opac"].shape
    assert (leaves["means2d"].grad[:, 2] == 0).all()


@pytest.mark.parametrize("bins", [1, 2, 4, 8])
def test_api_internal_integers_bit_exact(oracle, list_bin, bins):
    """Tile ranges, tile counts, radii and last blended index of the whole forward, bit for bit,
    whatever the bin size of the lists; with one list per tile also the sorted order itself
    (stable tie-break) and the number of keys."""
    from ds_splat_amd import stages
    list_bin(bins)
    sc = make_scene("cfg1", n=50000, width=640, height=360, sh_degree=1)
    cam = stages.camera_from_scene(sc, DEV)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    image, st = stages.forward(cam, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["opacities"], t["shs"])
    torch.cuda.synchronize()
    img_o, radii_o, S, _ = oracle_run(oracle, sc, 2.0, backward=False)
    assert S["num_keys"] > 100000
    if bins == 1:
        assert st.num_keys == S["num_keys"]
        assert (st.sorted_ids.cpu().numpy() == S["sorted_ids"]).all()
    else:
        assert 0 < st.num_keys < S["num_keys"] // 2
    assert (st.ranges.cpu().numpy() == S["ranges"]).all()
    assert (st.radii.cpu().numpy() == radii_o).all()
    sp = st.splats.cpu().numpy()
    assert (sp[:, 11].view(np.int32) == S["tiles_touched"]).all()
    ok = S["margin"] > 1e-4
    assert (st.final_idx.cpu().numpy()[ok] == S["final_idx"][ok]).all()


def test_api_opacity_as_vector_and_empty_scene(oracle):
    sc = make_scene("cfg0", n=2000, width=64, height=64, sh_degree=1)
    image, radii, leaves = api_run(sc, 3.0, opac_shape=(2000,))
    assert leaves["opac"].grad.shape == (2000,)
    # everything behind / outside: K = 0, image must be all zeros and backward all zeros
    sc2 = make_scene("cfg0", n=500, width=64, height=64, sh_degree=0)
    sc2["means_3d"][:, 0] += 1000.0
    image, radii, leaves = api_run(sc2)
    assert (image == 0).all() and (radii == 0).all()
    for v in leaves.values():
        assert (v.grad == 0).all()


def test_api_on_a_side_stream_matches_the_default_stream():
    """Every launch and the key-count copy go to torch's current stream: the result on a side
    stream (default priority) equals the one on the default stream bit for bit in the forward
    and within atomic reordering in the backward."""
    sc = make_scene("cfg1", n=20000, width=320, height=200, sh_degree=3)
    image0, radii0, leaves0 = api_run(sc, 2.0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        image1, radii1, leaves1 = api_run(sc, 2.0)
    side.synchronize()
    assert torch.equal(image0, image1) and torch.equal(radii0, radii1)
    for k in leaves0:
        a, b = leaves0[k].grad, leaves1[k].grad
        assert torch.allclose(a, b, rtol=1e-3, atol=1e-4 * max(1.0, float(a.abs().max())))


def test_only_the_gradients_asked_for_are_produced():
    """Inputs that take no gradient get none, and the others get what they get when every input
    takes one (the kernel skips the stores of unwanted outputs, nothing else changes)."""
    sc = make_scene("cfg1", n=20000, width=320, height=200, sh_degree=3)
    _, _, full = api_run(sc, 2.0)
    for wants in (("shs", "opac"), ("means", "scales", "rots"), ("means2d",)):
        _, _, part = api_run(sc, 2.0, wants=wants)
        for k in full:
            if k not in wants:
                assert part[k].grad is None, k
                continue
            a, b = full[k].grad, part[k].grad
            assert torch.allclose(a, b, rtol=1e-3, atol=1e-4 * max(1.0, float(a.abs().max()))), k
            assert float(b.abs().max()) > 0 or k == "means2d"


@pytest.mark.parametrize("pixels_per_lane", ["1", "4"])
@pytest.mark.parametrize("n", [20000, 20001])
def test_forward_prepares_the_accumulator_for_one_backward(blend_form, pixels_per_lane, n):
    """With prepare_grads the blend forward prepares the backward's accumulator on the side (both kernel
    forms, a Gaussian count that does and does not divide by the wavefronts' shares); a backward on
    it equals one that fills for itself, and a second backward on the same state fills again."""
    from ds_splat_amd import stages
    blend_form(pixels_per_lane)
    sc = make_scene("cfg1", n=n, width=320, height=200, sh_degree=3)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    cam = stages.camera_from_scene(sc, DEV)
    args = (t["means_3d"], t["scales"] * 2.0, t["rotations"], t["opacities"], t["shs"])
    image0, st0 = stages.forward(cam, *args)
    poison = torch.full((n, 12), float("nan"), device=DEV)      # the allocator hands this block out again
    del poison
    image1, st1 = stages.forward(cam, *args, prepare_grads=True)
    torch.cuda.synchronize()
    # nine sums zeroed, the conic (floats 4..6 of the splat record) in the three spare places
    records, marks = stages.accumulator_views(st1.grads, n)
    assert st0.grads is None and bool((records[:, :9] == 0).all()) and bool((marks == 0).all())
    assert torch.equal(records[:, 9:12], st1.splats[:, 4:7])
    assert torch.equal(image0, image1)
    bwd = lambda st: stages.backward(cam, st, 16, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["v_image"])
    o0, o1 = bwd(st0), bwd(st1)
    assert st1.grads is None
    o2 = bwd(st1)
    torch.cuda.synchronize()
    for k in o0:
        if k == "marks":
            continue
        cols = slice(0, 9) if k == "grads" else slice(None)   # the accumulator's spare places are not sums
        scale = max(1.0, float(o0[k].abs().max()))
        for other in (o1, o2):
            assert torch.allclose(o0[k][:, cols], other[k][:, cols], rtol=1e-3, atol=1e-4 * scale), k
    # the byte per Gaussian: set wherever a sum is, the same set every time, and some but not all
    for o in (o0, o1, o2):
        unmarked = o["marks"] == 0
        assert bool((o["grads"][unmarked][:, :9] == 0).all()) and torch.equal(o["marks"], o0["marks"])
        assert 0 < int(unmarked.sum()) < n
        for k in ("v_mean3d", "v_shs", "v_scale", "v_quat", "v_opacity"):
            assert bool((o[k][unmarked] == 0).all()), k


def test_backward_takes_ids_only_up_to_the_last_gaussian():
    """The blend kernels gather splat records at the ids they find in the lists.  Lists in disorder
    (a sort that gave up its bounded wait, a caller that handed the backward another forward's ids)
    must give wrong numbers, not a fetch outside the records: every id is clamped to n - 1.  Here a
    backward runs on lists in which every fifth id has been replaced by a value far outside."""
    from ds_splat_amd import stages
    n = 20000
    sc = make_scene("cfg1", n=n, width=320, height=200, sh_degree=3)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    cam = stages.camera_from_scene(sc, DEV)
    args = (t["means_3d"], t["scales"] * 2.0, t["rotations"], t["opacities"], t["shs"])
    _, st = stages.forward(cam, *args)
    bad = torch.tensor([0x7fffffff, -1, n, 1 << 30, -(1 << 31)], dtype=torch.int32, device=DEV)
    st.ids[::5] = bad[torch.arange(st.ids[::5].numel(), device=DEV) % 5]
    o = stages.backward(cam, st, 16, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["v_image"])
    torch.cuda.synchronize()
    # the replaced entries all read as Gaussian n - 1: it is marked, and nothing outside the arrays was touched
    assert int(o["marks"][n - 1]) == 1 and bool(torch.isfinite(o["v_opacity"]).all())


def test_backward_twice_through_the_api_gives_the_same_gradients():
    """retain_graph: the second backward finds the accumulator used and clears it for itself."""
    from ds_splat import GaussianRasterizationSettings, GaussianRasterizer
    sc = make_scene("cfg1", n=20000, width=320, height=200, sh_degree=3)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    settings = GaussianRasterizationSettings(
        image_height=sc["height"], image_width=sc["width"], tanfovx=sc["tanfovx"], tanfovy=sc["tanfovy"], bg=t["bg"],
        scale_modifier=1.0, viewmatrix=t["viewmatrix"], projmatrix=t["projmatrix"], sh_degree=sc["sh_degree"],
        max_sh_degree=3, campos=t["campos"], prefiltered=False, debug=False)
    means = t["means_3d"].clone().requires_grad_(True)
    shs = t["shs"].clone().requires_grad_(True)
    image, _ = GaussianRasterizer(settings)(means, torch.zeros_like(means), shs, None, t["opacities"],
                                            t["scales"] * 2.0, t["rotations"], None)
    image.backward(t["v_image"], retain_graph=True)
    first = (means.grad.clone(), shs.grad.clone())
    means.grad = None
    shs.grad = None
    image.backward(t["v_image"])
    torch.cuda.synchronize()
    for a, b in zip(first, (means.grad, shs.grad)):
        assert float(a.abs().max()) > 0
        assert torch.allclose(a, b, rtol=1e-3, atol=1e-4 * max(1.0, float(a.abs().max())))


def test_inria_adaptor_composites_the_background_and_keeps_the_gradients(oracle):
    """Channel-first image = the oracle's image + the oracle's final_T * bg (the reference's forward leaves the
    background out, cpp/rasterizer_kernels.cu:417-422, and its backward differentiates exactly that
    product); gradients against the oracle's backward with the same background, and equal to those of the
    wrapped API for the same upstream gradient."""
    from ds_splat_amd import inria_compat, stages
    sc = make_scene("cfg1", n=20000, width=320, height=200, sh_degree=3)
    bg = (0.3, 0.6, 0.1)
    image, radii, leaves = api_run(sc, 2.0, bg=bg)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    settings = inria_compat.GaussianRasterizationSettings(
        image_height=sc["height"], image_width=sc["width"], tanfovx=sc["tanfovx"], tanfovy=sc["tanfovy"],
        bg=torch.tensor(bg, dtype=torch.float32, device=DEV), scale_modifier=1.0, viewmatrix=t["viewmatrix"],
        projmatrix=t["projmatrix"], sh_degree=sc["sh_degree"], campos=t["campos"])
    p = dict(means=t["means_3d"].clone().requires_grad_(True), shs=t["shs"].clone().requires_grad_(True),
             opac=t["opacities"].clone().requires_grad_(True), scales=(t["scales"] * 2.0).clone().requires_grad_(True),
             rots=t["rotations"].clone().requires_grad_(True))
    color, radii2 = inria_compat.GaussianRasterizer(settings)(
        means3D=p["means"], means2D=torch.zeros_like(p["means"]), opacities=p["opac"], shs=p["shs"],
        scales=p["scales"], rotations=p["rots"])
    assert color.shape == (3, sc["height"], sc["width"]) and torch.equal(radii, radii2)
    cam = stages.camera_from_scene(sc, DEV, bg=torch.tensor(bg))
    _, st = stages.forward(cam, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["opacities"], t["shs"])
    want = image.detach() + st.final_T.unsqueeze(-1) * torch.tensor(bg, device=DEV).view(1, 1, 3)
    assert torch.allclose(color.detach().permute(1, 2, 0), want, rtol=0, atol=1e-6)
    assert (st.final_T > 0.5).any() and float((color.detach().permute(1, 2, 0) - image.detach()).abs().max()) > 0.05
    # against the CPU oracle: its image and final_T, composited here
    img_o, radii_o, S, B = oracle_run(oracle, sc, 2.0, bg=np.asarray(bg, np.float32))
    assert (radii2.cpu().numpy() == radii_o).all()
    ok = S["margin"] > 1e-4
    assert ok.mean() > 0.98
    want_o = img_o + S["final_T"][..., None] * np.asarray(bg, np.float32).reshape(1, 1, 3)
    got = color.detach().permute(1, 2, 0).cpu().numpy()
    np.testing.assert_allclose(got[ok], want_o[ok], rtol=1e-4, atol=1e-5)
    assert float(np.abs(want_o - img_o)[ok].max()) > 0.05          # the background does show
    color.backward(t["v_image"].permute(2, 0, 1))
    torch.cuda.synchronize()
    fT, fidx, _ = gpu_forward_state(sc, 2.0)
    gok = comparable_gaussians(S, B, sc["width"], fT, fidx)
    got_grads = {"v_mean3d": p["means"].grad, "v_shs": p["shs"].grad, "v_opacity": p["opac"].grad,
                 "v_scale": p["scales"].grad, "v_quat": p["rots"].grad}
    check_grads_against_bounds({k: v.cpu().numpy() for k, v in got_grads.items()}, B, B["bounds"], gok,
                               "inria adaptor")
    for k in p:
        a, b = leaves[k].grad, p[k].grad
        assert torch.allclose(a, b, rtol=1e-3, atol=1e-4 * max(1.0, float(a.abs().max()))), k


def test_api_precomputed_colors_and_cov3d(oracle):
    sc = make_scene("cfg0", n=5000, width=128, height=96, sh_degree=2)
    A = arrays(sc)
    s = scene_settings(sc)
    base = oracle.project_fwd(s, A["means_3d"], A["scales"] * 2, A["rotations"], A["shs"])
    cols = torch.rand(5000, 3, generator=torch.Generator().manual_seed(1))
    img_o, radii_o, st = oracle.forward(s, A["means_3d"], A["scales"] * 2, A["rotations"], A["opacities"], A["shs"],
                                        colors_precomp=cols.numpy())
    S = oracle.state(s, st, 5000)
    oracle.free(st)
    image, radii, _ = api_run(sc, 2.0, backward=False, colors=cols.to(DEV))
    ok = S["margin"] > 1e-4
    np.testing.assert_allclose(image.cpu().numpy()[ok], img_o[ok], rtol=1e-4, atol=1e-5)
    # cov3D_precomp path renders the same image as scales+rotations
    img_a, radii_a, _ = api_run(sc, 2.0, backward=False)
    img_b, radii_b, _ = api_run(sc, 2.0, backward=False, cov3d=torch.from_numpy(base["cov3d"]).to(DEV))
    assert (radii_a == radii_b).all() and torch.equal(img_a, img_b)


def test_api_backward_with_precomputed_inputs():
    """Gradients on the optional-input paths: cov3D_precomp takes v_cov3d (and the backward reads the
    covariances that were passed in, not rebuilt ones), colors_precomp takes the colour sums; the
    other gradients equal those of the scales + rotations + SH run, which the oracle tests pin."""
    from ds_splat_amd import stages
    sc = make_scene("cfg0", n=5000, width=128, height=96, sh_degree=2)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    cam = stages.camera_from_scene(sc, DEV)
    _, st = stages.forward(cam, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["opacities"], t["shs"])
    o = stages.backward(cam, st, 16, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["v_image"])
    torch.cuda.synchronize()
    close = lambda a, b: torch.allclose(a, b.reshape(a.shape), rtol=1e-3, atol=1e-4 * max(1.0, float(b.abs().max())))

    cov = st.cov3d.clone().requires_grad_(True)
    _, _, leaves = api_run(sc, 2.0, cov3d=cov)
    assert float(o["v_cov3d"].abs().max()) > 0 and close(cov.grad, o["v_cov3d"])
    assert close(leaves["means"].grad, o["v_mean3d"]) and close(leaves["shs"].grad, o["v_shs"])
    assert close(leaves["opac"].grad, o["v_opacity"])
    assert leaves["scales"].grad is None and leaves["rots"].grad is None

    cols = st.splats[:, 8:11].clone().requires_grad_(True)      # the colours the SH run blended with
    image_c, _, leaves = api_run(sc, 2.0, colors=cols)
    assert float(o["v_colors"].abs().max()) > 0 and close(cols.grad, o["v_colors"])
    assert close(leaves["means"].grad, o["v_mean3d"]) and close(leaves["scales"].grad, o["v_scale"])
    assert close(leaves["rots"].grad, o["v_quat"]) and leaves["shs"].grad is None


def test_forward_core_raw_pointer_entry(oracle):
    """dsx_forward_core: device pointers in, image out (the reference's torch-free entry)."""
    import ctypes as C
    from ds_splat_amd import _native
    lib = _native.load()
    sc = make_scene("cfg0", n=8000, width=160, height=128, sh_degree=3)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    view = t["viewmatrix"].t().contiguous()
    proj = t["projmatrix"].t().contiguous()
    image = torch.empty(128, 160, 3, device=DEV)
    p = lambda x: C.c_void_p(x.data_ptr())
    rc = lib.dsx_forward_core(p(t["means_3d"]), p(t["shs"]), p(t["opacities"]), p(t["scales"]), p(t["rotations"]),
                              8000, p(view), p(proj), p(t["campos"]), 160, 128, sc["tanfovx"], sc["tanfovy"], 1.0, 3,
                              3, p(image), C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    img_o, _, S, _ = oracle_run(oracle, sc, backward=False)
    ok = S["margin"] > 1e-4
    np.testing.assert_allclose(image.cpu().numpy()[ok], img_o[ok], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("name,n,W,H,scale_mul", [
    ("cfg3", 200_000, 7680, 4320, 1.0),     # 129600 tiles: 32-bit slots, 3 partition passes, corner grid in global memory
    ("cfg1", 300, 8000, 8000, 30.0),        # 250000 tiles, rectangles of thousands of tiles
    ("cfg2", 300, 16, 16, 1.0),             # one tile
    ("cfg4", 100_000, 1920, 1080, 1.0),     # ~850 tiles per Gaussian
])
def test_forward_lists_equal_the_64_bit_route(list_bin, name, n, W, H, scale_mul):
    """The whole forward's sorted ids and ranges (depth order + tile partition, one list per tile)
    against the reference-shaped route (64-bit keys, radix sort, ranges from keys) at shapes the
    oracle is too slow for."""
    from ds_splat_amd import stages
    list_bin(1)
    sc = make_scene(name, n=n, width=W, height=H)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    cam = stages.camera_from_scene(sc, DEV)
    img, st = stages.forward(cam, t["means_3d"], t["scales"] * scale_mul, t["rotations"], t["opacities"], t["shs"])
    k = st.num_keys
    tiles = st.splats[:, 11].view(torch.int32).to(torch.int64).clone()
    tiles[-1] = 0
    assert k == int(tiles.sum().item()) > 0
    block_sums = torch.cat([tiles, torch.zeros((-n) % 256, dtype=torch.int64, device=DEV)]).view(-1, 256).sum(1)
    block_sums = block_sums.to(torch.int32)
    stages.scan_u32(block_sums)
    keys, vals = stages.emit_keys(cam, n, k, st.splats, block_sums)
    stages.sort_pairs(keys, vals, cam.num_tiles)
    ranges = stages.tile_ranges(keys, cam.num_tiles)
    assert torch.equal(vals, st.sorted_ids) and torch.equal(ranges, st.ranges)
    assert torch.isfinite(img).all()


# ------------------------------------------------------------------------- properties at full size
def test_full_size_properties_cfg2(list_bin):
    """3M Gaussians, 1920x1080, SH3 (the headline shape): properties that need no oracle (one list per tile)."""
    from ds_splat_amd import stages
    list_bin(1)
    sc = make_scene("cfg2")
    n = sc["n"]
    cam = stages.camera_from_scene(sc, DEV)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    order = stages.new_order(cam, n, DEV)
    splats, radii, cov3d, block_sums = stages.project_fwd(cam, t["means_3d"], t["scales"], t["rotations"],
                                                          t["opacities"], t["shs"], order=order)
    tiles = splats[:, 11].view(torch.int32).to(torch.int64)
    tiles_eff = tiles.clone()
    tiles_eff[-1] = 0
    total = stages.scan_u32(block_sums)
    k = int(total.item())
    assert k == int(tiles_eff.sum().item()) and k > 10_000_000
    assert ((radii > 0) == (tiles > 0)).all() or ((radii > 0) | (tiles == 0)).all()
    keys, vals = stages.emit_keys(cam, n, k, splats, block_sums)
    # every Gaussian appears exactly tiles_touched times, keys carry its depth bits
    counts = torch.bincount(vals.to(torch.int64), minlength=n)
    assert torch.equal(counts, tiles_eff)
    depth_bits = splats[:, 2].view(torch.int32).to(torch.int64)
    assert torch.equal(keys & 0xFFFFFFFF, depth_bits[vals.to(torch.int64)])
    checksum = int(keys.sum().item()) ^ int(vals.to(torch.int64).sum().item())
    stages.sort_pairs(keys, vals, cam.num_tiles)
    assert int(keys.sum().item()) ^ int(vals.to(torch.int64).sum().item()) == checksum   # a permutation
    assert (keys[1:] >= keys[:-1]).all()                                                   # sorted
    same = keys[1:] == keys[:-1]
    assert (vals[1:][same] > vals[:-1][same]).all()                                        # stable tie-break
    assert torch.equal(keys & 0xFFFFFFFF, depth_bits[vals.to(torch.int64)])                # pairs stay together
    ranges = stages.tile_ranges(keys, cam.num_tiles)
    assert (ranges[1:] >= ranges[:-1]).all() and int(ranges[-1]) == k and int(ranges[0]) == 0
    # the fast route (depth order of the Gaussians, ordered emission, tile partition) gives the
    # same lists as the 64-bit sort of all keys
    perm, offsets = stages.depth_order(cam, n, order)
    assert int(offsets[-1]) == k
    # unsigned order of the depth bits; Gaussians that emit nothing come last (all-ones key)
    sort_key = torch.where(tiles_eff > 0, depth_bits & 0xFFFFFFFF, torch.full_like(depth_bits, 0xFFFFFFFF))
    d_sorted = sort_key[perm.to(torch.int64)]
    assert (d_sorted[1:] >= d_sorted[:-1]).all()
    ids_fast, ranges_fast, flags = stages.tile_lists(cam, n, k, order, return_flags=True)
    assert flags == (0, 0)
    assert torch.equal(ids_fast, vals) and torch.equal(ranges_fast, ranges)
    del ids_fast, ranges_fast, perm, offsets, d_sorted
    tile_of = (keys >> 32).to(torch.int64)
    r = ranges.to(torch.int64)
    t_last = int(tile_of[-1])
    probe = torch.randint(0, t_last, (2000,), device=DEV)
    for tt in probe.tolist()[:200]:
        seg = tile_of[int(r[tt]):int(r[tt + 1])]
        assert (seg == tt).all()
    image, final_T, final_idx = stages.blend_fwd(cam, ranges, vals, splats)
    assert torch.isfinite(image).all() and (image >= 0).all()
    assert (final_T <= 1).all() and (final_T >= 9.9e-5).all()
    # all-white scene: image telescopes to 1 - final_T in every channel
    white = splats.clone()
    white[:, 8:11] = 1.0
    img_w, T_w, _ = stages.blend_fwd(cam, ranges, vals, white)
    assert torch.allclose(img_w, (1 - T_w).unsqueeze(-1).expand(-1, -1, 3), rtol=0, atol=2e-5)
    assert torch.equal(T_w, final_T)
    # determinism of the forward, linearity of the backward in the upstream gradient
    image2, _, _ = stages.blend_fwd(cam, ranges, vals, splats)
    assert torch.equal(image, image2)
    g1 = stages.blend_bwd(cam, n, ranges, vals, splats, final_T, final_idx, t["v_image"])
    g2 = stages.blend_bwd(cam, n, ranges, vals, splats, final_T, final_idx, 2.0 * t["v_image"])
    assert torch.allclose(g2, 2.0 * g1, rtol=2e-3, atol=2e-3 * float(g1.abs().max()))
    # v_rgb of a Gaussian nobody blended is zero; gradient of culled Gaussians is zero
    assert (g1[radii <= 0] == 0).all()
    o = stages.gaussian_bwd(cam, 16, t["means_3d"], t["scales"], t["rotations"], splats, cov3d, radii, g1)
    for key in ("v_mean3d", "v_scale", "v_quat", "v_cov3d", "v_shs"):
        assert torch.isfinite(o[key]).all()
        assert (o[key][radii <= 0] == 0).all()


def test_full_size_properties_cfg4_heavy_overlap(list_bin):
    """The heavy-overlap shape at full size (1 M large Gaussians, 1080p, K = 858 M pairs: too many for
    the 64-bit route's buffers and for the CPU oracle in a test): what the lists must satisfy
    whatever their size.  K equals the sum of the tile counts; every Gaussian appears exactly
    tiles_touched times; the ranges partition [0, K); inside a tile the pairs are ordered by
    (depth bits, Gaussian index); every pair of a tile's list covers that tile; the image of an
    all-white scene telescopes to 1 - final_T; forward and backward outputs are finite.  (One list per tile.)"""
    from ds_splat_amd import stages
    list_bin(1)
    sc = make_scene("cfg4")
    n = sc["n"]
    cam = stages.camera_from_scene(sc, DEV)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    image, st = stages.forward(cam, t["means_3d"], t["scales"], t["rotations"], t["opacities"], t["shs"],
                               prepare_grads=True)
    torch.cuda.synchronize()
    k = st.num_keys
    tiles = st.splats[:, 11].view(torch.int32).to(torch.int64)
    tiles[-1] = 0                                                    # the last Gaussian never emits
    assert k == int(tiles.sum().item()) and k > 500_000_000
    ids = st.sorted_ids.to(torch.int64)
    assert int(ids.min()) >= 0 and int(ids.max()) < n
    assert torch.equal(torch.bincount(ids, minlength=n), tiles)
    r = st.ranges.to(torch.int64)
    assert int(r[0]) == 0 and int(r[-1]) == k and bool((r[1:] >= r[:-1]).all())
    # (tile, depth bits) never decreases along the whole array; equal keys keep ascending indices
    tile_of = torch.repeat_interleave(torch.arange(cam.num_tiles, device=DEV), r[1:] - r[:-1])
    assert tile_of.numel() == k
    depth_bits = st.splats[:, 2].view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    key = (tile_of << 32) | depth_bits[ids]
    assert bool((key[1:] >= key[:-1]).all())
    same = key[1:] == key[:-1]
    assert bool((ids[1:][same] > ids[:-1][same]).all())
    del key, same
    # each pair's tile lies inside its Gaussian's rectangle (recomputed from centre and radius as the
    # reference does: truncation, +1 on the upper bound, clamped to the grid)
    ntx, nty = (cam.width + 15) // 16, (cam.height + 15) // 16
    cx, cy, d = st.splats[:, 0] / 16, st.splats[:, 1] / 16, st.radii.to(torch.float32) / 16
    sx = (cx - d).to(torch.int32).clamp(0, ntx)          # cpp/rasterizer_kernels.cu:239-247
    ex = (cx + d + 1).to(torch.int32).clamp(0, ntx)
    sy = (cy - d).to(torch.int32).clamp(0, nty)
    ey = (cy + d + 1).to(torch.int32).clamp(0, nty)
    assert torch.equal(((ex - sx) * (ey - sy)).to(torch.int64)[:-1] * (st.radii[:-1] > 0), tiles[:-1])
    step = 997                                                       # a sample of the pairs
    tt, gg = tile_of[::step], ids[::step]
    tx, ty = (tt % ntx).to(torch.int32), (tt // ntx).to(torch.int32)
    assert bool(((tx >= sx[gg]) & (tx < ex[gg]) & (ty >= sy[gg]) & (ty < ey[gg])).all())
    del tile_of, ids, tt, gg
    assert bool(torch.isfinite(image).all()) and bool((image >= 0).all())
    assert bool((st.final_T <= 1).all()) and bool((st.final_T >= 9.9e-5).all())
    white = st.splats.clone()
    white[:, 8:11] = 1.0
    img_w, T_w, _ = stages.blend_fwd(cam, st.ranges, st.sorted_ids, white)
    assert torch.allclose(img_w, (1 - T_w).unsqueeze(-1).expand(-1, -1, 3), rtol=0, atol=2e-5)
    assert torch.equal(T_w, st.final_T)
    o = stages.backward(cam, st, 16, t["means_3d"], t["scales"], t["rotations"], t["v_image"])
    torch.cuda.synchronize()
    for name in ("v_mean3d", "v_means2d", "v_shs", "v_opacity", "v_scale", "v_quat"):
        assert bool(torch.isfinite(o[name]).all()), name
        assert bool((o[name][st.radii <= 0] == 0).all()), name
    assert float(o["v_shs"].abs().max()) > 0


# share of the VISIBLE Gaussians whose gradients must be comparable at full size (the rest can be
# reached by a pixel with a borderline forward decision; more of them where lists are long)
GRADS_COMPARED_FLOOR = {"cfg1": 0.5, "cfg2": 0.5, "cfg4": 0.05, "dense": 0.05}


@pytest.mark.parametrize("workload", ["cfg1", "cfg2", "cfg4", "dense"])
def test_full_size_against_the_openmp_oracle(workload, list_bin):
    """The forward+backward shapes at full size (500 K Gaussians, the headline 3 M, the heavy-overlap
    1 M with its 858 M pairs, and the 2 M faint Gaussians of "dense", where every pixel walks its
    whole list, 5.5 G pixel-pairs, and every visible Gaussian receives a gradient; 1920x1080, SH3)
    against the oracle's OpenMP build (same source as the serial oracle, loops over Gaussians and
    tiles in parallel): integers, every sorted id included, bit for bit, image rtol 1e-4 / atol 1e-5
    and gradients within 1e-4 of the summed magnitudes of their terms, away from threshold decisions."""
    from oracle.binding import Oracle
    from ds_splat_amd import stages
    omp = Oracle(omp=True)
    sc = make_scene(workload)
    image, radii, leaves = api_run(sc)
    img_o, radii_o, S, B = oracle_run(omp, sc)
    assert (radii.cpu().numpy() == radii_o).all()
    ok = S["margin"] > 1e-4
    visible = radii_o > 0
    T_gpu, idx_gpu, st = gpu_forward_state(sc)
    gok = comparable_gaussians(S, B, sc["width"], T_gpu, idx_gpu)
    print("%s: %.2f %% of the pixels compared; %d Gaussians visible" % (workload, 100.0 * ok.mean(), int(visible.sum())))
    assert ok.mean() > 0.97, ok.mean()
    np.testing.assert_allclose(image.detach().cpu().numpy()[ok], img_o[ok], rtol=1e-4, atol=1e-5)
    check_grads(leaves, B, gok, workload)
    # the culled Gaussians compare trivially (all zeros): the floor is on the visible ones
    assert gok[visible].mean() > GRADS_COMPARED_FLOOR[workload], gok[visible].mean()
    if workload == "dense":
        # what the workload is for: the walks are deep and the gradients dense
        c = B["counters"]
        walked = c.pairs_fwd / (256.0 * np.diff(S["ranges"][:8161].astype(np.int64)).sum())
        moved = (B["abs_sums"].sum(axis=1) > 0).sum()
        print("dense: pixels walk %.1f %% of their tile's list, %d of %d visible Gaussians receive a gradient" % (
            100 * walked, moved, visible.sum()))
        assert walked > 0.8 and moved > 0.5 * visible.sum()
    del image, leaves
    # the API ran with the library's own bin size for the lists: ranges and last blended indices
    # are the reference's whatever that is ...
    assert (st.ranges.cpu().numpy() == S["ranges"]).all()
    assert (st.final_idx.cpu().numpy()[ok] == S["final_idx"][ok]).all()
    print("%s: lists of %d x %d tiles, %d pairs instead of %d" % (
        workload, stages.list_bin(stages.camera_from_scene(sc, DEV)), stages.list_bin(stages.camera_from_scene(sc, DEV)),
        st.num_keys, S["num_keys"]))
    del st
    # ... and with one list per tile the sorted order itself is the reference's
    list_bin(1)
    _, _, st = gpu_forward_state(sc)
    assert st.num_keys == S["num_keys"]
    assert (st.ranges.cpu().numpy() == S["ranges"]).all()
    assert (st.sorted_ids.cpu().numpy() == S["sorted_ids"]).all()
    assert (st.final_idx.cpu().numpy()[ok] == S["final_idx"][ok]).all()


@pytest.mark.parametrize("bins", [1, 0])
def test_full_size_forward_cfg3_4k(list_bin, bins):
    """6M Gaussians at 3840x2160 (forward only): runs, sorted, deterministic, and equal to the
    oracle's OpenMP build: radii, ranges (and, with one list per tile, the key count and the 36 M
    sorted ids) bit for bit, the image rtol 1e-4 / atol 1e-5 away from threshold decisions."""
    from oracle.binding import Oracle
    from ds_splat_amd import stages
    list_bin(bins)
    sc = make_scene("cfg3")
    cam = stages.camera_from_scene(sc, DEV)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    image, st = stages.forward(cam, t["means_3d"], t["scales"], t["rotations"], t["opacities"], t["shs"])
    image2, st2 = stages.forward(cam, t["means_3d"], t["scales"], t["rotations"], t["opacities"], t["shs"])
    torch.cuda.synchronize()
    assert st.num_keys == st2.num_keys > 1_000_000
    assert torch.equal(st.sorted_ids, st2.sorted_ids) and torch.equal(image, image2)
    assert (st.ranges[1:] >= st.ranges[:-1]).all() and (bins != 1 or int(st.ranges[-1]) == st.num_keys)
    assert torch.isfinite(image).all()
    del image2, st2
    img_o, radii_o, S, _ = oracle_run(Oracle(omp=True), sc, backward=False)
    assert (st.radii.cpu().numpy() == radii_o).all()
    assert (st.ranges.cpu().numpy() == S["ranges"]).all()
    if bins == 1:
        assert st.num_keys == S["num_keys"]
        assert (st.sorted_ids.cpu().numpy() == S["sorted_ids"]).all()
    ok = S["margin"] > 1e-4
    assert (st.final_idx.cpu().numpy()[ok] == S["final_idx"][ok]).all()
    assert ok.mean() > 0.97
    np.testing.assert_allclose(image.cpu().numpy()[ok], img_o[ok], rtol=1e-4, atol=1e-5)


def test_a_sort_that_gave_up_poisons_the_image():
    """The chained scans wait for their predecessors a bounded number of times and set a flag if
    they give up (never observed).  Force the depth sort's flag from the host between the two
    halves of the forward: the image must come back NaN, not plausible."""
    from ds_splat_amd import stages
    sc = make_scene("cfg1", n=5000, width=160, height=96, sh_degree=1)
    cam = stages.camera_from_scene(sc, DEV)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    args = (cam, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["opacities"], t["shs"])
    image, st = stages.forward(*args)
    assert torch.isfinite(image).all() and st.num_keys > 0

    def poke(order, n, k):
        ia, _ = stages.sort_flag_indices(cam, n, 0, order, order)
        assert ia is not None
        torch.cuda.synchronize()
        assert int(order.view(torch.int32)[ia].item()) == 0
        order.view(torch.int32)[ia] = 1

    image, st = stages.forward(*args, after_project=poke)
    torch.cuda.synchronize()
    assert torch.isnan(image).all()


def test_backward_uses_the_bin_size_of_its_own_forward(oracle, list_bin):
    """The bin size of the tile lists is an argument of every native call and the autograd context keeps the one
    its forward used: changing the package's default between a forward and its backward changes nothing for that
    backward (gradients against the oracle)."""
    from ds_splat import GaussianRasterizationSettings, GaussianRasterizer
    sc = make_scene("cfg1", n=20000, width=640, height=360, sh_degree=3)
    img_o, radii_o, S, B = oracle_run(oracle, sc, 2.0)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    settings = GaussianRasterizationSettings(
        image_height=sc["height"], image_width=sc["width"], tanfovx=sc["tanfovx"], tanfovy=sc["tanfovy"], bg=t["bg"],
        scale_modifier=1.0, viewmatrix=t["viewmatrix"], projmatrix=t["projmatrix"], sh_degree=sc["sh_degree"],
        max_sh_degree=3, campos=t["campos"], prefiltered=False, debug=False)
    fT, fidx, _ = gpu_forward_state(sc, 2.0)
    gok = comparable_gaussians(S, B, sc["width"], fT, fidx)
    for before, after in ((4, 1), (1, 4), (4, 8)):
        list_bin(before)
        means = t["means_3d"].clone().requires_grad_(True)
        scales = (t["scales"] * 2.0).requires_grad_(True)
        image, _ = GaussianRasterizer(settings)(means, torch.zeros_like(means), t["shs"], None, t["opacities"],
                                                scales, t["rotations"], None)
        list_bin(after)
        image.backward(t["v_image"])
        torch.cuda.synchronize()
        check_grads_against_bounds({"v_mean3d": means.grad.cpu().numpy(), "v_scale": scales.grad.cpu().numpy()}, B,
                                   B["bounds"], gok, "bins %d then %d" % (before, after))


def test_lists_of_another_bin_size_are_not_walked(list_bin):
    """A `ranges` buffer carries the bin size it was built for in its header word; a blend launch that is told
    another one (a caller's mix-up: the C ABI cannot see it on the host) reads no further: the forward stage
    writes a NaN image, the backward leaves every gradient zero, and nothing is fetched outside the buffers."""
    from ds_splat_amd import stages
    sc = make_scene("cfg1", n=20000, width=640, height=360, sh_degree=3)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    for built, told in ((4, 1), (1, 4), (4, 8), (8, 2)):
        cam = stages.camera_from_scene(sc, DEV, list_bin=built)
        image, st = stages.forward(cam, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["opacities"], t["shs"])
        assert int(stages.split_lists(cam, st.lists)["header"].item()) == {1: 0, 2: 1, 4: 2, 8: 3}[built]
        assert torch.isfinite(image).all() and float(image.max()) > 0
        other = cam.with_list_bin(told)
        # the stage forward on the wrong layout: NaN image (the buffer is as long as the larger layout wants)
        pad = torch.zeros(max(int(_ranges_words(other)), st.lists.numel()) + 8, dtype=torch.int32, device=DEV)
        pad[:st.lists.numel()] = st.lists
        img2, _, _ = stages.blend_fwd(other, pad, st.sorted_ids, st.splats)
        torch.cuda.synchronize()
        # (the stage entry takes per-tile ranges without a header too, dsx_tile_ranges' own, so it cannot refuse
        # when it is told "per tile": positions are clamped and the image is merely wrong)
        assert told == 1 or torch.isnan(img2).all(), (built, told)
        # the whole backward on the wrong layout: zeros
        st.lists = pad
        st.list_bin = told
        out = stages.backward(other, st, 16, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["v_image"])
        torch.cuda.synchronize()
        for key in ("v_mean3d", "v_shs", "v_opacity", "v_scale", "v_quat"):
            assert float(out[key].abs().max()) == 0.0, (built, told, key)


def _ranges_words(cam):
    from ds_splat_amd import _native
    return _native.load().dsx_ranges_count(cam.width, cam.height, cam.list_bin)


def test_list_positions_beyond_the_ids_are_not_followed():
    """Ranges whose ends lie beyond the entries of sorted_ids (a `ranges` buffer of another forward, a k that is
    too small): the blend kernels clamp every position to [0, k) and give wrong numbers, not a fetch outside
    sorted_ids.  Runs the stage entry points and the whole backward on per-tile and on binned lists."""
    from ds_splat_amd import stages
    sc = make_scene("cfg1", n=20000, width=640, height=360, sh_degree=3)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    for bins in (1, 4):
        cam = stages.camera_from_scene(sc, DEV, list_bin=bins)
        image, st = stages.forward(cam, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["opacities"], t["shs"])
        k = st.num_keys
        parts = stages.split_lists(cam, st.lists)
        which = "fine" if bins == 1 else "bins"
        assert int(parts[which][-1].item()) == k
        # only the first third of the pairs is handed over (ids and, for binned lists, their mask words), with
        # the full ranges
        third = k // 3
        short = torch.cat([st.sorted_ids[:third], st.sorted_ids[k:k + third]]) if bins > 1 else st.sorted_ids[:third].clone()
        img2, fT2, fidx2 = stages.blend_fwd(cam, st.lists, short, st.splats)
        torch.cuda.synchronize()
        assert torch.isfinite(img2).all()
        st.sorted_ids = short
        out = stages.backward(cam, st, 16, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["v_image"])
        torch.cuda.synchronize()
        assert all(torch.isfinite(out[key]).all() for key in ("v_mean3d", "v_shs", "v_scale"))


def test_api_rejects_bad_inputs_with_the_reference_messages():
    """cpp/rasterizer_torch.cu:176-190 and :124-129: every check fires before anything is launched."""
    from ds_splat import GaussianRasterizationSettings, GaussianRasterizer
    sc = make_scene("cfg0", n=64, width=32, height=32, sh_degree=1)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}

    def settings(sh_degree=1, max_sh_degree=3):
        return GaussianRasterizationSettings(32, 32, sc["tanfovx"], sc["tanfovy"], t["bg"], 1.0, t["viewmatrix"],
                                             t["projmatrix"], sh_degree, max_sh_degree, t["campos"], False, False)

    good = dict(means_3d=t["means_3d"], means_2d=torch.zeros_like(t["means_3d"]), shs=t["shs"], colors_precomp=None,
                opacities=t["opacities"], scales=t["scales"], rotations=t["rotations"], cov_3d_precomp=None)

    def run(s=None, **change):
        a = dict(good)
        a.update(change)
        return GaussianRasterizer(s or settings())(a["means_3d"], a["means_2d"], a["shs"], a["colors_precomp"],
                                                   a["opacities"], a["scales"], a["rotations"], a["cov_3d_precomp"])

    image, radii = run()
    assert image.shape == (32, 32, 3)
    cases = [
        (dict(means_3d=t["means_3d"].t().contiguous().t()), "means_3d must be contiguous"),
        (dict(opacities=sc["opacities"]), "opacities must be a CUDA tensor"),
        (dict(shs=t["shs"].transpose(1, 2)), "shs error"),
        (dict(scales=sc["scales"]), "scales error"),
        (dict(rotations=t["rotations"].t().contiguous().t()), "rotations error"),
        (dict(scales=None, rotations=None), "cov3D error"),
        (dict(shs=None), "SHS error"),
        (dict(scales=t["scales"].double()), "scales must be float32"),
        (dict(opacities=t["opacities"][:10].contiguous()), "opacities must have one entry per Gaussian"),
        (dict(shs=t["shs"][:, :4].contiguous()), r"shs must have shape"),
        (dict(rotations=t["rotations"][:, :3].contiguous()), r"scales must be \[N,3\] and rotations \[N,4\]"),
        (dict(scales=None, rotations=None, cov_3d_precomp=torch.zeros(10, 6, device=DEV)), r"cov3D_precomp must be"),
        (dict(shs=None, colors_precomp=torch.zeros(10, 3, device=DEV)), r"colors_precomp must be"),
    ]
    for change, message in cases:
        with pytest.raises(RuntimeError, match=message):
            run(**change)
    with pytest.raises(RuntimeError, match="sh_degree must be in"):
        run(s=settings(sh_degree=4))
    with pytest.raises(RuntimeError, match="sh_degree must be in"):
        run(s=settings(max_sh_degree=2))


def test_non_finite_gaussians_are_culled_and_leave_the_rest_alone():
    """NaN / infinite means and scales fail the frustum or determinant test (radius 0): the image
    and every other Gaussian's gradient equal those of a scene where the same Gaussians sit far
    outside the view.  A NaN opacity is not a culling criterion (the reference blends it with
    alpha 0.999, cpp/rasterizer_kernels.cu:341-431): that scene must simply run to completion."""
    sc = make_scene("cfg1", n=20000, width=320, height=200, sh_degree=2)
    bad = torch.arange(5000, 5030)
    clean = dict(sc)
    clean["means_3d"] = sc["means_3d"].clone()
    clean["means_3d"][bad, 0] += 1.0e4                      # far outside the frustum
    dirty = dict(sc)
    dirty["means_3d"] = sc["means_3d"].clone()
    dirty["scales"] = sc["scales"].clone()
    dirty["means_3d"][bad[:10], 1] = float("nan")
    dirty["scales"][bad[10:20], 2] = float("nan")
    dirty["scales"][bad[20:30], 0] = float("inf")
    img_c, radii_c, leaves_c = api_run(clean, 2.0)
    img_d, radii_d, leaves_d = api_run(dirty, 2.0)
    assert (radii_d[bad] == 0).all() and (radii_c[bad] == 0).all()
    assert torch.equal(radii_c, radii_d)
    assert torch.equal(img_c, img_d)
    keep = torch.ones(20000, dtype=torch.bool, device=DEV)
    keep[bad] = False
    for name in ("means", "shs", "opac", "scales", "rots"):
        gc, gd = leaves_c[name].grad, leaves_d[name].grad
        assert torch.isfinite(gd[keep]).all()
        scale = float(gc.abs().max())
        assert torch.allclose(gc[keep], gd[keep], rtol=1e-3, atol=1e-4 * max(1.0, scale)), name
    nan_opacity = dict(sc)
    nan_opacity["opacities"] = sc["opacities"].clone()
    nan_opacity["opacities"][bad[:5]] = float("nan")
    img_n, radii_n, _ = api_run(nan_opacity, 2.0)
    assert img_n.shape == img_c.shape and torch.equal(radii_n > 0, (radii_c > 0) | torch.isin(
        torch.arange(20000, device=DEV), bad.to(DEV)) & (radii_n > 0))



def test_forward_refuses_more_per_tile_pairs_than_32_bits_index():
    """Lists per bin hold a fraction of the pairs of per-tile lists, but the per-tile ranges, final_idx and the
    scan records still index the per-tile pairs as int32: 300 K Gaussians that each cover the whole 1920 x 1080
    image make 2.4 G per-tile pairs (beyond 2^31) and only 40 M pairs of the 8 x 8 bins (well below the 2^30 that
    the partition sorts).  The forward must say DSX_ERR_TOO_LARGE after its first half, not wrap the indices."""
    from ds_splat_amd import stages
    n = 300_000
    sc = make_scene("cfg1", n=n, width=1920, height=1080, sh_degree=0)
    sc["means_3d"][:, :2] *= 0.02                      # all near the optical axis
    sc["scales"] = torch.full_like(sc["scales"], 40.0)  # ... and far larger than the frustum
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    cam = stages.camera_from_scene(sc, DEV)
    assert stages.list_bin(cam) == 8
    with pytest.raises(RuntimeError, match="too many"):
        stages.forward(cam, t["means_3d"], t["scales"], t["rotations"], t["opacities"], t["shs"])
    torch.cuda.synchronize()
    # the same scene cut to a tenth fits both limits and renders
    m = n // 10
    image, st = stages.forward(cam, t["means_3d"][:m].contiguous(), t["scales"][:m].contiguous(),
                               t["rotations"][:m].contiguous(), t["opacities"][:m].contiguous(),
                               t["shs"][:m].contiguous())
    torch.cuda.synchronize()
    assert st.num_keys_per_tile == (m - 1) * 8160 and st.num_keys == (m - 1) * 135
    assert torch.isfinite(image).all()


@pytest.mark.parametrize("bins", [0, 2, 8])
def test_stage_entry_points_chain_on_binned_lists(oracle, bins):
    """The documented chain of stage entry points (projection, depth order, tile lists, blend forward, blend
    backward) on an image whose lists the library builds per bin of tiles: the same camera goes to every call,
    the whole `ranges` and `sorted_ids` buffers go from dsx_tile_lists to the blend stages, and the results are
    the oracle's."""
    from ds_splat_amd import stages
    sc = make_scene("cfg1", n=40000, width=1280, height=720, sh_degree=3, seed=77)      # 3600 tiles
    img_o, radii_o, S, B = oracle_run(oracle, sc, 2.0)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    cam = stages.camera_from_scene(sc, DEV, list_bin=bins)
    assert stages.list_bin(cam) == (4 if bins == 0 else bins)
    n = sc["n"]
    order = stages.new_order(cam, n, DEV)
    splats, radii, cov3d, _ = stages.project_fwd(cam, t["means_3d"], t["scales"] * 2.0, t["rotations"], t["opacities"],
                                                 t["shs"], order=order)
    stages.depth_order(cam, n, order)
    torch.cuda.synchronize()
    k = stages.key_count(cam, n, order)
    ids, lists = stages.tile_lists(cam, n, k, order, return_lists=True)
    image, final_T, final_idx = stages.blend_fwd(cam, lists, ids, splats)
    grads = stages.blend_bwd(cam, n, lists, ids, splats, final_T, final_idx, t["v_image"])
    torch.cuda.synchronize()
    assert (radii.cpu().numpy() == radii_o).all()
    assert (lists[:cam.num_tiles + 1].cpu().numpy() == S["ranges"]).all()
    ok = S["margin"] > 1e-4
    assert ok.mean() > 0.98
    np.testing.assert_allclose(image.cpu().numpy()[ok], img_o[ok], rtol=1e-4, atol=1e-5)
    assert (final_idx.cpu().numpy()[ok] == S["final_idx"][ok]).all()
    # the nine screen-space sums against the oracle's blend backward, each within 1e-4 of the summed magnitudes
    # of its terms, for the Gaussians that no borderline decision touches
    A = arrays(sc)
    Bb = oracle.blend_bwd(scene_settings(sc), S["ranges"], S["sorted_ids"], S["means2d"], S["conic"], S["rgb"],
                          A["opacities"], S["final_T"], S["final_idx"], A["v_image"])
    gok = comparable_gaussians(S, Bb, sc["width"], final_T.cpu().numpy(), final_idx.cpu().numpy())
    want = np.concatenate([Bb["v_xy"], Bb["v_conic"], Bb["v_opacity"].reshape(n, 1), Bb["v_rgb"]], axis=1).astype(np.float64)
    err = np.abs(grads.cpu().numpy()[:, :9].astype(np.float64) - want)[gok]
    bound = (1e-4 * Bb["abs_sums"].astype(np.float64) + 1e-7)[gok]
    assert gok.mean() > 0.5 and (err <= bound).all(), float((err / bound).max())
