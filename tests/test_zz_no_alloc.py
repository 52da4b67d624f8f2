"""dsx_backward_static (the backward whose gradient accumulator is a device array built into the
library, for callers that cannot allocate) against dsx_backward on the same forward state, through
the C ABI: two calls in a row, the second on a smaller scene, so that what the first call left in the
shared array must not leak into the second."""
import ctypes as C

import numpy as np
import pytest
import torch

from ds_splat_amd.synthetic import make_scene
from helpers import arrays, scene_settings, set_camera

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _static_call(lib, cam, st, n, t, scales, out):
    p = lambda x: None if x is None else C.c_void_p(x.data_ptr())
    return lib.dsx_backward_static(cam.ref, n, st.num_keys, 16, p(t["means_3d"]), p(scales), p(t["rotations"]),
                                   p(st.splats), None, p(st.radii), p(st.lists), p(st.sorted_ids), p(st.final_T),
                                   p(st.final_idx), p(t["v_image"]), p(out["v_mean3d"]), p(out["v_means2d"]),
                                   p(out["v_shs"]), p(out["v_colors"]), p(out["v_opacity"]), p(out["v_scale"]),
                                   p(out["v_quat"]), p(out["v_cov3d"]),
                                   C.c_void_p(torch.cuda.current_stream().cuda_stream))


def _backward_both_ways(oracle, n, W, H, camera, seed, list_bin=None, scale_mul=2.0):
    from ds_splat_amd import _native, stages
    lib = _native.load()
    sc = set_camera(make_scene("cfg1", n=n, width=W, height=H, sh_degree=3, seed=seed), camera)
    t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    scales = (t["scales"] * scale_mul).contiguous()
    cam = stages.camera_from_scene(sc, DEV, list_bin=list_bin)
    _, st = stages.forward(cam, t["means_3d"], scales, t["rotations"], t["opacities"], t["shs"])
    # the existing entry point, with a caller-provided accumulator
    ref = stages.backward(cam, st, 16, t["means_3d"], scales, t["rotations"], t["v_image"])
    # the entry point under test: same arguments, no accumulator
    out = stages._bwd_outputs(n, 16, torch.device(DEV))
    rc = _static_call(lib, cam, st, n, t, scales, out)
    assert rc == 0, _native.load().dsx_error_string(rc)
    torch.cuda.synchronize()
    # the call allocates nothing on the device: around a second call (the first one of a process may load
    # the kernels' code) the driver reports the same free memory
    free_before = torch.cuda.mem_get_info()[0]
    rc = _static_call(lib, cam, st, n, t, scales, out)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert rc == 0, _native.load().dsx_error_string(rc)
    torch.cuda.synchronize()
    # tolerances per element from the oracle: 1e-4 of the summed magnitudes of the terms of each sum
    # (both runs add them with float atomics, in an order of their own)
    A = arrays(sc)
    s = scene_settings(sc)
    osc = (A["scales"] * scale_mul).astype(np.float32)
    _, radii, ost = oracle.forward(s, A["means_3d"], osc, A["rotations"], A["opacities"], A["shs"])
    S = oracle.state(s, ost, n)
    B = oracle.backward(s, ost, 16, A["means_3d"], osc, A["rotations"], A["opacities"], A["v_image"])
    oracle.free(ost)
    bounds = oracle.gradient_bounds(s, 16, A["means_3d"], osc, A["rotations"], S["conic"], S["cov3d"],
                                    radii, B["abs_sums"], rel=1e-4)
    assert S["num_keys"] > n // 2 and st.num_keys > 0
    worst = 0.0
    for key in ("v_mean3d", "v_means2d", "v_shs", "v_colors", "v_opacity", "v_scale", "v_quat", "v_cov3d"):
        a, b = ref[key].cpu().numpy().astype(np.float64), out[key].cpu().numpy().astype(np.float64)
        assert np.isfinite(b).all() and np.abs(a).max() > 0, key
        ratio = np.abs(a - b) / (bounds[key].reshape(a.shape) + 1e-300)
        assert ratio.max() <= 1.0, "%s: static and caller-scratch backward differ by %.3e of the bound" % (
            key, ratio.max())
        worst = max(worst, float(ratio.max()))
    return worst


def test_backward_static_matches_backward_twice_in_a_row(oracle):
    first = _backward_both_ways(oracle, 30000, 640, 360, "rotated", seed=71)
    second = _backward_both_ways(oracle, 7000, 320, 200, "identity", seed=72)      # smaller: stale sums must be gone
    print("dsx_backward_static vs dsx_backward: largest difference / bound = %.4f, %.4f" % (first, second))


def test_backward_static_on_binned_lists_and_at_its_largest_n(oracle):
    """The two paths the small scenes above do not reach: lists per bin of tiles (the backward then reads the
    forward's scan records and the pairs' tile masks), and a scene of exactly DSX_STATIC_MAX_GAUSSIANS, whose
    marks end at the last byte of the built-in scratch."""
    binned = _backward_both_ways(oracle, 30000, 640, 360, "rotated", seed=73, list_bin=4)
    hd = _backward_both_ways(oracle, 40000, 1280, 720, "identity", seed=74)                  # 3600 tiles: binned by default
    largest = _backward_both_ways(oracle, 524288, 640, 360, "identity", seed=75, scale_mul=1.0)
    print("dsx_backward_static vs dsx_backward: largest difference / bound = %.4f (bins of 4 x 4), %.4f (1280 x 720), "
          "%.4f (n = 524288)" % (binned, hd, largest))


def test_backward_static_replayed_from_a_graph(oracle):
    """What the entry point is for: a caller that cannot allocate, such as code under graph capture.  The call is
    captured into a HIP graph (after a first call outside the capture, which looks up the scratch's address),
    replayed three times with other work between the replays (an eager static backward of another scene, which
    leaves its sums in the shared scratch), and every replay must reproduce the eager result."""
    from ds_splat_amd import _native, stages
    lib = _native.load()

    def prepare(n, W, H, seed):
        sc = make_scene("cfg1", n=n, width=W, height=H, sh_degree=3, seed=seed)
        t = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
        scales = (t["scales"] * 2.0).contiguous()
        cam = stages.camera_from_scene(sc, DEV)
        _, st = stages.forward(cam, t["means_3d"], scales, t["rotations"], t["opacities"], t["shs"])
        return cam, st, n, t, scales, stages._bwd_outputs(n, 16, torch.device(DEV))

    a = prepare(30000, 640, 360, 81)
    b = prepare(9000, 320, 200, 82)
    keys = ("v_mean3d", "v_means2d", "v_shs", "v_opacity", "v_scale", "v_quat")
    assert _static_call(lib, *a) == 0        # eager: the reference result (and the address look-up)
    torch.cuda.synchronize()
    want = {k: a[5][k].clone() for k in keys}
    assert all(float(want[k].abs().max()) > 0 for k in keys)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        rc = _static_call(lib, *a)           # (torch.cuda.graph makes `side` the current stream)
    assert rc == 0, lib.dsx_error_string(rc)
    torch.cuda.synchronize()
    for replay in range(3):
        for k in keys:
            a[5][k].fill_(float("nan"))
        assert _static_call(lib, *b) == 0    # other work on the shared scratch between the replays
        junk = torch.randn(1 << 20, device=DEV).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for k in keys:
            got = a[5][k]
            assert torch.isfinite(got).all(), (replay, k)
            # the same terms added by float atomics in another order
            assert torch.allclose(got, want[k], rtol=1e-3, atol=1e-4 * max(1.0, float(want[k].abs().max()))), (replay, k)
        del junk


def test_backward_static_rejects_more_gaussians_than_its_scratch_holds():
    from ds_splat_amd import _native
    lib = _native.load()
    cam = _native.Camera(64, 64, 0.5, 0.5, 1.0, 3, 3, 8, 8, 8, 8, 0)
    fake = 16
    rc = lib.dsx_backward_static(C.byref(cam), 524288 + 1, 5, 16, *([fake] * 11), *([None] * 8), None)
    assert rc == -6 and b"524288" in lib.dsx_error_string(rc)
