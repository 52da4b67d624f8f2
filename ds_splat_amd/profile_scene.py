"""Timing harness in the shape of the reference's (tests/rasterizer_test.cpp:145-212): load a
scene dump, run the rasterizer a number of times, print one "Timing step" line per iteration.

    python -m ds_splat_amd.profile_scene --scene garden.pt            # a TorchScript scene dump
    python -m ds_splat_amd.profile_scene --synthetic cfg2 --backward  # a synthetic workload
    python -m ds_splat_amd.profile_scene --synthetic cfg1 --core      # the raw-pointer forward

Unlike the reference's harness, which stops its host clock without waiting for the device, each
iteration is bracketed by a device synchronisation; ``--kernels`` adds the per-kernel times of
the last iteration (events on the launch stream).
"""
import argparse
import ctypes as C
import time

import torch

from . import _native, scene_io
from .rasterizer import GaussianRasterizationSettings, GaussianRasterizer


def _scene(args):
    if args.scene:
        return scene_io.load_scene(args.scene)
    from .synthetic import make_scene
    return scene_io.scene_from_synthetic(make_scene(args.synthetic))


def main(argv=None):
    """Runs the harness; returns the image of the last iteration (callers that check what was timed)."""
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    src = ap.add_mutually_exclusive_group(required=True)
    src.add_argument("--scene", help="TorchScript scene dump (see ds_splat_amd.scene_io)")
    src.add_argument("--synthetic", help="name of a synthetic workload (cfg0 .. cfg4)")
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--backward", action="store_true", help="time forward + backward (upstream gradient of ones)")
    ap.add_argument("--core", action="store_true", help="time the raw-pointer forward dsx_forward_core instead")
    ap.add_argument("--kernels", action="store_true", help="per-kernel times of the last iteration")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)

    lib = _native.load()
    dev = torch.device(args.device)
    sc = {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in _scene(args).items()}
    H, W = sc["image_height"], sc["image_width"]
    n = sc["means_3d"].shape[0]
    print("scene: %d Gaussians, %dx%d, SH degree %d" % (n, W, H, sc["sh_degree"]))

    if args.core:
        view = sc["viewmatrix"].t().contiguous()
        proj = sc["projmatrix"].t().contiguous()
        image = torch.empty((H, W, 3), dtype=torch.float32, device=dev)
        p = lambda t: C.c_void_p(t.data_ptr())
        tensors = [sc[k].contiguous() for k in ("means_3d", "shs", "opacities", "scales", "rotations")]

        def step():
            _native.check(lib.dsx_forward_core(*[p(t) for t in tensors], n, p(view), p(proj), p(sc["campos"]), W, H,
                                               sc["tanfovx"], sc["tanfovy"], sc["scale_modifier"], 3, sc["sh_degree"],
                                               p(image), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)))
            return image
        name = "rasterizer_core"
    else:
        settings = GaussianRasterizationSettings(
            image_height=H, image_width=W, tanfovx=sc["tanfovx"], tanfovy=sc["tanfovy"],
            bg=torch.zeros(3, device=dev), scale_modifier=sc["scale_modifier"], viewmatrix=sc["viewmatrix"],
            projmatrix=sc["projmatrix"], sh_degree=sc["sh_degree"], max_sh_degree=3, campos=sc["campos"],
            prefiltered=False, debug=False)
        rasterizer = GaussianRasterizer(settings)
        names = ("means_3d", "means_2d", "shs", "opacities", "scales", "rotations")
        leaves = {k: sc[k].clone().requires_grad_(args.backward) for k in names}
        v_image = torch.ones((H, W, 3), dtype=torch.float32, device=dev)

        def step():
            image, radii = rasterizer(leaves["means_3d"], leaves["means_2d"], leaves["shs"], None, leaves["opacities"],
                                      leaves["scales"], leaves["rotations"], None)
            if args.backward:
                for t in leaves.values():
                    t.grad = None
                image.backward(v_image)
            return image.detach()
        name = "rasterizer_forward_backward" if args.backward else "rasterizer_forward"

    rendered = None
    with torch.cuda.device(dev):
        for i in range(args.iters):
            last = i == args.iters - 1
            if args.kernels and last:
                _native.trace_enable(True)
                _native.trace_read()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            rendered = step()
            torch.cuda.synchronize()
            print("Timing step:%s took: %.3fms" % (name, (time.perf_counter() - t0) * 1e3))
            if args.kernels and last:
                for kernel, ms in _native.trace_read():
                    print("    %-36s %.4f ms" % (kernel, ms))
                _native.trace_enable(False)
    return rendered      # the last iteration's image [H, W, 3] (None without an iteration)


if __name__ == "__main__":
    main()
