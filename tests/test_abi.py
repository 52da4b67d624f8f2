"""The C-ABI library loads without a GPU and exports exactly what include/dsx.h declares;
the host-side helpers that need no device behave."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "dsx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dsx_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_functions():
    from ds_splat_amd import _native
    assert declared_functions() == sorted(_native.SIGNATURES)


def test_library_exports_every_declared_symbol():
    from ds_splat_amd import _native
    lib = _native.load()
    for name in declared_functions():
        assert getattr(lib, name) is not None


def test_torch_binding_loads_and_links_the_library():
    from ds_splat_amd import _native
    ext = _native.load_torch_ext()
    assert ext.version() == _native.load().dsx_version()
    assert callable(ext.forward) and callable(ext.backward)


def test_host_helpers():
    from ds_splat_amd import _native
    lib = _native.load()
    assert lib.dsx_version() >= 100
    assert lib.dsx_num_blocks(0) == 0 and lib.dsx_num_blocks(1) == 1 and lib.dsx_num_blocks(257) == 2
    assert lib.dsx_num_tiles(1920, 1080) == 120 * 68
    assert lib.dsx_num_tiles(40, 30) == 6
    # 32 depth bits + bits for tile ids 0..T (slot 0 = negative keys), at most 9 bits a pass
    assert lib.dsx_sort_passes(8160) == 5 and lib.dsx_sort_passes(255) == 5 and lib.dsx_sort_passes(32400) == 6
    assert lib.dsx_workspace_bytes(0, 0, 64, 64, 0) >= 0
    # tile lists: two slot buffers (16-bit slots up to 65534 lists, else 32-bit) and one id buffer
    assert (1 << 20) * 8 < lib.dsx_workspace_bytes(0, 1 << 20, 1920, 1080, 0) < (1 << 20) * 9
    assert (1 << 20) * 12 < lib.dsx_workspace_bytes(0, 1 << 20, 16400, 1040, 1) < (1 << 20) * 13
    # bins of the tile lists: an argument of every call (0: the library's choice); the `ranges` buffer is the
    # per-tile ranges and a header word, and grows with the bins
    assert lib.dsx_list_bin(1920, 1080, 1) == 1 and lib.dsx_ranges_count(1920, 1080, 1) == 8160 + 2
    assert lib.dsx_list_bin(1920, 1080, 3) == 0 and lib.dsx_ranges_count(1920, 1080, 3) == 0
    assert lib.dsx_order_bytes(100, 1920, 1080, 5) == 0 and lib.dsx_workspace_bytes(0, 10, 1920, 1080, -1) == 0
    # per tile below 2048 tiles; 8 x 8 where that needs one partition pass and 4 x 4 two (1080p: 135 against
    # 510 lists); 4 x 4 where it fits one pass itself (128 lists) or where both need two (4K: 510 against 2040)
    assert lib.dsx_list_bin(1920, 1080, 0) == 8 and lib.dsx_list_bin(1024, 512, 0) == 4
    assert lib.dsx_list_bin(1024, 496, 0) == 1 and lib.dsx_list_bin(3840, 2160, 0) == 4
    assert lib.dsx_list_bin(640, 480, 8) == 8 and lib.dsx_list_bin(640, 480, 0) == 1
    # a bin's slot shares its word with the tile mask (at most 65534 bins): larger bins, then per-tile lists
    assert lib.dsx_list_bin(16400, 16400, 0) == 8 and lib.dsx_list_bin(40000, 40000, 0) == 1
    assert lib.dsx_ranges_count(1920, 1080, 0) == (8160 + 1) + 1 + 1 + (15 * 9 + 1) + 8 * 8160
    assert lib.dsx_ranges_count(1920, 1080, 8) == lib.dsx_ranges_count(1920, 1080, 0)
    assert lib.dsx_ranges_count(240, 240, 0) == 225 + 2
    assert lib.dsx_sort_workspace_bytes(1 << 20, 8160) > (1 << 20) * 12
    assert lib.dsx_sort_u32_workspace_bytes(1 << 20, 32) > (1 << 20) * 8
    # order buffer: 4 uint32 arrays and two uint2 arrays per Gaussian
    assert lib.dsx_order_bytes(1 << 20, 1920, 1080, 0) > (1 << 20) * 32
    assert lib.dsx_order_bytes(0, 3840, 2160, 0) - lib.dsx_order_bytes(0, 16, 16, 0) >= 241 * 136 * 4 - 512
    assert b"workspace" in lib.dsx_error_string(-5)
    assert lib.dsx_error_string(0) == b"ok"


def test_bad_arguments_are_rejected_without_touching_the_gpu():
    from ds_splat_amd import _native
    lib = _native.load()
    assert lib.dsx_scan_u32(-1, None, None, None) == -1
    assert lib.dsx_sort_pairs(-5, 10, None, None, None, 0, None) == -1
    assert lib.dsx_sort_pairs(1 << 31, 10, 1, 1, 1, 0, None) == -4
    assert lib.dsx_tile_ranges(10, None, 4, None, None) == -1
    assert lib.dsx_project_fwd(None, 10, *([None] * 12), 0, None) == -1
    assert lib.dsx_sort_pairs_u32(10, 33, 1, 1, 1, 0, None) == -1
    assert lib.dsx_sort_pairs_u32(10, 32, 1, 1, 1, 0, None) == -5
    assert lib.dsx_depth_order(None, 10, None, 0, None) == -1
    assert lib.dsx_sort_flags(-1, 0, 16, 16, 0, None, None, None, None) == -1
    assert lib.dsx_sort_flags(10, 10, 16, 16, 3, None, None, None, None) == -1
    assert lib.dsx_sort_flags(10, 10, 16, 16, 0, None, None, None, None) == 0
    # with a well-formed camera (its pointers are only compared with null before these checks fail)
    import ctypes as C
    cam = _native.Camera(64, 64, 0.5, 0.5, 1.0, 3, 3, 8, 8, 8, 8, 0)
    ref = C.byref(cam)
    fake = 16   # any non-null address: nothing is launched
    # the per-Gaussian backward needs the stored covariances or scales + rotations to rebuild them
    assert lib.dsx_gaussian_bwd(ref, 10, 16, fake, None, None, fake, None, fake, fake, *([None] * 8), None) == -1
    # ... and takes either with every output absent (n = 0: nothing to do)
    assert lib.dsx_gaussian_bwd(ref, 0, 16, fake, None, None, fake, None, fake, fake, *([None] * 8), None) == 0
    assert lib.dsx_gaussian_bwd(ref, 10, 17, fake, fake, fake, fake, None, fake, fake, *([None] * 8), None) == -1
    # the forward's first half wants a place for K; the backward its saved tensors
    assert lib.dsx_forward_project(ref, 10, *([fake] * 7), fake, fake, None, fake, fake, 1 << 20, None, None) == -1
    assert lib.dsx_backward(ref, 10, 5, 16, fake, fake, fake, fake, None, fake, None, fake, fake, fake, fake, fake, 0,
                            *([None] * 8), None) == -1
    # list positions and ids are bounded by what the caller says it holds: a backward with entries but no
    # sorted_ids, negative counts, and counts beyond 32-bit indexing are refused before anything is launched
    full = [fake, fake, fake, fake, None, fake, fake]          # means3d .. radii, ranges
    tail = [fake, fake, fake, fake, 0] + [None] * 8 + [None]    # final_T, final_idx, v_image, grads, prepared, outputs, stream
    assert lib.dsx_backward(ref, 10, 5, 16, *full, None, *tail) == -1
    assert lib.dsx_backward(ref, 10, -1, 16, *full, fake, *tail) == -1
    assert lib.dsx_backward(ref, 10, 1 << 30, 16, *full, fake, *tail) == -4
    assert lib.dsx_blend_fwd(ref, 10, 5, fake, None, fake, fake, fake, fake, None) == -1
    assert lib.dsx_blend_fwd(ref, -1, 5, fake, fake, fake, fake, fake, fake, None) == -1
    assert lib.dsx_blend_fwd(ref, 10, 1 << 31, fake, fake, fake, fake, fake, fake, None) == -4
    assert lib.dsx_blend_bwd(ref, 10, 1 << 31, fake, fake, fake, fake, fake, fake, fake, None) == -4
    assert lib.dsx_blend_bwd(ref, 10, 5, fake, None, fake, fake, fake, fake, fake, None) == -1
    # a bin size that is none of 0, 1, 2, 4, 8 is a bad camera
    bad = _native.Camera(64, 64, 0.5, 0.5, 1.0, 3, 3, 8, 8, 8, 8, 3)
    assert lib.dsx_depth_order(C.byref(bad), 10, fake, 1 << 20, None) == -1
    assert lib.dsx_blend_fwd(C.byref(bad), 10, 5, fake, fake, fake, fake, fake, fake, None) == -1
    assert b"2^31" in lib.dsx_error_string(-4) and b"2^30" in lib.dsx_error_string(-4)


def test_python_api_surface():
    import dataclasses
    import ds_splat
    from ds_splat import GaussianRasterizationSettings, GaussianRasterizer
    names = [f.name for f in dataclasses.fields(GaussianRasterizationSettings)]
    assert names == ["image_height", "image_width", "tanfovx", "tanfovy", "bg", "scale_modifier", "viewmatrix",
                     "projmatrix", "sh_degree", "max_sh_degree", "campos", "prefiltered", "debug"]
    import inspect
    sig = list(inspect.signature(GaussianRasterizer.forward).parameters)
    assert sig == ["self", "means_3d", "means_2d", "shs", "colors_precomp", "opacities", "scales", "rotations",
                   "cov_3d_precomp"]


def test_native_settings_follow_the_settings_tensors():
    """The transposed camera matrices are cached per settings object: a replaced or modified matrix
    must be seen, and matrices made under torch.inference_mode (no version counter) must work."""
    import torch
    from ds_splat import GaussianRasterizationSettings, GaussianRasterizer
    from ds_splat_amd.synthetic import make_scene
    sc = make_scene("cfg0", n=8, width=32, height=32)
    s = GaussianRasterizationSettings(32, 32, sc["tanfovx"], sc["tanfovy"], sc["bg"], 1.0, sc["viewmatrix"].clone(),
                                      sc["projmatrix"].clone(), 0, 3, sc["campos"], False, False)
    r = GaussianRasterizer(s)
    a = r.settings_for_cpp_code
    assert r.settings_for_cpp_code is a                                  # unchanged: cached
    assert torch.equal(a.view_matrix, s.viewmatrix.t()) and torch.equal(a.proj_matrix, s.projmatrix.t())
    s.viewmatrix[3, 0] = 5.0                                             # modified in place
    b = r.settings_for_cpp_code
    assert b is not a and float(b.view_matrix[0, 3]) == 5.0
    s.viewmatrix = torch.eye(4) * 2.0                                    # replaced
    c = r.settings_for_cpp_code
    assert c is not b and float(c.view_matrix[1, 1]) == 2.0
    s.scale_modifier = 1.3
    assert r.settings_for_cpp_code.scale_modifier == 1.3
    with torch.inference_mode():
        s.viewmatrix = torch.eye(4) * 3.0
        s.projmatrix = torch.arange(16, dtype=torch.float32).reshape(4, 4)
        d = r.settings_for_cpp_code
    assert float(d.view_matrix[2, 2]) == 3.0 and float(d.proj_matrix[0, 1]) == 4.0


def test_scene_dump_round_trip(tmp_path):
    """The TorchScript scene dump carries the attribute names the reference's timing harness
    reads (tests/rasterizer_test.cpp:147-168)."""
    import torch
    from ds_splat_amd import scene_io
    from ds_splat_amd.synthetic import make_scene
    sc = make_scene("cfg0", n=64, width=48, height=32, sh_degree=2)
    path = str(tmp_path / "scene.pt")
    scene_io.save_scene(path, scene_io.scene_from_synthetic(sc))
    m = torch.jit.load(path)
    for name in ("means_3d", "means_2d", "shs", "opacities", "scales", "rotations", "viewmatrix", "projmatrix",
                 "campos", "image_height", "image_width", "tanfovx", "tanfovy", "scale_modifier", "sh_degree"):
        assert hasattr(m, name), name
    d = scene_io.load_scene(path)
    assert d["image_height"] == 32 and d["image_width"] == 48 and d["sh_degree"] == 2
    assert torch.equal(d["shs"], sc["shs"]) and torch.equal(d["projmatrix"], sc["projmatrix"])
    assert abs(d["tanfovx"] - sc["tanfovx"]) < 1e-12


def test_inria_adaptor_surface():
    import inspect
    from ds_splat_amd import inria_compat
    assert inria_compat.GaussianRasterizationSettings._fields == (
        "image_height", "image_width", "tanfovx", "tanfovy", "bg", "scale_modifier", "viewmatrix", "projmatrix",
        "sh_degree", "campos", "prefiltered", "debug")
    sig = list(inspect.signature(inria_compat.GaussianRasterizer.forward).parameters)
    assert sig == ["self", "means3D", "means2D", "opacities", "shs", "colors_precomp", "scales", "rotations",
                   "cov3D_precomp"]


def test_input_checks_mirror_the_reference_messages():
    import torch
    from ds_splat import GaussianRasterizationSettings, GaussianRasterizer
    from ds_splat_amd.synthetic import make_scene
    sc = make_scene("cfg0", n=8, width=32, height=32)
    s = GaussianRasterizationSettings(32, 32, sc["tanfovx"], sc["tanfovy"], sc["bg"], 1.0, sc["viewmatrix"],
                                      sc["projmatrix"], 0, 3, sc["campos"], False, False)
    r = GaussianRasterizer(s)
    with pytest.raises(RuntimeError, match="means_3d must be a CUDA tensor"):
        r(sc["means_3d"], sc["means_3d"], sc["shs"], None, sc["opacities"], sc["scales"], sc["rotations"], None)
