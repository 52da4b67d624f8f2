"""ctypes binding of libdsx.so (the C ABI declared in include/dsx.h).

The library is built in-tree by ``__graft_entry__.build()`` (or ``make -C ds_splat_amd/csrc``)
into ``ds_splat_amd/lib/libdsx.so``.  There is no fallback: if the library is missing or a
symbol is absent, loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdsx.so")

SPLAT_FLOATS = 12
GRAD_FLOATS = 12
PROJ_BLOCK = 256
TILE = 16


class Camera(C.Structure):
    """struct dsx_camera"""
    _fields_ = [
        ("image_height", C.c_int32),
        ("image_width", C.c_int32),
        ("tanfovx", C.c_float),
        ("tanfovy", C.c_float),
        ("scale_modifier", C.c_float),
        ("sh_degree", C.c_int32),
        ("max_sh_degree", C.c_int32),
        ("view", C.c_void_p),
        ("proj", C.c_void_p),
        ("campos", C.c_void_p),
        ("bg", C.c_void_p),
        ("list_bin", C.c_int32),
    ]


_P = C.c_void_p
_I64 = C.c_int64
_I32 = C.c_int32
_CAM = C.POINTER(Camera)

# name -> (restype, argtypes); must list every function include/dsx.h declares
SIGNATURES = {
    "dsx_error_string": (C.c_char_p, [C.c_int]),
    "dsx_version": (C.c_int, []),
    "dsx_num_blocks": (_I64, [_I64]),
    "dsx_num_tiles": (_I32, [_I32, _I32]),
    "dsx_sort_passes": (_I32, [_I32]),
    "dsx_workspace_bytes": (C.c_size_t, [_I64, _I64, _I32, _I32, _I32]),
    "dsx_sort_workspace_bytes": (C.c_size_t, [_I64, _I32]),
    "dsx_sort_u32_workspace_bytes": (C.c_size_t, [_I64, _I32]),
    "dsx_order_bytes": (C.c_size_t, [_I64, _I32, _I32, _I32]),
    "dsx_project_fwd": (C.c_int, [_CAM, _I64] + [_P] * 7 + [_P] * 4 + [_P, C.c_size_t, _P]),
    "dsx_scan_u32": (C.c_int, [_I64, _P, _P, _P]),
    "dsx_emit_keys": (C.c_int, [_CAM, _I64, _I64, _P, _P, _P, _P, _P]),
    "dsx_sort_pairs": (C.c_int, [_I64, _I32, _P, _P, _P, C.c_size_t, _P]),
    "dsx_tile_ranges": (C.c_int, [_I64, _P, _I32, _P, _P]),
    "dsx_sort_pairs_u32": (C.c_int, [_I64, _I32, _P, _P, _P, C.c_size_t, _P]),
    "dsx_depth_order": (C.c_int, [_CAM, _I64, _P, C.c_size_t, _P]),
    "dsx_order_view": (C.c_int, [_I64, _P, C.POINTER(_P), C.POINTER(_P)]),
    "dsx_sort_flags": (C.c_int, [_I64, _I64, _I32, _I32, _I32, _P, _P, C.POINTER(_P), C.POINTER(_P)]),
    "dsx_tile_lists": (C.c_int, [_CAM, _I64, _I64, _P, _P, _P, _P, C.c_size_t, _P]),
    "dsx_blend_fwd": (C.c_int, [_CAM, _I64, _I64] + [_P] * 6 + [_P]),
    "dsx_blend_bwd": (C.c_int, [_CAM, _I64, _I64] + [_P] * 7 + [_P]),
    "dsx_gaussian_bwd": (C.c_int, [_CAM, _I64, _I32] + [_P] * 7 + [_P] * 8 + [_P]),
    "dsx_forward_project": (C.c_int, [_CAM, _I64] + [_P] * 7 + [_P] * 4 + [_P, C.c_size_t, _P, _P]),
    "dsx_forward_finish": (C.c_int, [_CAM, _I64, _I64] + [_P] * 7 + [_P, C.c_size_t, _P, _P]),
    "dsx_backward": (C.c_int, [_CAM, _I64, _I64, _I32] + [_P] * 11 + [_P, _I32] + [_P] * 8 + [_P]),
    "dsx_backward_static": (C.c_int, [_CAM, _I64, _I64, _I32] + [_P] * 11 + [_P] * 8 + [_P]),
    "dsx_forward_core": (C.c_int, [_P] * 5 + [_I64] + [_P] * 3 + [_I32, _I32, C.c_float, C.c_float, C.c_float,
                                                                    _I32, _I32, _P, _P]),
}



class TraceEntry(C.Structure):
    """struct dsx_trace_entry"""
    _fields_ = [("name", C.c_char * 48), ("milliseconds", C.c_float)]


SIGNATURES["dsx_trace_enable"] = (C.c_int, [C.c_int])
SIGNATURES["dsx_trace_read"] = (C.c_int, [C.POINTER(TraceEntry), C.c_int])
SIGNATURES["dsx_set_blend_pixels_per_lane"] = (C.c_int, [C.c_int])
SIGNATURES["dsx_list_bin"] = (_I32, [_I32, _I32, _I32])
SIGNATURES["dsx_ranges_count"] = (_I64, [_I32, _I32, _I32])
SIGNATURES["dsx_sorted_ids_count"] = (_I64, [_I64, _I32, _I32, _I32])
SIGNATURES["dsx_grads_bytes"] = (C.c_size_t, [_I64])

_lib = None

# Tiles per side of the bins that the tile lists are built for when a caller does not say: 0 leaves the
# choice to the library (by image size).  A Python-side default for the callers in this package
# (rasterizer, stages, benchmark); the native library keeps no such setting: every call is told.
_default_list_bin = 0


def default_list_bin():
    return _default_list_bin


def set_default_list_bin(tiles_per_side):
    """0 (the library's choice by image size), 1, 2, 4 or 8.  Takes effect for forwards that start
    afterwards; a backward always uses the bin size of its own forward."""
    global _default_list_bin
    if int(tiles_per_side) not in (0, 1, 2, 4, 8):
        raise ValueError("list_bin must be 0, 1, 2, 4 or 8")
    _default_list_bin = int(tiles_per_side)


def load():
    """Loads libdsx.so once and attaches prototypes.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "ds_splat_amd: native library %s is missing — build it with "
            "`python -c 'import __graft_entry__ as g; g.build()'` or `make -C ds_splat_amd/csrc`" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


_ext = None


def load_torch_ext():
    """Imports the C++ torch binding (ds_splat_amd/lib/_dsx_torch*.so, built from csrc/torch_ext.cpp
    and linked against libdsx.so).  Raises if it is not built: there is no Python fallback."""
    global _ext
    if _ext is not None:
        return _ext
    import glob
    import importlib.util
    import torch  # noqa: F401  (the binding links against torch's libraries)
    load()
    found = sorted(glob.glob(os.path.join(_HERE, "lib", "_dsx_torch*.so")))
    if not found:
        raise RuntimeError(
            "ds_splat_amd: the torch binding ds_splat_amd/lib/_dsx_torch*.so is missing — build it with "
            "`python -c 'import __graft_entry__ as g; g.build()'` or `make -C ds_splat_amd/csrc`")
    spec = importlib.util.spec_from_file_location("_dsx_torch", found[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    _ext = mod
    return mod


def check(status):
    if status != 0:
        raise RuntimeError(load().dsx_error_string(status).decode())


def trace_enable(on):
    check(load().dsx_trace_enable(1 if on else 0))


def trace_read(max_entries=65536):
    """Returns [(kernel name, milliseconds), ...] in launch order and clears the trace."""
    buf = (TraceEntry * max_entries)()
    count = load().dsx_trace_read(buf, max_entries)
    return [(buf[i].name.decode(), float(buf[i].milliseconds)) for i in range(count)]
