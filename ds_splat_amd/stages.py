"""Per-stage wrappers over the C ABI for torch tensors that already live on the GPU.

Used by the rasterizer module, the GPU parity tests and the benchmark.  Every function
launches on torch's current stream of the tensors' device and allocates its outputs with
torch (the native library allocates nothing).
"""
import ctypes as C
import threading

import torch

from . import _native as N


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


class CameraArgs:
    """Holds the device tensors a ``dsx_camera`` points to (keeps them alive)."""

    def __init__(self, image_height, image_width, tanfovx, tanfovy, bg, scale_modifier, view_rowmajor,
                 proj_rowmajor, sh_degree, max_sh_degree, campos, list_bin=None):
        """list_bin: tiles per side of the bins of the tile lists (0: the library's choice by image size;
        None: _native.default_list_bin() at the time of construction)."""
        dev = view_rowmajor.device
        f32 = lambda t: t.to(device=dev, dtype=torch.float32).contiguous()
        self.view = f32(view_rowmajor)
        self.proj = f32(proj_rowmajor)
        self.campos = f32(campos)
        self.bg = f32(bg)
        self.height = int(image_height)
        self.width = int(image_width)
        self.sh_degree = int(sh_degree)
        self.device = dev
        c = N.Camera()
        c.image_height = self.height
        c.image_width = self.width
        c.tanfovx = float(tanfovx)
        c.tanfovy = float(tanfovy)
        c.scale_modifier = float(scale_modifier)
        c.sh_degree = self.sh_degree
        c.max_sh_degree = int(max_sh_degree)
        c.view = self.view.data_ptr()
        c.proj = self.proj.data_ptr()
        c.campos = self.campos.data_ptr()
        c.bg = self.bg.data_ptr()
        c.list_bin = N.default_list_bin() if list_bin is None else int(list_bin)
        self.c = c

    @property
    def ref(self):
        return C.byref(self.c)

    @property
    def num_tiles(self):
        return ((self.width + 15) // 16) * ((self.height + 15) // 16)

    @property
    def list_bin(self):
        """what the calls are told (0: the library's choice); stages.list_bin(cam) resolves it"""
        return int(self.c.list_bin)

    def with_list_bin(self, list_bin):
        """The same camera (same device tensors) asking for another bin size."""
        other = CameraArgs.__new__(CameraArgs)
        other.__dict__.update(self.__dict__)
        c = N.Camera()
        C.memmove(C.byref(c), C.byref(self.c), C.sizeof(N.Camera))
        c.list_bin = int(list_bin)
        other.c = c
        return other


def camera_from_scene(sc, device, bg=None, sh_degree=None, scale_modifier=None, list_bin=None):
    """CameraArgs for a ds_splat_amd.synthetic scene (API-convention matrices are transposed
    back to row-major here, as the rasterizer module does)."""
    return CameraArgs(sc["height"], sc["width"], sc["tanfovx"], sc["tanfovy"],
                      (sc["bg"] if bg is None else bg).to(device),
                      sc["scale_modifier"] if scale_modifier is None else scale_modifier,
                      sc["viewmatrix"].to(device).t().contiguous(), sc["projmatrix"].to(device).t().contiguous(),
                      sc["sh_degree"] if sh_degree is None else sh_degree, 3, sc["campos"].to(device), list_bin)


def project_fwd(cam, means3d, scales, quats, opacities, shs, cov3d_precomp=None, colors_precomp=None, order=None):
    """order: optional uint8 buffer of new_order(n) that also receives depth bits and tile rectangles."""
    lib = N.load()
    n = means3d.shape[0]
    dev = means3d.device
    splats = torch.empty((n, N.SPLAT_FLOATS), dtype=torch.float32, device=dev)
    radii = torch.empty((n,), dtype=torch.int32, device=dev)
    cov3d = torch.empty((n, 6), dtype=torch.float32, device=dev)
    block_sums = torch.empty((int(lib.dsx_num_blocks(n)),), dtype=torch.int32, device=dev)
    N.check(lib.dsx_project_fwd(cam.ref, n, _ptr(means3d), _ptr(scales), _ptr(quats), _ptr(opacities), _ptr(shs),
                                _ptr(cov3d_precomp), _ptr(colors_precomp), _ptr(splats), _ptr(radii), _ptr(cov3d),
                                _ptr(block_sums), _ptr(order), 0 if order is None else order.numel(), _stream()))
    return splats, radii, cov3d, block_sums


def new_order(cam, n, device):
    """The buffer that carries the depth order from the projection to the tile lists."""
    nbytes = int(N.load().dsx_order_bytes(n, cam.width, cam.height, cam.list_bin))
    return torch.empty((max(nbytes, 1),), dtype=torch.uint8, device=device)


def depth_order(cam, n, order):
    """Sorts the Gaussians of a projected `order` buffer by depth bits (stable).  Returns views
    (depth order int32[n], scanned pair counts of its 256-Gaussian blocks int32[blocks + 1]; pairs
    per bin when the lists are binned)."""
    lib = N.load()
    N.check(lib.dsx_depth_order(cam.ref, n, _ptr(order), order.numel(), _stream()))
    return depth_order_view(n, order)


def depth_order_view(n, order):
    lib = N.load()
    p_order, p_off = C.c_void_p(), C.c_void_p()
    N.check(lib.dsx_order_view(n, _ptr(order), C.byref(p_order), C.byref(p_off)))
    base = order.data_ptr()
    as_i32 = order.view(torch.int32)
    o0 = (p_order.value - base) // 4
    o1 = (p_off.value - base) // 4
    return as_i32[o0:o0 + n], as_i32[o1:o1 + int(lib.dsx_num_blocks(n)) + 1]


def list_bin(cam):
    """Tiles per side of the bins that the tile lists of this image size are built for (1: per tile)."""
    return int(N.load().dsx_list_bin(cam.width, cam.height, cam.list_bin))


def key_count(cam, n, order):
    """Number of pairs of the lists that dsx_tile_lists will build from a depth-ordered `order`
    buffer (per bin when the lists are binned): the last scanned block offset."""
    _, offsets = depth_order_view(n, order)
    return int(offsets[-1].item())


def split_lists(cam, lists):
    """The parts of a `ranges` buffer (dsx_ranges_count words): dict with 'fine' [T+1], 'header' [1]
    (log2 of the bin side) and, for binned lists, 'last_tile' (int tensor [1]), 'bins' [bins+1] and
    'walk' [T, 4, 2]."""
    t = cam.num_tiles
    out = {"fine": lists[:t + 1], "header": lists[t + 1:t + 2]}
    b = list_bin(cam)
    if b > 1:
        nbx, nby = (((cam.width + 15) // 16) + b - 1) // b, (((cam.height + 15) // 16) + b - 1) // b
        out["last_tile"] = lists[t + 2:t + 3]
        out["bins"] = lists[t + 3:t + 3 + nbx * nby + 1]
        out["walk"] = lists[t + 4 + nbx * nby:].view(t, 4, 2)
    return out


def tile_lists(cam, n, k, order, return_flags=False, return_lists=False):
    """(sorted_ids[k], ranges[T+1]) from a depth-ordered `order` buffer; with return_flags also
    the two give-up flags of the chained scans (depth sort, tile partition) as Python ints.
    The ranges are the per-tile ranges as the reference defines them whatever the bin size;
    sorted_ids holds the per-tile lists only with bins of one tile.  return_lists: the whole
    `ranges` buffer (see split_lists) instead of its first T+1 words."""
    lib = N.load()
    dev = order.device
    sorted_ids = new_sorted_ids(cam, k, dev)
    lists = torch.empty((int(lib.dsx_ranges_count(cam.width, cam.height, cam.list_bin)),), dtype=torch.int32, device=dev)
    nbytes = int(lib.dsx_workspace_bytes(n, k, cam.width, cam.height, cam.list_bin))
    ws = torch.empty((max(nbytes, 1),), dtype=torch.uint8, device=dev)
    N.check(lib.dsx_tile_lists(cam.ref, n, k, _ptr(order), _ptr(sorted_ids), _ptr(lists), _ptr(ws), nbytes, _stream()))
    ranges = lists if return_lists else lists[:cam.num_tiles + 1]
    if not return_lists:
        sorted_ids = sorted_ids[:k]      # the ids alone (binned lists carry a word of tile masks per pair behind them)
    if not return_flags:
        return sorted_ids, ranges
    p_a, p_b = C.c_void_p(), C.c_void_p()
    N.check(lib.dsx_sort_flags(n, k, cam.width, cam.height, cam.list_bin, _ptr(order), _ptr(ws) if k > 0 else None,
                               C.byref(p_a), C.byref(p_b)))
    torch.cuda.synchronize()
    read = lambda t, p: 0 if not p.value else int(t.view(torch.int32)[(p.value - t.data_ptr()) // 4].item())
    return sorted_ids, ranges, (read(order, p_a), read(ws, p_b))


def new_sorted_ids(cam, k, device):
    """The `sorted_ids` buffer for k pairs: k ids and, for binned lists, k more words (the pairs' tile masks)."""
    words = int(N.load().dsx_sorted_ids_count(k, cam.width, cam.height, cam.list_bin))
    return torch.empty((words,), dtype=torch.int32, device=device)


def sort_pairs_u32(keys, values, key_bits=32):
    """Stable ascending sort of (uint32 key, uint32 value) pairs held in int32 tensors, in place."""
    lib = N.load()
    count = keys.numel()
    nbytes = int(lib.dsx_sort_u32_workspace_bytes(count, key_bits))
    ws = torch.empty((max(nbytes, 1),), dtype=torch.uint8, device=keys.device)
    N.check(lib.dsx_sort_pairs_u32(count, key_bits, _ptr(keys), _ptr(values), _ptr(ws), nbytes, _stream()))
    return keys, values


def scan_u32(data):
    lib = N.load()
    total = torch.empty((1,), dtype=torch.int32, device=data.device)
    N.check(lib.dsx_scan_u32(data.numel(), _ptr(data), _ptr(total), _stream()))
    return total


def emit_keys(cam, n, k, splats, block_offsets):
    lib = N.load()
    keys = torch.empty((k,), dtype=torch.int64, device=splats.device)
    values = torch.empty((k,), dtype=torch.int32, device=splats.device)
    N.check(lib.dsx_emit_keys(cam.ref, n, k, _ptr(splats), _ptr(block_offsets), _ptr(keys), _ptr(values),
                              _stream()))
    return keys, values


def sort_pairs(keys, values, num_tiles, width=None, height=None):
    """Sorts in place."""
    lib = N.load()
    k = keys.numel()
    nbytes = int(lib.dsx_sort_workspace_bytes(k, num_tiles))
    ws = torch.empty((max(nbytes, 1),), dtype=torch.uint8, device=keys.device)
    N.check(lib.dsx_sort_pairs(k, num_tiles, _ptr(keys), _ptr(values), _ptr(ws), nbytes, _stream()))
    return keys, values


def tile_ranges(sorted_keys, num_tiles):
    lib = N.load()
    ranges = torch.empty((num_tiles + 1,), dtype=torch.int32, device=sorted_keys.device)
    N.check(lib.dsx_tile_ranges(sorted_keys.numel(), _ptr(sorted_keys), num_tiles, _ptr(ranges), _stream()))
    return ranges


def _pairs_in(cam, sorted_ids):
    """number of pairs k that a `sorted_ids` buffer of this camera's bin size holds"""
    return sorted_ids.numel() // (2 if list_bin(cam) > 1 else 1)


def blend_fwd(cam, ranges, sorted_ids, splats):
    """ranges, sorted_ids: the whole buffers of tile_lists(..., return_lists=True) for this camera's bin size,
    or, for per-tile lists, any tensor that starts with the T + 1 per-tile ranges and the ids."""
    lib = N.load()
    n, k = splats.shape[0], _pairs_in(cam, sorted_ids)
    dev = ranges.device
    image = torch.empty((cam.height, cam.width, 3), dtype=torch.float32, device=dev)
    final_T = torch.empty((cam.height, cam.width), dtype=torch.float32, device=dev)
    final_idx = torch.empty((cam.height, cam.width), dtype=torch.int32, device=dev)
    N.check(lib.dsx_blend_fwd(cam.ref, n, k, _ptr(ranges), _ptr(sorted_ids), _ptr(splats), _ptr(image),
                              _ptr(final_T), _ptr(final_idx), _stream()))
    return image, final_T, final_idx


def blend_bwd(cam, n, ranges, sorted_ids, splats, final_T, final_idx, v_image):
    lib = N.load()
    grads = torch.empty((n, N.GRAD_FLOATS), dtype=torch.float32, device=splats.device)
    N.check(lib.dsx_blend_bwd(cam.ref, n, _pairs_in(cam, sorted_ids), _ptr(ranges), _ptr(sorted_ids), _ptr(splats),
                              _ptr(final_T), _ptr(final_idx), _ptr(v_image), _ptr(grads), _stream()))
    return grads


def new_accumulator(n, dev):
    """The whole backward's accumulator as flat float32: dsx_grads_bytes(n) bytes, the n records of 12
    floats and, behind them, the byte per Gaussian (see accumulator_views)."""
    return torch.empty((int(N.load().dsx_grads_bytes(n)) // 4,), dtype=torch.float32, device=dev)


def accumulator_views(grads, n):
    """(records[n, 12] float32, marks[n] uint8) of a buffer of new_accumulator."""
    records = grads[:n * N.GRAD_FLOATS].view(n, N.GRAD_FLOATS)
    marks = grads[n * N.GRAD_FLOATS:].view(torch.uint8)[:n]
    return records, marks


def _bwd_outputs(n, num_bases, dev):
    e = lambda *s: torch.empty(s, dtype=torch.float32, device=dev)
    return dict(v_mean3d=e(n, 3), v_means2d=e(n, 3), v_shs=e(n, num_bases, 3) if num_bases > 0 else None,
                v_colors=e(n, 3), v_opacity=e(n, 1), v_scale=e(n, 3), v_quat=e(n, 4), v_cov3d=e(n, 6))


def gaussian_bwd(cam, num_bases, means3d, scales, quats, splats, cov3d, radii, grads):
    lib = N.load()
    n = means3d.shape[0]
    o = _bwd_outputs(n, num_bases, means3d.device)
    N.check(lib.dsx_gaussian_bwd(cam.ref, n, num_bases, _ptr(means3d), _ptr(scales), _ptr(quats), _ptr(splats),
                                 _ptr(cov3d), _ptr(radii), _ptr(grads), _ptr(o["v_mean3d"]), _ptr(o["v_means2d"]),
                                 _ptr(o["v_shs"]), _ptr(o["v_colors"]), _ptr(o["v_opacity"]), _ptr(o["v_scale"]),
                                 _ptr(o["v_quat"]), _ptr(o["v_cov3d"]), _stream()))
    return o


_pinned = threading.local()


def _pinned_i64():
    """Two pinned int64 per host thread: the landing place of the two pair counts."""
    t = getattr(_pinned, "slot", None)
    if t is None:
        t = torch.zeros((2,), dtype=torch.int64, pin_memory=True)
        _pinned.slot = t
    return t


class ForwardState:
    """What the forward keeps for the backward (the reference saves the analogous tensors
    on the autograd context, ds_splat/rasterizer.py:47-64)."""
    __slots__ = ("splats", "radii", "cov3d", "sorted_ids", "ids", "lists", "ranges", "final_T", "final_idx",
                 "num_keys", "num_keys_per_tile", "list_bin", "grads")


def sort_flag_indices(cam, n, k, order, workspace):
    """Positions (int32 index into `order`, int32 index into `workspace`; None where absent) of
    the give-up flags of the two chained scans."""
    lib = N.load()
    p_a, p_b = C.c_void_p(), C.c_void_p()
    N.check(lib.dsx_sort_flags(n, k, cam.width, cam.height, cam.list_bin, _ptr(order), _ptr(workspace) if k > 0 else None,
                               C.byref(p_a), C.byref(p_b)))
    ia = (p_a.value - order.data_ptr()) // 4 if p_a.value else None
    ib = (p_b.value - workspace.data_ptr()) // 4 if p_b.value else None
    return ia, ib


def forward(cam, means3d, scales, quats, opacities, shs, cov3d_precomp=None, colors_precomp=None,
            after_project=None, prepare_grads=False):
    """Whole forward: returns (image[H,W,3], ForwardState).  after_project(order, n, k), if given,
    runs between the two halves (diagnostics).  prepare_grads: also allocate the backward's gradient
    accumulator and let the blend kernel prepare it on the side: sums zeroed, conics in the spare
    places (one backward may then skip its fill and its reads of the splat records)."""
    lib = N.load()
    n = means3d.shape[0]
    dev = means3d.device
    st = ForwardState()
    st.splats = torch.empty((n, N.SPLAT_FLOATS), dtype=torch.float32, device=dev)
    st.radii = torch.empty((n,), dtype=torch.int32, device=dev)
    st.cov3d = torch.empty((n, 6), dtype=torch.float32, device=dev)
    block_sums = torch.empty((int(lib.dsx_num_blocks(n)),), dtype=torch.int32, device=dev)
    order = new_order(cam, n, dev)
    k_host = _pinned_i64()
    stream = _stream()
    N.check(lib.dsx_forward_project(cam.ref, n, _ptr(means3d), _ptr(scales), _ptr(quats), _ptr(opacities), _ptr(shs),
                                    _ptr(cov3d_precomp), _ptr(colors_precomp), _ptr(st.splats), _ptr(st.radii),
                                    _ptr(st.cov3d), _ptr(block_sums), _ptr(order), order.numel(),
                                    _ptr(k_host), stream))
    k = int(k_host[0].item())
    st.num_keys = k
    st.num_keys_per_tile = int(k_host[1].item())
    st.list_bin = cam.list_bin
    if after_project is not None:
        after_project(order, n, k)
    # (binned lists: k ids and, behind them, k words of tile masks; st.ids is the ids alone)
    st.sorted_ids = new_sorted_ids(cam, k, dev)
    st.ids = st.sorted_ids[:k]
    # the whole `ranges` buffer, and its first T+1 words: the per-tile ranges as the reference defines them
    st.lists = torch.empty((int(lib.dsx_ranges_count(cam.width, cam.height, cam.list_bin)),), dtype=torch.int32, device=dev)
    st.ranges = st.lists[:cam.num_tiles + 1]
    image = torch.empty((cam.height, cam.width, 3), dtype=torch.float32, device=dev)
    st.final_T = torch.empty((cam.height, cam.width), dtype=torch.float32, device=dev)
    st.final_idx = torch.empty((cam.height, cam.width), dtype=torch.int32, device=dev)
    nbytes = int(lib.dsx_workspace_bytes(n, k, cam.width, cam.height, cam.list_bin))
    ws = torch.empty((max(nbytes, 1),), dtype=torch.uint8, device=dev)
    st.grads = new_accumulator(n, dev) if prepare_grads else None
    N.check(lib.dsx_forward_finish(cam.ref, n, k, _ptr(st.splats), _ptr(order), _ptr(st.sorted_ids),
                                   _ptr(st.lists), _ptr(image), _ptr(st.final_T), _ptr(st.final_idx), _ptr(ws),
                                   nbytes, _ptr(st.grads), stream))
    return image, st


def backward(cam, st, num_bases, means3d, scales, quats, v_image):
    lib = N.load()
    n = means3d.shape[0]
    dev = means3d.device
    o = _bwd_outputs(n, num_bases, dev)
    if cam.list_bin != st.list_bin:
        raise RuntimeError("the forward built its tile lists for list_bin = %d, this camera asks for %d (a backward "
                           "must be given the list_bin of its forward)" % (st.list_bin, cam.list_bin))
    # an accumulator that the forward prepared serves one backward; after that it holds sums
    prepared = getattr(st, "grads", None) is not None
    grads = st.grads if prepared else new_accumulator(n, dev)
    st.grads = None
    N.check(lib.dsx_backward(cam.ref, n, _pairs_in(cam, st.sorted_ids), num_bases, _ptr(means3d), _ptr(scales), _ptr(quats), _ptr(st.splats),
                             _ptr(st.cov3d), _ptr(st.radii), _ptr(st.lists), _ptr(st.sorted_ids), _ptr(st.final_T),
                             _ptr(st.final_idx), _ptr(v_image), _ptr(grads), int(prepared), _ptr(o["v_mean3d"]),
                             _ptr(o["v_means2d"]), _ptr(o["v_shs"]), _ptr(o["v_colors"]), _ptr(o["v_opacity"]),
                             _ptr(o["v_scale"]), _ptr(o["v_quat"]), _ptr(o["v_cov3d"]), _stream()))
    o["grads"], o["marks"] = accumulator_views(grads, n)
    return o
