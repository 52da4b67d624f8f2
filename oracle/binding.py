"""ctypes binding of the CPU oracle (oracle/dsxo.cpp).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py.  Nothing in the ds_splat_amd package imports this module.
All arrays are numpy, C-contiguous; matrices are row-major "math convention" (what the
reference's native code sees after ds_splat/rasterizer.py:147-148).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


class Settings(C.Structure):
    _fields_ = [
        ("image_height", C.c_int32),
        ("image_width", C.c_int32),
        ("tanfovx", C.c_float),
        ("tanfovy", C.c_float),
        ("bg", C.c_float * 3),
        ("scale_modifier", C.c_float),
        ("view", C.c_float * 16),
        ("proj", C.c_float * 16),
        ("sh_degree", C.c_int32),
        ("max_sh_degree", C.c_int32),
        ("campos", C.c_float * 3),
    ]


class Counters(C.Structure):
    _fields_ = [
        ("pairs_fwd", C.c_int64),
        ("pairs_fwd_applied", C.c_int64),
        ("pairs_bwd", C.c_int64),
        ("pairs_bwd_valid", C.c_int64),
    ]


def make_settings(height, width, tanfovx, tanfovy, bg, scale_modifier, view_rowmajor, proj_rowmajor, sh_degree,
                  campos, max_sh_degree=3):
    s = Settings()
    s.image_height = int(height)
    s.image_width = int(width)
    s.tanfovx = float(tanfovx)
    s.tanfovy = float(tanfovy)
    s.bg[:] = [float(x) for x in np.asarray(bg, dtype=np.float32).reshape(3)]
    s.scale_modifier = float(scale_modifier)
    s.view[:] = [float(x) for x in np.asarray(view_rowmajor, dtype=np.float32).reshape(16)]
    s.proj[:] = [float(x) for x in np.asarray(proj_rowmajor, dtype=np.float32).reshape(16)]
    s.sh_degree = int(sh_degree)
    s.max_sh_degree = int(max_sh_degree)
    s.campos[:] = [float(x) for x in np.asarray(campos, dtype=np.float32).reshape(3)]
    return s


def build(force=False):
    """Compile the oracle (serial + OpenMP) with the Makefile next to this file."""
    args = ["make", "-C", _HERE, "-j2"]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def _f(a):
    return None if a is None else a.ctypes.data_as(C.POINTER(C.c_float))


def _d(a):
    return None if a is None else a.ctypes.data_as(C.POINTER(C.c_double))


def _i(a):
    return None if a is None else a.ctypes.data_as(C.POINTER(C.c_int32))


def _l(a):
    return None if a is None else a.ctypes.data_as(C.POINTER(C.c_int64))


def _c32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


class Oracle:
    """One loaded oracle library; ``omp=True`` loads the OpenMP build (CPU baseline)."""

    def __init__(self, omp=False):
        name = "libdsxo_omp.so" if omp else "libdsxo.so"
        path = os.path.join(_HERE, name)
        if not os.path.exists(path):
            build()
        self.lib = C.CDLL(path)
        L = self.lib
        L.dsxo_num_threads.restype = C.c_int
        L.dsxo_offsets.restype = C.c_int64
        L.dsxo_forward.restype = C.c_void_p
        L.dsxo_state_num_keys.restype = C.c_int64
        L.dsxo_state_num_keys.argtypes = [C.c_void_p]
        L.dsxo_state_free.argtypes = [C.c_void_p]
        L.dsxo_blend_loss_f64.restype = C.c_double

    def num_threads(self):
        return int(self.lib.dsxo_num_threads())

    # ---- per-stage -------------------------------------------------------------------
    def project_fwd(self, s, means3d, scales, quats, shs, cov3d_precomp=None, colors_precomp=None):
        n = means3d.shape[0]
        means3d, scales, quats, shs = _c32(means3d), _c32(scales), _c32(quats), _c32(shs)
        cov3d_precomp, colors_precomp = _c32(cov3d_precomp), _c32(colors_precomp)
        out = dict(
            means2d=np.empty((n, 3), np.float32), conic=np.empty((n, 3), np.float32),
            rgb=np.empty((n, 3), np.float32), radii=np.empty(n, np.int32),
            tiles_touched=np.empty(n, np.int32), cov3d=np.empty((n, 6), np.float32))
        self.lib.dsxo_project_fwd(C.byref(s), C.c_int64(n), _f(means3d), _f(scales), _f(quats), _f(shs),
                                  _f(cov3d_precomp), _f(colors_precomp), _f(out["means2d"]), _f(out["conic"]),
                                  _f(out["rgb"]), _i(out["radii"]), _i(out["tiles_touched"]), _f(out["cov3d"]))
        return out

    def offsets(self, tiles_touched):
        tiles_touched = np.ascontiguousarray(tiles_touched, np.int32)
        off = np.empty_like(tiles_touched)
        k = self.lib.dsxo_offsets(C.c_int64(len(tiles_touched)), _i(tiles_touched), _i(off))
        return off, int(k)

    def emit_keys(self, s, means2d, radii, offsets, k):
        n = means2d.shape[0]
        keys = np.empty(k, np.int64)
        vals = np.empty(k, np.int32)
        self.lib.dsxo_emit_keys(C.byref(s), C.c_int64(n), C.c_int64(k), _f(_c32(means2d)),
                                _i(np.ascontiguousarray(radii, np.int32)),
                                _i(np.ascontiguousarray(offsets, np.int32)), _l(keys), _i(vals))
        return keys, vals

    def sort_pairs(self, keys, vals):
        keys = np.array(keys, dtype=np.int64, copy=True)
        vals = np.array(vals, dtype=np.int32, copy=True)
        self.lib.dsxo_sort_pairs(C.c_int64(len(keys)), _l(keys), _i(vals))
        return keys, vals

    def tile_ranges(self, keys, num_tiles):
        keys = np.ascontiguousarray(keys, np.int64)
        ranges = np.empty(num_tiles + 1, np.int32)
        self.lib.dsxo_tile_ranges(C.c_int64(len(keys)), _l(keys), C.c_int32(num_tiles), _i(ranges))
        return ranges

    def blend_fwd(self, s, ranges, sorted_ids, means2d, conic, rgb, opacities):
        H, W = s.image_height, s.image_width
        image = np.empty((H, W, 3), np.float32)
        final_T = np.empty((H, W), np.float32)
        final_idx = np.empty((H, W), np.int32)
        margin = np.empty((H, W), np.float32)
        cnt = Counters()
        self.lib.dsxo_blend_fwd(C.byref(s), _i(np.ascontiguousarray(ranges, np.int32)),
                                _i(np.ascontiguousarray(sorted_ids, np.int32)), _f(_c32(means2d)), _f(_c32(conic)),
                                _f(_c32(rgb)), _f(_c32(opacities).reshape(-1)), _f(image), _f(final_T),
                                _i(final_idx), _f(margin), C.byref(cnt))
        return dict(image=image, final_T=final_T, final_idx=final_idx, margin=margin, counters=cnt)

    def blend_bwd(self, s, ranges, sorted_ids, means2d, conic, rgb, opacities, final_T, final_idx, v_out,
                  v_out_alpha=None):
        n = means2d.shape[0]
        out = dict(v_xy=np.empty((n, 2), np.float32), v_conic=np.empty((n, 3), np.float32),
                   v_rgb=np.empty((n, 3), np.float32), v_opacity=np.empty((n, 1), np.float32),
                   g_margin=np.empty(n, np.float32), abs_sums=np.empty((n, 9), np.float32))
        cnt = Counters()
        self.lib.dsxo_blend_bwd_ex(C.byref(s), C.c_int64(n), _i(np.ascontiguousarray(ranges, np.int32)),
                                _i(np.ascontiguousarray(sorted_ids, np.int32)), _f(_c32(means2d)), _f(_c32(conic)),
                                _f(_c32(rgb)), _f(_c32(opacities).reshape(-1)), _f(_c32(final_T)),
                                _i(np.ascontiguousarray(final_idx, np.int32)), _f(_c32(v_out)), _f(_c32(v_out_alpha)),
                                _f(out["v_xy"]), _f(out["v_conic"]), _f(out["v_rgb"]), _f(out["v_opacity"]),
                                _f(out["g_margin"]), C.byref(cnt), _f(out["abs_sums"]))
        out["counters"] = cnt
        return out

    def sh_bwd(self, s, num_bases, means3d, v_rgb):
        n = means3d.shape[0]
        v_shs = np.empty((n, num_bases, 3), np.float32)
        self.lib.dsxo_sh_bwd(C.byref(s), C.c_int64(n), C.c_int32(num_bases), _f(_c32(means3d)), _f(_c32(v_rgb)),
                             _f(v_shs))
        return v_shs

    def project_bwd(self, s, means3d, scales, quats, conic, cov3d, radii, v_xy, v_conic):
        n = means3d.shape[0]
        out = dict(v_mean3d=np.empty((n, 3), np.float32), v_scale=np.empty((n, 3), np.float32),
                   v_quat=np.empty((n, 4), np.float32), v_cov3d=np.empty((n, 6), np.float32),
                   v_cov2d=np.empty((n, 3), np.float32))
        self.lib.dsxo_project_bwd(C.byref(s), C.c_int64(n), _f(_c32(means3d)), _f(_c32(scales)), _f(_c32(quats)),
                                  _f(_c32(conic)), _f(_c32(cov3d)), _i(np.ascontiguousarray(radii, np.int32)),
                                  _f(_c32(v_xy)), _f(_c32(v_conic)), _f(out["v_mean3d"]), _f(out["v_scale"]),
                                  _f(out["v_quat"]), _f(out["v_cov3d"]), _f(out["v_cov2d"]))
        return out

    # ---- whole pipeline --------------------------------------------------------------
    def forward(self, s, means3d, scales, quats, opacities, shs, cov3d_precomp=None, colors_precomp=None,
                want_state=True, keep_emitted=False):
        """Returns (image, radii, handle).  ``handle`` must go to backward() or free()."""
        n = means3d.shape[0]
        H, W = s.image_height, s.image_width
        self._in = [_c32(means3d), _c32(scales), _c32(quats), _c32(opacities).reshape(-1), _c32(shs),
                    _c32(cov3d_precomp), _c32(colors_precomp)]
        image = np.empty((H, W, 3), np.float32)
        radii = np.empty(n, np.int32)
        self.lib.dsxo_keep_emitted(C.c_int(1 if keep_emitted else 0))
        st = self.lib.dsxo_forward(C.byref(s), C.c_int64(n), *[_f(a) for a in self._in], _f(image), _i(radii))
        st = C.c_void_p(st)
        if not want_state:
            self.free(st)
            st = None
        return image, radii, st

    def state(self, s, st, n, emitted=False):
        H, W = s.image_height, s.image_width
        T = ((H + 15) // 16) * ((W + 15) // 16)
        k = int(self.lib.dsxo_state_num_keys(st))
        o = dict(means2d=np.empty((n, 3), np.float32), conic=np.empty((n, 3), np.float32),
                 rgb=np.empty((n, 3), np.float32), tiles_touched=np.empty(n, np.int32),
                 offsets=np.empty(n, np.int32), cov3d=np.empty((n, 6), np.float32),
                 sorted_keys=np.empty(k, np.int64), sorted_ids=np.empty(k, np.int32),
                 ranges=np.empty(T + 1, np.int32), final_T=np.empty((H, W), np.float32),
                 final_idx=np.empty((H, W), np.int32), margin=np.empty((H, W), np.float32))
        cnt = Counters()
        self.lib.dsxo_state_get(st, _f(o["means2d"]), _f(o["conic"]), _f(o["rgb"]), _i(o["tiles_touched"]),
                                _i(o["offsets"]), _f(o["cov3d"]), _l(o["sorted_keys"]), _i(o["sorted_ids"]),
                                _i(o["ranges"]), _f(o["final_T"]), _i(o["final_idx"]), _f(o["margin"]),
                                C.byref(cnt))
        o["counters"] = cnt
        o["num_keys"] = k
        if emitted:
            o["emitted_keys"] = np.empty(k, np.int64)
            o["emitted_values"] = np.empty(k, np.int32)
            self.lib.dsxo_state_get_emitted(st, _l(o["emitted_keys"]), _i(o["emitted_values"]))
        return o

    def backward(self, s, st, num_bases, means3d, scales, quats, opacities, v_image):
        n = means3d.shape[0]
        o = dict(v_mean3d=np.empty((n, 3), np.float32), v_means2d=np.empty((n, 3), np.float32),
                 v_shs=np.empty((n, num_bases, 3), np.float32), v_colors=np.empty((n, 3), np.float32),
                 v_opacity=np.empty((n, 1), np.float32), v_scale=np.empty((n, 3), np.float32),
                 v_quat=np.empty((n, 4), np.float32), v_cov3d=np.empty((n, 6), np.float32),
                 g_margin=np.empty(n, np.float32), abs_sums=np.empty((n, 9), np.float32))
        self.lib.dsxo_backward_ex(st, C.byref(s), C.c_int64(n), C.c_int32(num_bases), _f(_c32(means3d)),
                               _f(_c32(scales)), _f(_c32(quats)), _f(_c32(opacities).reshape(-1)),
                               _f(_c32(v_image)), _f(o["v_mean3d"]), _f(o["v_means2d"]), _f(o["v_shs"]),
                               _f(o["v_colors"]), _f(o["v_opacity"]), _f(o["v_scale"]), _f(o["v_quat"]),
                               _f(o["v_cov3d"]), _f(o["g_margin"]), _f(o["abs_sums"]))
        cnt = Counters()
        self.lib.dsxo_state_get(st, *([None] * 12), C.byref(cnt))
        o["counters"] = cnt
        return o

    def free(self, st):
        if st is not None:
            self.lib.dsxo_state_free(st)

    def gradient_bounds(self, s, num_bases, means3d, scales, quats, conic, cov3d, radii, abs_sums, rel=1e-3,
                        floor=1e-7):
        """Per-element tolerances for the gradients of a backward whose nine screen-space sums were
        accumulated in another order than the oracle's (float atomics).

        abs_sums[N,9] (from blend_bwd / backward) is, per Gaussian, the sum of the absolute values
        of the terms of each screen-space sum: a reordered float summation may be off by
        ``rel * abs_sums + floor`` there.  The outputs of the per-Gaussian backward are linear in
        those sums; the Jacobian's columns come from running the oracle's projection backward on
        unit inputs, and the bound of an output element is own = sum_k |J_k| * (rel * abs_sums_k + floor)
        plus, for the outputs that come out of chains of small matrix products (v_mean3d, v_scale,
        v_quat, v_cov3d, v_shs), the largest `own` of the same Gaussian's row of that output: an
        element that is small because its chain cancels carries rounding errors of the size of its
        neighbours (measured on the GPU against this oracle: up to 4e-3 of `own`, never above 2e-5
        of the row's largest).  Nothing is scaled by a whole tensor.
        Returns a dict with the keys of backward()."""
        n = means3d.shape[0]
        eps = (rel * np.asarray(abs_sums, np.float64) + floor)          # x y | a b c | opacity | r g b
        out = dict(v_means2d=np.concatenate([eps[:, 0:2], np.zeros((n, 1))], axis=1), v_opacity=eps[:, 5:6].copy(),
                   v_colors=eps[:, 6:9].copy())
        ones = np.ones((n, 3), np.float32)
        Y = np.abs(self.sh_bwd(s, num_bases, means3d, ones)[:, :, 0].astype(np.float64))   # |Y_b| per Gaussian
        with_row_max = lambda own: own + own.reshape(n, -1).max(axis=1).reshape((n,) + (1,) * (own.ndim - 1))
        out["v_shs"] = with_row_max(Y[:, :, None] * eps[:, None, 6:9])
        acc = None
        for k in range(5):
            v_xy = np.zeros((n, 2), np.float32)
            v_conic = np.zeros((n, 3), np.float32)
            if k < 2:
                v_xy[:, k] = 1.0
            else:
                v_conic[:, k - 2] = 1.0
            J = self.project_bwd(s, means3d, scales, quats, conic, cov3d, radii, v_xy, v_conic)
            if acc is None:
                acc = {key: np.zeros(J[key].shape, np.float64) for key in ("v_mean3d", "v_scale", "v_quat", "v_cov3d")}
            for key in acc:
                acc[key] += np.abs(J[key].astype(np.float64)) * eps[:, k:k + 1]
        out.update({key: with_row_max(own) for key, own in acc.items()})
        return out

    # ---- float64 instances -----------------------------------------------------------
    def blend_loss_f64(self, width, height, ranges, sorted_ids, xy, conic, rgb, opac, weights, alpha_clamp,
                       bg=None):
        a = [np.ascontiguousarray(x, np.float64) for x in (xy, conic, rgb, opac, weights)]
        bg = None if bg is None else np.ascontiguousarray(bg, np.float64)
        return float(self.lib.dsxo_blend_loss_f64(
            C.c_int32(width), C.c_int32(height), _i(np.ascontiguousarray(ranges, np.int32)),
            _i(np.ascontiguousarray(sorted_ids, np.int32)), C.c_int64(xy.shape[0]), *[_d(x) for x in a],
            _d(bg), C.c_double(alpha_clamp)))
