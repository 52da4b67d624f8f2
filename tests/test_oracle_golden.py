"""The oracle against every vector the reference's own tests hold for this path
(tests/rasterizer_test.cpp): the two tile-range known-answer tests, the key-packing helper,
and the expected keys/indices of the (upstream commented-out) PrepareKeysIndicesSimple."""
import json
import os
import struct

import numpy as np

from oracle.binding import make_settings

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _key(tile, depth):
    return (int(tile) << 32) | int(depth)


def test_tile_ranges_reference_kats(oracle):
    g = json.load(open(os.path.join(GOLD, "tile_ranges_kat.json")))
    tiles = ((g["image_width"] + 15) // 16) * ((g["image_height"] + 15) // 16)
    assert tiles == 6
    for case in g["cases"]:
        keys = np.array([_key(t, d) for t, d in case["tile_depth"]], np.int64)
        got = oracle.tile_ranges(keys, tiles)
        assert got.tolist() == case["expected"], case["name"]


def test_key_packing_first_golden_key():
    # tests/rasterizer_test.cpp:52 first key: tile 10*120+88, depth bits of 315.0f
    bits = struct.unpack("<i", struct.pack("<f", 315.0))[0]
    assert bits == 0x439D8000
    assert _key(10 * 120 + 88, bits) == 5533052272640


def test_prepare_keys_reference_vector(oracle):
    """Tile rect, row-major emission order, key packing and the 'last Gaussian never
    emits' rule, against the reference authors' expected 40 keys and indices."""
    g = json.load(open(os.path.join(GOLD, "prepare_keys_kat.json")))
    W, H = g["image_width"], g["image_height"]
    s = make_settings(H, W, 1.0, 1.0, [0, 0, 0], 1.0, np.eye(4), np.eye(4), 0, [0, 0, 0])
    m = np.array(g["xy_depth"], np.float32)
    r = np.array(g["radii"], np.int32)
    tx, ty = (W + 15) // 16, (H + 15) // 16
    # independent count: tiles whose index lies in the truncated, clamped rect
    cnt = []
    for (px, py, _), rad in zip(m, r):
        lo_x, hi_x = int(px / 16 - rad / 16), int(px / 16 + rad / 16 + 1)
        lo_y, hi_y = int(py / 16 - rad / 16), int(py / 16 + rad / 16 + 1)
        nx = sum(1 for t in range(tx) if lo_x <= t < hi_x)
        ny = sum(1 for t in range(ty) if lo_y <= t < hi_y)
        cnt.append(nx * ny)
    off, k = oracle.offsets(np.array(cnt, np.int32))
    assert k == len(g["ref_keys"]) == 40          # Gaussian 9 (20 tiles) is the last: no keys
    keys, vals = oracle.emit_keys(s, m, r, off, k)
    assert keys.tolist() == g["ref_keys"]
    assert vals.tolist() == g["ref_indices"]
