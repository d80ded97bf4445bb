"""ctypes/numpy front end of the CPU oracle (oracle/fgs_oracle.cpp).

Test infrastructure only: the test-suite, the smoke check and the CPU-baseline leg of the
benchmark load it; the shipped package never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libfgs_oracle.so")
_lib = None


def build(force=False):
    """Compile the oracle with the Makefile next to this file."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a, t=C.c_void_p):
    return a.ctypes.data_as(t) if a is not None else None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.fgs_oracle_log2f.restype = C.c_float
        L.fgs_oracle_log2f.argtypes = [C.c_float]
        L.fgs_oracle_higher_msb.restype = C.c_uint32
        L.fgs_oracle_higher_msb.argtypes = [C.c_uint32]
        L.fgs_oracle_tile_test.restype = C.c_int
        L.fgs_oracle_tile_test.argtypes = [C.c_int] * 4 + [C.c_float] * 6
        L.fgs_oracle_view_proj.restype = None
        L.fgs_oracle_view_proj.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int] + [C.c_float] * 4 + [C.c_void_p] * 2
        L.fgs_oracle_cov2d.restype = None
        L.fgs_oracle_cov2d.argtypes = [C.c_void_p] + [C.c_float] * 4 + [C.c_void_p] * 3
        L.fgs_oracle_sh_color.restype = None
        L.fgs_oracle_sh_color.argtypes = [C.c_void_p] * 4
        L.fgs_oracle_rect.restype = None
        L.fgs_oracle_rect.argtypes = [C.c_float, C.c_float] + [C.c_int] * 6 + [C.c_void_p] * 2
        L.fgs_oracle_cov3d.restype = None
        L.fgs_oracle_cov3d.argtypes = [C.c_int] + [C.c_void_p] * 3
        L.fgs_oracle_preprocess.restype = C.c_int
        L.fgs_oracle_preprocess.argtypes = (
            [C.c_int] + [C.c_void_p] * 4 + [C.c_int] * 4 + [C.c_void_p] * 2 + [C.c_float] * 4
            + [C.c_void_p] * 5 + [C.c_int64, C.c_void_p, C.c_void_p, C.c_int])
        L.fgs_oracle_sort.restype = None
        L.fgs_oracle_sort.argtypes = [C.c_int] * 5 + [C.c_void_p] * 4 + [C.c_int]
        L.fgs_oracle_ranges.restype = None
        L.fgs_oracle_ranges.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int]
        L.fgs_oracle_render.restype = None
        L.fgs_oracle_render.argtypes = [C.c_int] * 4 + [C.c_void_p] * 9 + [C.c_int]
        _lib = L
    return _lib


def default_threads():
    return max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "64"))))


# ---- scalar helpers -------------------------------------------------------------------------

def log2f(x):
    L = lib()
    x = _f32(x)
    return np.array([L.fgs_oracle_log2f(float(v)) for v in x.ravel()], dtype=np.float32).reshape(x.shape)


def higher_msb(n):
    return int(lib().fgs_oracle_higher_msb(int(n)))


def view_proj(pos, rot, width, height, fx, fy, zfar, znear):
    pos, rot = _f32(pos), _f32(rot).reshape(9)
    view = np.zeros(16, np.float32)
    proj = np.zeros(16, np.float32)
    lib().fgs_oracle_view_proj(_p(pos), _p(rot), width, height, fx, fy, zfar, znear, _p(view), _p(proj))
    return view, proj


def cov2d(p, fx, fy, tan_fovx, tan_fovy, cov3d, view):
    p, cov3d, view = _f32(p), _f32(cov3d), _f32(view)
    out = np.zeros(3, np.float32)
    lib().fgs_oracle_cov2d(_p(p), fx, fy, tan_fovx, tan_fovy, _p(cov3d), _p(view), _p(out))
    return out


def tile_test(pix_min, pix_max, center, conic, power):
    return bool(lib().fgs_oracle_tile_test(int(pix_min[0]), int(pix_min[1]), int(pix_max[0]), int(pix_max[1]),
                                           float(center[0]), float(center[1]),
                                           float(conic[0]), float(conic[1]), float(conic[2]), float(power)))


def sh_color(p, campos, sh):
    p, campos, sh = _f32(p), _f32(campos), _f32(sh).reshape(48)
    out = np.zeros(3, np.float32)
    lib().fgs_oracle_sh_color(_p(p), _p(campos), _p(sh), _p(out))
    return out


def rect(px, py, width, height, gx, gy, bx, by):
    rmin = np.zeros(2, np.int32)
    rmax = np.zeros(2, np.int32)
    lib().fgs_oracle_rect(float(px), float(py), width, height, gx, gy, bx, by, _p(rmin), _p(rmax))
    return rmin, rmax


def cov3d(scale, rot):
    scale, rot = _f32(scale), _f32(rot)
    n = scale.shape[0]
    out = np.zeros((n, 6), np.float32)
    lib().fgs_oracle_cov3d(n, _p(scale), _p(rot), _p(out))
    return out


# ---- stages ---------------------------------------------------------------------------------

def preprocess(positions, shs, opacities, cov3ds, width, height, block_x, block_y, cam_pos, cam_rot,
               fx, fy, zfar, znear, capacity, points_xy=None, rgb_depth=None, conic_opacity=None,
               start_offset=0, threads=None):
    """Returns dict(points_xy, rgb_depth, conic_opacity, keys, values, num_rendered, rc, counts)."""
    positions, shs, opacities, cov3ds = _f32(positions), _f32(shs), _f32(opacities), _f32(cov3ds)
    n = opacities.shape[0]
    assert positions.shape == (n, 3) and shs.shape == (n, 48) and cov3ds.shape == (n, 6)
    if points_xy is None:
        points_xy = np.zeros((n, 2), np.float32)
    if rgb_depth is None:
        rgb_depth = np.zeros((n, 4), np.float32)
    if conic_opacity is None:
        conic_opacity = np.zeros((n, 4), np.float32)
    keys = np.zeros(capacity, np.uint64)
    values = np.zeros(capacity, np.uint32)
    off = np.array([start_offset], np.int32)
    counts = np.zeros(4, np.int64)
    cam_pos, cam_rot = _f32(cam_pos).reshape(3), _f32(cam_rot).reshape(9)
    rc = lib().fgs_oracle_preprocess(
        n, _p(positions), _p(shs), _p(opacities), _p(cov3ds), width, height, block_x, block_y,
        _p(cam_pos), _p(cam_rot), fx, fy, zfar, znear,
        _p(points_xy), _p(rgb_depth), _p(conic_opacity), _p(keys), _p(values),
        capacity, _p(off), _p(counts), threads or default_threads())
    return dict(points_xy=points_xy, rgb_depth=rgb_depth, conic_opacity=conic_opacity, keys=keys,
                values=values, num_rendered=int(off[0]), rc=rc,
                counts=dict(n_pass=int(counts[0]), visible=int(counts[1]), keys=int(counts[2]),
                            candidates=int(counts[3])))


def sort(num_rendered, width, height, block_x, block_y, keys, values, threads=None):
    keys = np.ascontiguousarray(keys, dtype=np.uint64)
    values = np.ascontiguousarray(values, dtype=np.uint32)
    ko = np.zeros(max(num_rendered, 1), np.uint64)
    vo = np.zeros(max(num_rendered, 1), np.uint32)
    lib().fgs_oracle_sort(num_rendered, width, height, block_x, block_y, _p(keys), _p(values), _p(ko), _p(vo),
                          threads or default_threads())
    return ko[:num_rendered], vo[:num_rendered]


def ranges(num_rendered, keys_sorted, num_tiles):
    keys_sorted = np.ascontiguousarray(keys_sorted, dtype=np.uint64)
    r = np.full((num_tiles, 2), -1, np.int32)
    lib().fgs_oracle_ranges(num_rendered, _p(keys_sorted), _p(r), num_tiles)
    return r


def render(width, height, block_x, block_y, points_xy, rgb_depth, conic_opacity, values_sorted, rng, bg,
           want_u8=True, want_f32=True, threads=None):
    """Returns (u8 image or None, f32 image or None, walked)."""
    points_xy, rgb_depth, conic_opacity = _f32(points_xy), _f32(rgb_depth), _f32(conic_opacity)
    values_sorted = np.ascontiguousarray(values_sorted, dtype=np.uint32)
    rng = np.ascontiguousarray(rng, dtype=np.int32)
    bg = _f32(bg).reshape(3)
    u8 = np.zeros((height, width, 3), np.uint8) if want_u8 else None
    f32 = np.zeros((height, width, 3), np.float32) if want_f32 else None
    walked = np.zeros(1, np.int64)
    lib().fgs_oracle_render(width, height, block_x, block_y, _p(points_xy), _p(rgb_depth), _p(conic_opacity),
                            _p(values_sorted), _p(rng), _p(bg), _p(u8), _p(f32), _p(walked),
                            threads or default_threads())
    return u8, f32, int(walked[0])
