"""ctypes binding of libflashgs_hip.so (the C ABI declared in include/flashgs_hip.h).

Arguments are raw device addresses (ints) and host numpy arrays; nothing here depends on torch.
Every wrapper raises ``RuntimeError`` with the library's message when a call returns non-zero,
the way the reference's extension turns C++ exceptions into Python errors
(FlashGS ``sort.cu:40-43``).  There is no CPU fallback: a missing library is an ImportError.
"""
import ctypes as C
import os

import numpy as np

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libflashgs_hip.so")

FGS_OK, FGS_E_INVALID, FGS_E_WORKSPACE, FGS_E_HIP, FGS_E_NOMEM = 0, -1, -2, -3, -4
FGS_MAX_RENDERED = (1 << 30) - 1

_RENDER_ARGS = [C.c_int] * 3 + [C.c_void_p] * 8 + [C.c_void_p]

SIGNATURES = {
    "fgs_preprocess": (C.c_int, [C.c_int] + [C.c_void_p] * 4 + [C.c_int] * 4 + [C.c_void_p] * 2 + [C.c_float] * 4
                       + [C.c_void_p] * 6 + [C.c_int64, C.c_void_p]),
    "fgs_preprocess_static": (C.c_int, [C.c_int] + [C.c_void_p] * 4 + [C.c_int] * 4 + [C.c_void_p] * 2 + [C.c_float] * 4
                              + [C.c_void_p] * 6 + [C.c_int64, C.c_void_p]),
    "fgs_preprocess_mirrored": (C.c_int, [C.c_int] + [C.c_void_p] * 4 + [C.c_int] * 4 + [C.c_void_p] * 2 + [C.c_float] * 4
                                + [C.c_void_p] * 6 + [C.c_int64, C.c_void_p, C.c_void_p]),
    "fgs_wait_count": (C.c_int, [C.c_void_p, C.c_double, C.c_void_p]),
    "fgs_sort_gaussian": (C.c_int, [C.c_int] * 5 + [C.c_void_p, C.c_size_t] + [C.c_void_p] * 4 + [C.c_void_p]),
    "fgs_get_sort_buffer_size": (C.c_size_t, [C.c_int]),
    "fgs_render_16x16": (C.c_int, _RENDER_ARGS),
    "fgs_render_32x16": (C.c_int, _RENDER_ARGS),
    "fgs_render_32x32": (C.c_int, _RENDER_ARGS),
    "fgs_render_f32": (C.c_int, [C.c_int] * 5 + [C.c_void_p] * 9 + [C.c_void_p]),
    "fgs_tile_ranges": (C.c_int, [C.c_int] * 5 + [C.c_void_p] * 3),
    "fgs_blend": (C.c_int, [C.c_int] * 4 + [C.c_void_p] * 9),
    "fgs_render_ex": (C.c_int, [C.c_int] * 5 + [C.c_void_p] * 9 + [C.c_int, C.c_void_p]),
    "fgs_blend_ex": (C.c_int, [C.c_int] * 4 + [C.c_void_p] * 8 + [C.c_int, C.c_void_p]),
    "fgs_blend_kernel_name": (C.c_char_p, [C.c_int] * 5),
    "fgs_camera_matrices": (None, [C.c_void_p] * 2 + [C.c_int] * 2 + [C.c_float] * 4 + [C.c_void_p] * 2),
    "fgs_set_scan_spin_limit": (C.c_uint, [C.c_uint]),
    "fgs_reset_scan": (C.c_int, [C.c_void_p]),
    "fgs_set_colour_sums": (C.c_int, [C.c_int]),
    "fgs_last_error": (C.c_char_p, []),
    "fgs_abi_version": (C.c_int, []),
}

_lib = None


def load():
    """Load the library once; fails loudly if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: run `python -m flashgs_amd.build` first" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def last_error():
    return load().fgs_last_error().decode()


def _check(rc, what):
    if rc != FGS_OK:
        raise RuntimeError("%s failed (%d): %s" % (what, rc, last_error()))


def _host_f32(a, n):
    a = np.ascontiguousarray(np.asarray(a, dtype=np.float32).reshape(-1))
    if a.size != n:
        raise ValueError("expected %d floats, got %d" % (n, a.size))
    return a


def camera_matrices(position, rotation, width, height, focal_x, focal_y, zFar, zNear):
    pos, rot = _host_f32(position, 3), _host_f32(rotation, 9)
    view = np.zeros(16, np.float32)
    proj = np.zeros(16, np.float32)
    load().fgs_camera_matrices(pos.ctypes.data, rot.ctypes.data, width, height, focal_x, focal_y, zFar, zNear,
                               view.ctypes.data, proj.ctypes.data)
    return view, proj


COUNT_PENDING = -2147483647       # FGS_COUNT_PENDING: what the caller puts into the count mirror before the call


def preprocess(P, positions, shs, opacities, cov3ds, width, height, block_x, block_y, position, rotation,
               focal_x, focal_y, zFar, zNear, points_xy, rgb_depth, conic_opacity, keys, values, curr_offset,
               key_capacity=0, stream=0, static=False, count_mirror=None):
    """``static=True`` calls fgs_preprocess_static, the variant that allocates nothing;
    ``count_mirror`` (address of a word of pinned host memory holding COUNT_PENDING) calls
    fgs_preprocess_mirrored, which also stores the pair count there for `wait_count`."""
    pos, rot = _host_f32(position, 3), _host_f32(rotation, 9)
    name = "fgs_preprocess_mirrored" if count_mirror is not None else "fgs_preprocess_static" if static else "fgs_preprocess"
    if count_mirror is not None and static:
        raise ValueError("static and count_mirror exclude each other")
    tail = (key_capacity, count_mirror, stream) if count_mirror is not None else (key_capacity, stream)
    rc = getattr(load(), name)(P, positions, shs, opacities, cov3ds, width, height, block_x, block_y,
                               pos.ctypes.data, rot.ctypes.data, focal_x, focal_y, zFar, zNear,
                               points_xy, rgb_depth, conic_opacity, keys, values, curr_offset, *tail)
    _check(rc, name)


def wait_count(count_mirror, timeout_seconds=10.0):
    """Polls the count mirror of a `preprocess(..., count_mirror=...)` call; the pair count (negative: the launch gave up)."""
    out = C.c_int(0)
    _check(load().fgs_wait_count(count_mirror, float(timeout_seconds), C.addressof(out)), "fgs_wait_count")
    return out.value


COLOUR_SUMS_MATRIX_F16, COLOUR_SUMS_FP32 = 0, 1
BLEND_DEFAULT, BLEND_FP32, BLEND_MATRIX_F16 = 0, 1, 2       # the flags of render_f32 / blend / blend_kernel_name


def set_colour_sums(mode):
    """The process default of how blends form their colour sums (fp32 multiply-add, or the matrix
    unit with f16 operands); returns the previous default."""
    prev = int(load().fgs_set_colour_sums(int(mode)))
    if prev < 0:
        raise RuntimeError("fgs_set_colour_sums failed: %s" % last_error())
    return prev


def set_scan_spin_limit(polls):
    """Polls after which a wait inside the preprocess launch gives up; returns the previous value."""
    return int(load().fgs_set_scan_spin_limit(polls))


def reset_scan(stream=0):
    """Clears the scan status of preprocess on `stream` (the way back after a negative pair count)."""
    _check(load().fgs_reset_scan(stream), "fgs_reset_scan")


def get_sort_buffer_size(num_rendered):
    return int(load().fgs_get_sort_buffer_size(num_rendered))


def sort_gaussian(num_rendered, width, height, block_x, block_y, sorting_space, sorting_size,
                  keys_unsorted, values_unsorted, keys_sorted, values_sorted, stream=0):
    rc = load().fgs_sort_gaussian(num_rendered, width, height, block_x, block_y, sorting_space, sorting_size,
                                  keys_unsorted, values_unsorted, keys_sorted, values_sorted, stream)
    _check(rc, "fgs_sort_gaussian")


def render(block_x, block_y, num_rendered, width, height, points_xy, rgb_depth, conic_opacity,
           keys_sorted, values_sorted, ranges, bg_color, out_color, stream=0):
    name = "fgs_render_%dx%d" % (block_x, block_y)
    if name not in SIGNATURES:
        raise ValueError("no entry point for %dx%d tiles" % (block_x, block_y))
    bg = _host_f32(bg_color, 3)
    rc = getattr(load(), name)(num_rendered, width, height, points_xy, rgb_depth, conic_opacity,
                               keys_sorted, values_sorted, ranges, bg.ctypes.data, out_color, stream)
    _check(rc, name)


def render_f32(block_x, block_y, num_rendered, width, height, points_xy, rgb_depth, conic_opacity,
               keys_sorted, values_sorted, ranges, bg_color, out_u8, out_f32, stream=0, flags=None):
    """fgs_render_f32, or fgs_render_ex when `flags` (BLEND_*) is given."""
    bg = _host_f32(bg_color, 3)
    if flags is None:
        rc = load().fgs_render_f32(block_x, block_y, num_rendered, width, height, points_xy, rgb_depth, conic_opacity,
                                   keys_sorted, values_sorted, ranges, bg.ctypes.data, out_u8, out_f32, stream)
        _check(rc, "fgs_render_f32")
    else:
        rc = load().fgs_render_ex(block_x, block_y, num_rendered, width, height, points_xy, rgb_depth, conic_opacity,
                                  keys_sorted, values_sorted, ranges, bg.ctypes.data, out_u8, out_f32, int(flags), stream)
        _check(rc, "fgs_render_ex")


def blend_kernel_name(block_x, block_y, width, height, flags=BLEND_DEFAULT):
    """The kernel(s) a blend of this tile and frame size launches on the current device."""
    return load().fgs_blend_kernel_name(block_x, block_y, width, height, int(flags)).decode()


def tile_ranges(block_x, block_y, num_rendered, width, height, keys_sorted, ranges, stream=0):
    _check(load().fgs_tile_ranges(block_x, block_y, num_rendered, width, height, keys_sorted, ranges, stream),
           "fgs_tile_ranges")


def blend(block_x, block_y, width, height, points_xy, rgb_depth, conic_opacity, values_sorted, ranges, bg_color,
          out_u8, out_f32, stream=0, flags=None):
    """fgs_blend, or fgs_blend_ex when `flags` (BLEND_*) is given."""
    bg = _host_f32(bg_color, 3)
    if flags is None:
        _check(load().fgs_blend(block_x, block_y, width, height, points_xy, rgb_depth, conic_opacity, values_sorted,
                                ranges, bg.ctypes.data, out_u8, out_f32, stream), "fgs_blend")
    else:
        _check(load().fgs_blend_ex(block_x, block_y, width, height, points_xy, rgb_depth, conic_opacity, values_sorted,
                                   ranges, bg.ctypes.data, out_u8, out_f32, int(flags), stream), "fgs_blend_ex")
