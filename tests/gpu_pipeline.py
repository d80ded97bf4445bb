"""Test-side driver: runs the stages of the HIP path through the C ABI (ctypes) with torch
tensors as device memory, in the call order of FlashGS ``example.py:67-94``."""
import numpy as np
import torch

from flashgs_amd import cabi

DEV = "cuda:0"


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


class SceneOnDevice:
    def __init__(self, scene):
        self.n = scene.num_vertex
        self.position = dev(scene.position)
        self.shs = dev(scene.shs)
        self.opacity = dev(scene.opacity)
        self.cov3d = dev(scene.cov3d)


def preprocess(sd, cam, capacity, block=(16, 16), sentinel=None, start_offset=0, guard=True, pad=0, static=False,
               mirror=False):
    """Returns dict of torch tensors + num_rendered (after a sync).  The key and value buffers are
    allocated with `pad` entries beyond the capacity the library is told about.  With `mirror` the
    call is fgs_preprocess_mirrored and `mirrored` is what fgs_wait_count found in the pinned word."""
    n = sd.n
    fillv = 0.0 if sentinel is None else sentinel
    points_xy = torch.full((n, 2), fillv, device=DEV, dtype=torch.float32)
    rgb_depth = torch.full((n, 4), fillv, device=DEV, dtype=torch.float32)
    conic_opacity = torch.full((n, 4), fillv, device=DEV, dtype=torch.float32)
    keys = torch.zeros(capacity + pad, device=DEV, dtype=torch.int64)
    values = torch.zeros(capacity + pad, device=DEV, dtype=torch.int32)
    curr_offset = torch.full((1,), start_offset, device=DEV, dtype=torch.int32)
    word = torch.full((1,), 777, dtype=torch.int32).pin_memory() if mirror else None     # stale: the call marks it pending itself
    cabi.preprocess(n, sd.position.data_ptr(), sd.shs.data_ptr(), sd.opacity.data_ptr(), sd.cov3d.data_ptr(),
                    cam.width, cam.height, block[0], block[1], cam.position, cam.rotation,
                    cam.focal_x, cam.focal_y, cam.zFar, cam.zNear,
                    points_xy.data_ptr(), rgb_depth.data_ptr(), conic_opacity.data_ptr(),
                    keys.data_ptr(), values.data_ptr(), curr_offset.data_ptr(),
                    capacity if guard else 0, torch.cuda.current_stream().cuda_stream, static=static,
                    count_mirror=word.data_ptr() if mirror else None)
    mirrored = cabi.wait_count(word.data_ptr()) if mirror else None
    num = int(curr_offset.cpu()[0])
    return dict(points_xy=points_xy, rgb_depth=rgb_depth, conic_opacity=conic_opacity, keys=keys, values=values,
                num_rendered=num, mirrored=mirrored)


def sort(num, width, height, keys, values, block=(16, 16), space_for=None):
    size = cabi.get_sort_buffer_size(num if space_for is None else space_for)
    space = torch.zeros(max(size, 1), device=DEV, dtype=torch.int8)
    ks = torch.zeros(max(num, 1), device=DEV, dtype=torch.int64)
    vs = torch.zeros(max(num, 1), device=DEV, dtype=torch.int32)
    cabi.sort_gaussian(num, width, height, block[0], block[1], space.data_ptr(), size,
                       keys.data_ptr(), values.data_ptr(), ks.data_ptr(), vs.data_ptr(),
                       torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return ks, vs


def render(num, width, height, points_xy, rgb_depth, conic_opacity, ks, vs, bg, block=(16, 16), f32=True, flags=None):
    """fgs_render_f32 (or the plain fgs_render_<bx>x<by> with f32=False); with `flags` (cabi.BLEND_*)
    fgs_render_ex, which chooses the colour-sum mode for this call."""
    gx, gy = (width + block[0] - 1) // block[0], (height + block[1] - 1) // block[1]
    ranges = torch.full((gx * gy, 2), -7, device=DEV, dtype=torch.int32)
    out_u8 = torch.full((height, width, 3), 77, device=DEV, dtype=torch.uint8)
    out_f32 = torch.full((height, width, 3), -1.0, device=DEV, dtype=torch.float32) if f32 else None
    st = torch.cuda.current_stream().cuda_stream
    if f32 or flags is not None:
        cabi.render_f32(block[0], block[1], num, width, height, points_xy.data_ptr(), rgb_depth.data_ptr(),
                        conic_opacity.data_ptr(), ks.data_ptr(), vs.data_ptr(), ranges.data_ptr(), bg,
                        out_u8.data_ptr(), out_f32.data_ptr() if f32 else 0, st, flags=flags)
    else:
        cabi.render(block[0], block[1], num, width, height, points_xy.data_ptr(), rgb_depth.data_ptr(),
                    conic_opacity.data_ptr(), ks.data_ptr(), vs.data_ptr(), ranges.data_ptr(), bg,
                    out_u8.data_ptr(), st)
    torch.cuda.synchronize()
    return ranges, out_u8, out_f32


def u64(t):
    return t.cpu().numpy().view(np.uint64)


def u32(t):
    return t.cpu().numpy().view(np.uint32)


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def psnr(a, b):
    mse = float(np.mean((a.astype(np.float64) - b.astype(np.float64)) ** 2))
    return 200.0 if mse == 0 else 10.0 * np.log10(1.0 / mse)
