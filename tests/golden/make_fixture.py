"""Writes tests/golden/frame_small.npz: the CPU oracle's outputs for one small seeded frame.

The reference ships no vectors for this path, so this fixture does not pin the oracle against
the reference; it freezes what the pinned oracle produced when the fixture was made, so that a
later change of the scene generator, the oracle or the HIP path that alters keys, order or image
shows up as a diff against committed data.  Run from the repository root:

    python tests/golden/make_fixture.py
"""
import hashlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from flashgs_amd import scenes          # noqa: E402
from oracle import fgs_oracle as orc    # noqa: E402

N, WIDTH, HEIGHT, BLOCK, BG = 3000, 400, 240, (16, 16), (0.25, 0.5, 0.75)
CAPACITY = 1 << 18


def small_frame():
    """The fixture's scene and camera: config0's generator at 400x240."""
    sc = scenes.config0(n=N)
    cam = sc.cameras[0]
    scale = HEIGHT / cam.height
    cam.width, cam.height = WIDTH, HEIGHT
    cam.focal_x *= scale
    cam.focal_y *= scale
    return sc, cam


def input_digest(sc):
    h = hashlib.sha256()
    for a in (sc.position, sc.shs, sc.opacity, sc.cov3d):
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def main():
    sc, cam = small_frame()
    pre = orc.preprocess(sc.position, sc.shs, sc.opacity, sc.cov3d, cam.width, cam.height, BLOCK[0], BLOCK[1],
                         cam.position, cam.rotation, cam.focal_x, cam.focal_y, cam.zFar, cam.zNear, CAPACITY)
    K = pre["num_rendered"]
    ks, vs = orc.sort(K, cam.width, cam.height, BLOCK[0], BLOCK[1], pre["keys"], pre["values"])
    gx, gy = (cam.width + BLOCK[0] - 1) // BLOCK[0], (cam.height + BLOCK[1] - 1) // BLOCK[1]
    rg = orc.ranges(K, ks, gx * gy)
    u8, f32, walked = orc.render(cam.width, cam.height, BLOCK[0], BLOCK[1], pre["points_xy"], pre["rgb_depth"],
                                 pre["conic_opacity"], vs, rg, BG)
    visible = np.unique(pre["values"][:K])
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "frame_small.npz")
    np.savez_compressed(
        out,
        input_sha256=np.frombuffer(bytes.fromhex(input_digest(sc)), np.uint8),
        num_rendered=np.int64(K), walked=np.int64(walked),
        keys_unsorted=pre["keys"][:K], values_unsorted=pre["values"][:K],
        keys_sorted=ks[:K], values_sorted=vs[:K], ranges=rg,
        visible=visible.astype(np.uint32),
        points_xy=pre["points_xy"][visible], conic_opacity=pre["conic_opacity"][visible],
        rgb_depth=pre["rgb_depth"][visible],
        image_u8=u8)
    print("wrote %s: K=%d walked=%d visible=%d, %d bytes" % (out, K, walked, visible.size, os.path.getsize(out)))


if __name__ == "__main__":
    main()
