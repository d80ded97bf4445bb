"""Driver with the shape of FlashGS's ``example.py``: ``Scene``, ``Camera``, a statically allocated
``Rasterizer`` whose ``forward`` runs preprocess -> pair count -> sort_gaussian -> render_16x16
through ``flash_gaussian_splatting.ops``, ``savePpm`` and ``render_scene``.

Differences from the reference driver: the output image is allocated once instead of per frame,
the pair count is polled in pinned host memory, where the preprocess launch stores it as soon as
it is known (``ops.preprocess_mirrored`` / ``ops.wait_count``), instead of being copied back with
a blocking read,
the too-many-pairs condition raises a real exception (``example.py:82`` raises a string), a
preprocess whose bounded waits gave up is launched once more after ``ops.reset_scan`` and raises
``ScanGaveUp`` if that fails too, and the tile size is a constructor argument.  ``BatchRasterizer``
renders a list of cameras with several frames in flight on streams of their own.
"""
import json
import os
import time

import numpy as np
import torch

_ops = None


def ops():
    """The compiled operator module; importing it fails loudly if it has not been built."""
    global _ops
    if _ops is None:
        import flash_gaussian_splatting
        _ops = flash_gaussian_splatting.ops
    return _ops


class Scene:
    """example.py:10-27"""

    def __init__(self, device):
        self.device = device
        self.num_vertex = 0
        self.position = None
        self.shs = None
        self.opacity = None
        self.cov3d = None

    def loadPly(self, scene_path):
        self.num_vertex, position, shs, opacity, cov3d = ops().loadPly(scene_path)
        self._to_device(position, shs, opacity, cov3d)

    def from_arrays(self, position, shs, opacity, cov3d):
        """Same tensors from host arrays (numpy or torch), e.g. ``flashgs_amd.scenes``."""
        t = [torch.as_tensor(np.ascontiguousarray(a), dtype=torch.float32) for a in (position, shs, opacity, cov3d)]
        self.num_vertex = int(t[2].shape[0])
        self._to_device(*t)
        return self

    def _to_device(self, position, shs, opacity, cov3d):
        self.position = position.to(self.device).contiguous()
        self.shs = shs.to(self.device).contiguous()
        self.opacity = opacity.to(self.device).contiguous()
        self.cov3d = cov3d.to(self.device).contiguous()


class Camera:
    """example.py:30-41: one entry of a 3DGS ``cameras.json``."""

    def __init__(self, camera_json):
        self.id = camera_json.get('id', 0)
        self.img_name = camera_json.get('img_name', str(self.id))
        self.width = int(camera_json['width'])
        self.height = int(camera_json['height'])
        self.position = torch.tensor(camera_json['position'], dtype=torch.float32)
        self.rotation = torch.tensor(camera_json['rotation'], dtype=torch.float32)
        self.focal_x = float(camera_json['fx'])
        self.focal_y = float(camera_json['fy'])
        self.zFar = 100.0
        self.zNear = 0.01

    @classmethod
    def from_synthetic(cls, cam, cam_id=0):
        return cls(dict(id=cam_id, img_name="%05d" % cam_id, width=cam.width, height=cam.height,
                        position=[float(v) for v in cam.position],
                        rotation=[[float(v) for v in row] for row in np.asarray(cam.rotation).reshape(3, 3)],
                        fx=cam.focal_x, fy=cam.focal_y))


class TooManyPairs(RuntimeError):
    """More (tile, Gaussian) pairs than the key buffers hold (example.py:81-82)."""


class ScanGaveUp(RuntimeError):
    """A wait inside the preprocess launch ran into its poll limit, twice in a row: the pair
    count came back negative although the frame was launched again on cleared scan status."""


class Rasterizer:
    """example.py:44-94: all buffers are allocated once, ``forward`` allocates nothing."""

    RENDER = {(16, 16): "render_16x16", (32, 16): "render_32x16", (32, 32): "render_32x32"}

    def __init__(self, scene, MAX_NUM_RENDERED, MAX_NUM_TILES, tile=(16, 16), max_width=0, max_height=0):
        dev = scene.device
        self.tile = tuple(tile)
        self._render = getattr(ops(), self.RENDER[self.tile])
        self.gaussian_keys_unsorted = torch.zeros(MAX_NUM_RENDERED, device=dev, dtype=torch.int64)
        self.gaussian_values_unsorted = torch.zeros(MAX_NUM_RENDERED, device=dev, dtype=torch.int32)
        self.gaussian_keys_sorted = torch.zeros(MAX_NUM_RENDERED, device=dev, dtype=torch.int64)
        self.gaussian_values_sorted = torch.zeros(MAX_NUM_RENDERED, device=dev, dtype=torch.int32)
        self.MAX_NUM_RENDERED = MAX_NUM_RENDERED
        self.MAX_NUM_TILES = MAX_NUM_TILES
        self.SORT_BUFFER_SIZE = ops().get_sort_buffer_size(MAX_NUM_RENDERED)
        self.list_sorting_space = torch.zeros(self.SORT_BUFFER_SIZE, device=dev, dtype=torch.int8)
        self.ranges = torch.zeros((MAX_NUM_TILES, 2), device=dev, dtype=torch.int32)
        self.curr_offset = torch.zeros(1, device=dev, dtype=torch.int32)
        self.points_xy = torch.zeros((scene.num_vertex, 2), device=dev, dtype=torch.float32)
        self.rgb_depth = torch.zeros((scene.num_vertex, 4), device=dev, dtype=torch.float32)
        self.conic_opacity = torch.zeros((scene.num_vertex, 4), device=dev, dtype=torch.float32)
        # the launch stores the pair count here as soon as it has it; forward polls this word
        # instead of the blocking device-to-host copy of example.py:79
        self._count = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        self._out = None
        if max_width and max_height:
            self._out = torch.zeros((max_height, max_width, 3), device=dev, dtype=torch.uint8)
        self.num_rendered = 0

    def _image(self, camera, device):
        if self._out is None or self._out.shape[0] != camera.height or self._out.shape[1] != camera.width:
            self._out = torch.zeros((camera.height, camera.width, 3), device=device, dtype=torch.uint8)
        return self._out

    def forward(self, scene, camera, bg_color, out=None):
        """One frame.  The image is the rasterizer's own buffer (overwritten by the next frame) or,
        if given, `out`: a contiguous uint8 (or int8) GPU tensor of height x width x 3."""
        o = ops()
        bx, by = self.tile
        tiles = ((camera.width + bx - 1) // bx) * ((camera.height + by - 1) // by)
        if tiles > self.MAX_NUM_TILES:
            raise ValueError("image needs %d tiles, MAX_NUM_TILES is %d" % (tiles, self.MAX_NUM_TILES))
        if self.num_rendered >= 0 and int(self._count[0]) < 0:
            # the count of the last frame was good when it arrived, and a wait of one workgroup gave up after that
            self.num_rendered = -1
            o.reset_scan(self.curr_offset)
            raise ScanGaveUp("a workgroup of the previous frame's preprocess gave up waiting after the pair count "
                             "had been reported; that frame's image is not to be used")
        for attempt in range(2):
            self.curr_offset.zero_()
            o.preprocess_mirrored(scene.position, scene.shs, scene.opacity, scene.cov3d,
                                  camera.width, camera.height, bx, by,
                                  camera.position, camera.rotation,
                                  camera.focal_x, camera.focal_y, camera.zFar, camera.zNear,
                                  self.points_xy, self.rgb_depth, self.conic_opacity,
                                  self.gaussian_keys_unsorted, self.gaussian_values_unsorted, self.curr_offset, self._count)
            # the count arrives while the launch is still writing keys; the sort below is enqueued
            # behind it on the same stream
            num_rendered = o.wait_count(self._count, 60.0)
            if num_rendered >= 0:
                break
            # a bounded wait of the launch gave up: clear the scan status and launch once more
            o.reset_scan(self.curr_offset)
        self.num_rendered = num_rendered
        if num_rendered < 0:
            raise ScanGaveUp("preprocess gave up waiting for its scan over workgroups twice in a row "
                             "(fgs_set_scan_spin_limit polls); the frame was not rendered")
        if num_rendered >= self.MAX_NUM_RENDERED:
            raise TooManyPairs("Too many k-v pairs! (%d, capacity %d)" % (num_rendered, self.MAX_NUM_RENDERED))
        o.sort_gaussian(num_rendered, camera.width, camera.height, bx, by, self.list_sorting_space,
                        self.gaussian_keys_unsorted, self.gaussian_values_unsorted,
                        self.gaussian_keys_sorted, self.gaussian_values_sorted)
        out_color = self._image(camera, scene.device) if out is None else out
        self._render(num_rendered, camera.width, camera.height,
                     self.points_xy, self.rgb_depth, self.conic_opacity,
                     self.gaussian_keys_sorted, self.gaussian_values_sorted,
                     self.ranges, bg_color, out_color)
        return out_color


class BatchRasterizer:
    """Renders a list of cameras with several frames in flight (no counterpart in the reference,
    whose driver renders one frame after the other on one stream).

    Every frame in flight has a `Rasterizer` - key, sort and attribute buffers - and a stream of
    its own; the cameras go to them in turn.  The stages of one frame still follow each other,
    but one frame's blend, which is bound by instruction issue, runs beside the next frame's
    preprocess and sort, which are bound by memory, and a launch that leaves CUs idle (the tail
    of a preprocess, the short kernels of a small frame) has the other frame's work to fill them.
    The images are what `Rasterizer.forward` renders, frame by frame."""

    def __init__(self, scene, MAX_NUM_RENDERED, MAX_NUM_TILES, frames_in_flight=2, tile=(16, 16)):
        if frames_in_flight < 1:
            raise ValueError("frames_in_flight must be at least 1")
        self.rasterizers = [Rasterizer(scene, MAX_NUM_RENDERED, MAX_NUM_TILES, tile) for _ in range(frames_in_flight)]
        self.streams = [torch.cuda.Stream(device=scene.device) for _ in range(frames_in_flight)]

    def render(self, scene, cameras, bg_color, out=None):
        """All `cameras` (of one image size); returns a uint8 tensor [len(cameras), height, width, 3]
        (or fills `out`), ready for use on the current stream of the scene's device."""
        cameras = list(cameras)
        if not cameras:
            return out
        h, w = cameras[0].height, cameras[0].width
        if any(c.height != h or c.width != w for c in cameras):
            raise ValueError("the cameras of a batch must have one image size")
        if out is None:
            out = torch.empty((len(cameras), h, w, 3), device=scene.device, dtype=torch.uint8)
        if tuple(out.shape) != (len(cameras), h, w, 3) or not out.is_contiguous():
            raise ValueError("out must be a contiguous tensor of shape %r" % ((len(cameras), h, w, 3),))
        caller = torch.cuda.current_stream(scene.device)
        for s in self.streams:
            s.wait_stream(caller)              # the scene and `out` as the caller's stream leaves them
        for i, camera in enumerate(cameras):
            j = i % len(self.streams)
            with torch.cuda.stream(self.streams[j]):
                self.rasterizers[j].forward(scene, camera, bg_color, out=out[i])
        for s in self.streams:
            caller.wait_stream(s)
        return out


def savePpm(image, path):
    """example.py:97-102: binary P6."""
    image = image.cpu()
    assert image.dim() >= 3 and image.size(2) == 3
    with open(path, 'wb') as f:
        f.write(b'P6\n' + f'{image.size(1)} {image.size(0)}\n255\n'.encode() + image.numpy().tobytes())


def render_scene(model_path, test_performance=False, device='cuda:0', MAX_NUM_RENDERED=2 ** 27, MAX_NUM_TILES=2 ** 20,
                 frames_in_flight=1):
    """example.py:105-144: render every camera of ``<model_path>/cameras.json`` to ``test_out/*.ppm``.
    With ``frames_in_flight`` above 1 and ``test_performance`` the cameras of one image size are
    also timed as a batch through ``BatchRasterizer``."""
    scene_path = os.path.join(model_path, "point_cloud", "iteration_30000", "point_cloud.ply")
    camera_path = os.path.join(model_path, "cameras.json")
    device = torch.device(device)
    bg_color = torch.zeros(3, dtype=torch.float32)
    scene = Scene(device)
    scene.loadPly(scene_path)
    print("num_vertex = %d" % scene.num_vertex)
    with open(camera_path, 'r') as camera_file:
        cameras_json = json.load(camera_file)
    image_dir = os.path.join(model_path, "test_out")
    os.makedirs(image_dir, exist_ok=True)
    rasterizer = Rasterizer(scene, MAX_NUM_RENDERED, MAX_NUM_TILES)
    for camera_json in cameras_json:
        camera = Camera(camera_json)
        print("image name = %s" % camera.img_name)
        image = rasterizer.forward(scene, camera, bg_color)
        if test_performance:
            n = 10
            torch.cuda.synchronize()
            t0 = time.time()
            for _ in range(n):
                image = rasterizer.forward(scene, camera, bg_color)
            torch.cuda.synchronize()
            t1 = time.time()
            print("elapsed time = %f ms" % ((t1 - t0) / n * 1000))
            print("fps = %f" % (n / (t1 - t0)))
        savePpm(image, os.path.join(image_dir, "%s.ppm" % camera.img_name))
    if test_performance and frames_in_flight > 1 and cameras_json:
        cameras = [Camera(c) for c in cameras_json]
        cameras = [c for c in cameras if (c.width, c.height) == (cameras[0].width, cameras[0].height)]
        del rasterizer
        batch = BatchRasterizer(scene, MAX_NUM_RENDERED, MAX_NUM_TILES, frames_in_flight=frames_in_flight)
        out = batch.render(scene, cameras, bg_color)
        torch.cuda.synchronize()
        t0 = time.time()
        batch.render(scene, cameras, bg_color, out=out)
        torch.cuda.synchronize()
        t1 = time.time()
        print("batch of %d cameras, %d frames in flight: elapsed time per frame = %f ms, fps = %f"
              % (len(cameras), frames_in_flight, (t1 - t0) / len(cameras) * 1000, len(cameras) / (t1 - t0)))


if __name__ == "__main__":
    import sys
    if len(sys.argv) < 2:
        sys.exit("usage: python -m flashgs_amd.rasterizer <model_path>")
    render_scene(sys.argv[1], True)
