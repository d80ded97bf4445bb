"""The op surface on the GPU, used the way FlashGS's example.py uses it: ``Rasterizer.forward``
through ``flash_gaussian_splatting.ops`` against the oracle, and the error behaviour of the ops."""
import numpy as np
import pytest
import torch

from flashgs_amd import scenes
from flashgs_amd.rasterizer import Camera, Rasterizer, Scene, TooManyPairs, savePpm

pytestmark = pytest.mark.gpu


def _setup(n=40_000, cap=1 << 19, tile=(16, 16)):
    sc = scenes.config0(n=n)
    scene = Scene(torch.device("cuda:0")).from_arrays(sc.position, sc.shs, sc.opacity, sc.cov3d)
    return sc, scene, Camera.from_synthetic(sc.cameras[0]), Rasterizer(scene, cap, 1 << 14, tile=tile)


@pytest.mark.parametrize("tile", [(16, 16), (32, 16), (32, 32)])
def test_rasterizer_forward_matches_oracle(oracle, tile, tmp_path):
    sc, scene, cam, rast = _setup(tile=tile)
    c0 = sc.cameras[0]
    bg = torch.tensor([0.0, 0.2, 0.4])
    img = rast.forward(scene, cam, bg)
    img2 = rast.forward(scene, cam, bg).cpu().numpy()          # a second frame reuses every buffer
    K = rast.num_rendered
    pre = oracle.preprocess(sc.position, sc.shs, sc.opacity, sc.cov3d, c0.width, c0.height, tile[0], tile[1],
                            c0.position, c0.rotation, c0.focal_x, c0.focal_y, c0.zFar, c0.zNear, 1 << 19)
    assert pre["num_rendered"] == K
    ks, vs = oracle.sort(K, c0.width, c0.height, tile[0], tile[1], pre["keys"], pre["values"])
    assert np.array_equal(rast.gaussian_keys_sorted[:K].cpu().numpy().view(np.uint64), ks)
    assert np.array_equal(rast.gaussian_values_sorted[:K].cpu().numpy().view(np.uint32), vs)
    gx, gy = (c0.width + tile[0] - 1) // tile[0], (c0.height + tile[1] - 1) // tile[1]
    rg = oracle.ranges(K, ks, gx * gy)
    assert np.array_equal(rast.ranges[:gx * gy].cpu().numpy(), rg)
    u8, _, _ = oracle.render(c0.width, c0.height, tile[0], tile[1], pre["points_xy"], pre["rgb_depth"],
                             pre["conic_opacity"], vs, rg, bg.numpy(), want_f32=False)
    d = np.abs(img2.astype(np.int16) - u8.astype(np.int16))
    assert d.max() <= 1 and (d > 0).mean() < 0.02
    path = tmp_path / "frame.ppm"
    savePpm(img, str(path))
    data = path.read_bytes()
    assert data.startswith(b"P6\n%d %d\n255\n" % (c0.width, c0.height))


def test_int8_image_like_the_reference_driver():
    """example.py:89 allocates the image as int8; the op accepts any 1-byte dtype."""
    import flash_gaussian_splatting as fgs
    sc, scene, cam, rast = _setup(n=5000)
    bg = torch.zeros(3)
    ref = rast.forward(scene, cam, bg).clone()
    out = torch.zeros((cam.height, cam.width, 3), device="cuda:0", dtype=torch.int8)
    fgs.ops.render_16x16(rast.num_rendered, cam.width, cam.height, rast.points_xy, rast.rgb_depth, rast.conic_opacity,
                         rast.gaussian_keys_sorted, rast.gaussian_values_sorted, rast.ranges, bg, out)
    assert torch.equal(out.view(torch.uint8), ref)


def test_too_many_pairs_raises():
    sc, scene, cam, _ = _setup(n=40_000)
    small = Rasterizer(scene, 1000, 1 << 14)
    with pytest.raises(TooManyPairs):
        small.forward(scene, cam, torch.zeros(3))


def test_ops_errors_on_the_gpu():
    import flash_gaussian_splatting as fgs
    sc, scene, cam, rast = _setup(n=5000)
    rast.forward(scene, cam, torch.zeros(3))
    K = rast.num_rendered
    tiny = torch.zeros(64, device="cuda:0", dtype=torch.int8)
    with pytest.raises(RuntimeError, match="needed"):            # workspace too small
        fgs.ops.sort_gaussian(K, cam.width, cam.height, 16, 16, tiny, rast.gaussian_keys_unsorted,
                              rast.gaussian_values_unsorted, rast.gaussian_keys_sorted, rast.gaussian_values_sorted)
    with pytest.raises(RuntimeError, match="contiguous"):
        fgs.ops.preprocess(scene.position, scene.shs, scene.opacity, scene.cov3d, cam.width, cam.height, 16, 16,
                           cam.position, cam.rotation, cam.focal_x, cam.focal_y, cam.zFar, cam.zNear,
                           torch.zeros((scene.num_vertex, 4), device="cuda:0")[:, :2], rast.rgb_depth, rast.conic_opacity,
                           rast.gaussian_keys_unsorted, rast.gaussian_values_unsorted, rast.curr_offset)
    with pytest.raises(RuntimeError, match="dtype"):
        fgs.ops.preprocess(scene.position, scene.shs, scene.opacity, scene.cov3d, cam.width, cam.height, 16, 16,
                           cam.position, cam.rotation, cam.focal_x, cam.focal_y, cam.zFar, cam.zNear,
                           rast.points_xy, rast.rgb_depth, rast.conic_opacity,
                           rast.gaussian_keys_unsorted.to(torch.int32), rast.gaussian_values_unsorted, rast.curr_offset)
    with pytest.raises(RuntimeError, match="too small"):
        fgs.ops.render_16x16(K, cam.width, cam.height, rast.points_xy, rast.rgb_depth, rast.conic_opacity,
                             rast.gaussian_keys_sorted, rast.gaussian_values_sorted, rast.ranges[:10], torch.zeros(3),
                             torch.zeros((cam.height, cam.width, 3), device="cuda:0", dtype=torch.uint8))


def _write_ply(path, recs):
    props = ["x", "y", "z", "nx", "ny", "nz"] + ["f_dc_%d" % i for i in range(3)] + ["f_rest_%d" % i for i in range(45)] \
        + ["opacity"] + ["scale_%d" % i for i in range(3)] + ["rot_%d" % i for i in range(4)]
    head = "ply\nformat binary_little_endian 1.0\nelement vertex %d\n" % len(recs)
    head += "".join("property float %s\n" % p for p in props) + "end_header\n"
    with open(path, "wb") as fh:
        fh.write(head.encode())
        fh.write(np.ascontiguousarray(recs, dtype="<f4").tobytes())


def test_render_scene_from_ply_and_cameras_json(oracle, tmp_path, capsys):
    """The file path of example.py:105-144: a 3DGS model directory (point_cloud.ply of 62-float
    records + cameras.json) goes through loadPly -> device -> preprocess -> sort -> render -> .ppm,
    and every image is the oracle's image of the same Gaussians (those loadPly returns)."""
    import json
    import flash_gaussian_splatting as fgs
    from flashgs_amd.rasterizer import render_scene
    rng = np.random.default_rng(21)
    n = 30_000
    recs = np.zeros((n, 62), np.float32)
    recs[:, 0:3] = rng.uniform(-5.0, 5.0, (n, 3))
    recs[:, 3:6] = rng.standard_normal((n, 3))                   # normals: ignored by the loader
    recs[:, 6:9] = 0.5 * rng.standard_normal((n, 3))             # f_dc
    recs[:, 9:54] = 0.05 * rng.standard_normal((n, 45))          # f_rest, planar
    recs[:, 54] = 1.5 * rng.standard_normal(n)                   # opacity logit
    recs[:, 55:58] = -3.2 + 0.6 * rng.standard_normal((n, 3))    # log-scales
    recs[:, 58:62] = rng.standard_normal((n, 4)) * 3.0           # quaternion, not normalised
    model = tmp_path / "model"
    ply_dir = model / "point_cloud" / "iteration_30000"
    ply_dir.mkdir(parents=True)
    _write_ply(str(ply_dir / "point_cloud.ply"), recs)
    cams = []
    for k, (w, h, pos) in enumerate([(1280, 720, [0.0, 0.0, -15.0]), (1000, 600, [1.0, -0.5, -13.0])]):
        c = scenes.look_at(pos, [0, 0, 0], w, h, 50.0)
        cams.append(dict(id=k, img_name="view_%d" % k, width=w, height=h, position=[float(v) for v in c.position],
                         rotation=[[float(v) for v in row] for row in c.rotation], fx=c.focal_x, fy=c.focal_y))
    (model / "cameras.json").write_text(json.dumps(cams))

    render_scene(str(model), test_performance=True, MAX_NUM_RENDERED=1 << 20, MAX_NUM_TILES=1 << 13, frames_in_flight=2)
    out = capsys.readouterr().out
    assert "num_vertex = %d" % n in out and "fps = " in out
    assert "batch of 1 cameras, 2 frames in flight" in out          # the second camera has another image size

    num, position, shs, opacity, cov3d = fgs.ops.loadPly(str(ply_dir / "point_cloud.ply"))
    assert num == n
    for cj in cams:
        w, h = cj["width"], cj["height"]
        pos = np.array(cj["position"], np.float32)
        rot = np.array(cj["rotation"], np.float32)
        pre = oracle.preprocess(position.numpy(), shs.numpy(), opacity.numpy(), cov3d.numpy(), w, h, 16, 16, pos, rot,
                                cj["fx"], cj["fy"], 100.0, 0.01, 1 << 20)
        K = pre["num_rendered"]
        assert K > 10_000
        ks, vs = oracle.sort(K, w, h, 16, 16, pre["keys"], pre["values"])
        rg = oracle.ranges(K, ks, ((w + 15) // 16) * ((h + 15) // 16))
        u8, _, _ = oracle.render(w, h, 16, 16, pre["points_xy"], pre["rgb_depth"], pre["conic_opacity"], vs, rg,
                                 np.zeros(3, np.float32), want_f32=False)
        data = (model / "test_out" / ("%s.ppm" % cj["img_name"])).read_bytes()
        head = b"P6\n%d %d\n255\n" % (w, h)
        assert data.startswith(head) and len(data) == len(head) + 3 * w * h
        img = np.frombuffer(data[len(head):], np.uint8).reshape(h, w, 3)
        d = np.abs(img.astype(np.int16) - u8.astype(np.int16))
        assert d.max() <= 1 and (d > 0).mean() < 0.02
        assert img.max() > 100          # not an empty frame


def test_two_rasterizers_on_two_streams_overlapping(oracle):
    """Two renderers with their own buffers on two streams of one device, frames enqueued back to
    back without any ordering between the streams: the library keeps its scratch per stream, so
    both produce exactly what each produces alone (and what the oracle produces)."""
    sc_a = scenes.config0(n=60_000)
    sc_b = scenes.make(1, n=150_000)
    dev = torch.device("cuda:0")
    jobs = []
    for sc in (sc_a, sc_b):
        scene = Scene(dev).from_arrays(sc.position, sc.shs, sc.opacity, sc.cov3d)
        cam = Camera.from_synthetic(sc.cameras[0])
        rast = Rasterizer(scene, 1 << 21, 1 << 14)
        jobs.append((sc, scene, cam, rast, torch.cuda.Stream()))
    bg = torch.tensor([0.1, 0.3, 0.5])
    alone = []
    for sc, scene, cam, rast, _ in jobs:
        alone.append(rast.forward(scene, cam, bg).clone())
        assert rast.num_rendered > 50_000
    torch.cuda.synchronize()
    # both frames are small enough to rank their tiles (the table the blend keeps per stream)
    outs = [[], []]
    for rep in range(6):
        for k, (sc, scene, cam, rast, stream) in enumerate(jobs):
            with torch.cuda.stream(stream):
                outs[k].append(rast.forward(scene, cam, bg).clone())
    torch.cuda.synchronize()
    for k in range(2):
        for img in outs[k]:
            assert torch.equal(img, alone[k])
    # and the image is the oracle's
    sc, scene, cam, rast, _ = jobs[0]
    c0 = sc.cameras[0]
    pre = oracle.preprocess(sc.position, sc.shs, sc.opacity, sc.cov3d, c0.width, c0.height, 16, 16,
                            c0.position, c0.rotation, c0.focal_x, c0.focal_y, c0.zFar, c0.zNear, 1 << 21)
    K = pre["num_rendered"]
    ks, vs = oracle.sort(K, c0.width, c0.height, 16, 16, pre["keys"], pre["values"])
    rg = oracle.ranges(K, ks, ((c0.width + 15) // 16) * ((c0.height + 15) // 16))
    u8, _, _ = oracle.render(c0.width, c0.height, 16, 16, pre["points_xy"], pre["rgb_depth"], pre["conic_opacity"], vs, rg,
                             bg.numpy(), want_f32=False)
    d = np.abs(alone[0].cpu().numpy().astype(np.int16) - u8.astype(np.int16))
    assert d.max() <= 1 and (d > 0).mean() < 0.02
