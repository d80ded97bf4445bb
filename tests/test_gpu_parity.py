"""GPU parity: every stage of the HIP path, called through the C ABI, against the CPU oracle on
the same seeded inputs.  Keys, values, sort order, ranges and the preprocess attributes must be
bit-exact; images are compared before the 8-bit encode with max-abs <= 2e-3 and PSNR > 55 dB."""
import numpy as np
import pytest

from flashgs_amd import scenes

pytestmark = pytest.mark.gpu

IMG_MAX_ABS = 2e-3
IMG_PSNR_DB = 55.0
# 8-bit values that lie within the exponent's rounding of a step of the encode move by one.
IMG_U8_FRACTION = 0.01
# With the colour sums on the matrix unit (opt-in) weights and colours are rounded to f16 (products
# and sums in fp32): a pixel's colour is within 2^-10 of itself of the oracle's, which moves a few
# more of those 8-bit values.
IMG_U8_FRACTION_F16 = 0.03     # a guard against a systematic shift only: the bound proper is the per-pixel one (2^-10 of the colour)


def _oracle_frame(oracle, sc, cam, capacity, block=(16, 16), bg=(0, 0, 0), sentinel=0.0):
    n = sc.num_vertex
    pre = oracle.preprocess(sc.position, sc.shs, sc.opacity, sc.cov3d, cam.width, cam.height, block[0], block[1],
                            cam.position, cam.rotation, cam.focal_x, cam.focal_y, cam.zFar, cam.zNear, capacity,
                            points_xy=np.full((n, 2), sentinel, np.float32),
                            rgb_depth=np.full((n, 4), sentinel, np.float32),
                            conic_opacity=np.full((n, 4), sentinel, np.float32))
    K = pre["num_rendered"]
    ks, vs = oracle.sort(K, cam.width, cam.height, block[0], block[1], pre["keys"], pre["values"])
    gx, gy = (cam.width + block[0] - 1) // block[0], (cam.height + block[1] - 1) // block[1]
    rg = oracle.ranges(K, ks, gx * gy)
    u8, f32, walked = oracle.render(cam.width, cam.height, block[0], block[1], pre["points_xy"], pre["rgb_depth"],
                                    pre["conic_opacity"], vs, rg, bg)
    return dict(pre=pre, K=K, ks=ks, vs=vs, ranges=rg, u8=u8, f32=f32, walked=walked)


def _check_frame(oracle, sc, cam, capacity, block=(16, 16), bg=(0, 0, 0)):
    import gpu_pipeline as gp
    sentinel = -123.25
    ref = _oracle_frame(oracle, sc, cam, capacity, block, bg, sentinel)
    sd = gp.SceneOnDevice(sc)
    got = gp.preprocess(sd, cam, capacity, block, sentinel=sentinel)
    K = ref["K"]
    assert got["num_rendered"] == K
    # unsorted list: same pairs in the same canonical order
    assert np.array_equal(gp.u64(got["keys"])[:K], ref["pre"]["keys"][:K])
    assert np.array_equal(gp.u32(got["values"])[:K], ref["pre"]["values"][:K])
    # attributes: bit-exact everywhere, which includes the untouched (sentinel) rows
    for name in ("points_xy", "conic_opacity", "rgb_depth"):
        a, b = gp.bits(got[name].cpu().numpy()), gp.bits(ref["pre"][name])
        bad = np.flatnonzero((a != b).any(axis=1))
        assert bad.size == 0, "%s differs in %d rows, first %d: %r vs %r" % (
            name, bad.size, bad[0], got[name][int(bad[0])].cpu().numpy(), ref["pre"][name][bad[0]])

    ks, vs = gp.sort(K, cam.width, cam.height, got["keys"], got["values"], block)
    assert np.array_equal(gp.u64(ks)[:K], ref["ks"])
    assert np.array_equal(gp.u32(vs)[:K], ref["vs"])

    # the library default: every operation of the blend in fp32, as render.cu:40-52
    rg, u8, f32 = gp.render(K, cam.width, cam.height, got["points_xy"], got["rgb_depth"], got["conic_opacity"],
                            ks, vs, bg, block)
    assert np.array_equal(rg.cpu().numpy(), ref["ranges"])
    f32 = f32.cpu().numpy()
    err = np.abs(f32 - ref["f32"])
    assert err.max() <= IMG_MAX_ABS, "max abs image error %g" % err.max()
    assert gp.psnr(f32, ref["f32"]) > IMG_PSNR_DB
    d8 = np.abs(u8.cpu().numpy().astype(np.int16) - ref["u8"].astype(np.int16))
    assert d8.max() <= 1, "8-bit image differs by more than one step"
    assert (d8 > 0).mean() < IMG_U8_FRACTION
    # the opt-in mode with the colour sums on the matrix unit, chosen for this call only
    from flashgs_amd import cabi
    _, u8h, f16 = gp.render(K, cam.width, cam.height, got["points_xy"], got["rgb_depth"], got["conic_opacity"],
                            ks, vs, bg, block, flags=cabi.BLEND_MATRIX_F16)
    f16 = f16.cpu().numpy()
    err16 = np.abs(f16 - ref["f32"])
    assert err16.max() <= IMG_MAX_ABS, "f16 colour operands: max abs image error %g" % err16.max()
    # pixel by pixel: the f16 operands of the colour sums cost at most 2^-10 of the colour itself
    over = err16 - (2.0 ** -10 * np.abs(ref["f32"]) + 2e-4)
    assert over.max() <= 0, "a pixel is %g further from the oracle than f16 colour operands explain" % over.max()
    assert gp.psnr(f16, ref["f32"]) > IMG_PSNR_DB
    d8 = np.abs(u8h.cpu().numpy().astype(np.int16) - ref["u8"].astype(np.int16))
    assert d8.max() <= 1 and (d8 > 0).mean() < IMG_U8_FRACTION_F16
    return ref


def test_config0_full_frame(oracle):
    sc = scenes.make(0)
    _check_frame(oracle, sc, sc.cameras[0], 1 << 20)


def test_small_scene_white_background(oracle):
    sc = scenes.config0(n=5000)
    _check_frame(oracle, sc, sc.cameras[0], 1 << 16, bg=(1.0, 0.5, 0.25))


def test_config1_partial_tile_rows(oracle):
    """1920x1080: the last tile row is half outside the image."""
    sc = scenes.make(1, n=200_000)
    _check_frame(oracle, sc, sc.cameras[0], 1 << 20)


def _big_splat_scene(n=4000, seed=7):
    """Splats whose candidate rectangles exceed 64 tiles, so the whole-wave tile test runs."""
    sc = scenes.config0(n=n)
    rng = np.random.default_rng(seed)
    ls = rng.normal(-2.2, 0.9, (n, 3))
    ls[: n // 50] += 2.5                      # a few enormous ones, some covering the screen
    sc.cov3d = scenes.cov3d_from_scale_rotation(np.exp(ls).astype(np.float32), scenes._unit_quats(rng, n))
    return sc


@pytest.mark.parametrize("block", [(16, 16), (32, 16), (32, 32)])
def test_large_splats_all_tile_sizes(oracle, block):
    sc = _big_splat_scene()
    cam = sc.cameras[0]
    cam.width, cam.height = 1000, 600            # neither a multiple of 16 nor of 32
    ref = _check_frame(oracle, sc, cam, 1 << 22, block=block, bg=(0.3, 0.1, 0.9))
    assert ref["pre"]["counts"]["candidates"] > 64 * 20


@pytest.mark.parametrize("block", [(32, 16), (32, 32)])
def test_wide_tiles_on_a_frame_with_many_tiles(oracle, block):
    """5120x2880 has more tiles than the chip holds at once even at 32x32 (160x90 = 14 400):
    the blend then runs its variant with fewer resident waves."""
    sc = scenes.config0(n=40_000)
    cam = sc.cameras[0]
    scale = 2880 / cam.height
    cam.width, cam.height = 5120, 2880
    cam.focal_x *= scale
    cam.focal_y *= scale
    _check_frame(oracle, sc, cam, 1 << 22, block=block, bg=(0.1, 0.2, 0.3))


def test_random_frames_with_odd_sizes_and_cameras(oracle):
    """Twenty random frames: 1 to 150 000 Gaussians, images from 1x1 to 4000x1080 including sizes
    one below and one above a tile, fields of view from 10 to 120 degrees, cameras inside and
    outside the cloud, all three tile shapes.  Keys, values, their order, the attribute records,
    the sorted lists and the ranges are compared bit for bit, the image within the tolerance."""
    import gpu_pipeline as gp
    for seed in range(20):
        rng = np.random.default_rng(1000 + seed)
        n = int(rng.choice([1, 7, 63, 257, 5000, 40000, 150000]))
        sc = scenes.config0(n=n)
        sc.position = (sc.position * rng.uniform(0.2, 3.0)).astype(np.float32)
        ls = rng.normal(rng.uniform(-5, -1.0), rng.uniform(0.3, 1.5), (n, 3))
        sc.cov3d = scenes.cov3d_from_scale_rotation(np.exp(ls).astype(np.float32), scenes._unit_quats(rng, n))
        W = int(rng.choice([1, 15, 16, 17, 100, 333, 640, 1280, 1921, 4000]))
        H = int(rng.choice([1, 16, 31, 200, 360, 721, 1080]))
        cam = scenes.look_at(rng.uniform(-6, 6, 3), rng.uniform(-2, 2, 3), W, H, rng.uniform(10, 120))
        block = [(16, 16), (32, 16), (32, 32)][seed % 3]
        bg = rng.uniform(0, 1, 3).astype(np.float32)
        cap = 1 << 24
        r = oracle.preprocess(sc.position, sc.shs, sc.opacity, sc.cov3d, W, H, block[0], block[1], cam.position, cam.rotation,
                              cam.focal_x, cam.focal_y, cam.zFar, cam.zNear, cap)
        K = r["num_rendered"]
        assert r["rc"] == 0 and K <= cap
        where = "seed %d: %d Gaussians, %dx%d, tile %s, %d pairs" % (seed, n, W, H, block, K)
        got = gp.preprocess(gp.SceneOnDevice(sc), cam, cap, block=block)
        assert got["num_rendered"] == K, where
        assert np.array_equal(gp.u64(got["keys"])[:K], r["keys"][:K]), where
        assert np.array_equal(gp.u32(got["values"])[:K], r["values"][:K]), where
        vis = np.zeros(n, bool)
        vis[r["values"][:K]] = True
        for name in ("points_xy", "conic_opacity", "rgb_depth"):
            assert np.array_equal(gp.bits(got[name].cpu().numpy()[vis]), gp.bits(r[name][vis])), where + ", " + name
        ks, vs = oracle.sort(K, W, H, block[0], block[1], r["keys"][:K], r["values"][:K])
        gks, gvs = gp.sort(K, W, H, got["keys"], got["values"], block)
        assert np.array_equal(gp.u64(gks)[:K], ks) and np.array_equal(gp.u32(gvs)[:K], vs), where
        gx, gy = (W + block[0] - 1) // block[0], (H + block[1] - 1) // block[1]
        rg = oracle.ranges(K, ks, gx * gy)
        _, ref, _ = oracle.render(W, H, block[0], block[1], r["points_xy"], r["rgb_depth"], r["conic_opacity"], vs, rg, bg,
                                  want_u8=False)
        grg, _, f32 = gp.render(K, W, H, got["points_xy"], got["rgb_depth"], got["conic_opacity"], gks, gvs, bg, block)
        assert np.array_equal(grg.cpu().numpy(), rg), where
        err = np.abs(f32.cpu().numpy() - ref).max()
        assert err <= IMG_MAX_ABS, where + ": max abs image error %g" % err


def test_degenerate_inputs_match_the_oracle(oracle):
    """NaN / infinite / zero / enormous entries in every input tensor: the kernels must neither fault
    nor disagree with the oracle about which keys such Gaussians emit (the float->int conversions
    saturate and map NaN to 0 on both sides)."""
    sc = scenes.config0(n=20_000)
    rng = np.random.default_rng(5)
    bad = [np.nan, np.inf, -np.inf, 0.0, 1e30, -1e30, 1e-30]
    for arr in (sc.position, sc.opacity, sc.cov3d, sc.shs):
        flat = arr.reshape(-1)
        where = rng.choice(flat.size, 300, replace=False)
        flat[where] = rng.choice(bad, where.size).astype(np.float32)
    sc.cov3d[100:140] = 0.0                      # degenerate covariances
    sc.cov3d[200:220] *= 1e6                     # splats far larger than the screen
    sc.opacity[300:320] = 1.0
    sc.opacity[320:340] = 1.0 / 255.0
    import gpu_pipeline as gp
    cam = sc.cameras[0]
    cap = 1 << 22
    pre = oracle.preprocess(sc.position, sc.shs, sc.opacity, sc.cov3d, cam.width, cam.height, 16, 16,
                            cam.position, cam.rotation, cam.focal_x, cam.focal_y, cam.zFar, cam.zNear, cap)
    K = pre["num_rendered"]
    assert 0 < K < cap
    got = gp.preprocess(gp.SceneOnDevice(sc), cam, cap)
    assert got["num_rendered"] == K
    assert np.array_equal(gp.u64(got["keys"])[:K], pre["keys"][:K])
    assert np.array_equal(gp.u32(got["values"])[:K], pre["values"][:K])
    vis = np.unique(pre["values"][:K])
    for name in ("points_xy", "conic_opacity", "rgb_depth"):
        a, b = got[name].cpu().numpy()[vis], pre[name][vis]
        # bit-exact, except that a NaN may carry another sign or payload
        same = (gp.bits(a) == gp.bits(b)) | (np.isnan(a) & np.isnan(b))
        rows = np.flatnonzero(~same.all(axis=1))
        assert rows.size == 0, "%s: %d rows differ, first Gaussian %d: %r vs %r" % (
            name, rows.size, vis[rows[0]], a[rows[0]], b[rows[0]])
    ks, vs = gp.sort(K, cam.width, cam.height, got["keys"], got["values"])
    oks, ovs = oracle.sort(K, cam.width, cam.height, 16, 16, pre["keys"], pre["values"])
    assert np.array_equal(gp.u64(ks)[:K], oks) and np.array_equal(gp.u32(vs)[:K], ovs)
    # the image may hold NaN where a NaN colour was blended: only require that the blend runs
    rg, u8, _ = gp.render(K, cam.width, cam.height, got["points_xy"], got["rgb_depth"], got["conic_opacity"],
                          ks, vs, (0, 0, 0), f32=False)
    assert np.array_equal(rg.cpu().numpy(), oracle.ranges(K, oks, rg.shape[0]))


@pytest.mark.parametrize("aniso_last", [False, True])
def test_anisotropic_splats_near_camera(oracle, aniso_last):
    """Needle-shaped splats close to the camera: the exact ellipse test rejects most candidates.
    As a random subset of the scene and stored as its last tenth (then the last workgroups hold
    nothing else and their lists of big rectangles run full)."""
    sc = scenes.config4(n=60_000, width=1280, height=720, n_poses=3, aniso_last=aniso_last)
    for cam in sc.cameras:
        ref = _check_frame(oracle, sc, cam, 1 << 22)
        assert ref["K"] < ref["pre"]["counts"]["candidates"]


def test_empty_inputs(oracle):
    import gpu_pipeline as gp
    import torch
    from flashgs_amd import cabi
    # no Gaussian survives the culls: zero pairs, background image, ranges all zero
    sc = scenes.config0(n=1000)
    sc.position[:, 2] = -100.0                    # all behind the camera
    ref = _check_frame(oracle, sc, sc.cameras[0], 1 << 10, bg=(0.25, 0.5, 0.75))
    assert ref["K"] == 0
    # P == 0 is accepted and leaves the counter alone
    off = torch.full((1,), 5, device=gp.DEV, dtype=torch.int32)
    cabi.preprocess(0, 0, 0, 0, 0, 64, 64, 16, 16, [0, 0, 0], np.eye(3), 50.0, 50.0, 100.0, 0.01, 0, 0, 0, 0, 0,
                    off.data_ptr(), 16, 0)
    assert int(off.cpu()[0]) == 5


def test_start_offset_and_capacity_guard(oracle):
    """Pairs are appended after the caller's starting offset (preprocess.cu:330,395 add to the
    counter); pairs beyond key_capacity are dropped but still counted."""
    import gpu_pipeline as gp
    sc = scenes.config0(n=30_000)
    cam = sc.cameras[0]
    sd = gp.SceneOnDevice(sc)
    full = gp.preprocess(sd, cam, 1 << 18)
    K = full["num_rendered"]
    assert K > 1000
    shifted = gp.preprocess(sd, cam, 1 << 18, start_offset=777)
    assert shifted["num_rendered"] == K + 777
    assert np.array_equal(gp.u64(shifted["keys"])[777:777 + K], gp.u64(full["keys"])[:K])
    assert np.all(gp.u64(shifted["keys"])[:777] == 0)
    cap = K // 2
    n = sd.n
    import torch
    keys = torch.zeros(cap + 64, device=gp.DEV, dtype=torch.int64)
    values = torch.full((cap + 64,), -1, device=gp.DEV, dtype=torch.int32)
    off = torch.zeros(1, device=gp.DEV, dtype=torch.int32)
    from flashgs_amd import cabi
    cabi.preprocess(n, sd.position.data_ptr(), sd.shs.data_ptr(), sd.opacity.data_ptr(), sd.cov3d.data_ptr(),
                    cam.width, cam.height, 16, 16, cam.position, cam.rotation, cam.focal_x, cam.focal_y, cam.zFar, cam.zNear,
                    full["points_xy"].data_ptr(), full["rgb_depth"].data_ptr(), full["conic_opacity"].data_ptr(),
                    keys.data_ptr(), values.data_ptr(), off.data_ptr(), cap, 0)
    torch.cuda.synchronize()
    assert int(off.cpu()[0]) == K                                     # still the full count
    assert np.array_equal(gp.u64(keys)[:cap], gp.u64(full["keys"])[:cap])
    assert np.all(gp.u64(keys)[cap:] == 0) and np.all(values.cpu().numpy()[cap:] == -1)   # nothing past the capacity


def test_mirrored_preprocess_stores_the_count_in_pinned_memory():
    """fgs_preprocess_mirrored: the word of pinned host memory receives the pair count the launch
    leaves in *curr_offset (with a starting offset too), everything else is what fgs_preprocess
    writes; a launch that gives up stores a negative count there; memory that is not pinned is refused."""
    import gpu_pipeline as gp
    import torch
    from flashgs_amd import cabi
    sc = scenes.config1(n=400_000)
    cam = sc.cameras[0]
    sd = gp.SceneOnDevice(sc)
    cap = 1 << 21
    plain = gp.preprocess(sd, cam, cap)
    K = plain["num_rendered"]
    assert K > 100_000
    for start in (0, 1000):
        got = gp.preprocess(sd, cam, cap, start_offset=start, mirror=True)
        assert got["mirrored"] == got["num_rendered"] == K + start
        assert np.array_equal(gp.u64(got["keys"])[start:start + K], gp.u64(plain["keys"])[:K])
        assert np.array_equal(gp.u32(got["values"])[start:start + K], gp.u32(plain["values"])[:K])
        assert torch.equal(got["rgb_depth"], plain["rgb_depth"])
    # no Gaussians: the count is the starting offset
    st = torch.cuda.current_stream().cuda_stream
    word = torch.full((1,), cabi.COUNT_PENDING, dtype=torch.int32).pin_memory()
    offset = torch.full((1,), 37, device=gp.DEV, dtype=torch.int32)
    cabi.preprocess(0, 0, 0, 0, 0, cam.width, cam.height, 16, 16, cam.position, cam.rotation, cam.focal_x, cam.focal_y,
                    cam.zFar, cam.zNear, 0, 0, 0, 0, 0, offset.data_ptr(), 0, st, count_mirror=word.data_ptr())
    assert cabi.wait_count(word.data_ptr()) == 37
    # a launch whose scan gives up
    previous = cabi.set_scan_spin_limit(0)
    try:
        bad = gp.preprocess(gp.SceneOnDevice(scenes.config0(n=1_200_000)), scenes.config0(n=1_200_000).cameras[0], 1 << 22,
                            mirror=True)
    finally:
        cabi.set_scan_spin_limit(previous)
    assert bad["num_rendered"] < 0 and bad["mirrored"] < 0
    cabi.reset_scan(st)
    again = gp.preprocess(sd, cam, cap, mirror=True)
    assert again["mirrored"] == K
    # pageable memory cannot be written by the launch
    pageable = torch.full((1,), cabi.COUNT_PENDING, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="pinned"):
        cabi.preprocess(0, 0, 0, 0, 0, cam.width, cam.height, 16, 16, cam.position, cam.rotation, cam.focal_x, cam.focal_y,
                        cam.zFar, cam.zNear, 0, 0, 0, 0, 0, offset.data_ptr(), 0, st, count_mirror=pageable.data_ptr())
    torch.cuda.synchronize()
    assert int(torch.zeros(1, device=gp.DEV).sum()) == 0          # the refused call left no error behind


def test_scan_that_gives_up_reports_a_negative_count_until_reset():
    """With the spin limit at 0 every wait of the preprocess launch that is not satisfied at its
    first poll gives up: the kernel still runs to its end (no wave is left waiting) and the pair
    count comes back negative, which the sort refuses.  The frame has more workgroups than the chip
    holds at once, so some are dispatched only after the scanner has given up.  The scan status is
    then marked unusable: the next launch - another scene, normal limit - reports a negative count
    as well and writes nothing; after fgs_reset_scan both scenes come out right again.  Both entry
    points (the allocated scan status and the built-in one)."""
    import gpu_pipeline as gp
    import torch
    from flashgs_amd import cabi
    big = scenes.config0(n=1_200_000)            # 4689 workgroups
    other = scenes.config1(n=300_000)
    cam, cam_o = big.cameras[0], other.cameras[0]
    sd, sd_o = gp.SceneOnDevice(big), gp.SceneOnDevice(other)
    cap = 1 << 22
    good, good_o = gp.preprocess(sd, cam, cap), gp.preprocess(sd_o, cam_o, cap)
    K, K_o = good["num_rendered"], good_o["num_rendered"]
    assert K > 1_000_000 and K_o > 100_000
    st = torch.cuda.current_stream().cuda_stream
    for static in (False, True):
        previous = cabi.set_scan_spin_limit(0)
        try:
            bad = gp.preprocess(sd, cam, cap, static=static)
        finally:
            assert cabi.set_scan_spin_limit(previous) == 0
        assert previous == 1 << 22
        assert bad["num_rendered"] < 0
        with pytest.raises(RuntimeError, match="negative"):
            gp.sort(bad["num_rendered"], cam.width, cam.height, bad["keys"], bad["values"])
        # sticky: another scene with the normal limit is refused at once and nothing is written
        stuck = gp.preprocess(sd_o, cam_o, cap, sentinel=-3.5, static=static)
        assert stuck["num_rendered"] < 0
        assert not gp.u64(stuck["keys"]).any()
        assert np.all(stuck["rgb_depth"].cpu().numpy() == -3.5)
        cabi.reset_scan(st)
        for scene_d, c, want, n in ((sd_o, cam_o, good_o, K_o), (sd, cam, good, K), (sd_o, cam_o, good_o, K_o)):
            again = gp.preprocess(scene_d, c, cap, static=static)
            assert again["num_rendered"] == n
            assert np.array_equal(gp.u64(again["keys"])[:n], gp.u64(want["keys"])[:n])
            assert np.array_equal(gp.u32(again["values"])[:n], gp.u32(want["values"])[:n])


@pytest.mark.parametrize("frames_in_flight", [1, 2, 3])
def test_batch_rasterizer_renders_what_the_rasterizer_renders(frames_in_flight):
    """BatchRasterizer: the poses of an orbit on two or three streams, each with buffers of its
    own - the images are those of Rasterizer.forward, pose by pose, also when the batch is
    rendered a second time into the same tensor."""
    import gpu_pipeline as gp
    import torch
    from flashgs_amd.rasterizer import BatchRasterizer, Camera, Rasterizer, Scene
    sc = scenes.config4(n=120_000, width=1280, height=720, n_poses=7)
    scene = Scene(torch.device(gp.DEV)).from_arrays(sc.position, sc.shs, sc.opacity, sc.cov3d)
    cams = [Camera.from_synthetic(c, i) for i, c in enumerate(sc.cameras)]
    bg = torch.tensor([0.1, 0.2, 0.3])
    one = Rasterizer(scene, 1 << 22, 1 << 14)
    want = torch.stack([one.forward(scene, c, bg).clone() for c in cams])
    batch = BatchRasterizer(scene, 1 << 22, 1 << 14, frames_in_flight=frames_in_flight)
    got = batch.render(scene, cams, bg)
    assert got.shape == want.shape and torch.equal(got, want)        # read on the current stream, no synchronisation here
    again = batch.render(scene, cams[::-1], bg, out=got)
    assert again is got and torch.equal(got, want.flip(0))
    assert batch.render(scene, [], bg) is None
    with pytest.raises(ValueError, match="one image size"):
        batch.render(scene, [cams[0], Camera.from_synthetic(scenes.config1(n=10).cameras[0])], bg)


def test_rasterizer_relaunches_once_after_a_scan_that_gave_up():
    """Rasterizer.forward clears the scan status and launches the frame once more when the pair
    count comes back negative; with the waits still failing it raises ScanGaveUp, not TooManyPairs."""
    import gpu_pipeline as gp
    import torch
    from flashgs_amd import cabi
    from flashgs_amd.rasterizer import Camera, Rasterizer, ScanGaveUp, Scene
    sc = scenes.config0(n=400_000)
    scene = Scene(torch.device(gp.DEV)).from_arrays(sc.position, sc.shs, sc.opacity, sc.cov3d)
    cam = Camera.from_synthetic(sc.cameras[0])
    rast = Rasterizer(scene, 1 << 21, 1 << 14)
    bg = torch.zeros(3)
    want = rast.forward(scene, cam, bg).clone()
    K = rast.num_rendered
    # leave the stream's scan status marked unusable, as a scan that gave up does
    previous = cabi.set_scan_spin_limit(0)
    try:
        with pytest.raises(ScanGaveUp):
            rast.forward(scene, cam, bg)
    finally:
        cabi.set_scan_spin_limit(previous)
    # the status is still marked; forward recovers by itself
    got = rast.forward(scene, cam, bg)
    assert rast.num_rendered == K and torch.equal(got, want)
    # a workgroup that gives up after the count has gone out lowers the mirrored count later: the
    # next forward reports the frame before, once, and renders again after that
    torch.cuda.synchronize()
    rast._count[0] = -2147483648
    with pytest.raises(ScanGaveUp, match="previous frame"):
        rast.forward(scene, cam, bg)
    got = rast.forward(scene, cam, bg)
    assert rast.num_rendered == K and torch.equal(got, want)


def test_preprocess_replayed_from_a_captured_graph():
    """The preprocess entry points keep no per-launch state on the host, so a captured launch
    (here the one that also mirrors its count into pinned memory) can be replayed: every replay
    (with eager launches of other sizes in between) gives the eager result."""
    import gpu_pipeline as gp
    import torch
    from flashgs_amd import cabi
    sc = scenes.config0(n=70_000)
    cam = sc.cameras[0]
    sd = gp.SceneOnDevice(sc)
    cap = 1 << 20
    eager = gp.preprocess(sd, cam, cap)
    K = eager["num_rendered"]
    ref_keys = gp.u64(eager["keys"])[:K].copy()
    ref_vals = gp.u32(eager["values"])[:K].copy()
    n = sd.n
    xy = torch.zeros((n, 2), device=gp.DEV); rgb = torch.zeros((n, 4), device=gp.DEV); co = torch.zeros((n, 4), device=gp.DEV)
    keys = torch.zeros(cap, device=gp.DEV, dtype=torch.int64)
    values = torch.zeros(cap, device=gp.DEV, dtype=torch.int32)
    off = torch.zeros(1, device=gp.DEV, dtype=torch.int32)
    word = torch.full((1,), cabi.COUNT_PENDING, dtype=torch.int32).pin_memory()     # the captured launch also mirrors its count
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        off.zero_()                     # a fill kernel, not a memset node
        cabi.preprocess(n, sd.position.data_ptr(), sd.shs.data_ptr(), sd.opacity.data_ptr(), sd.cov3d.data_ptr(),
                        cam.width, cam.height, 16, 16, cam.position, cam.rotation, cam.focal_x, cam.focal_y,
                        cam.zFar, cam.zNear, xy.data_ptr(), rgb.data_ptr(), co.data_ptr(),
                        keys.data_ptr(), values.data_ptr(), off.data_ptr(), cap, torch.cuda.current_stream().cuda_stream,
                        count_mirror=word.data_ptr())
    small = gp.SceneOnDevice(scenes.config0(n=3000))
    for replay in range(4):
        keys.zero_(); values.zero_()
        word[0] = cabi.COUNT_PENDING
        graph.replay()
        assert cabi.wait_count(word.data_ptr()) == K, "replay %d" % replay
        torch.cuda.synchronize()
        assert int(off.cpu()[0]) == K, "replay %d" % replay
        assert np.array_equal(gp.u64(keys)[:K], ref_keys), "replay %d" % replay
        assert np.array_equal(gp.u32(values)[:K], ref_vals), "replay %d" % replay
        for name, t in (("points_xy", xy), ("rgb_depth", rgb), ("conic_opacity", co)):
            vis = np.unique(ref_vals)
            assert np.array_equal(gp.bits(t.cpu().numpy()[vis]), gp.bits(eager[name].cpu().numpy()[vis])), name
        # eager launches of another size between the replays
        for _ in range(replay + 1):
            gp.preprocess(small, cam, 1 << 16)
        torch.cuda.synchronize()


def test_captured_preprocess_survives_a_larger_eager_call_on_its_stream():
    """Warm-up, capture, then a larger P on the same stream: the stream gets a larger scan status,
    and the one whose address the captured launch holds must stay alive and consistent.  Replays
    before and after the larger call give the eager result."""
    import gpu_pipeline as gp
    import torch
    from flashgs_amd import cabi
    small = scenes.config0(n=70_000)
    large = scenes.config0(n=1_200_000)          # 4689 workgroups: more than the first allocation holds
    cam = small.cameras[0]
    sd, sd_large = gp.SceneOnDevice(small), gp.SceneOnDevice(large)
    cap = 1 << 22
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        eager = gp.preprocess(sd, cam, cap)                 # allocates the stream's scan status
    K = eager["num_rendered"]
    n = sd.n
    xy = torch.zeros((n, 2), device=gp.DEV); rgb = torch.zeros((n, 4), device=gp.DEV); co = torch.zeros((n, 4), device=gp.DEV)
    keys = torch.zeros(cap, device=gp.DEV, dtype=torch.int64)
    values = torch.zeros(cap, device=gp.DEV, dtype=torch.int32)
    off = torch.zeros(1, device=gp.DEV, dtype=torch.int32)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        off.zero_()
        cabi.preprocess(n, sd.position.data_ptr(), sd.shs.data_ptr(), sd.opacity.data_ptr(), sd.cov3d.data_ptr(),
                        cam.width, cam.height, 16, 16, cam.position, cam.rotation, cam.focal_x, cam.focal_y,
                        cam.zFar, cam.zNear, xy.data_ptr(), rgb.data_ptr(), co.data_ptr(),
                        keys.data_ptr(), values.data_ptr(), off.data_ptr(), cap, torch.cuda.current_stream().cuda_stream)

    def replay_and_check(what):
        keys.zero_(); values.zero_()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            graph.replay()
        torch.cuda.synchronize()
        assert int(off.cpu()[0]) == K, what
        assert np.array_equal(gp.u64(keys)[:K], gp.u64(eager["keys"])[:K]), what
        assert np.array_equal(gp.u32(values)[:K], gp.u32(eager["values"])[:K]), what

    replay_and_check("replay before the larger call")
    with torch.cuda.stream(side):
        big1 = gp.preprocess(sd_large, cam, cap)            # the stream moves to a larger scan status
    replay_and_check("replay after the larger call")
    with torch.cuda.stream(side):
        big2 = gp.preprocess(sd_large, cam, cap)
    replay_and_check("second replay after the larger call")
    Kl = big1["num_rendered"]
    assert Kl > 1_000_000 and big2["num_rendered"] == Kl
    assert np.array_equal(gp.u64(big1["keys"])[:Kl], gp.u64(big2["keys"])[:Kl])
    ref_large = gp.preprocess(sd_large, cam, cap)           # on the default stream, its own scan status
    assert np.array_equal(gp.u64(big1["keys"])[:Kl], gp.u64(ref_large["keys"])[:Kl])


def test_sort_and_render_replayed_from_a_captured_graph():
    """The other two stages keep no state at all between calls: sort + render of a fixed pair count,
    captured once and replayed with eager work in between, reproduce the eager image."""
    import gpu_pipeline as gp
    import torch
    from flashgs_amd import cabi
    sc = scenes.config0(n=60_000)
    cam = sc.cameras[0]
    sd = gp.SceneOnDevice(sc)
    pre = gp.preprocess(sd, cam, 1 << 20)
    K = pre["num_rendered"]
    ks_e, vs_e = gp.sort(K, cam.width, cam.height, pre["keys"], pre["values"])
    rg_e, u8_e, _ = gp.render(K, cam.width, cam.height, pre["points_xy"], pre["rgb_depth"], pre["conic_opacity"],
                              ks_e, vs_e, (0.2, 0.4, 0.6), f32=False)
    size = cabi.get_sort_buffer_size(K)
    space = torch.zeros(size, device=gp.DEV, dtype=torch.int8)
    ks = torch.zeros(K, device=gp.DEV, dtype=torch.int64)
    vs = torch.zeros(K, device=gp.DEV, dtype=torch.int32)
    gx, gy = (cam.width + 15) // 16, (cam.height + 15) // 16
    ranges = torch.zeros((gx * gy, 2), device=gp.DEV, dtype=torch.int32)
    out = torch.zeros((cam.height, cam.width, 3), device=gp.DEV, dtype=torch.uint8)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        st = torch.cuda.current_stream().cuda_stream
        cabi.sort_gaussian(K, cam.width, cam.height, 16, 16, space.data_ptr(), size,
                           pre["keys"].data_ptr(), pre["values"].data_ptr(), ks.data_ptr(), vs.data_ptr(), st)
        cabi.render(16, 16, K, cam.width, cam.height, pre["points_xy"].data_ptr(), pre["rgb_depth"].data_ptr(),
                    pre["conic_opacity"].data_ptr(), ks.data_ptr(), vs.data_ptr(), ranges.data_ptr(), (0.2, 0.4, 0.6),
                    out.data_ptr(), st)
    for replay in range(3):
        ks.zero_(); vs.zero_(); out.zero_(); ranges.fill_(-3); space.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(gp.u64(ks), gp.u64(ks_e)[:K]), "replay %d" % replay
        assert np.array_equal(gp.u32(vs), gp.u32(vs_e)[:K]), "replay %d" % replay
        assert torch.equal(ranges, rg_e) and torch.equal(out, u8_e), "replay %d" % replay
        gp.sort(1000, cam.width, cam.height, pre["keys"], pre["values"])       # eager work of another size
        torch.cuda.synchronize()


def test_repeated_frames_are_deterministic():
    import gpu_pipeline as gp
    sc = scenes.config0(n=50_000)
    cam = sc.cameras[0]
    sd = gp.SceneOnDevice(sc)
    first = gp.preprocess(sd, cam, 1 << 18)
    K = first["num_rendered"]
    ks0, vs0 = gp.sort(K, cam.width, cam.height, first["keys"], first["values"])
    for _ in range(5):
        again = gp.preprocess(sd, cam, 1 << 18)
        assert again["num_rendered"] == K
        assert np.array_equal(gp.u64(again["keys"])[:K], gp.u64(first["keys"])[:K])
        ks, vs = gp.sort(K, cam.width, cam.height, again["keys"], again["values"], space_for=1 << 18)
        assert np.array_equal(gp.u64(ks)[:K], gp.u64(ks0)[:K]) and np.array_equal(gp.u32(vs)[:K], gp.u32(vs0)[:K])


@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 2047, 2048, 2049, 4096, 100_003, 1_500_000])
def test_sort_sizes_against_numpy(n):
    """Ragged sizes around the wave (64) and workgroup tile (2048) boundaries, with many equal keys."""
    import gpu_pipeline as gp
    rng = np.random.default_rng(n)
    W, H = 3840, 2160
    tiles = 240 * 135
    tile = rng.integers(0, tiles, n).astype(np.uint64)
    depth = rng.uniform(0.2, 80.0, n).astype(np.float32)
    if n > 100:
        depth[: n // 3] = depth[0]
        tile[: n // 5] = tile[1]
    keys = (tile << np.uint64(32)) | depth.view(np.uint32).astype(np.uint64)
    vals = rng.permutation(n).astype(np.uint32)
    ks, vs = gp.sort(n, W, H, gp.dev(keys.view(np.int64)), gp.dev(vals.view(np.int32)))
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(gp.u64(ks)[:n], keys[order])
    assert np.array_equal(gp.u32(vs)[:n], vals[order])


def test_sort_8k_frame_wide_partition_digits():
    """7680x4320 has 129 600 tiles: 17 tile bits, partitioned in two passes of 9-bit digits.  Against numpy."""
    rng = np.random.default_rng(8)
    n = 1_200_000
    tile = rng.integers(0, 480 * 270, n).astype(np.uint32)
    tile[: n // 6] = 129_599                      # one very long segment in the last tile
    depth = rng.uniform(0.2, 90.0, n).astype(np.float32)
    depth[::7] = np.float32(3.25)
    _sort_case(tile, depth.view(np.uint32), 7680, 4320, seed=8)


def test_sort_120M_pairs_properties():
    """120M pairs on an 8K frame (the size the large-scale configuration speaks of), without the
    oracle: output non-decreasing, pairs stay together, equal keys keep their input order, and
    the output is a permutation of the input."""
    import gpu_pipeline as gp
    import torch
    n = 120_000_000
    g = torch.Generator(device=gp.DEV).manual_seed(3)
    tile = torch.randint(0, 480 * 270, (n,), device=gp.DEV, generator=g, dtype=torch.int64)
    depth = (torch.rand(n, device=gp.DEV, generator=g) * 90 + 0.2).to(torch.float32).view(torch.int32).to(torch.int64)
    depth[: n // 8] = depth[0]
    keys = (tile << 32) | depth
    del tile, depth
    vals = torch.arange(n, device=gp.DEV, dtype=torch.int32)        # value = input position
    ks, vs = gp.sort(n, 7680, 4320, keys, vals)
    assert bool((ks[1:] >= ks[:-1]).all())
    assert bool((keys[vs.long()] == ks).all())                        # pairs stayed together
    tie = ks[1:] == ks[:-1]
    assert bool((vs[1:][tie] > vs[:-1][tie]).all())                   # stable
    del tie
    seen = torch.zeros(n, device=gp.DEV, dtype=torch.bool)
    seen[vs.long()] = True
    assert bool(seen.all())                                           # a permutation


def test_sort_full_size_properties():
    """At the headline size (8M pairs, 47 key bits) without the oracle: output is a permutation of
    the input, non-decreasing, and equal keys keep their input order."""
    import gpu_pipeline as gp
    import torch
    n = 8_115_406
    g = torch.Generator(device=gp.DEV).manual_seed(1)
    tile = torch.randint(0, 32400, (n,), device=gp.DEV, generator=g, dtype=torch.int64)
    depth = (torch.rand(n, device=gp.DEV, generator=g) * 60 + 0.2).to(torch.float32).view(torch.int32).to(torch.int64)
    depth[: n // 4] = depth[0]
    keys = (tile << 32) | depth
    vals = torch.arange(n, device=gp.DEV, dtype=torch.int32)        # value = input position
    ks, vs = gp.sort(n, 3840, 2160, keys, vals)
    assert bool((ks[1:] >= ks[:-1]).all())
    assert bool((keys[vs.long()] == ks).all())                        # pairs stayed together
    tie = ks[1:] == ks[:-1]
    assert bool((vs[1:][tie] > vs[:-1][tie]).all())                   # stable
    assert int(torch.bincount(vs.long(), minlength=n).max()) == 1     # a permutation


def test_blend_long_lists_shared_between_waves(oracle):
    """A small frame blends its long lists with four waves: the owner takes the head of the list,
    the rest is cut into four runs that start from T = 1 and are folded front to back.  Crafted
    lists around the lengths where that sets in, with odd and even lengths, one that saturates in
    its head, one that saturates inside a run and faint ones that never do; blended through
    fgs_blend on ranges made here, against the oracle's blend of the same lists."""
    import gpu_pipeline as gp
    from flashgs_amd import cabi
    import torch
    W, H = 320, 232                      # 20 x 15 tiles, the last row half a tile
    gx, gy = 20, 15
    rng = np.random.default_rng(11)
    # (tile, list length, opacity): faint lists never reach the stop
    lists = [(0, 767, 0.002), (21, 768, 0.002), (22, 769, 0.002), (45, 770, 0.002), (66, 1501, 0.002),
             (107, 3000, 0.0015), (150, 5003, 0.001), (171, 2000, 0.9), (212, 2000, 0.02), (253, 1024, 0.004),
             (299, 900, 0.003), (280, 2048, 0.002)]
    lists += [(t, int(rng.integers(0, 300)), 0.05) for t in range(300) if t not in {l[0] for l in lists}]
    xy, co, rgbd, vals, ranges = [], [], [], [], np.zeros((gx * gy, 2), np.int32)
    at = 0
    for t, n, op in sorted(lists):
        tx, ty = t % gx, t // gx
        c = np.stack([tx * 16 + rng.uniform(-4, 20, n), ty * 16 + rng.uniform(-4, 20, n)], 1)
        sig = rng.uniform(3.0, 12.0, (n, 2))
        rho = rng.uniform(-0.6, 0.6, n)
        det = (sig[:, 0] * sig[:, 1]) ** 2 * (1 - rho ** 2)
        cx, cz = sig[:, 1] ** 2 / det, sig[:, 0] ** 2 / det
        cy = -rho * sig[:, 0] * sig[:, 1] / det
        log2e = 1.4426950408889634
        xy.append(c)
        co.append(np.stack([-0.5 * log2e * cx, -log2e * cy, -0.5 * log2e * cz, np.log2(np.full(n, op))], 1))
        rgbd.append(np.concatenate([rng.uniform(0, 1.5, (n, 3)), rng.uniform(1, 50, (n, 1))], 1))
        ranges[t] = (at, at + n)
        at += n
    xy = np.concatenate(xy).astype(np.float32)
    co = np.concatenate(co).astype(np.float32)
    rgbd = np.concatenate(rgbd).astype(np.float32)
    vals = rng.permutation(at).astype(np.uint32)          # list position -> Gaussian index
    inv = np.empty(at, np.int64); inv[vals] = np.arange(at)
    xy_g, co_g, rgbd_g = xy[inv], co[inv], rgbd[inv]      # attributes by Gaussian index
    bg = np.array([0.2, 0.4, 0.6], np.float32)
    _, ref, walked = oracle.render(W, H, 16, 16, xy_g, rgbd_g, co_g, vals, ranges, bg, want_u8=False)
    assert walked < at                                     # the opaque lists did stop early
    out = torch.full((H, W, 3), -1.0, device=gp.DEV, dtype=torch.float32)
    d = [gp.dev(a) for a in (xy_g, rgbd_g, co_g)]
    dv, dr = gp.dev(vals.view(np.int32)), gp.dev(ranges)
    # the second call reuses the tile ranking buffer; then the same with the colour sums on the matrix unit
    for flags, bound in ((None, 2e-4), (None, 2e-4), (cabi.BLEND_MATRIX_F16, 1e-3)):
        cabi.blend(16, 16, W, H, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), dv.data_ptr(), dr.data_ptr(),
                   bg, 0, out.data_ptr(), torch.cuda.current_stream().cuda_stream, flags=flags)
        torch.cuda.synchronize()
        err = np.abs(out.cpu().numpy() - ref)
        # 1e-4 for the runs that stop on their own T, plus 2^-10 of a colour with f16 operands
        assert err.max() <= bound, "max abs image error %g (flags %r)" % (err.max(), flags)


def _blend_lists(oracle, lists, W, H, bg, seed, colour_hi=1.5, flags=None):
    """Builds the attribute tensors and ranges for hand-made per-tile lists (tile, length, opacity),
    blends them with fgs_blend (fgs_blend_ex when `flags` is given) and with the oracle; returns
    (GPU float image, oracle float image)."""
    import gpu_pipeline as gp
    from flashgs_amd import cabi
    import torch
    gx, gy = (W + 15) // 16, (H + 15) // 16
    rng = np.random.default_rng(seed)
    xy, co, rgbd, ranges = [], [], [], np.zeros((gx * gy, 2), np.int32)
    at = 0
    for t, n, op in sorted(lists):
        tx, ty = t % gx, t // gx
        c = np.stack([tx * 16 + rng.uniform(-4, 20, n), ty * 16 + rng.uniform(-4, 20, n)], 1)
        sig = rng.uniform(3.0, 12.0, (n, 2))
        rho = rng.uniform(-0.6, 0.6, n)
        det = (sig[:, 0] * sig[:, 1]) ** 2 * (1 - rho ** 2)
        cx, cz = sig[:, 1] ** 2 / det, sig[:, 0] ** 2 / det
        cy = -rho * sig[:, 0] * sig[:, 1] / det
        log2e = 1.4426950408889634
        xy.append(c)
        co.append(np.stack([-0.5 * log2e * cx, -log2e * cy, -0.5 * log2e * cz, np.log2(np.full(n, op))], 1))
        rgbd.append(np.concatenate([rng.uniform(0, colour_hi, (n, 3)), rng.uniform(1, 50, (n, 1))], 1))
        ranges[t] = (at, at + n)
        at += n
    xy = np.concatenate(xy).astype(np.float32)
    co = np.concatenate(co).astype(np.float32)
    rgbd = np.concatenate(rgbd).astype(np.float32)
    vals = np.arange(at, dtype=np.uint32)
    bg = np.asarray(bg, np.float32)
    _, ref, _ = oracle.render(W, H, 16, 16, xy, rgbd, co, vals, ranges, bg, want_u8=False)
    out = torch.full((H, W, 3), -1.0, device=gp.DEV, dtype=torch.float32)
    d = [gp.dev(a) for a in (xy, rgbd, co)]
    dv, dr = gp.dev(vals.view(np.int32)), gp.dev(ranges)
    cabi.blend(16, 16, W, H, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), dv.data_ptr(), dr.data_ptr(),
               bg, 0, out.data_ptr(), torch.cuda.current_stream().cuda_stream, flags=flags)
    torch.cuda.synchronize()
    return out.cpu().numpy(), ref


@pytest.mark.parametrize("W,H", [(320, 240), (3840, 400)])       # the kernel of small frames and the one of large frames
def test_blend_faint_weights_keep_their_relative_accuracy(oracle, W, H):
    """With FGS_BLEND_MATRIX_F16 the colour sums take their weights as f16.  Lists of thousands of Gaussians whose weights
    alpha*T lie between 1e-8 and 1e-5, far below f16's smallest normal number 6e-5, still add up to
    colours that are right to 2^-10 of themselves: the weights are scaled before the conversion."""
    gx = (W + 15) // 16
    lists = [(t, 1500 + 37 * (t % 5), op) for t, op in zip(range(0, 12 * gx, gx + 3), [1e-5, 3e-6, 1e-6, 3e-7, 1e-7, 1e-8] * 2)]
    from flashgs_amd import cabi
    got, ref = _blend_lists(oracle, lists, W, H, (0.0, 0.0, 0.0), seed=5, flags=cabi.BLEND_MATRIX_F16)
    lit = ref > 0
    assert lit.any() and ref[lit].max() < 0.05                      # faint sums, nothing near 1
    assert np.all(np.abs(got - ref)[lit] <= 2.0 ** -10 * ref[lit] + 1e-9)
    assert np.all(got[~lit] == 0)


def test_blend_colours_up_to_the_f16_range(oracle):
    """Colours far above 1 (up to 6e4, just inside f16) blend like any other with f16 operands:
    within 2^-10 of the pixel's own colour."""
    from flashgs_amd import cabi
    lists = [(t, 40 + t, 0.3) for t in range(0, 300, 7)]
    got, ref = _blend_lists(oracle, lists, 320, 240, (0.1, 0.2, 0.3), seed=9, colour_hi=6.0e4, flags=cabi.BLEND_MATRIX_F16)
    assert ref.max() > 1.0e4
    assert np.all(np.abs(got - ref) <= 2.0 ** -10 * np.abs(ref) + 1e-4)


@pytest.mark.parametrize("W,H,block", [(1280, 720, (16, 16)), (5120, 2880, (16, 16)), (1000, 600, (32, 16)), (1000, 600, (32, 32))])
def test_colour_sum_modes_per_call_and_by_default(oracle, W, H, block):
    """The colour sums by fp32 multiply-add (the default) and on the matrix unit with f16 operands
    (FGS_BLEND_MATRIX_F16), on the kernel of small frames, the one of large frames and both wide
    tiles.  The fp32 image is as close to the oracle as the exponent's evaluation order allows, far
    inside the f16 bound.  A per-call flag wins over the process default; the entry points without
    flags follow fgs_set_colour_sums."""
    import gpu_pipeline as gp
    from flashgs_amd import cabi
    sc = scenes.config0(n=60_000)
    cam = sc.cameras[0]
    scale = H / cam.height
    cam.width, cam.height = W, H
    cam.focal_x *= scale
    cam.focal_y *= scale
    bg = np.array([0.3, 0.5, 0.7], np.float32)
    ref = _oracle_frame(oracle, sc, cam, 1 << 22, block=block, bg=bg)
    K = ref["K"]
    got = gp.preprocess(gp.SceneOnDevice(sc), cam, 1 << 22, block=block)
    assert got["num_rendered"] == K
    ks, vs = gp.sort(K, W, H, got["keys"], got["values"], block)

    def image(flags):
        _, u8, f32 = gp.render(K, W, H, got["points_xy"], got["rgb_depth"], got["conic_opacity"], ks, vs, bg, block, flags=flags)
        return u8.cpu().numpy(), f32.cpu().numpy()

    assert "true>" in cabi.blend_kernel_name(block[0], block[1], W, H)                # the default is fp32
    assert "true>" in cabi.blend_kernel_name(block[0], block[1], W, H, cabi.BLEND_FP32)
    assert "false>" in cabi.blend_kernel_name(block[0], block[1], W, H, cabi.BLEND_MATRIX_F16)
    by_default, fp32, f16 = image(None), image(cabi.BLEND_FP32), image(cabi.BLEND_MATRIX_F16)
    assert np.array_equal(by_default[1], fp32[1]) and np.array_equal(by_default[0], fp32[0])
    assert not np.array_equal(fp32[1], f16[1])
    err32, err16 = np.abs(fp32[1] - ref["f32"]), np.abs(f16[1] - ref["f32"])
    assert err32.max() <= 2e-4, "fp32 colour sums: max abs image error %g" % err32.max()
    assert err16.max() <= IMG_MAX_ABS and err32.mean() < err16.mean()
    d8 = np.abs(fp32[0].astype(np.int16) - ref["u8"].astype(np.int16))
    assert d8.max() <= 1 and (d8 > 0).mean() < 0.005
    prev = cabi.set_colour_sums(cabi.COLOUR_SUMS_MATRIX_F16)
    try:
        assert prev == cabi.COLOUR_SUMS_FP32
        assert "false>" in cabi.blend_kernel_name(block[0], block[1], W, H)
        assert np.array_equal(image(None)[1], f16[1])                 # flag-less calls follow the process default ...
        assert np.array_equal(image(cabi.BLEND_FP32)[1], fp32[1])     # ... a flag does not
    finally:
        cabi.set_colour_sums(prev)


def test_ranges_kernel_against_searchsorted():
    import gpu_pipeline as gp
    import torch
    from flashgs_amd import cabi
    rng = np.random.default_rng(33)
    W, H = 1920, 1080
    tiles = 120 * 68
    for n, top, beyond in ((0, tiles, 0), (1, tiles, 0), (5, tiles, 0), (70_001, tiles, 0), (3000, tiles - 700, 0),
                           (70_001, tiles - 3, 40)):
        # tiles 1000..1300 and everything from `top` up stay empty; `beyond` pairs carry tile ids
        # outside the image (they sort to the end and belong to no range)
        tile = np.sort(rng.integers(0, top, n)).astype(np.uint64)
        tile = tile[(tile < 1000) | (tile > 1300)]
        tile = np.concatenate([tile, np.sort(rng.integers(tiles, tiles + 9, beyond)).astype(np.uint64)])
        n = tile.size
        keys = (tile << np.uint64(32)) | rng.integers(0, 1 << 32, n).astype(np.uint64)
        dk = gp.dev(keys.view(np.int64)) if n else torch.zeros(1, device=gp.DEV, dtype=torch.int64)
        rg = torch.full((tiles, 2), -9, device=gp.DEV, dtype=torch.int32)
        cabi.tile_ranges(16, 16, n, W, H, dk.data_ptr(), rg.data_ptr(), 0)
        torch.cuda.synchronize()
        lo = np.searchsorted(tile, np.arange(tiles), side="left")
        hi = np.searchsorted(tile, np.arange(tiles), side="right")
        want = np.where((lo == hi)[:, None], 0, np.stack([lo, hi], 1)).astype(np.int32)
        assert np.array_equal(rg.cpu().numpy(), want)


@pytest.mark.parametrize("config", [1, 2, 4])
def test_full_size_configs(oracle, config):
    """The 1080p / 1M, the 4K / 3M and (every sixth pose of) the 2M orbit configurations end to
    end against the oracle.  The orbit has needle-shaped splats next to the camera whose candidate
    rectangles cover the screen: most of its candidates are rejected by the exact tile test."""
    sc = scenes.make(config)
    for cam in sc.cameras[::6] if config == 4 else (sc.cameras[0],):
        ref = _check_frame(oracle, sc, cam, 1 << 24)
        if config == 4:
            assert ref["pre"]["counts"]["candidates"] > 3 * ref["K"]


def test_orbit_config_at_4k(oracle):
    """The 2M orbit at 3840x2160, every sixth pose and the last: the needles next to the camera have
    candidate rectangles of thousands of tiles, which the workgroup tests from column and row spans."""
    sc = scenes.make(4, width=3840, height=2160)
    for cam in sc.cameras[::6] + [sc.cameras[-1]]:
        ref = _check_frame(oracle, sc, cam, 1 << 25)
        assert ref["pre"]["counts"]["candidates"] > 5 * ref["K"]


def test_orbit_config_at_4k_with_the_needles_stored_last(oracle):
    """The same scene with its anisotropic tenth stored last: the last 780 workgroups hold nothing
    but needles, up to the 27 listed rectangles each and more.  Three poses."""
    sc = scenes.make(6, width=3840, height=2160)
    for cam in sc.cameras[::25]:
        ref = _check_frame(oracle, sc, cam, 1 << 25)
        assert ref["pre"]["counts"]["candidates"] > 5 * ref["K"]


@pytest.fixture(scope="module")
def config3_scene():
    return scenes.make(3)


def test_config3_8k_frame(oracle, config3_scene):
    """8M Gaussians at 7680x4320 (129 600 tiles, two partition passes of 9-bit digits, the blend
    variant with fewer resident waves), 2 % of the splats enlarged: the whole frame against the oracle."""
    sc = config3_scene
    ref = _check_frame(oracle, sc, sc.cameras[0], 1 << 25)
    assert ref["K"] > 10_000_000


def test_config3_more_than_100M_pairs(oracle, config3_scene):
    """The same scene with every splat five times as large: more than 100M pairs in a key buffer of
    2^27 entries (example.py:123), slot arithmetic far beyond 2^24, hundreds of tiles with more
    than 8192 pairs.  The whole frame against the oracle; then with a key buffer smaller than the
    pair count: the count is still the full one and nothing is written past the capacity
    (the reference would write out of bounds there, preprocess.cu:330,395; example.py:79-82 only
    checks afterwards)."""
    import gpu_pipeline as gp
    sc = scenes.config3_dense(base=config3_scene)
    cam = sc.cameras[0]
    ref = _check_frame(oracle, sc, cam, 1 << 27)
    K = ref["K"]
    assert K > 100_000_000
    assert ((ref["ranges"][:, 1] - ref["ranges"][:, 0]) > 8192).sum() > 100
    cap = 100_000_000
    got = gp.preprocess(gp.SceneOnDevice(sc), cam, cap, pad=1 << 20)
    assert got["num_rendered"] == K
    assert np.array_equal(gp.u64(got["keys"])[:cap], ref["pre"]["keys"][:cap])
    assert np.array_equal(gp.u32(got["values"])[:cap], ref["pre"]["values"][:cap])
    assert not gp.u64(got["keys"])[cap:].any() and not gp.u32(got["values"])[cap:].any()


def _sort_case(tile, depth_bits, W, H, junk=None, seed=0, ascending=False):
    """`ascending`: the values are the input positions, as the pairs of a tile leave the preprocess
    (ascending Gaussian indices): the sorting networks then break ties of depth by the value itself.
    Otherwise a random permutation, where they have to carry positions."""
    import gpu_pipeline as gp
    rng = np.random.default_rng(seed)
    n = tile.size
    keys = (tile.astype(np.uint64) << np.uint64(32)) | depth_bits.astype(np.uint64)
    gx, gy = (W + 15) // 16, (H + 15) // 16
    end_bit = 32 + int(gx * gy).bit_length()
    if junk is not None:
        keys = keys | (junk.astype(np.uint64) << np.uint64(end_bit))
    vals = rng.permutation(n).astype(np.uint32)
    if ascending:
        vals = np.arange(n, dtype=np.uint32)
        far = rng.integers(0, n, 3)                      # three tiles' segments that do not ascend among all that do
        vals[far] = vals[far][::-1] + np.uint32(1 << 30)
    ks, vs = gp.sort(n, W, H, gp.dev(keys.view(np.int64)), gp.dev(vals.view(np.int32)))
    masked = keys & np.uint64((1 << end_bit) - 1)
    order = np.argsort(masked, kind="stable")
    assert np.array_equal(gp.u64(ks)[:n], keys[order])
    assert np.array_equal(gp.u32(vs)[:n], vals[order])


@pytest.mark.parametrize("dense", [False, True])
@pytest.mark.parametrize("seg", [1500, 3000, 5000, 8000, 8192, 8193, 12000, 16384, 16385, 40000])
def test_sort_segment_size_classes(seg, dense):
    """Tiles holding 1500 ... 40000 pairs: every size class of the per-tile depth sort, with many
    equal depths and with depths that agree in whole bytes (skipped passes); on a frame of many
    tiles with few pairs and on one of 16 tiles with thousands of pairs each."""
    rng = np.random.default_rng(seg)
    if dense:
        W, H = 64, 64
        tile = np.repeat(np.array([5, 6, 9, 15, 1], np.uint32), [seg, 7, seg // 2, seg, 20000])
    else:
        W, H = 1920, 1080
        tile = np.repeat(np.array([5, 6, 4000, 8159], np.uint32), [seg, 7, seg // 2, seg])
    rng.shuffle(tile)
    depth = rng.uniform(1.0, 1.9, tile.size).astype(np.float32)      # same exponent: top byte constant
    depth[::3] = np.float32(1.5)
    _sort_case(tile, depth.view(np.uint32), W, H, seed=seg)


@pytest.mark.parametrize("ascending", [False, True])
@pytest.mark.parametrize("W,H", [(1920, 1080), (3840, 2160)])
def test_sort_every_segment_length_up_to_1100(W, H, ascending):
    """One tile per length 1 ... 1100: every padding of the register sorting networks (64, 128, ... 1024
    elements) and the first lengths of the next class, with many equal depths (ties must keep input
    order) and with depths of all magnitudes, 0 and 0xffffffff included.  At 1080p one launch sorts
    every segment of up to 1024 pairs, at 4K those above 512 come from a list in a launch of their own."""
    rng = np.random.default_rng(1100)
    lengths = np.arange(1, 1101)
    tiles = rng.permutation(((W + 15) // 16) * ((H + 15) // 16))[:lengths.size].astype(np.uint32)
    tile = np.repeat(tiles, lengths)
    depth = rng.integers(0, 1 << 32, tile.size, dtype=np.uint64).astype(np.uint32)
    depth[::5] = depth[1::5][: depth[::5].size]          # duplicates next to each other before the shuffle
    depth[rng.integers(0, tile.size, 2000)] = 0
    depth[rng.integers(0, tile.size, 2000)] = 0xFFFFFFFF
    order = rng.permutation(tile.size)
    _sort_case(tile[order], depth[order], W, H, seed=7, ascending=ascending)


@pytest.mark.parametrize("n,W,H", [(262_144, 1280, 720), (262_145, 1280, 720), (524_288, 1920, 1080), (524_289, 1920, 1080),
                                   (262_144, 7680, 4320), ((1 << 24) - 1, 3840, 2160), ((1 << 24) + 1, 3840, 2160)])
def test_sort_around_the_list_lengths_where_the_launches_change(n, W, H):
    """The partition blocks are smaller up to 262 144 pairs, the last segment launch takes the
    classes above 1024 pairs up to 2^19 pairs and the one above 4096 up to 2^24: lists of just those
    lengths and one more, with crowded tiles of every class among evenly filled ones, values in
    input order (the networks' tie-break) and many equal depths."""
    rng = np.random.default_rng(n % 1000 + W)
    tiles = ((W + 15) // 16) * ((H + 15) // 16)
    tile = rng.integers(0, tiles, n).astype(np.uint32)
    pos = 0
    for length in (600, 1024, 1025, 3000, 4096, 4097, 8192, 8193, 20000, 70000):
        if pos + length > n // 2:
            break
        tile[pos:pos + length] = rng.integers(0, tiles)
        pos += length
    rng.shuffle(tile)
    depth = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    depth[::7] = depth[3]
    _sort_case(tile, depth, W, H, seed=n % 97, ascending=True)


def test_sort_bits_above_the_range_stay_with_their_pair():
    """Bits above 32 + bit_length(tiles) are outside the sorted range (sort.cu:34-39) but travel
    with the key; segments whose keys differ there take the general path."""
    rng = np.random.default_rng(77)
    W, H = 640, 480                                   # 1200 tiles -> 11 tile bits
    n = 60000
    tile = rng.integers(0, 1200, n).astype(np.uint32)
    tile[:20000] = 17                                 # one long segment
    tile[20000:23000] = 18                            # and one of the classes that are sorted in LDS
    tile[23000:29500] = 19
    depth = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    junk = rng.integers(0, 1 << 10, n).astype(np.uint32)
    junk[30000:] = 0
    _sort_case(tile, depth, W, H, junk=junk, seed=1)
    # the same on a frame whose list is long enough for the classes to have launches of their own
    W, H = 1920, 1080
    n = 700_000
    tile = rng.integers(0, 8160, n).astype(np.uint32)
    tile[:20000] = 17
    tile[20000:23000] = 18
    tile[23000:29500] = 19
    depth = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    junk = rng.integers(0, 1 << 10, n).astype(np.uint32)
    junk[30000:] = 0
    _sort_case(tile, depth, W, H, junk=junk, seed=2)


@pytest.mark.parametrize("W,H,n", [(16, 16, 5000), (256, 16, 9000), (160, 128, 70_000), (3840, 2160, 300),
                                   (7680, 4320, 40), (8208, 8208, 200_000), (8208, 8208, 90)])
def test_sort_segment_table_shapes(W, H, n):
    """The table of segment starts under every way it is produced: one partition pass (up to 256 tile
    ids, one of them a frame of a single tile), two passes on a sparse frame (one workgroup owns every
    entry, most tile ids empty, first and last tile in use), and 263 169 tiles (19 tile bits, three
    passes, where a launch of its own reads the sorted keys)."""
    rng = np.random.default_rng(W + n)
    tiles = ((W + 15) // 16) * ((H + 15) // 16)
    tile = rng.integers(0, tiles, n).astype(np.uint32)
    tile[:3] = tiles - 1
    tile[3:5] = 0
    depth = rng.uniform(0.2, 90.0, n).astype(np.float32)
    depth[::4] = np.float32(2.5)
    _sort_case(tile, depth.view(np.uint32), W, H, seed=n)


def test_sort_low_digit_changes_at_block_boundaries():
    """Second partition pass whose input blocks (4096 pairs) end exactly where the low tile digit
    changes, with low digits that no pair has in between: every entry of the segment table still
    has exactly one writer."""
    rng = np.random.default_rng(4096)
    W, H = 3840, 2160
    lows = np.array([3, 7, 7, 200, 201, 255], np.uint32)
    high = rng.integers(0, 126, (lows.size, 4096)).astype(np.uint32)
    tile = (high * 256 + lows[:, None]).reshape(-1)
    tile = tile[rng.permutation(tile.size)]
    depth = rng.integers(0, 1 << 32, tile.size, dtype=np.uint64).astype(np.uint32)
    _sort_case(tile, depth, W, H, seed=3)


def test_sort_more_tile_ids_than_the_segment_table():
    """16400 x 16400 pixels = 1 050 625 tiles: 21 tile bits, three partition passes of 9-bit digits,
    and segment bounds found by search instead of the table."""
    rng = np.random.default_rng(78)
    W = H = 16400
    n = 300_000
    tile = rng.integers(0, 1025 * 1025, n).astype(np.uint32)
    tile[:5000] = 1_050_624
    tile[5000:9000] = 0
    depth = rng.uniform(0.2, 90.0, n).astype(np.float32)
    _sort_case(tile, depth.view(np.uint32), W, H, seed=2)
