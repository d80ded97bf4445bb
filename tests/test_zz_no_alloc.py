"""fgs_preprocess_static - the entry point that allocates nothing - against fgs_preprocess on the
same inputs: pair count, keys, values and their order, and the three attribute tensors (untouched
rows included) must be bit-identical.  Two calls in a row share the built-in scan status, the
second with a smaller input; the size limit is an error, not a fault."""
import numpy as np
import pytest

from flashgs_amd import scenes

pytestmark = pytest.mark.gpu


def _same(a, b, K):
    import gpu_pipeline as gp
    assert a["num_rendered"] == b["num_rendered"] == K
    assert np.array_equal(gp.u64(a["keys"])[:K], gp.u64(b["keys"])[:K])
    assert np.array_equal(gp.u32(a["values"])[:K], gp.u32(b["values"])[:K])
    for name in ("points_xy", "conic_opacity", "rgb_depth"):
        assert np.array_equal(gp.bits(a[name].cpu().numpy()), gp.bits(b[name].cpu().numpy())), name


def test_static_entry_point_matches_the_allocating_one():
    import gpu_pipeline as gp
    big = scenes.config0(n=300_000)
    small = scenes.config0(n=41_000)
    cam = big.cameras[0]
    cap = 1 << 22
    sds = {id(sc): gp.SceneOnDevice(sc) for sc in (big, small)}
    want = {id(sc): gp.preprocess(sds[id(sc)], cam, cap, sentinel=-5.5) for sc in (big, small)}
    for sc in (big, small, big):            # in a row: larger, smaller, larger again; the status arrays are reused
        got = gp.preprocess(sds[id(sc)], cam, cap, sentinel=-5.5, static=True)
        assert want[id(sc)]["num_rendered"] > 10_000
        _same(got, want[id(sc)], want[id(sc)]["num_rendered"])
    # mixed with the allocating entry point and with another tile size
    sd = gp.SceneOnDevice(small)
    want = gp.preprocess(sd, cam, cap, block=(32, 16), sentinel=1.25)
    got = gp.preprocess(sd, cam, cap, block=(32, 16), sentinel=1.25, static=True)
    _same(got, want, want["num_rendered"])


def test_static_entry_point_allocates_nothing_and_runs_under_capture():
    """What the entry point is for.  The first call on a fresh stream leaves the device's free
    memory as it was (the allocating entry point takes its scan status there); the call can be
    captured into a graph on a stream that has never run a preprocess, which fails if anything
    allocates or synchronises; replays, alternating with eager static calls of another size on
    another scene, give the allocating entry point's result every time."""
    import gpu_pipeline as gp
    import torch
    from flashgs_amd import cabi
    a, b = scenes.config0(n=200_000), scenes.config1(n=90_000)
    cam, cam_b = a.cameras[0], b.cameras[0]
    sd, sd_b = gp.SceneOnDevice(a), gp.SceneOnDevice(b)
    cap = 1 << 22
    want, want_b = gp.preprocess(sd, cam, cap), gp.preprocess(sd_b, cam_b, cap)
    K, K_b = want["num_rendered"], want_b["num_rendered"]
    n = sd.n
    xy = torch.zeros((n, 2), device=gp.DEV); rgb = torch.zeros((n, 4), device=gp.DEV); co = torch.zeros((n, 4), device=gp.DEV)
    keys = torch.zeros(cap, device=gp.DEV, dtype=torch.int64)
    values = torch.zeros(cap, device=gp.DEV, dtype=torch.int32)
    off = torch.zeros(1, device=gp.DEV, dtype=torch.int32)

    def launch(stream):
        cabi.preprocess(n, sd.position.data_ptr(), sd.shs.data_ptr(), sd.opacity.data_ptr(), sd.cov3d.data_ptr(),
                        cam.width, cam.height, 16, 16, cam.position, cam.rotation, cam.focal_x, cam.focal_y,
                        cam.zFar, cam.zNear, xy.data_ptr(), rgb.data_ptr(), co.data_ptr(),
                        keys.data_ptr(), values.data_ptr(), off.data_ptr(), cap, stream, static=True)

    def check(what):
        torch.cuda.synchronize()
        assert int(off.cpu()[0]) == K, what
        assert np.array_equal(gp.u64(keys)[:K], gp.u64(want["keys"])[:K]), what
        assert np.array_equal(gp.u32(values)[:K], gp.u32(want["values"])[:K]), what

    fresh = torch.cuda.Stream()
    fresh.wait_stream(torch.cuda.current_stream())
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    launch(fresh.cuda_stream)
    check("first static call on a fresh stream")
    assert torch.cuda.mem_get_info()[0] == free_before, "the static entry point took device memory"

    side = torch.cuda.Stream()                   # has never run a preprocess: nothing to fall back on but the built-in status
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        off.zero_()
        launch(torch.cuda.current_stream().cuda_stream)
    for replay in range(3):
        keys.zero_(); values.zero_()
        graph.replay()
        check("replay %d" % replay)
        got_b = gp.preprocess(sd_b, cam_b, cap, static=True)            # another scene and size on the same status
        assert got_b["num_rendered"] == K_b
        assert np.array_equal(gp.u64(got_b["keys"])[:K_b], gp.u64(want_b["keys"])[:K_b])


def test_static_entry_point_rejects_what_its_status_cannot_hold():
    from flashgs_amd import cabi
    with pytest.raises(RuntimeError, match="exceeds"):
        cabi.preprocess((1 << 24) + 1, 1, 1, 1, 1, 64, 64, 16, 16, [0, 0, 0], np.eye(3), 50.0, 50.0, 100.0, 0.01,
                        1, 1, 1, 1, 1, 1, 16, 0, static=True)
