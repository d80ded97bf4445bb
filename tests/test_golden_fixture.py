"""The committed fixture tests/golden/frame_small.npz against the oracle (CPU) and the HIP path (GPU).

The fixture holds what the oracle produced for one small seeded frame when it was written
(tests/golden/make_fixture.py); the reference ships no vectors of its own for this path.
"""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import make_fixture as mf   # noqa: E402

FIXTURE = os.path.join(HERE, "golden", "frame_small.npz")


@pytest.fixture(scope="module")
def golden():
    return np.load(FIXTURE)       # allow_pickle stays False


def test_scene_generator_reproduces_the_fixture_inputs(golden):
    sc, _ = mf.small_frame()
    assert bytes(golden["input_sha256"]).hex() == mf.input_digest(sc)


def test_oracle_reproduces_the_fixture(oracle, golden):
    sc, cam = mf.small_frame()
    bx, by = mf.BLOCK
    pre = oracle.preprocess(sc.position, sc.shs, sc.opacity, sc.cov3d, cam.width, cam.height, bx, by,
                            cam.position, cam.rotation, cam.focal_x, cam.focal_y, cam.zFar, cam.zNear, mf.CAPACITY)
    K = int(golden["num_rendered"])
    assert pre["num_rendered"] == K
    assert np.array_equal(pre["keys"][:K], golden["keys_unsorted"])
    assert np.array_equal(pre["values"][:K], golden["values_unsorted"])
    vis = golden["visible"]
    for name in ("points_xy", "conic_opacity", "rgb_depth"):
        assert np.array_equal(pre[name][vis].view(np.uint32), golden[name].view(np.uint32)), name
    ks, vs = oracle.sort(K, cam.width, cam.height, bx, by, pre["keys"], pre["values"])
    assert np.array_equal(ks[:K], golden["keys_sorted"])
    assert np.array_equal(vs[:K], golden["values_sorted"])
    rg = oracle.ranges(K, ks, golden["ranges"].shape[0])
    assert np.array_equal(rg, golden["ranges"])
    u8, _, walked = oracle.render(cam.width, cam.height, bx, by, pre["points_xy"], pre["rgb_depth"],
                                  pre["conic_opacity"], vs, rg, mf.BG)
    assert walked == int(golden["walked"])
    # exp2f comes from the host's libm: allow the last 8-bit step to differ between machines
    assert np.abs(u8.astype(np.int16) - golden["image_u8"].astype(np.int16)).max() <= 1


@pytest.mark.gpu
def test_hip_path_reproduces_the_fixture(golden):
    import gpu_pipeline as gp
    sc, cam = mf.small_frame()
    K = int(golden["num_rendered"])
    sd = gp.SceneOnDevice(sc)
    got = gp.preprocess(sd, cam, mf.CAPACITY, mf.BLOCK)
    assert got["num_rendered"] == K
    assert np.array_equal(gp.u64(got["keys"])[:K], golden["keys_unsorted"])
    assert np.array_equal(gp.u32(got["values"])[:K], golden["values_unsorted"])
    vis = golden["visible"].astype(np.int64)
    for name in ("points_xy", "conic_opacity", "rgb_depth"):
        assert np.array_equal(gp.bits(got[name].cpu().numpy()[vis]), gp.bits(golden[name])), name
    ks, vs = gp.sort(K, cam.width, cam.height, got["keys"], got["values"], mf.BLOCK)
    assert np.array_equal(gp.u64(ks)[:K], golden["keys_sorted"])
    assert np.array_equal(gp.u32(vs)[:K], golden["values_sorted"])
    rg, u8, _ = gp.render(K, cam.width, cam.height, got["points_xy"], got["rgb_depth"], got["conic_opacity"],
                          ks, vs, mf.BG, mf.BLOCK)
    assert np.array_equal(rg.cpu().numpy(), golden["ranges"])
    d8 = np.abs(u8.cpu().numpy().astype(np.int16) - golden["image_u8"].astype(np.int16))
    assert d8.max() <= 1 and (d8 > 0).mean() < 0.01
