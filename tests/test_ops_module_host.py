"""The Python op surface without a GPU: the module has the reference's name and operators
(``csrc/pybind.cpp:233-271`` of FlashGS), refuses host tensors where device tensors are needed,
and ``loadPly`` parses the 62-float records of a 3DGS .ply."""
import math
import struct

import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def ops():
    import flash_gaussian_splatting
    return flash_gaussian_splatting.ops


def test_operator_names(ops):
    for name in ("loadPly", "preprocess", "sort_gaussian", "get_sort_buffer_size", "render_16x16", "render_32x16", "render_32x32",
                 "reset_scan", "preprocess_mirrored", "wait_count"):
        assert callable(getattr(ops, name))
    assert ops.get_sort_buffer_size(2 ** 20) >= 12 * 2 ** 20
    with pytest.raises(RuntimeError):
        ops.get_sort_buffer_size(-1)


def test_host_tensors_are_refused(ops):
    n = 4
    f = lambda *s: torch.zeros(*s, dtype=torch.float32)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ops.preprocess(f(n, 3), f(n, 48), f(n), f(n, 6), 64, 64, 16, 16, f(3), torch.eye(3), 50.0, 50.0, 100.0, 0.01,
                       f(n, 2), f(n, 4), f(n, 4), torch.zeros(16, dtype=torch.int64), torch.zeros(16, dtype=torch.int32),
                       torch.zeros(1, dtype=torch.int32))
    with pytest.raises(RuntimeError):
        ops.sort_gaussian(0, 64, 64, 16, 16, torch.zeros(8, dtype=torch.int8), torch.zeros(1, dtype=torch.int64),
                          torch.zeros(1, dtype=torch.int32), torch.zeros(1, dtype=torch.int64), torch.zeros(1, dtype=torch.int32))
    with pytest.raises(RuntimeError):
        ops.render_16x16(0, 64, 64, f(n, 2), f(n, 4), f(n, 4), torch.zeros(1, dtype=torch.int64),
                         torch.zeros(1, dtype=torch.int32), torch.zeros(16, 2, dtype=torch.int32), f(3),
                         torch.zeros(64, 64, 3, dtype=torch.int8))


def _write_ply(path, recs):
    props = ["x", "y", "z", "nx", "ny", "nz"] + ["f_dc_%d" % i for i in range(3)] + ["f_rest_%d" % i for i in range(45)] \
        + ["opacity"] + ["scale_%d" % i for i in range(3)] + ["rot_%d" % i for i in range(4)]
    head = "ply\nformat binary_little_endian 1.0\nelement vertex %d\n" % len(recs)
    head += "".join("property float %s\n" % p for p in props) + "end_header\n"
    with open(path, "wb") as fh:
        fh.write(head.encode())
        for r in recs:
            fh.write(struct.pack("<62f", *r))


def test_load_ply(ops, tmp_path, oracle):
    rng = np.random.default_rng(5)
    n = 37
    recs = rng.standard_normal((n, 62)).astype(np.float32)
    path = str(tmp_path / "point_cloud.ply")
    _write_ply(path, recs)
    num, pos, shs, opac, cov3d = ops.loadPly(path)
    assert num == n and pos.shape == (n, 3) and shs.shape == (n, 48) and opac.shape == (n,) and cov3d.shape == (n, 6)
    assert np.array_equal(pos.numpy(), recs[:, 0:3])
    sh = recs[:, 6:54]
    want = np.empty((n, 16, 3), np.float32)
    want[:, 0] = sh[:, 0:3]
    for j in range(1, 16):        # planar f_rest (15 r, 15 g, 15 b) -> interleaved per coefficient
        want[:, j, 0] = sh[:, 3 + j - 1]
        want[:, j, 1] = sh[:, 3 + 15 + j - 1]
        want[:, j, 2] = sh[:, 3 + 30 + j - 1]
    assert np.array_equal(shs.numpy(), want.reshape(n, 48))
    np.testing.assert_allclose(opac.numpy(), 1 / (1 + np.exp(-recs[:, 54].astype(np.float64))), rtol=1e-6)
    scale = np.exp(recs[:, 55:58].astype(np.float64))
    q = recs[:, 58:62].astype(np.float64)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    ref = oracle.cov3d(scale.astype(np.float32), q.astype(np.float32))
    np.testing.assert_allclose(cov3d.numpy(), ref, rtol=2e-5, atol=1e-7)


def test_load_ply_errors(ops, tmp_path):
    with pytest.raises(RuntimeError, match="Failed to open"):
        ops.loadPly(str(tmp_path / "missing.ply"))
    bad = tmp_path / "bad.ply"
    bad.write_bytes(b"ply\nformat binary_little_endian 1.0\nelement vertex 3\n")
    with pytest.raises(RuntimeError, match="end of header"):
        ops.loadPly(str(bad))
    neg = tmp_path / "neg.ply"
    neg.write_bytes(b"ply\nelement vertex 0\nend_header\n")
    with pytest.raises(RuntimeError, match="not positive"):
        ops.loadPly(str(neg))
    short = tmp_path / "short.ply"
    short.write_bytes(b"ply\nelement vertex 2\nend_header\n" + b"\0" * 100)
    with pytest.raises(RuntimeError, match="exceeds the 0 records"):
        ops.loadPly(str(short))
    # a header may claim any count: it is checked against the file's size before anything is allocated
    # (2^31 - 1 vertices would be 532 GB of tensors)
    huge = tmp_path / "huge.ply"
    huge.write_bytes(b"ply\nelement vertex 2147483647\nend_header\n" + b"\0" * (62 * 4 * 3))
    with pytest.raises(RuntimeError, match="exceeds the 3 records"):
        ops.loadPly(str(huge))
