"""Deterministic synthetic scenes and cameras for the five benchmark configurations.

Every array is float32 in the layouts the ops take (``example.py:23-27`` of FlashGS):
``position [N,3]``, ``shs [N,48]`` (16 coefficients x RGB interleaved), ``opacity [N]`` (already
sigmoid-ed) and ``cov3d [N,6]`` (xx,xy,xz,yy,yz,zz).  Generation uses numpy's PCG64 stream seeded
with the configuration's seed and a fixed call order, so the CPU oracle and the GPU path see the
same bytes.

Camera convention (FlashGS ``preprocess.cu:420-427``, ``pybind.cpp:140-143``): ``rotation`` is the
camera-to-world matrix, row-major; the camera looks along its +z axis, +x is right and +y is DOWN
the image.  World "up" in the generated scenes is +y.
"""
from dataclasses import dataclass, field
import math

import numpy as np

TILE = 16
Z_FAR = 100.0   # example.py:40-41
Z_NEAR = 0.01


@dataclass
class Camera:
    width: int
    height: int
    position: np.ndarray          # float32 [3]
    rotation: np.ndarray          # float32 [3,3], camera-to-world, row-major
    focal_x: float
    focal_y: float
    zFar: float = Z_FAR
    zNear: float = Z_NEAR


@dataclass
class Scene:
    name: str
    position: np.ndarray
    shs: np.ndarray
    opacity: np.ndarray
    cov3d: np.ndarray
    cameras: list = field(default_factory=list)

    @property
    def num_vertex(self):
        return int(self.opacity.shape[0])


def focal_from_fov_y(height, fov_y_deg):
    return float(np.float32(height / (2.0 * math.tan(math.radians(fov_y_deg) / 2.0))))


def look_at(position, target, width, height, fov_y_deg):
    """Camera at ``position`` whose +z axis points at ``target``; image y runs down (world -y)."""
    position = np.asarray(position, np.float64)
    f = np.asarray(target, np.float64) - position
    f /= np.linalg.norm(f)
    down0 = np.array([0.0, -1.0, 0.0])
    r = np.cross(down0, f)
    r /= np.linalg.norm(r)
    d = np.cross(f, r)
    rot = np.stack([r, d, f], axis=1)   # columns are the camera axes in world space
    foc = focal_from_fov_y(height, fov_y_deg)
    return Camera(width, height, position.astype(np.float32), rot.astype(np.float32), foc, foc)


def cov3d_from_scale_rotation(scale, quat):
    """Sigma = R S^2 R^T with R from the (r,x,y,z) quaternion, as ``computeCov3D``
    (FlashGS ``pybind.cpp:22-56``) defines it; returns [N,6] float32 (xx,xy,xz,yy,yz,zz)."""
    scale = np.asarray(scale, np.float32)
    q = np.asarray(quat, np.float32)
    r, x, y, z = q[:, 0], q[:, 1], q[:, 2], q[:, 3]
    one, two = np.float32(1.0), np.float32(2.0)
    R = np.empty((q.shape[0], 3, 3), np.float32)
    R[:, 0, 0] = one - two * (y * y + z * z)
    R[:, 0, 1] = two * (x * y - r * z)
    R[:, 0, 2] = two * (x * z + r * y)
    R[:, 1, 0] = two * (x * y + r * z)
    R[:, 1, 1] = one - two * (x * x + z * z)
    R[:, 1, 2] = two * (y * z - r * x)
    R[:, 2, 0] = two * (x * z - r * y)
    R[:, 2, 1] = two * (y * z + r * x)
    R[:, 2, 2] = one - two * (x * x + y * y)
    M = R * scale[:, None, :]                      # M[r,k] = R[r,k] * s_k
    out = np.empty((q.shape[0], 6), np.float32)
    idx = [(0, 0), (0, 1), (0, 2), (1, 1), (1, 2), (2, 2)]
    for j, (a, b) in enumerate(idx):
        out[:, j] = M[:, a, 0] * M[:, b, 0] + M[:, a, 1] * M[:, b, 1] + M[:, a, 2] * M[:, b, 2]
    return out


def _sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def _unit_quats(rng, n):
    q = rng.standard_normal((n, 4))
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    return q.astype(np.float32)


def _shs(rng, n):
    shs = np.empty((n, 16, 3), np.float32)
    shs[:, 0, :] = (rng.standard_normal((n, 3)) * 0.5).astype(np.float32)
    shs[:, 1:, :] = (rng.standard_normal((n, 15, 3)) * 0.05).astype(np.float32)
    return shs.reshape(n, 48)


def _finish(name, rng, means, log_scales, opacity_mean, opacity_sigma, cameras, quats=None):
    n = means.shape[0]
    if quats is None:
        quats = _unit_quats(rng, n)
    opacity = _sigmoid(opacity_mean + opacity_sigma * rng.standard_normal(n)).astype(np.float32)
    shs = _shs(rng, n)
    cov3d = cov3d_from_scale_rotation(np.exp(log_scales).astype(np.float32), quats)
    return Scene(name, np.ascontiguousarray(means, np.float32), shs, opacity, cov3d, cameras)


def _clusters(rng, n, n_clusters=32, lo=-20.0, hi=20.0, sigma=3.0):
    centres = rng.uniform(lo, hi, (n_clusters, 3))
    which = rng.integers(0, n_clusters, n)
    return centres[which] + sigma * rng.standard_normal((n, 3))


def _city(rng, n, half_extent, n_boxes=200):
    """Noisy ground plane (half of the points) plus box-shaped buildings sampled on their
    four walls and roof (the other half)."""
    n_ground = n // 2
    n_build = n - n_ground
    ground = np.empty((n_ground, 3))
    ground[:, 0] = rng.uniform(-half_extent, half_extent, n_ground)
    ground[:, 1] = 0.5 * rng.standard_normal(n_ground)
    ground[:, 2] = rng.uniform(-half_extent, half_extent, n_ground)

    s = half_extent / 50.0
    cx = rng.uniform(-0.9 * half_extent, 0.9 * half_extent, n_boxes)
    cz = rng.uniform(-0.9 * half_extent, 0.9 * half_extent, n_boxes)
    wx = rng.uniform(2.0, 8.0, n_boxes) * s
    wz = rng.uniform(2.0, 8.0, n_boxes) * s
    hy = rng.uniform(3.0, 25.0, n_boxes) * s
    # face areas: +x, -x, +z, -z walls and the roof
    areas = np.stack([wz * hy, wz * hy, wx * hy, wx * hy, wx * wz], axis=1)
    flat = areas.ravel() / areas.sum()
    pick = rng.choice(n_boxes * 5, size=n_build, p=flat)
    b, face = pick // 5, pick % 5
    u = rng.uniform(-0.5, 0.5, n_build)
    v = rng.uniform(0.0, 1.0, n_build)
    pts = np.empty((n_build, 3))
    sgn = np.where(face % 2 == 0, 0.5, -0.5)
    xw = face < 2
    zw = (face >= 2) & (face < 4)
    roof = face == 4
    pts[:, 0] = np.where(xw, cx[b] + sgn * wx[b], cx[b] + u * wx[b])
    pts[:, 2] = np.where(xw, cz[b] + u * wz[b],
                         np.where(zw, cz[b] + sgn * wz[b], cz[b] + (v - 0.5) * wz[b]))
    pts[:, 1] = np.where(roof, hy[b], v * hy[b])
    return np.concatenate([ground, pts], axis=0)


# ---------------------------------------------------------------------------------------------

def config0(n=100_000):
    """1280x720, 100k Gaussians in [-5,5]^3, camera at (0,0,-15) looking at the origin."""
    rng = np.random.default_rng(0)
    means = rng.uniform(-5.0, 5.0, (n, 3))
    log_scales = -4.0 + 0.5 * rng.standard_normal((n, 3))
    foc = focal_from_fov_y(720, 50.0)
    cam = Camera(1280, 720, np.array([0, 0, -15], np.float32), np.eye(3, dtype=np.float32), foc, foc)
    return _finish("cfg0_100k_720p", rng, means, log_scales, 0.0, 1.5, [cam])


def config1(n=1_000_000):
    """1920x1080, 1M Gaussians in 32 clusters, camera on a radius-40 sphere."""
    rng = np.random.default_rng(1)
    means = _clusters(rng, n)
    log_scales = -3.5 + 0.7 * rng.standard_normal((n, 3))
    az, el = math.radians(30.0), math.radians(20.0)
    pos = 40.0 * np.array([math.cos(el) * math.sin(az), math.sin(el), -math.cos(el) * math.cos(az)])
    cam = look_at(pos, [0, 0, 0], 1920, 1080, 60.0)
    return _finish("cfg1_1M_1080p", rng, means, log_scales, 0.0, 2.0, [cam])


def _city_scene(name, seed, n, half_extent, width, height, fov_y, big_fraction=0.0):
    rng = np.random.default_rng(seed)
    means = _city(rng, n, half_extent)
    log_scales = -3.0 + 0.8 * rng.standard_normal((n, 3))
    log_scales[:, 2] -= 1.5                       # flat splats
    if big_fraction > 0.0:
        big = rng.uniform(0.0, 1.0, n) < big_fraction
        log_scales[big] += 2.0
    pos = np.array([0.0, 8.0, -0.9 * half_extent])
    pitch = math.radians(-15.0)
    target = pos + np.array([0.0, math.sin(pitch), math.cos(pitch)])
    cam = look_at(pos, target, width, height, fov_y)
    return _finish(name, rng, means, log_scales, 0.5, 2.0, [cam])


def config2(n=3_000_000):
    """Headline: 3840x2160, 3M Gaussians, ground plane + 200 buildings, camera 8 above ground."""
    return _city_scene("cfg2_3M_4K", 2, n, 50.0, 3840, 2160, 60.0)


def config3(n=8_000_000):
    """7680x4320, 8M Gaussians on [-200,200], 2 % of them with log-scales +2."""
    return _city_scene("cfg3_8M_8K", 3, n, 200.0, 7680, 4320, 70.0, big_fraction=0.02)


def config3_dense(n=8_000_000, base=None):
    """The 8K scene with every splat five times as large (covariances x 25): more than 100M pairs and
    hundreds of tiles with more than 8192 of them, the regime the 8K configuration is meant to
    stress.  `base` may be an already generated config3 scene of the same n, whose arrays are shared."""
    sc = base if base is not None else config3(n)
    return Scene("cfg3_dense_8M_8K", sc.position, sc.shs, sc.opacity, (sc.cov3d * np.float32(25.0)).astype(np.float32),
                 list(sc.cameras))


def config4(n=2_000_000, width=1920, height=1080, n_poses=60, aniso_last=False):
    """Orbit of 60 poses (radius 30, height 5, 6 degree steps) around the cluster scene; 10 % of
    the Gaussians are 100:1 anisotropic and lie within 1 unit of the camera path.  They are a
    random subset of the indices; with `aniso_last` they are stored as the last tenth of the
    scene instead (name ..._needles_last), which is the worst case for a preprocess that hands
    out key slots in index order: the workgroups that hold them then all run at the end."""
    rng = np.random.default_rng(4)
    n_aniso = n // 10
    n_reg = n - n_aniso
    means = _clusters(rng, n_reg)
    log_scales = -3.5 + 0.7 * rng.standard_normal((n_reg, 3))
    ang = rng.uniform(0.0, 2.0 * math.pi, n_aniso)
    off = rng.standard_normal((n_aniso, 3))
    off *= (rng.uniform(0.0, 1.0, (n_aniso, 1)) ** (1.0 / 3.0)) / np.linalg.norm(off, axis=1, keepdims=True)
    path = np.stack([30.0 * np.sin(ang), np.full(n_aniso, 5.0), -30.0 * np.cos(ang)], axis=1)
    a_means = path + off
    a_ls = -4.5 + 0.5 * rng.standard_normal((n_aniso, 1)) + np.zeros((1, 3))
    a_ls[:, 0] += math.log(100.0)                 # one long axis: ratio 100:1
    means = np.concatenate([means, a_means], axis=0)
    log_scales = np.concatenate([log_scales, a_ls], axis=0)
    if not aniso_last:
        place = np.random.default_rng(44).permutation(n)       # a generator of its own: everything else is drawn as before
        means, log_scales = means[place], log_scales[place]
    cams = []
    for k in range(n_poses):
        a = math.radians(6.0 * k)
        pos = np.array([30.0 * math.sin(a), 5.0, -30.0 * math.cos(a)])
        cams.append(look_at(pos, [0, 0, 0], width, height, 60.0))
    name = "cfg4_2M_orbit_%dx%d%s" % (width, height, "_needles_last" if aniso_last else "")
    return _finish(name, rng, means, log_scales, 0.0, 2.0, cams)


def config4_needles_last(**kw):
    """The orbit scene with its anisotropic tenth stored last (see config4)."""
    return config4(aniso_last=True, **kw)


CONFIGS = {0: config0, 1: config1, 2: config2, 3: config3, 4: config4, 5: config3_dense, 6: config4_needles_last}


def make(config, **kw):
    return CONFIGS[int(config)](**kw)
