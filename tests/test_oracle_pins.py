"""Pins for the CPU oracle: every function is checked against something that does not come from
the oracle's own source - float64 closed forms, library routines (numpy stable argsort,
searchsorted, scipy spherical harmonics), a convex-QP solution of the ellipse/rectangle problem,
brute force over pixel centres.  The reference ships no golden vectors for this path, so these
are what fixes the oracle; each check is chosen so that a dropped term, a wrong sign or a
transposed operand fails it.  Runs on the CPU only.
"""
import math

import numpy as np
import pytest
from scipy import special

LOG2E = 1.4426950408889634


# ---- log2 -------------------------------------------------------------------------------------------

def test_log2_against_float64(oracle):
    rng = np.random.default_rng(10)
    x = np.concatenate([rng.uniform(1 / 255, 1.0, 20000), 2.0 ** rng.uniform(-20, 20, 5000),
                        [1.0, 0.5, 0.25, 2.0, 1 / 255, 1.41421354, 1.4142137, 0.70710677]]).astype(np.float32)
    got = oracle.log2f(x).astype(np.float64)
    want = np.log2(x.astype(np.float64))
    ulp = np.spacing(np.abs(want).astype(np.float32)).astype(np.float64)
    assert np.all(np.abs(got - want) <= 4 * ulp + 1e-9)          # measured worst case: 3 ulp
    assert np.all(np.abs(got - want) <= 5e-7 * np.abs(want) + 1e-9)
    assert oracle.log2f(np.float32([1.0]))[0] == 0.0
    assert oracle.log2f(np.float32([0.25]))[0] == -2.0


def test_higher_msb_is_bit_length(oracle):
    for n in list(range(1, 600)) + [3600, 8160, 32400, 129600, 65535, 65536, 2 ** 20, 2 ** 31 - 1, 2 ** 32 - 1]:
        assert oracle.higher_msb(n) == int(n).bit_length()


# ---- camera matrices ------------------------------------------------------------------------------------

def _rot(seed):
    rng = np.random.default_rng(seed)
    q, _ = np.linalg.qr(rng.standard_normal((3, 3)))
    if np.linalg.det(q) < 0:
        q[:, 0] = -q[:, 0]
    return q


def test_view_proj_closed_forms(oracle):
    W, H, fx, fy = 1280, 720, 772.0, 760.0
    pos = np.array([1.0, -2.0, -15.0])
    view, proj = oracle.view_proj(pos, np.eye(3), W, H, fx, fy, 100.0, 0.01)
    V = view.reshape(4, 4).T          # column-major storage -> conventional matrix
    Pm = proj.reshape(4, 4).T
    assert np.array_equal(V[:3, :3], np.eye(3, dtype=np.float32))
    assert np.array_equal(V[:3, 3], (-pos).astype(np.float32))
    np.testing.assert_allclose(Pm[0, 0], 2 * fx / W, rtol=1e-6)
    np.testing.assert_allclose(Pm[1, 1], 2 * fy / H, rtol=1e-6)
    assert np.array_equal(Pm[3], V[2])                 # p_hom.w is the view-space depth


def test_view_proj_general_rotation(oracle):
    for seed in range(5):
        R = _rot(seed)                                  # camera-to-world, row-major as in cameras.json
        pos = np.random.default_rng(seed).uniform(-10, 10, 3)
        W, H, fx, fy, zf, zn = 1920, 1080, 935.3, 935.3, 100.0, 0.01
        view, proj = oracle.view_proj(pos, R, W, H, fx, fy, zf, zn)
        V = view.reshape(4, 4).T.astype(np.float64)
        Vd = np.eye(4)
        Vd[:3, :3] = R.T
        Vd[:3, 3] = -R.T @ pos
        np.testing.assert_allclose(V, Vd, atol=2e-6)
        Pd = np.array([[2 * fx / W, 0, 0, 0], [0, 2 * fy / H, 0, 0],
                       [0, 0, zf / (zf - zn), -zf * zn / (zf - zn)], [0, 0, 1, 0]])
        np.testing.assert_allclose(proj.reshape(4, 4).T, Pd @ Vd, rtol=2e-5, atol=2e-5)


# ---- 2D covariance -----------------------------------------------------------------------------------------

def _cov2d_f64(p, fx, fy, tfx, tfy, cov3d, R, pos):
    t = R.T @ (p - pos)
    x = min(1.3 * tfx, max(-1.3 * tfx, t[0] / t[2])) * t[2]
    y = min(1.3 * tfy, max(-1.3 * tfy, t[1] / t[2])) * t[2]
    J = np.array([[fx / t[2], 0, -fx * x / t[2] ** 2], [0, fy / t[2], -fy * y / t[2] ** 2]])
    S = np.array([[cov3d[0], cov3d[1], cov3d[2]], [cov3d[1], cov3d[3], cov3d[4]], [cov3d[2], cov3d[4], cov3d[5]]])
    Wm = R.T
    c = J @ Wm @ S @ Wm.T @ J.T
    return np.array([c[0, 0] + 0.3, c[0, 1], c[1, 1] + 0.3])


def test_cov2d_against_float64_ewa(oracle):
    rng = np.random.default_rng(11)
    W, H, f = 1920, 1080, 935.3
    tfx, tfy = W / (2 * f), H / (2 * f)
    worst = 0.0
    for k in range(300):
        R = _rot(100 + k)
        pos = rng.uniform(-5, 5, 3)
        t = np.array([rng.uniform(-1.5, 1.5) * 8, rng.uniform(-1.0, 1.0) * 8, rng.uniform(0.5, 30)])   # some get clamped
        p = (R @ t + pos)
        A = rng.standard_normal((3, 3)) * rng.uniform(0.01, 0.5)
        S = A @ A.T
        c3 = np.array([S[0, 0], S[0, 1], S[0, 2], S[1, 1], S[1, 2], S[2, 2]])
        view, _ = oracle.view_proj(pos, R, W, H, f, f, 100.0, 0.01)
        got = oracle.cov2d(p, f, f, tfx, tfy, c3, view).astype(np.float64)
        want = _cov2d_f64(p, f, f, tfx, tfy, c3, R, pos)
        scale = np.abs(want).max()
        worst = max(worst, np.abs(got - want).max() / scale)
    assert worst < 1e-4


def test_cov2d_isotropic_on_axis_closed_form(oracle):
    f, z, s = 800.0, 10.0, 0.05
    view, _ = oracle.view_proj([0, 0, 0], np.eye(3), 1280, 720, f, f, 100.0, 0.01)
    got = oracle.cov2d([0, 0, z], f, f, 0.8, 0.45, [s * s, 0, 0, s * s, 0, s * s], view)
    want = (s * f / z) ** 2 + 0.3
    np.testing.assert_allclose(got[[0, 2]], [want, want], rtol=1e-6)
    assert abs(got[1]) < 1e-9


# ---- whole preprocess on one crafted Gaussian: power, radius, ndc2pix, conic, key packing ------------------------

def _one(oracle, p, sigma_world, opacity, W=1280, H=720, f=800.0, sh=None, block=(16, 16), campos=(0, 0, 0)):
    cov3d = np.array([[sigma_world ** 2, 0, 0, sigma_world ** 2, 0, sigma_world ** 2]], np.float32)
    shs = np.zeros((1, 48), np.float32) if sh is None else np.asarray(sh, np.float32).reshape(1, 48)
    return oracle.preprocess(np.array([p], np.float32), shs, np.array([opacity], np.float32), cov3d, W, H,
                             block[0], block[1], campos, np.eye(3), f, f, 100.0, 0.01, 4096, threads=1)


def test_single_gaussian_attributes_closed_form(oracle):
    W, H, f = 1280, 720, 800.0
    p, s, op = np.array([0.7, -0.3, 10.0]), 0.08, 0.6
    r = _one(oracle, p, s, op)
    assert r["num_rendered"] >= 1
    # pixel position: x_pix = f x / z + (W - 1) / 2
    np.testing.assert_allclose(r["points_xy"][0], [f * p[0] / p[2] + (W - 1) / 2, f * p[1] / p[2] + (H - 1) / 2], rtol=1e-5)
    # conic of the EWA covariance (J at the point, float64), scaled by -0.5 log2e / -log2e; w = log2(opacity)
    x, y, z = p
    J = np.array([[f / z, 0, -f * x / z ** 2], [0, f / z, -f * y / z ** 2]])
    c = (s * s) * J @ J.T + 0.3 * np.eye(2)
    ci = np.linalg.inv(c)
    want = [-0.5 * LOG2E * ci[0, 0], -LOG2E * ci[0, 1], -0.5 * LOG2E * ci[1, 1], math.log2(op)]
    np.testing.assert_allclose(r["conic_opacity"][0], want, rtol=2e-5, atol=1e-7)
    # depth in the attribute row and in the low key bits
    assert r["rgb_depth"][0, 3] == np.float32(10.0)
    assert np.all((r["keys"][:r["num_rendered"]] & 0xffffffff) == np.float32(10.0).view(np.uint32))
    # SH all zero: colour 0.5
    np.testing.assert_allclose(r["rgb_depth"][0, :3], 0.5, rtol=1e-6)


def test_emitted_tiles_of_a_circle(oracle):
    """Isotropic splat in the image plane: the ellipse q <= 2*power is a circle of radius
    sqrt(2 ln(256 op) c) around the projected centre, c the 2D variance.  The emitted tiles must be
    exactly the tiles whose pixel-centre rectangle [16i, 16i+15]^2 comes within that radius."""
    W, H, f = 1280, 720, 800.0
    rng = np.random.default_rng(12)
    checked = 0
    for _ in range(200):
        z = rng.uniform(2, 30)
        p = np.array([rng.uniform(-0.9, 0.9) * z * W / (2 * f), rng.uniform(-0.9, 0.9) * z * H / (2 * f), z])
        s, op = rng.uniform(0.01, 0.4), rng.uniform(0.02, 0.99)
        # keep the on-axis closed form valid: J's off-diagonal terms vanish only on the axis, so use
        # the float64 EWA covariance and require it to be close to isotropic
        x, y = p[0], p[1]
        J = np.array([[f / z, 0, -f * x / z ** 2], [0, f / z, -f * y / z ** 2]])
        c = (s * s) * J @ J.T + 0.3 * np.eye(2)
        ci = np.linalg.inv(c)
        power = math.log(256 * op)
        cx, cy = f * x / z + (W - 1) / 2, f * y / z + (H - 1) / 2
        r = _one(oracle, p, s, op)
        K = r["num_rendered"]
        got = set(int(k >> 32) for k in r["keys"][:K])
        want, ambiguous = set(), False
        for ty in range(H // 16):
            for tx in range(W // 16):
                qmin = _min_quadratic_over_rect(ci, cx, cy, 16 * tx, 16 * ty, 16 * tx + 15, 16 * ty + 15)
                if abs(qmin - 2 * power) < 1e-3 * max(1.0, 2 * power):
                    ambiguous = True
                if qmin <= 2 * power:
                    want.add(ty * (W // 16) + tx)
        if ambiguous:
            continue
        assert got == want
        # radius closed form: the candidate rectangle must cover the circle's bounding box
        checked += 1
    assert checked > 150


def _min_quadratic_over_rect(Q, cx, cy, x0, y0, x1, y1):
    """min over the closed rectangle of d^T Q d, d = (x - cx, y - cy), Q symmetric positive definite."""
    if x0 <= cx <= x1 and y0 <= cy <= y1:
        return 0.0
    best = math.inf
    a, b, c = Q[0, 0], Q[0, 1], Q[1, 1]
    for xe in (x0, x1):       # vertical edges: minimise over y
        dx = xe - cx
        t = min(max(-b * dx / c, y0 - cy), y1 - cy)
        best = min(best, a * dx * dx + 2 * b * dx * t + c * t * t)
    for ye in (y0, y1):       # horizontal edges: minimise over x
        dy = ye - cy
        t = min(max(-b * dy / a, x0 - cx), x1 - cx)
        best = min(best, a * t * t + 2 * b * t * dy + c * dy * dy)
    return best


def test_tile_test_against_convex_qp(oracle):
    """Random anisotropic conics against the float64 minimum of the quadratic over the rectangle."""
    rng = np.random.default_rng(13)
    n_checked = 0
    for _ in range(20000):
        ang = rng.uniform(0, math.pi)
        s1, s2 = rng.uniform(0.6, 40.0), rng.uniform(0.6, 40.0)
        Rm = np.array([[math.cos(ang), -math.sin(ang)], [math.sin(ang), math.cos(ang)]])
        cov = Rm @ np.diag([s1 * s1, s2 * s2]) @ Rm.T
        Q = np.linalg.inv(cov)
        power = rng.uniform(0.01, 5.5)
        tx, ty = rng.integers(0, 20, 2)
        bx, by = (16, 16) if rng.uniform() < 0.7 else (32, 16)
        x0, y0 = int(tx * bx), int(ty * by)
        x1, y1 = x0 + bx - 1, y0 + by - 1
        cx = np.float32(rng.uniform(x0 - 80, x1 + 80))
        cy = np.float32(rng.uniform(y0 - 80, y1 + 80))
        con = np.float32([Q[0, 0], Q[0, 1], Q[1, 1]])
        Qf = np.array([[con[0], con[1]], [con[1], con[2]]], np.float64)
        qmin = _min_quadratic_over_rect(Qf, float(cx), float(cy), x0, y0, x1, y1)
        w = 2 * float(np.float32(power))
        if abs(qmin - w) < 2e-4 * max(1.0, w, qmin):
            continue
        n_checked += 1
        assert oracle.tile_test((x0, y0), (x1, y1), (cx, cy), con, np.float32(power)) == (qmin <= w)
    assert n_checked > 19000


def test_emission_is_sound_against_pixel_brute_force(oracle):
    """Every pixel centre with alpha >= 1/256 lies in an emitted tile; emitted tiles lie in the
    candidate rectangle implied by the radius."""
    from flashgs_amd import scenes
    sc = scenes.config0(n=300)
    rng = np.random.default_rng(14)
    # make them big enough to span several tiles
    scale = np.exp(rng.normal(-2.0, 0.6, (300, 3))).astype(np.float32)
    cov3d = scenes.cov3d_from_scale_rotation(scale, scenes._unit_quats(rng, 300))
    cam = sc.cameras[0]
    W, H = 320, 240
    f = 200.0
    r = oracle.preprocess(sc.position, sc.shs, sc.opacity, cov3d, W, H, 16, 16, cam.position, cam.rotation, f, f,
                          100.0, 0.01, 1 << 16, threads=2)
    K = r["num_rendered"]
    gx = W // 16
    emitted = {}
    for k, v in zip(r["keys"][:K], r["values"][:K]):
        emitted.setdefault(int(v), set()).add(int(k >> 32))
    ys, xs = np.mgrid[0:H, 0:W]
    n_vis = 0
    for g, tiles in emitted.items():
        co = r["conic_opacity"][g].astype(np.float64)
        px, py = r["points_xy"][g].astype(np.float64)
        dx, dy = px - xs, py - ys
        alpha = np.exp2(co[3] + co[0] * dx * dx + co[2] * dy * dy + co[1] * dx * dy)
        inside = alpha >= (1 / 256) * (1 + 1e-4)
        need = set((ys[inside] // 16 * gx + xs[inside] // 16).tolist())
        assert need <= tiles, "Gaussian %d: a visible pixel lies in a tile without a key" % g
        n_vis += 1
    assert n_vis > 50


def test_rect_integer_model(oracle):
    rng = np.random.default_rng(15)
    gx, gy, bx, by = 80, 45, 16, 16
    for _ in range(5000):
        px = float(np.float32(rng.integers(-2000, 4000) / 8.0))     # exactly representable
        py = float(np.float32(rng.integers(-2000, 3000) / 8.0))
        w, h = int(rng.integers(1, 500)), int(rng.integers(1, 500))
        rmin, rmax = oracle.rect(px, py, w, h, gx, gy, bx, by)
        trunc = lambda v: int(v)                                     # C truncation toward zero
        assert rmin[0] == min(gx, max(0, trunc((px - w) / bx)))
        assert rmin[1] == min(gy, max(0, trunc((py - h) / by)))
        assert rmax[0] == min(gx, max(0, trunc((px + w) / bx) + 1))
        assert rmax[1] == min(gy, max(0, trunc((py + h) / by) + 1))
    # a splat wholly left of the image still probes tile column 0: (int)(-0.5) + 1 == 1
    rmin, rmax = oracle.rect(-10.0, 100.0, 2, 2, gx, gy, bx, by)
    assert (rmin[0], rmax[0]) == (0, 1)


def test_key_list_invariants_and_stale_rows(oracle):
    from flashgs_amd import scenes
    sc = scenes.config0(n=20000)
    cam = sc.cameras[0]
    n = sc.num_vertex
    sentinel = np.float32(-123.25)
    r = oracle.preprocess(sc.position, sc.shs, sc.opacity, sc.cov3d, cam.width, cam.height, 16, 16, cam.position,
                          cam.rotation, cam.focal_x, cam.focal_y, cam.zFar, cam.zNear, 1 << 18,
                          points_xy=np.full((n, 2), sentinel), rgb_depth=np.full((n, 4), sentinel),
                          conic_opacity=np.full((n, 4), sentinel))
    K = r["num_rendered"]
    keys, vals = r["keys"][:K], r["values"][:K]
    tiles = (cam.width // 16) * (cam.height // 16)
    assert K == r["counts"]["keys"] and K > 0
    assert np.all((keys >> 32) < tiles)
    depth = (keys & 0xffffffff).astype(np.uint32).view(np.float32)
    assert np.all(depth > 0.2)
    assert np.all(np.diff(vals.astype(np.int64)) >= 0)                 # ascending Gaussian index
    same = np.diff(vals.astype(np.int64)) == 0
    assert np.all(np.diff((keys >> 32).astype(np.int64))[same] > 0)    # row-major tiles inside one Gaussian
    assert np.array_equal(depth, r["rgb_depth"][vals, 3])
    emitting = np.zeros(n, bool)
    emitting[vals] = True
    # rows are written for the Gaussians that emit, plus the few whose one-tile rectangle failed
    # the test (test_one_tile_rectangle_gets_its_record_without_a_key); every other row is stale
    written = r["rgb_depth"][:, 3] != sentinel
    assert written.sum() == r["counts"]["visible"]
    assert np.all(written[emitting]) and (written & ~emitting).sum() <= 0.01 * emitting.sum()
    for name in ("points_xy", "rgb_depth", "conic_opacity"):
        assert np.all(r[name][~written] == sentinel)
        assert not np.any(r[name][written][:, -1] == sentinel)
    # single-threaded and multi-threaded runs give the same list
    r1 = oracle.preprocess(sc.position, sc.shs, sc.opacity, sc.cov3d, cam.width, cam.height, 16, 16, cam.position,
                           cam.rotation, cam.focal_x, cam.focal_y, cam.zFar, cam.zNear, 1 << 18, threads=1)
    assert np.array_equal(r1["keys"][:K], keys) and np.array_equal(r1["values"][:K], vals)


def test_one_tile_rectangle_gets_its_record_without_a_key(oracle):
    """preprocess.cu:317,411-417: vertex_valid starts as single_tile, so a Gaussian whose candidate
    rectangle is one tile has its attribute rows written even when that tile fails the ellipse
    test.  A small splat 12 pixels left of the image: the rectangle is clamped to tile (0, 6), which
    the ellipse (about 6 pixels at the opacity threshold) does not reach."""
    W, H, f, z = 1280, 720, 800.0, 10.0
    p = np.array([[(-12.0 - (W - 1) / 2) * z / f, (104.0 - (H - 1) / 2) * z / f, z]], np.float32)
    s2 = (math.sqrt(3.4) * z / f) ** 2
    cov3d = np.array([[s2, 0, 0, s2, 0, s2]], np.float32)
    sentinel = np.float32(-7.5)
    r = oracle.preprocess(p, np.zeros((1, 48), np.float32), np.array([0.6], np.float32), cov3d, W, H, 16, 16,
                          (0, 0, 0), np.eye(3), f, f, 100.0, 0.01, 16, threads=1,
                          points_xy=np.full((1, 2), sentinel), rgb_depth=np.full((1, 4), sentinel),
                          conic_opacity=np.full((1, 4), sentinel))
    assert r["counts"]["candidates"] == 1 and r["num_rendered"] == 0
    assert r["counts"]["visible"] == 1
    np.testing.assert_allclose(r["points_xy"][0], [-12.0, 104.0], atol=1e-3)
    assert r["rgb_depth"][0, 3] == np.float32(z) and r["conic_opacity"][0, 3] == np.float32(oracle.log2f(np.float32(0.6)))
    # two tiles high instead (centre on a tile border): no key, and now no record either
    p2 = p.copy()
    p2[0, 1] = (96.0 - (H - 1) / 2) * z / f
    r = oracle.preprocess(p2, np.zeros((1, 48), np.float32), np.array([0.6], np.float32), cov3d, W, H, 16, 16,
                          (0, 0, 0), np.eye(3), f, f, 100.0, 0.01, 16, threads=1,
                          points_xy=np.full((1, 2), sentinel), rgb_depth=np.full((1, 4), sentinel),
                          conic_opacity=np.full((1, 4), sentinel))
    assert r["counts"]["candidates"] == 2 and r["num_rendered"] == 0 and r["counts"]["visible"] == 0
    assert np.all(r["rgb_depth"] == sentinel) and np.all(r["points_xy"] == sentinel)


def test_cull_rules(oracle):
    # behind the near plane (z <= 0.2) and below 1/255 opacity emit nothing
    assert _one(oracle, [0, 0, 0.2], 0.01, 0.9)["num_rendered"] == 0
    assert _one(oracle, [0, 0, 0.21], 0.001, 0.9)["num_rendered"] >= 1
    assert _one(oracle, [0, 0, 5.0], 0.05, 1 / 255 - 1e-5)["num_rendered"] == 0
    assert _one(oracle, [0, 0, 5.0], 0.05, 1 / 255 + 1e-5)["num_rendered"] >= 1
    # far off-screen: nothing
    assert _one(oracle, [500.0, 0, 5.0], 0.05, 0.9)["num_rendered"] == 0


def test_capacity_overflow_is_reported(oracle):
    r = _one(oracle, [0, 0, 1.0], 0.5, 0.9)     # a huge splat: many tiles
    assert r["num_rendered"] > 100
    cov3d = np.array([[0.25, 0, 0, 0.25, 0, 0.25]], np.float32)
    rr = oracle.preprocess(np.array([[0, 0, 1.0]], np.float32), np.zeros((1, 48), np.float32), np.array([0.9], np.float32),
                           cov3d, 1280, 720, 16, 16, [0, 0, 0], np.eye(3), 800.0, 800.0, 100.0, 0.01, 50, threads=1)
    assert rr["rc"] == -1 and rr["num_rendered"] == r["num_rendered"]


# ---- SH colour -----------------------------------------------------------------------------------------------------

def _real_sh_basis(d):
    """Real spherical harmonics of degree <= 3 at unit vector d in the sign convention 3DGS uses:
    sqrt(2) Im / Re of scipy's complex harmonics (Condon-Shortley phase kept), index l*l + l + m."""
    x, y, z = d
    theta = math.acos(max(-1.0, min(1.0, z)))   # polar
    phi = math.atan2(y, x)                      # azimuth
    out = []
    for l in range(4):
        for m in range(-l, l + 1):
            Y = special.sph_harm_y(l, abs(m), theta, phi)
            if m == 0:
                out.append(Y.real)
            elif m > 0:
                out.append(math.sqrt(2) * Y.real)
            else:
                out.append(math.sqrt(2) * Y.imag)
    return np.array(out)


def test_sh_colour_against_scipy(oracle):
    rng = np.random.default_rng(16)
    for _ in range(200):
        p = rng.uniform(-5, 5, 3)
        cam = rng.uniform(-5, 5, 3)
        sh = rng.standard_normal((16, 3)) * 0.4
        got = oracle.sh_color(p, cam, sh.reshape(48)).astype(np.float64)
        d = (p.astype(np.float32) - cam.astype(np.float32)).astype(np.float64)
        d /= np.linalg.norm(d)
        want = np.maximum(0.0, 0.5 + _real_sh_basis(d) @ sh.astype(np.float32).astype(np.float64))
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=2e-6)


def test_sh_degree0_and_clamp(oracle):
    sh = np.zeros((16, 3))
    sh[0] = [1.0, -3.0, 0.25]
    got = oracle.sh_color([1, 2, 3], [0, 0, 0], sh.reshape(48))
    np.testing.assert_allclose(got, [0.5 + 0.28209479177387814, 0.0, 0.5 + 0.25 * 0.28209479177387814], rtol=1e-6)


# ---- cov3d ---------------------------------------------------------------------------------------------------------

def test_cov3d_against_float64(oracle):
    from flashgs_amd import scenes
    rng = np.random.default_rng(17)
    n = 500
    scale = np.exp(rng.normal(-3, 1, (n, 3))).astype(np.float32)
    q = scenes._unit_quats(rng, n)
    got = oracle.cov3d(scale, q).astype(np.float64)
    r, x, y, z = [q[:, i].astype(np.float64) for i in range(4)]
    R = np.stack([np.stack([1 - 2 * (y * y + z * z), 2 * (x * y - r * z), 2 * (x * z + r * y)], 1),
                  np.stack([2 * (x * y + r * z), 1 - 2 * (x * x + z * z), 2 * (y * z - r * x)], 1),
                  np.stack([2 * (x * z - r * y), 2 * (y * z + r * x), 1 - 2 * (x * x + y * y)], 1)], 1)
    S2 = scale.astype(np.float64) ** 2
    Sig = np.einsum("nik,nk,njk->nij", R, S2, R)
    want = np.stack([Sig[:, 0, 0], Sig[:, 0, 1], Sig[:, 0, 2], Sig[:, 1, 1], Sig[:, 1, 2], Sig[:, 2, 2]], 1)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-9)
    # the scene generator's vectorised version agrees
    np.testing.assert_allclose(scenes.cov3d_from_scale_rotation(scale, q), got, rtol=1e-5, atol=1e-9)
    # identity rotation: diag(s^2)
    one = oracle.cov3d(np.float32([[1, 2, 3]]), np.float32([[1, 0, 0, 0]]))
    assert np.array_equal(one[0], np.float32([1, 0, 0, 4, 0, 9]))


# ---- sort and ranges --------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("n", [0, 1, 2, 255, 4097, 200000])
def test_sort_against_numpy_stable(oracle, n):
    rng = np.random.default_rng(18 + n)
    W, H = 1920, 1080
    tiles = 120 * 68
    tile = rng.integers(0, tiles, n).astype(np.uint64)
    depth = rng.uniform(0.2, 50, n).astype(np.float32)
    if n > 10:
        depth[: n // 3] = depth[0]               # many ties
        tile[: n // 4] = tile[0]
    keys = (tile << np.uint64(32)) | depth.view(np.uint32).astype(np.uint64)
    vals = rng.permutation(n).astype(np.uint32)
    ks, vs = oracle.sort(n, W, H, 16, 16, keys, vals, threads=3)
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(ks, keys[order]) and np.array_equal(vs, vals[order])


def test_sort_ignores_bits_above_the_range(oracle):
    # bits above 32 + bit_length(tiles) are outside the sorted range (sort.cu:34-39)
    n = 1000
    rng = np.random.default_rng(19)
    W, H = 64, 64                                 # 16 tiles -> bit_length 5 -> end bit 37
    low = rng.integers(0, 1 << 37, n).astype(np.uint64)
    junk = rng.integers(0, 1 << 20, n).astype(np.uint64) << np.uint64(37)
    ks, vs = oracle.sort(n, W, H, 16, 16, low | junk, np.arange(n, dtype=np.uint32), threads=2)
    order = np.argsort(low, kind="stable")
    assert np.array_equal(vs, order.astype(np.uint32))


def test_ranges_against_searchsorted(oracle):
    rng = np.random.default_rng(20)
    tiles = 500
    for n in (0, 1, 7, 5000):
        tile = np.sort(rng.integers(0, tiles, n)).astype(np.uint64)
        if n > 100:
            tile = tile[(tile < 100) | (tile > 130)]          # a run of empty tiles
        n = tile.size
        keys = (tile << np.uint64(32)) | rng.integers(0, 1 << 32, n).astype(np.uint64)
        rg = oracle.ranges(n, keys, tiles)
        lo = np.searchsorted(tile, np.arange(tiles), side="left")
        hi = np.searchsorted(tile, np.arange(tiles), side="right")
        empty = lo == hi
        assert np.array_equal(rg[~empty, 0], lo[~empty]) and np.array_equal(rg[~empty, 1], hi[~empty])
        assert np.all(rg[empty] == 0)


# ---- blend ------------------------------------------------------------------------------------------------------------

def _blend_setup(gaussians, W=64, H=48, block=(16, 16)):
    """gaussians: list of (cx, cy, sigma, opacity, rgb); every Gaussian is put in every tile, in list order."""
    n = len(gaussians)
    xy = np.array([[g[0], g[1]] for g in gaussians], np.float32)
    co = np.array([[-0.5 * LOG2E / g[2] ** 2, 0.0, -0.5 * LOG2E / g[2] ** 2, math.log2(g[3])] for g in gaussians], np.float32)
    rgbd = np.array([list(g[4]) + [1.0] for g in gaussians], np.float32)
    gx, gy = (W + block[0] - 1) // block[0], (H + block[1] - 1) // block[1]
    vals = np.tile(np.arange(n, dtype=np.uint32), gx * gy)
    rng_ = np.stack([np.arange(gx * gy) * n, (np.arange(gx * gy) + 1) * n], 1).astype(np.int32)
    return xy, rgbd, co, vals, rng_


def test_blend_one_gaussian_closed_form(oracle):
    W, H = 64, 48
    g = (30.5, 20.25, 6.0, 0.8, (0.9, 0.4, 0.1))
    bg = np.array([0.2, 0.3, 0.6])
    xy, rgbd, co, vals, rg = _blend_setup([g], W, H)
    u8, f32, walked = oracle.render(W, H, 16, 16, xy, rgbd, co, vals, rg, bg)
    ys, xs = np.mgrid[0:H, 0:W]
    a = g[3] * np.exp(-0.5 * ((xs - g[0]) ** 2 + (ys - g[1]) ** 2) / g[2] ** 2)
    want = a[..., None] * np.array(g[4]) + (1 - a)[..., None] * bg
    np.testing.assert_allclose(f32, want, atol=2e-6)
    assert np.array_equal(u8, np.minimum(np.maximum(f32 * np.float32(255.0), 0), 255).astype(np.uint8))
    assert walked == 12


def test_rotated_gaussian_image_closed_form(oracle):
    """One anisotropic, rotated Gaussian through preprocess -> sort -> ranges -> render: inside the
    emitted tiles the image is op * exp(-1/2 d^T S^-1 d) * rgb + (1 - alpha) * bg with S the EWA
    covariance J W Sigma W^T J^T + 0.3 I inverted in float64.  The off-diagonal term of S^-1 enters
    the blend as conic.y * dx * dy: a wrong sign or a swapped axis there mirrors the ellipse."""
    W, H, f = 256, 192, 400.0
    rng = np.random.default_rng(5)
    bg = np.array([0.1, 0.2, 0.7])
    for trial in range(4):
        p = np.array([rng.uniform(-1, 1), rng.uniform(-0.6, 0.6), rng.uniform(6, 9)])
        th = rng.uniform(0.3, 1.2) * (1 if trial % 2 else -1)              # rotation about the view axis: both signs
        tilt = rng.uniform(-0.4, 0.4)                                       # and a little out of the image plane
        Rz = np.array([[math.cos(th), -math.sin(th), 0], [math.sin(th), math.cos(th), 0], [0, 0, 1]])
        Rx = np.array([[1, 0, 0], [0, math.cos(tilt), -math.sin(tilt)], [0, math.sin(tilt), math.cos(tilt)]])
        R = Rz @ Rx
        S3 = R @ np.diag([0.35, 0.06, 0.12]) ** 2 @ R.T
        cov3d = np.array([[S3[0, 0], S3[0, 1], S3[0, 2], S3[1, 1], S3[1, 2], S3[2, 2]]], np.float32)
        op = 0.85
        sh = np.zeros((1, 48), np.float32)
        sh[0, :3] = (np.array([0.9, 0.5, 0.2]) - 0.5) / 0.28209479177387814      # degree 0 only: colour = 0.5 + C0 * dc
        pre = oracle.preprocess(p[None].astype(np.float32), sh, np.array([op], np.float32), cov3d, W, H, 16, 16,
                                (0, 0, 0), np.eye(3), f, f, 100.0, 0.01, 4096, threads=1)
        K = pre["num_rendered"]
        assert K >= 4
        ks, vs = oracle.sort(K, W, H, 16, 16, pre["keys"], pre["values"])
        gx, gy = W // 16, H // 16
        rg = oracle.ranges(K, ks, gx * gy)
        _, img, _ = oracle.render(W, H, 16, 16, pre["points_xy"], pre["rgb_depth"], pre["conic_opacity"], vs, rg, bg)
        x, y, z = p
        J = np.array([[f / z, 0, -f * x / z ** 2], [0, f / z, -f * y / z ** 2]])
        S2 = J @ S3 @ J.T + 0.3 * np.eye(2)
        assert abs(S2[0, 1]) > 0.2 * math.sqrt(S2[0, 0] * S2[1, 1])            # really tilted on the screen
        Si = np.linalg.inv(S2)
        cx, cy = f * x / z + (W - 1) / 2, f * y / z + (H - 1) / 2
        ys, xs = np.mgrid[0:H, 0:W]
        dx, dy = xs - cx, ys - cy
        alpha = op * np.exp(-0.5 * (Si[0, 0] * dx * dx + 2 * Si[0, 1] * dx * dy + Si[1, 1] * dy * dy))
        want = alpha[..., None] * np.array([0.9, 0.5, 0.2]) + (1 - alpha)[..., None] * bg
        emitted = np.zeros((gy, gx), bool)
        emitted.reshape(-1)[(ks >> 32).astype(np.int64)] = True
        mask = np.kron(emitted, np.ones((16, 16), bool))
        assert alpha[mask].max() > 0.5
        np.testing.assert_allclose(img[mask], want[mask], atol=3e-4)
        # outside the emitted tiles the splat is below the 1/255 threshold and the image is the background
        assert alpha[~mask].max() < 1 / 255 + 1e-4
        np.testing.assert_allclose(img[~mask], np.broadcast_to(bg, img.shape)[~mask], atol=1e-6)


def test_blend_two_gaussians_order_matters(oracle):
    W, H = 32, 32
    a = (12.0, 15.0, 5.0, 0.7, (1.0, 0.0, 0.0))
    b = (18.0, 17.0, 7.0, 0.9, (0.0, 0.0, 1.0))
    ys, xs = np.mgrid[0:H, 0:W]

    def alpha(g):
        return g[3] * np.exp(-0.5 * ((xs - g[0]) ** 2 + (ys - g[1]) ** 2) / g[2] ** 2)

    for first, second in ((a, b), (b, a)):
        xy, rgbd, co, vals, rg = _blend_setup([first, second], W, H)
        _, f32, _ = oracle.render(W, H, 16, 16, xy, rgbd, co, vals, rg, [0, 0, 0])
        a1, a2 = alpha(first), alpha(second)
        want = a1[..., None] * np.array(first[4]) + ((1 - a1) * a2)[..., None] * np.array(second[4])
        np.testing.assert_allclose(f32, want, atol=2e-6)


def _blend_f64(W, H, block, xy, rgbd, co, vals, rg, bg, early_out=True):
    """Per-pixel float64 restatement of the rule: pairs, tile-wide stop when every pixel has T < 1e-4."""
    out = np.zeros((H, W, 3))
    gx = (W + block[0] - 1) // block[0]
    gy = (H + block[1] - 1) // block[1]
    for t in range(gx * gy):
        tx, ty = t % gx, t // gx
        ys, xs = np.mgrid[ty * block[1]:(ty + 1) * block[1], tx * block[0]:(tx + 1) * block[0]]
        T = np.ones(xs.shape)
        C = np.zeros(xs.shape + (3,))
        k = rg[t, 0]
        while k < rg[t, 1]:
            for g in vals[k:min(k + 2, rg[t, 1])]:
                dx, dy = xy[g, 0] - xs, xy[g, 1] - ys
                al = np.exp2(co[g, 3] + co[g, 0] * dx * dx + co[g, 2] * dy * dy + co[g, 1] * dx * dy)
                C += (al * T)[..., None] * rgbd[g, :3]
                T = T - al * T
            k += 2
            if early_out and np.all(T < 1e-4):
                break
        T = np.where(T < 1e-4, 0.0, T)
        res = C + T[..., None] * np.asarray(bg)
        yy, xx = ys < H, xs < W
        m = yy & xx
        out[ys[m], xs[m]] = res[m]
    return out


@pytest.mark.parametrize("block", [(16, 16), (32, 16), (32, 32)])
def test_blend_against_float64_brute_force(oracle, block):
    from flashgs_amd import scenes
    sc = scenes.config0(n=3000)
    rng = np.random.default_rng(21)
    scale = np.exp(rng.normal(-1.8, 0.5, (3000, 3))).astype(np.float32)
    cov3d = scenes.cov3d_from_scale_rotation(scale, scenes._unit_quats(rng, 3000))
    cam = sc.cameras[0]
    W, H, f = 200, 120, 120.0          # not multiples of the tile: partial tiles on both edges
    pre = oracle.preprocess(sc.position, sc.shs, sc.opacity, cov3d, W, H, block[0], block[1], cam.position,
                            cam.rotation, f, f, 100.0, 0.01, 1 << 18)
    K = pre["num_rendered"]
    ks, vs = oracle.sort(K, W, H, block[0], block[1], pre["keys"], pre["values"])
    gx, gy = (W + block[0] - 1) // block[0], (H + block[1] - 1) // block[1]
    rg = oracle.ranges(K, ks, gx * gy)
    bg = [0.1, 0.0, 0.3]
    u8, f32, walked = oracle.render(W, H, block[0], block[1], pre["points_xy"], pre["rgb_depth"], pre["conic_opacity"],
                                    vs, rg, bg)
    want = _blend_f64(W, H, block, pre["points_xy"].astype(np.float64), pre["rgb_depth"].astype(np.float64),
                      pre["conic_opacity"].astype(np.float64), vs, rg, bg)
    assert np.abs(f32 - want).max() < 2e-5
    assert 0 < walked <= K


def test_blend_early_out_rule(oracle):
    """A tile of opaque splats: the walk stops after the pair that drives every T below 1e-4, the
    result differs from the full walk by less than 1e-4 * sum(rgb), and T is snapped to zero."""
    W, H = 16, 16
    gs = [(8.0, 8.0, 400.0, 0.995, (0.3, 0.6, 0.9))] * 2 + [(8.0, 8.0, 400.0, 0.995, (1.0, 1.0, 1.0))] * 9
    xy, rgbd, co, vals, rg = _blend_setup(gs, W, H)
    bg = [1.0, 1.0, 1.0]
    _, f32, walked = oracle.render(W, H, 16, 16, xy, rgbd, co, vals, rg, bg)
    assert walked == 2          # T = 0.005^2 = 2.5e-5 < 1e-4 after the first pair
    full = _blend_f64(W, H, (16, 16), xy.astype(np.float64), rgbd.astype(np.float64), co.astype(np.float64), vals, rg,
                      bg, early_out=False)
    assert np.abs(f32 - full).max() < 1e-4 * 3
    # background is not added once T < 1e-4
    np.testing.assert_allclose(f32[8, 8], (1 - 2.5e-5) * np.array([0.3, 0.6, 0.9]), rtol=1e-4)
    # odd tail: 3 Gaussians, no stop possible before the single one
    xy, rgbd, co, vals, rg = _blend_setup(gs[:3], W, H)
    assert oracle.render(W, H, 16, 16, xy, rgbd, co, vals, rg, bg)[2] == 2
    gs2 = [(8.0, 8.0, 400.0, 0.5, (0.3, 0.6, 0.9))] * 3
    xy, rgbd, co, vals, rg = _blend_setup(gs2, W, H)
    assert oracle.render(W, H, 16, 16, xy, rgbd, co, vals, rg, bg)[2] == 3


def test_blend_empty_and_partial_tiles(oracle):
    W, H = 40, 24
    xy, rgbd, co, vals, rg = _blend_setup([], W, H)
    u8, f32, walked = oracle.render(W, H, 16, 16, np.zeros((1, 2), np.float32), np.zeros((1, 4), np.float32),
                                    np.zeros((1, 4), np.float32), np.zeros(1, np.uint32), rg, [0.5, 1.0, 2.0])
    assert walked == 0
    assert np.all(u8 == np.array([127, 255, 255], np.uint8))
    np.testing.assert_allclose(f32, np.broadcast_to(np.float32([0.5, 1.0, 2.0]), f32.shape))
