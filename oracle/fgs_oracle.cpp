/*
 * CPU oracle for the FlashGS forward rasterizer path.  TEST INFRASTRUCTURE ONLY:
 * see fgs_oracle.h.  Build with -ffp-contract=off (the Makefile does): every
 * fp32 expression below is written in the operand order of the reference and
 * must be evaluated as written, one IEEE operation at a time.
 *
 * Citations "file:line" are relative to the FlashGS source tree.
 *
 * Pin status (what checks each function independently of this file; the tests
 * named live in tests/test_oracle_*.py):
 *   log2f                 float64 numpy log2, <= 4 ulp over 25k samples         pinned
 *   view_proj             closed forms (identity rotation, fx/W), float64      pinned
 *   cov2d                 float64 EWA model J W S W^T J^T + 0.3 I, closed form pinned
 *   conic/power/radius    closed forms ln(256 op), floor(sqrt(2 p c)+1)        pinned
 *   ndc2pix               closed form fx x/z + (W-1)/2                         pinned
 *   rect                  integer model on exactly representable inputs        pinned
 *   tile_test             float64 convex-QP minimum over the rectangle, and
 *                         brute-force soundness over pixel centres             pinned
 *   key packing           integer identities, multiset invariants              pinned
 *   sh_color              scipy real spherical harmonics + 3DGS sign table     pinned
 *   stale rows            sentinel test; one-tile rectangle without a key      pinned
 *   sort                  numpy stable argsort                                 pinned
 *   ranges                numpy searchsorted                                   pinned
 *   render                closed form 1 and 2 Gaussians, float64 per-pixel
 *                         brute force on small scenes, early-out bound         pinned
 *   preprocess -> render  rotated anisotropic Gaussian: op exp(-d^T S^-1 d/2)
 *                         with S inverted in float64 (the conic's cross term)  pinned
 *   cov3d                 float64 R S S R^T                                    pinned
 * Not pinnable by anything available offline: the bit patterns of the PTX
 * .approx instructions the reference executes, nvcc's FMA contraction choices
 * and the atomics-dependent emission order; the deterministic replacements in
 * this file are the contract for those.
 */
#include "fgs_oracle.h"

#include <math.h>
#include <limits.h>
#include <string.h>
#include <stdlib.h>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

/* ---- bit casts, saturating conversion ---------------------------------- */

inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* (int)f with the saturating behaviour of the device conversion
 * (preprocess.cu:93-98, :309-310 rely on it): NaN -> 0, clamp to int range. */
inline int f2i_sat(float f)
{
    if (!(f == f)) return 0;
    if (f >= 2147483648.0f) return INT_MAX;
    if (f <= -2147483648.0f) return INT_MIN;
    return (int)f;
}

/* min / max of preprocess.cu:116-117 and max.f32 of :36-41: a NaN operand yields the other one. */
inline float fminf_(float a, float b)
{
    if (!(a == a)) return b;
    if (!(b == b)) return a;
    return a < b ? a : b;
}
inline float fmaxf_(float a, float b)
{
    if (!(a == a)) return b;
    if (!(b == b)) return a;
    return a > b ? a : b;
}
inline int imin(int a, int b) { return a < b ? a : b; }
inline int imax(int a, int b) { return a > b ? a : b; }

/* ---- GLM restatements: mat3 stored [col][row] --------------------------- */

struct M3 { float c[3][3]; };

/* glm/detail/type_mat3x3.inl:486-519 */
inline M3 m3_mul(const M3& a, const M3& b)
{
    M3 r;
    for (int col = 0; col < 3; col++)
        for (int row = 0; row < 3; row++)
            r.c[col][row] = a.c[0][row] * b.c[col][0] + a.c[1][row] * b.c[col][1] + a.c[2][row] * b.c[col][2];
    return r;
}

/* glm/detail/func_matrix.inl:86-105 */
inline M3 m3_transpose(const M3& m)
{
    M3 r;
    for (int col = 0; col < 3; col++)
        for (int row = 0; row < 3; row++)
            r.c[col][row] = m.c[row][col];
    return r;
}

/* glm/detail/type_mat3x3.inl:50-66: nine scalars fill columns */
inline M3 m3_from9(float x0, float y0, float z0, float x1, float y1, float z1, float x2, float y2, float z2)
{
    M3 r;
    r.c[0][0] = x0; r.c[0][1] = y0; r.c[0][2] = z0;
    r.c[1][0] = x1; r.c[1][1] = y1; r.c[1][2] = z1;
    r.c[2][0] = x2; r.c[2][1] = y2; r.c[2][2] = z2;
    return r;
}

/* ---- constants (preprocess.cu:13-34) ------------------------------------ */

const float kLog2e = 1.4426950216293334961f;
const float kLn2 = 0.69314718055f;
const float SH_C0 = 0.28209479177387814f;
const float SH_C1 = 0.4886025119029199f;
const float SH_C2[5] = { 1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                         -1.0925484305920792f, 0.5462742152960396f };
const float SH_C3[7] = { -0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
                         0.3731763325901154f, -0.4570457994644658f, 1.445305721320277f,
                         -0.5900435899266435f };

/* ---- deterministic replacement for lg2.approx.f32 (preprocess.cu:57-62) -- */

inline float sw_log2f(float x)
{
    uint32_t b = f2u(x);
    int e = (int)(b >> 23) - 127;
    float m = u2f((b & 0x007fffffu) | 0x3f800000u);   /* [1,2) */
    if (m > 1.41421354f) { m = m * 0.5f; e += 1; }     /* (0.7071, 1.4142] */
    float s = (m - 1.0f) / (m + 1.0f);
    float s2 = s * s;
    float p = 0.111111111f;
    p = p * s2 + 0.142857143f;
    p = p * s2 + 0.2f;
    p = p * s2 + 0.333333333f;
    p = p * s2 + 1.0f;
    float r = (s * 2.88539008f) * p;                    /* 2/ln 2 */
    return (float)e + r;
}

/* ---- preprocess.cu:64-67: the literals 1.0 and 0.5 make this fp64 -------- */

inline float ndc2pix(float v, int S)
{
    return (float)((((double)v + 1.0) * (double)S - 1.0) * 0.5);
}

/* ---- preprocess.cu:69-88 ------------------------------------------------- */

inline void xform4x3(const float p[3], const float* m, float out[3])
{
    out[0] = m[0] * p[0] + m[4] * p[1] + m[8] * p[2] + m[12];
    out[1] = m[1] * p[0] + m[5] * p[1] + m[9] * p[2] + m[13];
    out[2] = m[2] * p[0] + m[6] * p[1] + m[10] * p[2] + m[14];
}

inline void xform4x4(const float p[3], const float* m, float out[4])
{
    out[0] = m[0] * p[0] + m[4] * p[1] + m[8] * p[2] + m[12];
    out[1] = m[1] * p[0] + m[5] * p[1] + m[9] * p[2] + m[13];
    out[2] = m[2] * p[0] + m[6] * p[1] + m[10] * p[2] + m[14];
    out[3] = m[3] * p[0] + m[7] * p[1] + m[11] * p[2] + m[15];
}

/* ---- preprocess.cu:90-100 ------------------------------------------------ */

inline void get_rect(float px, float py, int width, int height, int gx, int gy, int bx, int by,
                     int rmin[2], int rmax[2])
{
    rmin[0] = imin(gx, imax(0, f2i_sat((px - (float)width) / (float)bx)));
    rmin[1] = imin(gy, imax(0, f2i_sat((py - (float)height) / (float)by)));
    /* the "+ 1" wraps at INT_MAX as the device's integer add does (the rectangle is then empty) */
    rmax[0] = imin(gx, imax(0, (int)((uint32_t)f2i_sat((px + (float)width) / (float)bx) + 1u)));
    rmax[1] = imin(gy, imax(0, (int)((uint32_t)f2i_sat((py + (float)height) / (float)by) + 1u)));
}

/* ---- preprocess.cu:103-143 ----------------------------------------------- */

inline void cov2d(const float p[3], float fx, float fy, float tan_fovx, float tan_fovy,
                  const float s[6], const float* vm, float out[3])
{
    float t[3];
    xform4x3(p, vm, t);
    const float limx = 1.3f * tan_fovx;
    const float limy = 1.3f * tan_fovy;
    const float txtz = t[0] / t[2];
    const float tytz = t[1] / t[2];
    t[0] = fminf_(limx, fmaxf_(-limx, txtz)) * t[2];
    t[1] = fminf_(limy, fmaxf_(-limy, tytz)) * t[2];

    M3 J = m3_from9(fx / t[2], 0.0f, -(fx * t[0]) / (t[2] * t[2]),
                    0.0f, fy / t[2], -(fy * t[1]) / (t[2] * t[2]),
                    0.0f, 0.0f, 0.0f);
    M3 W = m3_from9(vm[0], vm[4], vm[8], vm[1], vm[5], vm[9], vm[2], vm[6], vm[10]);
    M3 T = m3_mul(W, J);
    M3 Vrk = m3_from9(s[0], s[1], s[2], s[1], s[3], s[4], s[2], s[4], s[5]);
    M3 cov = m3_mul(m3_mul(m3_transpose(T), m3_transpose(Vrk)), T);
    cov.c[0][0] += 0.3f;
    cov.c[1][1] += 0.3f;
    out[0] = cov.c[0][0];
    out[1] = cov.c[0][1];
    out[2] = cov.c[1][1];
}

/* ---- preprocess.cu:145-185 ----------------------------------------------- */

inline void sh_color(const float p[3], const float cam[3], const float* sh, float rgb[3])
{
    float dx = p[0] - cam[0], dy = p[1] - cam[1], dz = p[2] - cam[2];
    float l2 = dx * dx + dy * dy + dz * dz;
    float r = 1.0f / sqrtf(l2);   /* replaces rsqrt.approx.f32 */
    float x = dx * r, y = dy * r, z = dz * r;
    float xx = x * x, yy = y * y, zz = z * z;
    float xy = x * y, yz = y * z, xz = x * z;
    for (int c = 0; c < 3; c++) {
        const float* v = sh + c;  /* v[3*j] = coefficient j of channel c (ops.h:26-30) */
        float res = SH_C0 * v[0] + 0.5f;
        res = res - SH_C1 * y * v[3 * 1] + SH_C1 * z * v[3 * 2] - SH_C1 * x * v[3 * 3];
        res = res +
              SH_C2[0] * xy * v[3 * 4] +
              SH_C2[1] * yz * v[3 * 5] +
              SH_C2[2] * (2.0f * zz - xx - yy) * v[3 * 6] +
              SH_C2[3] * xz * v[3 * 7] +
              SH_C2[4] * (xx - yy) * v[3 * 8];
        res = res +
              SH_C3[0] * y * (3.0f * xx - yy) * v[3 * 9] +
              SH_C3[1] * xy * z * v[3 * 10] +
              SH_C3[2] * y * (4.0f * zz - xx - yy) * v[3 * 11] +
              SH_C3[3] * z * (2.0f * zz - 3.0f * xx - 3.0f * yy) * v[3 * 12] +
              SH_C3[4] * x * (4.0f * zz - xx - yy) * v[3 * 13] +
              SH_C3[5] * z * (xx - yy) * v[3 * 14] +
              SH_C3[6] * x * (xx - 3.0f * yy) * v[3 * 15];
        rgb[c] = fmaxf_(res, 0.0f);
    }
}

/* ---- preprocess.cu:187-194 ----------------------------------------------- */

inline bool segment_hits(float a, float b, float c, float d, float l, float r)
{
    float delta = b * b - 4.0f * a * c;
    float t1 = (l - d) * (2.0f * a) + b;
    float t2 = (r - d) * (2.0f * a) + b;
    return delta >= 0.0f && (t1 <= 0.0f || t1 * t1 <= delta) && (t2 >= 0.0f || t2 * t2 <= delta);
}

/* ---- preprocess.cu:196-236 ----------------------------------------------- */

inline bool block_hits_ellipse(int minx, int miny, int maxx, int maxy, float cx, float cy,
                               float conx, float cony, float conz, float power)
{
    float a, b, c, dx, dy;
    float w = 2.0f * power;
    /* int + int, then int -> float for the comparison, as in the reference */
    if (cx * 2.0f < (float)(minx + maxx)) dx = cx - (float)minx; else dx = cx - (float)maxx;
    a = conz;
    b = -2.0f * cony * dx;
    c = conx * dx * dx - w;
    if (segment_hits(a, b, c, cy, (float)miny, (float)maxy)) return true;
    if (cy * 2.0f < (float)(miny + maxy)) dy = cy - (float)miny; else dy = cy - (float)maxy;
    a = conx;
    b = -2.0f * cony * dy;
    c = conz * dy * dy - w;
    if (segment_hits(a, b, c, cx, (float)minx, (float)maxx)) return true;
    return false;
}

/* ---- preprocess.cu:238-241 ----------------------------------------------- */

inline bool block_has_center(int minx, int miny, int maxx, int maxy, float cx, float cy)
{
    return cx >= (float)minx && cx <= (float)maxx && cy >= (float)miny && cy <= (float)maxy;
}

inline bool tile_test(int minx, int miny, int maxx, int maxy, float cx, float cy,
                      float conx, float cony, float conz, float power)
{
    return block_has_center(minx, miny, maxx, maxy, cx, cy) ||
           block_hits_ellipse(minx, miny, maxx, maxy, cx, cy, conx, cony, conz, power);
}

/* ---- sort.cu:9-24 -------------------------------------------------------- */

inline uint32_t higher_msb(uint32_t n)
{
    uint32_t msb = sizeof(n) * 4;
    uint32_t step = msb;
    while (step > 1) {
        step /= 2;
        if (n >> msb) msb += step; else msb -= step;
    }
    if (n >> msb) msb++;
    return msb;
}

/* ---- host camera set-up: preprocess.cu:420-448, pybind.cpp:140-143 -------- */

void view_proj(const float pos[3], const float rot[9], int width, int height,
               float fx, float fy, float zFar, float zNear, float view[16], float proj[16])
{
    /* GLM mat3 column c = rot[3c .. 3c+2]; getViewMatrix (preprocess.cu:420-427) */
    float np[3] = { -pos[0], -pos[1], -pos[2] };
    for (int c = 0; c < 3; c++) {
        for (int r = 0; r < 3; r++) view[4 * c + r] = rot[3 * c + r];
        view[4 * c + 3] = 0.0f;
    }
    /* mat3 * vec3: glm/detail/type_mat3x3.inl:468-474 */
    for (int r = 0; r < 3; r++)
        view[12 + r] = rot[0 + r] * np[0] + rot[3 + r] * np[1] + rot[6 + r] * np[2];
    view[15] = 1.0f;

    /* getProjectionMatrix (preprocess.cu:429-448); P indexed [col][row] */
    float top = (float)height / (2.0f * fy) * zNear;
    float bottom = -top;
    float right = (float)width / (2.0f * fx) * zNear;
    float left = -right;
    float P[4][4];
    memset(P, 0, sizeof P);
    float z_sign = 1.0f;
    P[0][0] = 2.0f * zNear / (right - left);
    P[1][1] = 2.0f * zNear / (top - bottom);
    P[0][2] = (right + left) / (right - left);
    P[1][2] = (top + bottom) / (top - bottom);
    P[3][2] = z_sign;
    P[2][2] = z_sign * zFar / (zFar - zNear);
    P[2][3] = -(zFar * zNear) / (zFar - zNear);
    float Pt[4][4];
    for (int c = 0; c < 4; c++)
        for (int r = 0; r < 4; r++) Pt[c][r] = P[r][c];
    /* mat4 * mat4: glm/detail/type_mat4x4.inl:630-648 */
    for (int c = 0; c < 4; c++)
        for (int r = 0; r < 4; r++)
            proj[4 * c + r] = Pt[0][r] * view[4 * c + 0] + Pt[1][r] * view[4 * c + 1] +
                              Pt[2][r] * view[4 * c + 2] + Pt[3][r] * view[4 * c + 3];
}

/* per-Gaussian state after preprocess.cu:282-316 */
struct GState {
    bool valid;
    float p_view[3];
    float point_xy[2];
    float conic[3];
    float power;
    float log2_opacity;
    int rmin[2], rmax[2];
};

struct Cam {
    float view[16], proj[16], campos[3];
    int W, H, bx, by, gx, gy;
    float tan_fovx, tan_fovy, fx, fy;
};

/* returns: 0 culled by near plane or opacity, 1 passed both culls */
inline int gaussian_state(int i, const float* positions, const float* opacities,
                          const float* cov3ds, const Cam& cam, GState& g)
{
    g.valid = false;
    const float* p = positions + 3 * (size_t)i;
    xform4x3(p, cam.view, g.p_view);
    if (g.p_view[2] <= 0.2f) return 0;
    float opacity = opacities[i];
    if (255.0f * opacity < 1.0f) return 0;

    float hom[4];
    xform4x4(p, cam.proj, hom);
    float p_w = 1.0f / (hom[3] + 0.0000001f);
    float proj_x = hom[0] * p_w, proj_y = hom[1] * p_w;

    float cov[3];
    cov2d(p, cam.fx, cam.fy, cam.tan_fovx, cam.tan_fovy, cov3ds + 6 * (size_t)i, cam.view, cov);
    float det = cov[0] * cov[2] - cov[1] * cov[1];
    float det_inv = 1.0f / det;
    g.conic[0] = cov[2] * det_inv;
    g.conic[1] = -cov[1] * det_inv;
    g.conic[2] = cov[0] * det_inv;

    g.log2_opacity = sw_log2f(opacity);
    g.power = kLn2 * 8.0f + kLn2 * g.log2_opacity;
    int width = f2i_sat(1.414214f * sqrtf(cov[0] * g.power) + 1.0f);
    int height = f2i_sat(1.414214f * sqrtf(cov[2] * g.power) + 1.0f);

    g.point_xy[0] = ndc2pix(proj_x, cam.W);
    g.point_xy[1] = ndc2pix(proj_y, cam.H);
    get_rect(g.point_xy[0], g.point_xy[1], width, height, cam.gx, cam.gy, cam.bx, cam.by, g.rmin, g.rmax);
    g.valid = (g.rmax[0] - g.rmin[0]) * (g.rmax[1] - g.rmin[1]) > 0;
    return 1;
}

} // namespace

extern "C" {

float fgs_oracle_log2f(float x) { return sw_log2f(x); }

void fgs_oracle_view_proj(const float pos[3], const float rot[9], int width, int height,
                          float focal_x, float focal_y, float zFar, float zNear,
                          float view[16], float proj[16])
{
    view_proj(pos, rot, width, height, focal_x, focal_y, zFar, zNear, view, proj);
}

void fgs_oracle_cov2d(const float p[3], float focal_x, float focal_y, float tan_fovx,
                      float tan_fovy, const float cov3d[6], const float view[16], float cov[3])
{
    cov2d(p, focal_x, focal_y, tan_fovx, tan_fovy, cov3d, view, cov);
}

int fgs_oracle_tile_test(int pix_min_x, int pix_min_y, int pix_max_x, int pix_max_y,
                         float cx, float cy, float conic_x, float conic_y, float conic_z, float power)
{
    return tile_test(pix_min_x, pix_min_y, pix_max_x, pix_max_y, cx, cy, conic_x, conic_y, conic_z, power) ? 1 : 0;
}

void fgs_oracle_sh_color(const float p[3], const float campos[3], const float sh[48], float rgb[3])
{
    sh_color(p, campos, sh, rgb);
}

void fgs_oracle_rect(float px, float py, int width, int height, int grid_x, int grid_y,
                     int block_x, int block_y, int rect_min[2], int rect_max[2])
{
    get_rect(px, py, width, height, grid_x, grid_y, block_x, block_y, rect_min, rect_max);
}

uint32_t fgs_oracle_higher_msb(uint32_t n) { return higher_msb(n); }

/* pybind.cpp:22-56 */
void fgs_oracle_cov3d(int n, const float* scale, const float* rot, float* cov3d)
{
    for (int i = 0; i < n; i++) {
        const float* sc = scale + 3 * (size_t)i;
        const float* q = rot + 4 * (size_t)i;
        M3 S = m3_from9(1.0f, 0, 0, 0, 1.0f, 0, 0, 0, 1.0f);
        S.c[0][0] = 1.0f * sc[0];
        S.c[1][1] = 1.0f * sc[1];
        S.c[2][2] = 1.0f * sc[2];
        float r = q[0], x = q[1], y = q[2], z = q[3];
        M3 R = m3_from9(
            1.f - 2.f * (y * y + z * z), 2.f * (x * y - r * z), 2.f * (x * z + r * y),
            2.f * (x * y + r * z), 1.f - 2.f * (x * x + z * z), 2.f * (y * z - r * x),
            2.f * (x * z - r * y), 2.f * (y * z + r * x), 1.f - 2.f * (x * x + y * y));
        M3 M = m3_mul(S, R);
        M3 Sigma = m3_mul(m3_transpose(M), M);
        float* o = cov3d + 6 * (size_t)i;
        o[0] = Sigma.c[0][0]; o[1] = Sigma.c[0][1]; o[2] = Sigma.c[0][2];
        o[3] = Sigma.c[1][1]; o[4] = Sigma.c[1][2]; o[5] = Sigma.c[2][2];
    }
}

int fgs_oracle_preprocess(int P, const float* positions, const float* shs,
                          const float* opacities, const float* cov3ds,
                          int width, int height, int block_x, int block_y,
                          const float cam_pos[3], const float cam_rot[9],
                          float focal_x, float focal_y, float zFar, float zNear,
                          float* points_xy, float* rgb_depth, float* conic_opacity,
                          uint64_t* keys_unsorted, uint32_t* values_unsorted,
                          int64_t capacity, int* curr_offset, int64_t counts[4],
                          int num_threads)
{
    Cam cam;
    cam.W = width; cam.H = height; cam.bx = block_x; cam.by = block_y;
    cam.gx = (width + block_x - 1) / block_x;   /* preprocess.cu:461 */
    cam.gy = (height + block_y - 1) / block_y;
    view_proj(cam_pos, cam_rot, width, height, focal_x, focal_y, zFar, zNear, cam.view, cam.proj);
    cam.tan_fovx = (float)width / (2.0f * focal_x);   /* preprocess.cu:465-466 */
    cam.tan_fovy = (float)height / (2.0f * focal_y);
    cam.fx = focal_x; cam.fy = focal_y;
    memcpy(cam.campos, cam_pos, sizeof cam.campos);

    if (num_threads < 1) num_threads = 1;
    const int T = num_threads;
    std::vector<std::vector<uint64_t> > tkeys(T);
    std::vector<std::vector<uint32_t> > tvals(T);
    std::vector<int64_t> npass(T, 0), nvis(T, 0), ncand(T, 0);

    /* Each thread owns a contiguous chunk of Gaussians, so concatenating the
     * per-thread lists in thread order gives ascending Gaussian index. */
#pragma omp parallel num_threads(T)
    {
#ifdef _OPENMP
        int t = omp_get_thread_num();
#else
        int t = 0;
#endif
        int64_t lo = (int64_t)P * t / T, hi = (int64_t)P * (t + 1) / T;
        std::vector<uint64_t>& K = tkeys[t];
        std::vector<uint32_t>& V = tvals[t];
        for (int64_t i = lo; i < hi; i++) {
            GState g = GState();
            npass[t] += gaussian_state((int)i, positions, opacities, cov3ds, cam, g);
            if (!g.valid) continue;
            bool any = false;
            /* preprocess.cu:318-335 and :371-409 emit the same set; order fixed row-major here */
            for (int y = g.rmin[1]; y < g.rmax[1]; y++) {
                for (int x = g.rmin[0]; x < g.rmax[0]; x++) {
                    ncand[t]++;
                    int minx = x * block_x, miny = y * block_y;
                    int maxx = minx + block_x - 1, maxy = miny + block_y - 1;
                    if (!tile_test(minx, miny, maxx, maxy, g.point_xy[0], g.point_xy[1],
                                   g.conic[0], g.conic[1], g.conic[2], g.power))
                        continue;
                    uint64_t key = (uint64_t)(uint32_t)(y * cam.gx + x);
                    key <<= 32;
                    key |= f2u(g.p_view[2]);
                    K.push_back(key);
                    V.push_back((uint32_t)i);
                    any = true;
                }
            }
            /* preprocess.cu:317,411-417: a rectangle of one tile gets its record whether or not
             * the tile passed the test (vertex_valid starts as single_tile) */
            const bool single_tile = (g.rmax[0] - g.rmin[0]) * (g.rmax[1] - g.rmin[1]) == 1;
            if (any || single_tile) {
                nvis[t]++;
                points_xy[2 * i + 0] = g.point_xy[0];
                points_xy[2 * i + 1] = g.point_xy[1];
                conic_opacity[4 * i + 0] = (-0.5f * kLog2e) * g.conic[0];
                conic_opacity[4 * i + 1] = -kLog2e * g.conic[1];
                conic_opacity[4 * i + 2] = (-0.5f * kLog2e) * g.conic[2];
                conic_opacity[4 * i + 3] = g.log2_opacity;
                float rgb[3];
                sh_color(positions + 3 * i, cam.campos, shs + 48 * i, rgb);
                rgb_depth[4 * i + 0] = rgb[0];
                rgb_depth[4 * i + 1] = rgb[1];
                rgb_depth[4 * i + 2] = rgb[2];
                rgb_depth[4 * i + 3] = g.p_view[2];
            }
        }
    }

    int64_t base = *curr_offset;
    std::vector<int64_t> off(T + 1, 0);
    for (int t = 0; t < T; t++) off[t + 1] = off[t] + (int64_t)tkeys[t].size();
    int64_t total = off[T];
    if (counts) {
        counts[0] = counts[1] = counts[3] = 0;
        for (int t = 0; t < T; t++) { counts[0] += npass[t]; counts[1] += nvis[t]; counts[3] += ncand[t]; }
        counts[2] = total;
    }
    int rc = 0;
#pragma omp parallel for num_threads(T) schedule(static, 1)
    for (int t = 0; t < T; t++) {
        int64_t dst = base + off[t];
        int64_t n = (int64_t)tkeys[t].size();
        if (dst >= capacity || n == 0) continue;        // (an empty vector's data() may be null)
        if (dst + n > capacity) n = capacity - dst;
        memcpy(keys_unsorted + dst, tkeys[t].data(), (size_t)n * 8);
        memcpy(values_unsorted + dst, tvals[t].data(), (size_t)n * 4);
    }
    if (base + total > capacity) rc = -1;
    *curr_offset = (int)(base + total);
    return rc;
}

void fgs_oracle_sort(int num_rendered, int width, int height, int block_x, int block_y,
                     const uint64_t* keys_in, const uint32_t* values_in,
                     uint64_t* keys_out, uint32_t* values_out, int num_threads)
{
    const int64_t n = num_rendered;
    int gx = (width + block_x - 1) / block_x, gy = (height + block_y - 1) / block_y;
    int end_bit = 32 + (int)higher_msb((uint32_t)(gx * gy));   /* sort.cu:34-39 */
    if (num_threads < 1) num_threads = 1;
    const int T = num_threads;
    if (n <= 0) return;

    std::vector<uint64_t> kbuf[2];
    std::vector<uint32_t> vbuf[2];
    kbuf[0].assign(keys_in, keys_in + n);
    vbuf[0].assign(values_in, values_in + n);
    kbuf[1].resize(n);
    vbuf[1].resize(n);
    int cur = 0;
    std::vector<int64_t> hist((size_t)T * 256);
    for (int bit = 0; bit < end_bit; bit += 8) {
        int nb = end_bit - bit < 8 ? end_bit - bit : 8;
        uint32_t mask = (1u << nb) - 1u;
        const uint64_t* ks = kbuf[cur].data();
        const uint32_t* vs = vbuf[cur].data();
        uint64_t* kd = kbuf[cur ^ 1].data();
        uint32_t* vd = vbuf[cur ^ 1].data();
        std::fill(hist.begin(), hist.end(), 0);
#pragma omp parallel num_threads(T)
        {
#ifdef _OPENMP
            int t = omp_get_thread_num();
#else
            int t = 0;
#endif
            int64_t lo = n * t / T, hi = n * (t + 1) / T;
            int64_t* h = &hist[(size_t)t * 256];
            for (int64_t i = lo; i < hi; i++) h[(ks[i] >> bit) & mask]++;
#pragma omp barrier
#pragma omp single
            {
                int64_t run = 0;
                for (int d = 0; d < 256; d++)
                    for (int tt = 0; tt < T; tt++) {
                        int64_t c = hist[(size_t)tt * 256 + d];
                        hist[(size_t)tt * 256 + d] = run;
                        run += c;
                    }
            }
            for (int64_t i = lo; i < hi; i++) {
                int64_t dst = h[(ks[i] >> bit) & mask]++;
                kd[dst] = ks[i];
                vd[dst] = vs[i];
            }
        }
        cur ^= 1;
    }
    memcpy(keys_out, kbuf[cur].data(), (size_t)n * 8);
    memcpy(values_out, vbuf[cur].data(), (size_t)n * 4);
}

void fgs_oracle_ranges(int num_rendered, const uint64_t* keys, int* ranges, int num_tiles)
{
    memset(ranges, 0, sizeof(int) * 2 * (size_t)num_tiles);   /* render.cu:557 */
    const int L = num_rendered;
    for (int idx = 0; idx < L; idx++) {                          /* render.cu:9-31 */
        uint32_t currtile = (uint32_t)(keys[idx] >> 32);
        if (idx == 0) ranges[2 * (size_t)currtile + 0] = 0;
        else {
            uint32_t prevtile = (uint32_t)(keys[idx - 1] >> 32);
            if (currtile != prevtile) {
                ranges[2 * (size_t)prevtile + 1] = idx;
                ranges[2 * (size_t)currtile + 0] = idx;
            }
        }
        if (idx == L - 1) ranges[2 * (size_t)currtile + 1] = L;
    }
}

void fgs_oracle_render(int width, int height, int block_x, int block_y,
                       const float* points_xy, const float* rgb_depth,
                       const float* conic_opacity, const uint32_t* values_sorted,
                       const int* ranges, const float bg[3],
                       uint8_t* out_u8, float* out_f32, int64_t* walked, int num_threads)
{
    const int gx = (width + block_x - 1) / block_x, gy = (height + block_y - 1) / block_y;   /* render.cu:556 */
    const int npx = block_x * block_y;
    if (num_threads < 1) num_threads = 1;
    int64_t total_walked = 0;

#pragma omp parallel for num_threads(num_threads) schedule(dynamic, 4) reduction(+ : total_walked)
    for (int tile = 0; tile < gx * gy; tile++) {
        const int tx = tile % gx, ty = tile / gx;
        const int r0 = ranges[2 * (size_t)tile], r1 = ranges[2 * (size_t)tile + 1];
        std::vector<float> T(npx, 1.0f), Cr(npx, 0.0f), Cg(npx, 0.0f), Cb(npx, 0.0f);
        std::vector<float> pxf(npx), pyf(npx);
        for (int j = 0; j < npx; j++) {   /* render.cu:217-241: every pixel of the tile, in or out of the image */
            pxf[j] = (float)(tx * block_x + j % block_x);
            pyf[j] = (float)(ty * block_y + j / block_x);
        }
        int k = r0;
        bool done = false;
        /* render.cu:315-519: Gaussians are taken in pairs; the tile-wide stop is tested after each pair */
        while (k < r1 && !done) {
            int nthis = (k + 1 < r1) ? 2 : 1;
            for (int s = 0; s < nthis; s++) {
                uint32_t g = values_sorted[k + s];
                const float gxp = points_xy[2 * (size_t)g], gyp = points_xy[2 * (size_t)g + 1];
                const float* co = conic_opacity + 4 * (size_t)g;
                const float* rgb = rgb_depth + 4 * (size_t)g;
                for (int j = 0; j < npx; j++) {   /* render.cu:40-52 */
                    float dx = gxp - pxf[j], dy = gyp - pyf[j];
                    float power = co[3] + co[0] * dx * dx + co[2] * dy * dy + co[1] * dx * dy;
                    float alpha = exp2f(power);   /* replaces ex2.approx.ftz.f32 */
                    float at = alpha * T[j];
                    Cr[j] += rgb[0] * at;
                    Cg[j] += rgb[1] * at;
                    Cb[j] += rgb[2] * at;
                    T[j] -= at;
                }
            }
            total_walked += nthis;
            if (nthis == 1) break;   /* render.cu:486-487 */
            done = true;
            for (int j = 0; j < npx; j++) done = done && T[j] < 0.0001f;
            k += 2;
        }
        for (int j = 0; j < npx; j++) {   /* render.cu:59-73; stores guarded everywhere (the reference's empty-tile branch is not) */
            int px = tx * block_x + j % block_x, py = ty * block_y + j / block_x;
            if (px >= width || py >= height) continue;
            float Tj = T[j];
            if (Tj < 0.0001f) Tj = 0.0f;
            float c[3] = { Cr[j] + Tj * bg[0], Cg[j] + Tj * bg[1], Cb[j] + Tj * bg[2] };
            size_t pid = (size_t)width * py + px;
            for (int ch = 0; ch < 3; ch++) {
                if (out_f32) out_f32[3 * pid + ch] = c[ch];
                if (out_u8) {   /* render.cu:54-57 */
                    float v = fminf_(fmaxf_(c[ch] * 255.0f, 0.0f), 255.0f);
                    out_u8[3 * pid + ch] = (uint8_t)v;
                }
            }
        }
    }
    if (walked) *walked = total_walked;
}

} // extern "C"
