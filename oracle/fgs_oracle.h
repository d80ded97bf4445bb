/*
 * CPU oracle for the FlashGS forward rasterizer path
 * (preprocess -> sort_gaussian -> render_16x16).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates the reference
 * algorithm (file:line citations are relative to the FlashGS source tree) in
 * plain scalar C++ so that the HIP kernels can be checked against it.  Only the
 * test-suite, the smoke check and the CPU-baseline leg of the benchmark may
 * load it; the shipped library never links or calls anything declared here.
 *
 * Hardware-defined approximations of the reference (PTX lg2.approx,
 * sqrt.approx, rsqrt.approx, ex2.approx) are replaced by deterministic
 * routines: a fixed-order software log2, IEEE sqrtf, 1/sqrtf and libm exp2f.
 * Emission order of (key,value) pairs, which the reference leaves to atomics,
 * is fixed to: ascending Gaussian index, then row-major tile order.
 *
 * Pin status of every function is listed at the top of fgs_oracle.cpp.
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* --- scalar building blocks, exported so tests can pin each one ---------- */

/* software log2 for positive normal floats; fixed operation order */
float fgs_oracle_log2f(float x);

/* preprocess.cu:420-427 and :429-448: column-major 4x4 view and proj matrices,
 * rot = 9 floats packed as pybind.cpp:140-143 packs them (GLM columns). */
void fgs_oracle_view_proj(const float pos[3], const float rot[9], int width, int height,
                          float focal_x, float focal_y, float zFar, float zNear,
                          float view[16], float proj[16]);

/* preprocess.cu:103-143: returns cov = (c00, c01, c11) after the +0.3 low-pass */
void fgs_oracle_cov2d(const float p[3], float focal_x, float focal_y, float tan_fovx,
                      float tan_fovy, const float cov3d[6], const float view[16], float cov[3]);

/* preprocess.cu:238-241 || :196-236 for one tile; returns 0/1 */
int fgs_oracle_tile_test(int pix_min_x, int pix_min_y, int pix_max_x, int pix_max_y,
                         float cx, float cy, float conic_x, float conic_y, float conic_z,
                         float power);

/* preprocess.cu:145-185: deg-3 SH colour of one Gaussian, clamped at 0 */
void fgs_oracle_sh_color(const float p[3], const float campos[3], const float sh[48], float rgb[3]);

/* preprocess.cu:90-100 */
void fgs_oracle_rect(float px, float py, int width, int height, int grid_x, int grid_y,
                     int block_x, int block_y, int rect_min[2], int rect_max[2]);

/* sort.cu:9-24 */
uint32_t fgs_oracle_higher_msb(uint32_t n);

/* pybind.cpp:22-56 (computeCov3D) for n Gaussians: scale[n,3], rot[n,4] (r,x,y,z) */
void fgs_oracle_cov3d(int n, const float* scale, const float* rot, float* cov3d);

/* --- the four stages ------------------------------------------------------ */

/* preprocess.cu:243-418 + :452-488.  Writes attributes only for Gaussians that
 * emitted >= 1 key.  Keys start at *curr_offset and *curr_offset ends at the
 * total.  Returns 0, or -1 if the key count would exceed capacity (nothing
 * beyond capacity is written).  counts (nullable) receives
 * {N_pass, V, K, candidates}. */
int fgs_oracle_preprocess(int P, const float* positions, const float* shs,
                          const float* opacities, const float* cov3ds,
                          int width, int height, int block_x, int block_y,
                          const float cam_pos[3], const float cam_rot[9],
                          float focal_x, float focal_y, float zFar, float zNear,
                          float* points_xy, float* rgb_depth, float* conic_opacity,
                          uint64_t* keys_unsorted, uint32_t* values_unsorted,
                          int64_t capacity, int* curr_offset, int64_t counts[4],
                          int num_threads);

/* sort.cu:28-39: stable LSD radix sort on key bits [0, 32 + higher_msb(tiles)) */
void fgs_oracle_sort(int num_rendered, int width, int height, int block_x, int block_y,
                     const uint64_t* keys_in, const uint32_t* values_in,
                     uint64_t* keys_out, uint32_t* values_out, int num_threads);

/* render.cu:557 + :9-31 */
void fgs_oracle_ranges(int num_rendered, const uint64_t* keys_sorted, int* ranges, int num_tiles);

/* render.cu:199-547 for a block_x x block_y tile.  out_u8 [H,W,3] (nullable),
 * out_f32 [H,W,3] (nullable) = C + T*bg before quantisation, with T zeroed
 * below 1e-4 as write_color does.  walked (nullable) receives B = sum over
 * tiles of Gaussians blended before the tile-wide stop. */
void fgs_oracle_render(int width, int height, int block_x, int block_y,
                       const float* points_xy, const float* rgb_depth,
                       const float* conic_opacity, const uint32_t* values_sorted,
                       const int* ranges, const float bg[3],
                       uint8_t* out_u8, float* out_f32, int64_t* walked, int num_threads);

#ifdef __cplusplus
}
#endif
