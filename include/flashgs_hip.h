/*
 * flashgs_hip.h - C ABI of the MI355X (gfx950) 3D Gaussian Splatting forward rasterizer.
 *
 * One entry point per host function of FlashGS's csrc/ops.h:32-65; each comment cites the
 * reference interface it replaces (paths relative to the FlashGS source tree).  Everything is
 * plain pointers and sizes: device pointers are raw HIP device addresses, `stream` is a
 * hipStream_t passed as void* (NULL = the default stream), cameras and colours are host
 * arrays.  All buffers are caller-owned; calls are asynchronous on `stream` and never
 * synchronise.  Every function that can fail returns 0 on success or a negative FGS_E_* code,
 * with a per-thread message available from fgs_last_error().
 */
#ifndef FLASHGS_HIP_H
#define FLASHGS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FGS_OK            0
#define FGS_E_INVALID    -1   /* null pointer, negative size, unsupported tile size */
#define FGS_E_WORKSPACE  -2   /* list_sorting_space too small for num_rendered */
#define FGS_E_HIP        -3   /* a HIP runtime call or kernel launch failed */
#define FGS_E_NOMEM      -4   /* internal scratch allocation failed */
#define FGS_E_TIMEOUT    -5   /* fgs_wait_count: no pair count within the time given */

/* Largest key count the sort accepts (positions and block counts are kept in 32-bit integers). */
#define FGS_MAX_RENDERED ((1 << 30) - 1)

/*
 * Replaces flashgs::preprocess (csrc/ops.h:32-39, csrc/cuda_rasterizer/preprocess.cu:452-488).
 * Same arguments in the same order, with the camera as host arrays: cam_position[3] and
 * cam_rotation[9] exactly as csrc/pybind.cpp:131-143 reads them from the two CPU tensors
 * (cam_rotation[3*c + r] becomes element r of GLM column c).
 *
 * positions f32[P,3], shs f32[P,48], opacities f32[P], cov3Ds f32[P,6] are device inputs;
 * points_xy f32[P,2], rgb_depth f32[P,4], conic_opacity f32[P,4] are device outputs whose rows
 * are written only for Gaussians that emit at least one key or whose candidate rectangle is a
 * single tile (preprocess.cu:317,411-417); all other rows keep what they held; keys/values receive the
 * (tile << 32 | depth bits, Gaussian index) pairs starting at *curr_offset, in ascending
 * Gaussian index then row-major tile order; *curr_offset (device int, zeroed by the caller as
 * in example.py:69) ends at the total number of pairs.
 *
 * key_capacity is the one addition to the reference signature: number of elements the key and
 * value buffers hold.  Pairs that would land at or beyond it are dropped (the counter still
 * counts them, so the caller's check of example.py:79-82 keeps working); pass 0 to write
 * unchecked like the reference (preprocess.cu:330,395).
 *
 * The call is asynchronous on `stream`.  The library keeps a small scratch for the scan over
 * workgroups per (device, stream), allocated on the first call on that stream, so calls on
 * different streams of one device may overlap in time.  When a larger P arrives a larger scratch
 * is allocated and the earlier one is kept, never freed (32 bytes per 256 Gaussians it was sized
 * for), because a HIP graph captured on the stream holds its address.  Nothing on the host changes
 * from launch to launch, so a launch can be captured in a HIP graph and replayed, also after
 * larger eager calls on the same stream; a stream that is being captured and has no (large enough)
 * scratch yet cannot allocate one and uses the built-in scan status of fgs_preprocess_static, with
 * its limits.
 *
 * Every wait inside the launch is bounded (fgs_set_scan_spin_limit).  If one ever gives up,
 * *curr_offset ends negative (INT_MIN) and keys, values and attribute rows are not to be used.
 * When it was the scan itself that gave up, the scratch is left marked unusable: every later
 * fgs_preprocess on that stream (and every fgs_preprocess_static on that device, if it was the
 * built-in scratch) reports a negative count too, at once and without touching anything, until
 * fgs_reset_scan has been called on the stream.  So the caller's recovery is: see a negative
 * count, call fgs_reset_scan(stream), zero *curr_offset, call fgs_preprocess again.
 */
int fgs_preprocess(int P,
                   const float* positions, const float* shs, const float* opacities, const float* cov3Ds,
                   int width, int height, int block_x, int block_y,
                   const float cam_position[3], const float cam_rotation[9],
                   float focal_x, float focal_y, float zFar, float zNear,
                   float* points_xy, float* rgb_depth, float* conic_opacity,
                   uint64_t* gaussian_keys_unsorted, uint32_t* gaussian_values_unsorted,
                   int* curr_offset, int64_t key_capacity, void* stream);

/*
 * No counterpart in the reference.  fgs_preprocess for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * same arguments, same kernel, same results, but the scan status lives in a 2 MiB array inside
 * the library's device image (one copy per GPU, held until the process ends) instead of a
 * buffer from hipMalloc, so the call allocates and frees nothing and never synchronises.
 * P is limited to 16 777 216 Gaussians; a larger P returns FGS_E_INVALID.  Every call on one GPU
 * shares that GPU's array: calls that overlap in time on one GPU race (calls on one stream, or
 * otherwise ordered, do not).  May be mixed freely with fgs_preprocess.
 */
int fgs_preprocess_static(int P,
                          const float* positions, const float* shs, const float* opacities, const float* cov3Ds,
                          int width, int height, int block_x, int block_y,
                          const float cam_position[3], const float cam_rotation[9],
                          float focal_x, float focal_y, float zFar, float zNear,
                          float* points_xy, float* rgb_depth, float* conic_opacity,
                          uint64_t* gaussian_keys_unsorted, uint32_t* gaussian_values_unsorted,
                          int* curr_offset, int64_t key_capacity, void* stream);

/*
 * No counterpart in the reference, whose caller reads the pair count back with a blocking copy
 * (example.py:79).  fgs_preprocess that also stores the pair count into *count_mirror, a word of
 * pinned host memory (hipHostMalloc; anything else returns FGS_E_INVALID), for a host that polls
 * it instead (fgs_wait_count).  The call itself writes FGS_COUNT_PENDING into *count_mirror before
 * it launches; a captured launch that is replayed does not, there the caller does before every replay.
 * The count arrives as soon as the launch knows it, which is while it is still writing keys: the
 * caller can enqueue fgs_sort_gaussian on the same stream at once, stream order does the rest.
 * A launch that gives up (see fgs_preprocess) stores INT_MIN; if only one workgroup's wait gives up
 * after the count has been stored, INT_MIN overwrites it later, so a caller that wants to rule
 * that out looks at the word again, or at *curr_offset, when the stream has drained.
 */
#define FGS_COUNT_PENDING (-2147483647)
int fgs_preprocess_mirrored(int P,
                            const float* positions, const float* shs, const float* opacities, const float* cov3Ds,
                            int width, int height, int block_x, int block_y,
                            const float cam_position[3], const float cam_rotation[9],
                            float focal_x, float focal_y, float zFar, float zNear,
                            float* points_xy, float* rgb_depth, float* conic_opacity,
                            uint64_t* gaussian_keys_unsorted, uint32_t* gaussian_values_unsorted,
                            int* curr_offset, int64_t key_capacity, int* count_mirror, void* stream);

/*
 * Host only: polls *count_mirror until it differs from FGS_COUNT_PENDING and stores what it finds
 * in *count (negative: the launch gave up).  FGS_E_TIMEOUT after timeout_seconds without a count.
 */
int fgs_wait_count(const int* count_mirror, double timeout_seconds, int* count);

/*
 * Replaces flashgs::sort_gaussian (csrc/ops.h:41-45, csrc/cuda_rasterizer/sort.cu:28-44):
 * stable ascending sort of num_rendered (key, value) pairs on key bits
 * [0, 32 + bit_length(tiles_x * tiles_y)).  Inputs are left untouched.
 * list_sorting_space must hold at least fgs_get_sort_buffer_size(num_rendered) bytes and be
 * 256-byte aligned.
 */
int fgs_sort_gaussian(int num_rendered,
                      int width, int height, int block_x, int block_y,
                      char* list_sorting_space, size_t sorting_size,
                      const uint64_t* gaussian_keys_unsorted, const uint32_t* gaussian_values_unsorted,
                      uint64_t* gaussian_keys_sorted, uint32_t* gaussian_values_sorted, void* stream);

/*
 * Replaces flashgs::get_sort_buffer_size (csrc/ops.h:47, sort.cu:46-54).  Host only.
 * Monotonic in num_rendered; returns 0 for a negative or too large count.
 */
size_t fgs_get_sort_buffer_size(int num_rendered);

/*
 * Replace flashgs::render_16x16 / render_32x16 / render_32x32 (csrc/ops.h:49-65,
 * csrc/cuda_rasterizer/render.cu:549-608): zero `ranges`, find each tile's [start,end) in the
 * sorted keys, blend front to back and write out_color u8[H,W,3].  `ranges` int32[tiles,2] is
 * scratch that holds the tile ranges afterwards.  bg_color is a host array of 3 floats.
 * All arithmetic is fp32, as in render.cu:40-52, unless the process default was changed with
 * fgs_set_colour_sums (fgs_render_ex / fgs_blend_ex choose per call).
 * A frame of at most 8192 16x16 tiles first ranks its tiles by list length into a table the
 * library keeps per (device, stream) (32 KB, allocated on the first such call on that stream),
 * and the rest of a list of more than 768 entries is blended in four runs that each stop on
 * their own transmittance: the colour can differ from the pair-by-pair walk of
 * render.cu:315-408 by what lies behind T < 1e-4, i.e. by less than 1e-4 of a colour.  Calls on
 * different streams may overlap in time; a stream that is being captured and has no table yet
 * uses one table per device instead, so replays of such graphs on one device must not overlap.
 */
int fgs_render_16x16(int num_rendered, int width, int height,
                     const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                     const uint64_t* gaussian_keys_sorted, const uint32_t* gaussian_values_sorted,
                     int* ranges, const float bg_color[3], uint8_t* out_color, void* stream);
int fgs_render_32x16(int num_rendered, int width, int height,
                     const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                     const uint64_t* gaussian_keys_sorted, const uint32_t* gaussian_values_sorted,
                     int* ranges, const float bg_color[3], uint8_t* out_color, void* stream);
int fgs_render_32x32(int num_rendered, int width, int height,
                     const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                     const uint64_t* gaussian_keys_sorted, const uint32_t* gaussian_values_sorted,
                     int* ranges, const float bg_color[3], uint8_t* out_color, void* stream);

/*
 * No counterpart in the reference: the same pass as fgs_render_<bx>x<by> with the colour
 * C + T*bg stored as f32[H,W,3] before the truncating 8-bit encode of render.cu:54-57, so that
 * images can be compared below one 8-bit step.  out_color_u8 may be NULL.
 * block_x x block_y must be 16x16, 32x16 or 32x32.
 */
int fgs_render_f32(int block_x, int block_y, int num_rendered, int width, int height,
                   const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                   const uint64_t* gaussian_keys_sorted, const uint32_t* gaussian_values_sorted,
                   int* ranges, const float bg_color[3], uint8_t* out_color_u8, float* out_color_f32,
                   void* stream);

/*
 * The two halves of fgs_render_*, for callers that want them separately (per-stage timing, or
 * blending several images from one set of ranges).  fgs_tile_ranges is render.cu:556-563 (zero
 * `ranges`, then identifyTileRanges, render.cu:9-31); fgs_blend is the renderCUDA launch of
 * render.cu:566-575 reading `ranges`.  Either output of fgs_blend may be NULL, not both.
 */
int fgs_tile_ranges(int block_x, int block_y, int num_rendered, int width, int height,
                    const uint64_t* gaussian_keys_sorted, int* ranges, void* stream);
int fgs_blend(int block_x, int block_y, int width, int height,
              const float* points_xy, const float* rgb_depth, const float* conic_opacity,
              const uint32_t* gaussian_values_sorted, const int* ranges, const float bg_color[3],
              uint8_t* out_color_u8, float* out_color_f32, void* stream);

/*
 * No counterpart in the reference.  How a blend forms its colour sums C += (alpha T) c.
 *   FGS_COLOUR_SUMS_FP32 (default): by fp32 multiply-add, operation for operation what
 *     render.cu:40-52 does.
 *   FGS_COLOUR_SUMS_MATRIX_F16 (opt-in, about a fifth faster in the blend of a 4K frame): on the
 *     matrix unit; the weights alpha T and the colours are rounded to f16, products and sums are
 *     fp32: a pixel's colour is within 2^-10 of itself of the all-fp32 sum.  Colours beyond
 *     +-65504 are drawn as +-65504 and opacities above 3.97 as 3.97; a conic that is not positive
 *     definite (its exponent grows without bound away from the centre) can push a weight past
 *     f16's range, which the fp32 mode does not have - keep such inputs on the default.
 * Exponent, alpha and transmittance are fp32 in both.
 *
 * fgs_set_colour_sums sets the process-wide default, which the entry points without a flags
 * argument use at the time of the call (fgs_render_<bx>x<by>, fgs_render_f32, fgs_blend); it
 * returns the previous default, -1 for an unknown mode.  A caller that shares the process with
 * other renderers passes the mode per call instead: fgs_render_ex and fgs_blend_ex are
 * fgs_render_f32 and fgs_blend with a flags argument, 0 = the process default, FGS_BLEND_FP32 or
 * FGS_BLEND_MATRIX_F16 = that mode whatever the default is.
 */
#define FGS_COLOUR_SUMS_MATRIX_F16 0
#define FGS_COLOUR_SUMS_FP32       1
int fgs_set_colour_sums(int mode);

#define FGS_BLEND_FP32        1
#define FGS_BLEND_MATRIX_F16  2
int fgs_render_ex(int block_x, int block_y, int num_rendered, int width, int height,
                  const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                  const uint64_t* gaussian_keys_sorted, const uint32_t* gaussian_values_sorted,
                  int* ranges, const float bg_color[3], uint8_t* out_color_u8, float* out_color_f32,
                  int flags, void* stream);
int fgs_blend_ex(int block_x, int block_y, int width, int height,
                 const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                 const uint32_t* gaussian_values_sorted, const int* ranges, const float bg_color[3],
                 uint8_t* out_color_u8, float* out_color_f32, int flags, void* stream);

/*
 * No counterpart in the reference.  Name of the kernel(s) a blend with these flags launches on
 * the current device for this tile and frame size (the choice depends on how many tiles the frame
 * has against what the chip holds at once), as a profiler lists them; "" for an unsupported tile
 * size or unknown flags.  Lets a benchmark attribute its figures to the kernel that ran.
 */
const char* fgs_blend_kernel_name(int block_x, int block_y, int width, int height, int flags);

/*
 * Host-side camera set-up used by fgs_preprocess (preprocess.cu:420-448,461-466), exposed so
 * callers and tests can inspect it: column-major 4x4 view and projection matrices.
 */
void fgs_camera_matrices(const float cam_position[3], const float cam_rotation[9],
                         int width, int height, float focal_x, float focal_y, float zFar, float zNear,
                         float view[16], float proj[16]);

/*
 * No counterpart in the reference.  Number of polls after which a wait inside the preprocess
 * launch (the scanner for a workgroup's key count, a workgroup for its key offset) gives up and
 * the launch reports a negative pair count; applies to launches made after the call, returns the
 * previous value.  The default, 1 << 22, is seconds of waiting and is never reached by a healthy
 * launch.  A diagnostic knob: 0 makes every wait that is not satisfied at its first poll give up,
 * which is how the give-up path is tested without hanging anything.
 */
unsigned fgs_set_scan_spin_limit(unsigned polls);

/*
 * No counterpart in the reference.  Clears the scan status that fgs_preprocess keeps for `stream`
 * on the current device, and the built-in one of fgs_preprocess_static on that device, with a
 * small kernel enqueued on `stream` (so it is ordered after the launches already on it and may be
 * captured).  Needed only after a preprocess that reported a negative pair count, see there;
 * harmless otherwise.  Must not overlap a preprocess launch that uses the same scan status from
 * another stream.
 */
int fgs_reset_scan(void* stream);

/* Message of the last failing call on this thread ("" if none). */
const char* fgs_last_error(void);

/*
 * ABI version of this header as major * 1000 + minor: the major number changes when an existing
 * signature or default changes, the minor one when entry points are added.
 */
#define FGS_ABI_VERSION 2001
int fgs_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FLASHGS_HIP_H */
