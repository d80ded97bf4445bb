// Tile ranges and front-to-back alpha blending for gfx950 (wave64).
//
// Replaces FlashGS render<BX,BY> (csrc/cuda_rasterizer/render.cu:549-576): zero the ranges,
// identifyTileRanges (:9-31) and renderCUDA (:199-547).
//
// Blend layout: a workgroup of 256 threads (4 wave64) owns one tile.  A tile is made of
// 16x16-pixel sub-tiles (1 for 16x16, 2 for 32x16, 4 for 32x32); each wave owns the same 8x8
// quadrant of every sub-tile, so a thread shades one pixel per sub-tile.  Gaussians are staged
// 256 at a time into LDS by all threads together (index -> centre, conic+opacity, colour), then
// every wave walks the batch reading LDS at a wave-uniform address.  After every second Gaussian
// (the reference tests after each pair, render.cu:394-405) a wave checks with one ballot whether
// all of its pixels have T < 1e-4 and stops shading if so; the workgroup leaves when all four
// waves have stopped or the range is exhausted.
#include "fgs_internal.h"

namespace fgs {
namespace {

constexpr int kBlendThreads = 256;
constexpr int kBatch = 256;

__global__ __launch_bounds__(256) void fill_i32_kernel(int* p, size_t n, int v)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

// render.cu:9-31, with the tile index checked against the number of tiles
__global__ __launch_bounds__(256) void tile_ranges_kernel(int L, const uint64_t* __restrict__ keys,
                                                          int2* __restrict__ ranges, uint32_t num_tiles)
{
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= L) return;
    const uint32_t cur = (uint32_t)(keys[idx] >> 32);
    if (cur >= num_tiles) return;
    if (idx == 0) {
        ranges[cur].x = 0;
    } else {
        const uint32_t prev = (uint32_t)(keys[idx - 1] >> 32);
        if (cur != prev) {
            if (prev < num_tiles) ranges[prev].y = idx;
            ranges[cur].x = idx;
        }
    }
    if (idx == L - 1) ranges[cur].y = L;
}

// render.cu:54-57
__device__ __forceinline__ uint8_t encode_u8(float x)
{
    float v = x * 255.0f;
    v = v > 0.0f ? v : 0.0f;       // also maps NaN to 0
    v = v < 255.0f ? v : 255.0f;
    return (uint8_t)v;
}

template <int SX, int SY>
__global__ __launch_bounds__(kBlendThreads) void blend_kernel(
    const int2* __restrict__ ranges,
    const uint32_t* __restrict__ point_list,
    int width, int height, int tiles_x,
    const float2* __restrict__ points_xy,
    const float4* __restrict__ rgb_depth,
    const float4* __restrict__ conic_opacity,
    float bg_r, float bg_g, float bg_b,
    uint8_t* __restrict__ out_u8,
    float* __restrict__ out_f32)
{
    constexpr int kSub = SX * SY;              // pixels per thread
    __shared__ float2 s_xy[kBatch];
    __shared__ float4 s_co[kBatch];
    __shared__ float4 s_rgb[kBatch];
    __shared__ int s_waves_done;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int tile_x = blockIdx.x, tile_y = blockIdx.y;
    const int2 range = ranges[tile_y * tiles_x + tile_x];

    // this thread's pixel inside a 16x16 sub-tile: wave -> 8x8 quadrant, lane -> pixel of it
    const int lx = (wave & 1) * 8 + (lane & 7);
    const int ly = (wave >> 1) * 8 + (lane >> 3);
    int pix_x[kSub], pix_y[kSub];
    float pxf[kSub], pyf[kSub];
#pragma unroll
    for (int s = 0; s < kSub; s++) {
        pix_x[s] = tile_x * (16 * SX) + (s % SX) * 16 + lx;
        pix_y[s] = tile_y * (16 * SY) + (s / SX) * 16 + ly;
        pxf[s] = (float)pix_x[s];
        pyf[s] = (float)pix_y[s];
    }

    float T[kSub], Cr[kSub], Cg[kSub], Cb[kSub];
#pragma unroll
    for (int s = 0; s < kSub; s++) { T[s] = 1.0f; Cr[s] = 0.0f; Cg[s] = 0.0f; Cb[s] = 0.0f; }

    if (tid == 0) s_waves_done = 0;
    bool wave_done = false;
    const int n = range.y - range.x;

    for (int base = 0; base < n; base += kBatch) {
        const int cnt = min(kBatch, n - base);
        __syncthreads();                       // previous batch fully consumed; s_waves_done initialised
        if (s_waves_done == kBlendThreads / kWave) break;
        if (tid < cnt) {
            const uint32_t g = point_list[range.x + base + tid];
            s_xy[tid] = points_xy[g];
            s_co[tid] = conic_opacity[g];
            s_rgb[tid] = rgb_depth[g];
        }
        __syncthreads();
        if (!wave_done) {
            for (int j = 0; j < cnt; j++) {
                const float2 g = s_xy[j];
                const float4 co = s_co[j];
                const float4 col = s_rgb[j];
#pragma unroll
                for (int s = 0; s < kSub; s++) {       // render.cu:40-52
                    const float dx = g.x - pxf[s], dy = g.y - pyf[s];
                    const float power = co.w + co.x * dx * dx + co.z * dy * dy + co.y * dx * dy;
                    const float alpha = __builtin_amdgcn_exp2f(power);
                    const float at = alpha * T[s];
                    Cr[s] += col.x * at;
                    Cg[s] += col.y * at;
                    Cb[s] += col.z * at;
                    T[s] -= at;
                }
                if (j & 1) {
                    bool done = true;
#pragma unroll
                    for (int s = 0; s < kSub; s++) done = done && T[s] < 0.0001f;
                    if (ballot(!done) == 0) { wave_done = true; break; }
                }
            }
            if (wave_done && lane == 0) atomicAdd(&s_waves_done, 1);
        }
    }

    // render.cu:59-73
#pragma unroll
    for (int s = 0; s < kSub; s++) {
        if (pix_x[s] < width && pix_y[s] < height) {
            const size_t pid = (size_t)width * pix_y[s] + pix_x[s];
            float t = T[s];
            if (t < 0.0001f) t = 0.0f;
            const float r = Cr[s] + t * bg_r, g = Cg[s] + t * bg_g, b = Cb[s] + t * bg_b;
            if (out_u8) {
                out_u8[3 * pid + 0] = encode_u8(r);
                out_u8[3 * pid + 1] = encode_u8(g);
                out_u8[3 * pid + 2] = encode_u8(b);
            }
            if (out_f32) {
                out_f32[3 * pid + 0] = r;
                out_f32[3 * pid + 1] = g;
                out_f32[3 * pid + 2] = b;
            }
        }
    }
}

int check_tile(int block_x, int block_y, int* sx, int* sy, const char* who)
{
    if ((block_x == 16 && block_y == 16) || (block_x == 32 && block_y == 16) || (block_x == 32 && block_y == 32)) {
        *sx = block_x / 16;
        *sy = block_y / 16;
        return FGS_OK;
    }
    return fail(FGS_E_INVALID, "%s: tile %dx%d unsupported (16x16, 32x16, 32x32)", who, block_x, block_y);
}

// render.cu:556-563: zero the ranges, then mark where each tile starts and ends
int ranges_impl(int block_x, int block_y, int num_rendered, int width, int height,
                const uint64_t* keys_sorted, int* ranges, void* stream, const char* who)
{
    if (num_rendered < 0) return fail(FGS_E_INVALID, "%s: num_rendered = %d is negative", who, num_rendered);
    if (width <= 0 || height <= 0 || block_x <= 0 || block_y <= 0)
        return fail(FGS_E_INVALID, "%s: width/height/block must be positive", who);
    if (!ranges || (num_rendered > 0 && !keys_sorted)) return fail(FGS_E_INVALID, "%s: null buffer", who);
    if (((uintptr_t)keys_sorted | (uintptr_t)ranges) % 8 != 0)
        return fail(FGS_E_INVALID, "%s: keys and ranges must be 8-byte aligned", who);
    const int tiles_x = (width + block_x - 1) / block_x, tiles_y = (height + block_y - 1) / block_y;
    const size_t num_tiles = (size_t)tiles_x * tiles_y;
    hipStream_t st = (hipStream_t)stream;
    const size_t words = num_tiles * 2;
    size_t fill_blocks = (words + 1023) / 1024;
    if (fill_blocks > 1024) fill_blocks = 1024;
    hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)fill_blocks), dim3(256), 0, st, ranges, words, 0);
    if (num_rendered > 0)
        hipLaunchKernelGGL(tile_ranges_kernel, dim3((num_rendered + 255) / 256), dim3(256), 0, st,
                           num_rendered, keys_sorted, (int2*)ranges,
                           (uint32_t)(num_tiles > 0xffffffffu ? 0xffffffffu : num_tiles));
    return check_hip(hipGetLastError(), who);
}

// render.cu:566-575
int blend_impl(int block_x, int block_y, int width, int height,
               const float* points_xy, const float* rgb_depth, const float* conic_opacity,
               const uint32_t* values_sorted, const int* ranges, const float bg[3],
               uint8_t* out_u8, float* out_f32, void* stream, const char* who)
{
    int sx = 0, sy = 0;
    int rc = check_tile(block_x, block_y, &sx, &sy, who);
    if (rc != FGS_OK) return rc;
    if (width <= 0 || height <= 0) return fail(FGS_E_INVALID, "%s: width/height must be positive", who);
    if (!ranges || !bg || (!out_u8 && !out_f32)) return fail(FGS_E_INVALID, "%s: null ranges, bg_color or output", who);
    if (((uintptr_t)rgb_depth | (uintptr_t)conic_opacity) % 16 != 0 ||
        ((uintptr_t)points_xy | (uintptr_t)ranges) % 8 != 0)
        return fail(FGS_E_INVALID, "%s: rgb_depth/conic_opacity must be 16-byte aligned, points_xy/ranges 8-byte aligned", who);
    const int tiles_x = (width + block_x - 1) / block_x, tiles_y = (height + block_y - 1) / block_y;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(tiles_x, tiles_y);
#define FGS_LAUNCH_BLEND(SX, SY)                                                                        \
    hipLaunchKernelGGL((blend_kernel<SX, SY>), grid, dim3(kBlendThreads), 0, st,                        \
                       (const int2*)ranges, values_sorted, width, height, tiles_x,                      \
                       (const float2*)points_xy, (const float4*)rgb_depth, (const float4*)conic_opacity, \
                       bg[0], bg[1], bg[2], out_u8, out_f32)
    if (sx == 1 && sy == 1) FGS_LAUNCH_BLEND(1, 1);
    else if (sx == 2 && sy == 1) FGS_LAUNCH_BLEND(2, 1);
    else FGS_LAUNCH_BLEND(2, 2);
#undef FGS_LAUNCH_BLEND
    return check_hip(hipGetLastError(), who);
}

int render_impl(int block_x, int block_y, int num_rendered, int width, int height,
                const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                const uint64_t* keys_sorted, const uint32_t* values_sorted,
                int* ranges, const float bg[3], uint8_t* out_u8, float* out_f32, void* stream, const char* who)
{
    int sx = 0, sy = 0;
    int rc = check_tile(block_x, block_y, &sx, &sy, who);
    if (rc != FGS_OK) return rc;
    if (num_rendered > 0 && (!points_xy || !rgb_depth || !conic_opacity || !keys_sorted || !values_sorted))
        return fail(FGS_E_INVALID, "%s: null buffer", who);
    rc = ranges_impl(block_x, block_y, num_rendered, width, height, keys_sorted, ranges, stream, who);
    if (rc != FGS_OK) return rc;
    return blend_impl(block_x, block_y, width, height, points_xy, rgb_depth, conic_opacity, values_sorted, ranges,
                      bg, out_u8, out_f32, stream, who);
}

} // namespace
} // namespace fgs

#define FGS_DEFINE_RENDER(NAME, BX, BY)                                                                      \
    extern "C" int NAME(int num_rendered, int width, int height,                                             \
                        const float* points_xy, const float* rgb_depth, const float* conic_opacity,          \
                        const uint64_t* gaussian_keys_sorted, const uint32_t* gaussian_values_sorted,        \
                        int* ranges, const float bg_color[3], uint8_t* out_color, void* stream)              \
    {                                                                                                        \
        if (!out_color) return fgs::fail(FGS_E_INVALID, #NAME ": null out_color");                           \
        return fgs::render_impl(BX, BY, num_rendered, width, height, points_xy, rgb_depth, conic_opacity,    \
                                gaussian_keys_sorted, gaussian_values_sorted, ranges, bg_color, out_color,   \
                                nullptr, stream, #NAME);                                                     \
    }

FGS_DEFINE_RENDER(fgs_render_16x16, 16, 16)
FGS_DEFINE_RENDER(fgs_render_32x16, 32, 16)
FGS_DEFINE_RENDER(fgs_render_32x32, 32, 32)

extern "C" int fgs_render_f32(int block_x, int block_y, int num_rendered, int width, int height,
                              const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                              const uint64_t* gaussian_keys_sorted, const uint32_t* gaussian_values_sorted,
                              int* ranges, const float bg_color[3], uint8_t* out_color_u8, float* out_color_f32,
                              void* stream)
{
    return fgs::render_impl(block_x, block_y, num_rendered, width, height, points_xy, rgb_depth,
                            conic_opacity, gaussian_keys_sorted, gaussian_values_sorted, ranges, bg_color,
                            out_color_u8, out_color_f32, stream, "fgs_render_f32");
}

extern "C" int fgs_tile_ranges(int block_x, int block_y, int num_rendered, int width, int height,
                               const uint64_t* gaussian_keys_sorted, int* ranges, void* stream)
{
    return fgs::ranges_impl(block_x, block_y, num_rendered, width, height, gaussian_keys_sorted, ranges, stream,
                            "fgs_tile_ranges");
}

extern "C" int fgs_blend(int block_x, int block_y, int width, int height,
                         const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                         const uint32_t* gaussian_values_sorted, const int* ranges, const float bg_color[3],
                         uint8_t* out_color_u8, float* out_color_f32, void* stream)
{
    return fgs::blend_impl(block_x, block_y, width, height, points_xy, rgb_depth, conic_opacity,
                           gaussian_values_sorted, ranges, bg_color, out_color_u8, out_color_f32, stream, "fgs_blend");
}
