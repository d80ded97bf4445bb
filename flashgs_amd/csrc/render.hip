// Tile ranges and front-to-back alpha blending for gfx950 (wave64).
//
// Replaces FlashGS render<BX,BY> (csrc/cuda_rasterizer/render.cu:549-576): zero the ranges,
// identifyTileRanges (:9-31) and renderCUDA (:199-547).
//
// Blend layout: one wave64 owns one tile.  A tile is made of 16x16-pixel sub-tiles (1 for 16x16,
// 2 for 32x16, 4 for 32x32); lane l shades the 2x2 pixel quad at (2*(l%8), 2*(l/8)) of every
// sub-tile; the quadratic form is evaluated at one pixel of the quad and stepped to the others.  Gaussians are
// staged 64 at a time into LDS (one per lane: index -> centre, conic+opacity, colour) while the
// loads of the following batch are already in flight, and the wave walks the batch reading LDS
// at wave-uniform addresses.  After every second Gaussian one ballot tests whether all pixels of
// the tile have T < 1e-4, which is the reference's stop rule (render.cu:394-408).  A workgroup is
// a single wave, so no workgroup barrier is needed anywhere.
#include "fgs_internal.h"

namespace fgs {
namespace {


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

// One Gaussian applied to this lane's 2x2 pixel quad (render.cu:40-52 for each pixel).  The
// exponent q(dx, dy) = w + cx dx^2 + cz dy^2 + cy dx dy is evaluated once, at the quad's first
// pixel, and stepped to its neighbours with the exact differences of the quadratic
// (q(dx-1, dy) - q(dx, dy) = cx - 2 cx dx - cy dy, and likewise in y; the mixed step adds cy).
// dx, dy are offsets from the Gaussian's own centre, so every term has the magnitude of the
// exponent itself and the stepping loses nothing that matters against the 2e-3 image tolerance.
struct Quad {
    float T[2][2], r[2][2], g[2][2], b[2][2];
};

__device__ __forceinline__ void shade_quad(Quad& q, float px0, float py0, const float4 a, const float4 b4, const float blue)
{
    // a = (centre x, centre y, conic x, conic y), b4 = (conic z, log2 opacity, red, green)
    const float dx = a.x - px0, dy = a.y - py0;
    const float tx = a.z * dx, ty = b4.x * dy, txy = a.w * dx;
    float pw[2][2];
    pw[0][0] = b4.y + tx * dx + ty * dy + txy * dy;
    const float step_x = (a.z - 2.0f * tx) - a.w * dy;          // to the pixel at x + 1
    const float step_y = (b4.x - 2.0f * ty) - txy;             // to the pixel at y + 1
    pw[0][1] = pw[0][0] + step_x;
    pw[1][0] = pw[0][0] + step_y;
    pw[1][1] = (pw[0][1] + step_y) + a.w;
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const float alpha = __builtin_amdgcn_exp2f(pw[j][i]);
            const float at = alpha * q.T[j][i];
            q.r[j][i] += b4.z * at;
            q.g[j][i] += b4.w * at;
            q.b[j][i] += blue * at;
            q.T[j][i] -= at;
        }
}

template <int SX, int SY>
__global__ __launch_bounds__(kWave) void blend_kernel(
    const int2* __restrict__ ranges,
    const uint32_t* __restrict__ point_list,
    int width, int height, int tiles_x, int tiles_y,
    const float2* __restrict__ points_xy,
    const float4* __restrict__ rgb_depth,
    const float4* __restrict__ conic_opacity,
    float bg_r, float bg_g, float bg_b,
    uint8_t* __restrict__ out_u8,
    float* __restrict__ out_f32)
{
    constexpr int kSub = SX * SY;              // 16x16 sub-tiles per tile = quads per lane
    __shared__ float4 s_a[kWave];              // centre x, centre y, conic x, conic y
    __shared__ float4 s_b[kWave];              // conic z, log2 opacity, red, green
    __shared__ float s_c[kWave];               // blue

    const int lane = threadIdx.x;
    // Workgroup -> tile.  The hardware deals consecutive workgroups out to the 8 XCDs in turn, and
    // every XCD has its own L2.  Neighbouring tiles share most of their Gaussians, so each XCD is
    // given whole 8x8 blocks of tiles (its workgroups g = 8*slot + xcd walk blocks xcd, xcd+8, ...
    // 64 tiles at a time): a Gaussian's attribute lines are then fetched into one L2 once instead
    // of into several L2s once per tile.
    const int group = blockIdx.x;
    const int xcd = group & 7, slot = group >> 3;
    const int blocks_x = (tiles_x + 7) >> 3;
    const int block = (slot >> 6) * 8 + xcd, inner = slot & 63;
    const int tile_x = (block % blocks_x) * 8 + (inner & 7);
    const int tile_y = (block / blocks_x) * 8 + (inner >> 3);
    if (tile_x >= tiles_x || tile_y >= tiles_y) return;
    const int2 range = ranges[tile_y * tiles_x + tile_x];
    const int n = range.y - range.x;

    // lane -> 2x2 quad of every 16x16 sub-tile
    const int qx = (lane & 7) * 2, qy = (lane >> 3) * 2;
    int pix_x[kSub], pix_y[kSub];
    float pxf[kSub], pyf[kSub];
    Quad quad[kSub];
#pragma unroll
    for (int s = 0; s < kSub; s++) {
        pix_x[s] = tile_x * (16 * SX) + (s % SX) * 16 + qx;
        pix_y[s] = tile_y * (16 * SY) + (s / SX) * 16 + qy;
        pxf[s] = (float)pix_x[s];
        pyf[s] = (float)pix_y[s];
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                quad[s].T[j][i] = 1.0f;
                quad[s].r[j][i] = 0.0f; quad[s].g[j][i] = 0.0f; quad[s].b[j][i] = 0.0f;
            }
    }

    // registers hold the batch that is staged next; loads for it overlap the shading of the current one
    float2 nxy = make_float2(0.f, 0.f);
    float4 nco = make_float4(0.f, 0.f, 0.f, 0.f), nrgb = make_float4(0.f, 0.f, 0.f, 0.f);
    if (lane < n) {
        const uint32_t g = point_list[range.x + lane];
        nxy = points_xy[g]; nco = conic_opacity[g]; nrgb = rgb_depth[g];
    }

    bool done = false;
    for (int base = 0; base < n && !done; base += kWave) {
        const int cnt = min(kWave, n - base);
        __builtin_amdgcn_wave_barrier();
        s_a[lane] = make_float4(nxy.x, nxy.y, nco.x, nco.y);
        s_b[lane] = make_float4(nco.z, nco.w, nrgb.x, nrgb.y);
        s_c[lane] = nrgb.z;
        __builtin_amdgcn_wave_barrier();
        if (base + kWave + lane < n) {
            const uint32_t g = point_list[range.x + base + kWave + lane];
            nxy = points_xy[g]; nco = conic_opacity[g]; nrgb = rgb_depth[g];
        }
        // Gaussians go in pairs; the tile-wide stop is tested after each pair (render.cu:394-408)
        for (int j = 0; j < cnt; j += 2) {
            {
                const float4 a = s_a[j], b4 = s_b[j];
                const float blue = s_c[j];
#pragma unroll
                for (int s = 0; s < kSub; s++) shade_quad(quad[s], pxf[s], pyf[s], a, b4, blue);
            }
            if (j + 1 >= cnt) break;            // odd tail (render.cu:486-487)
            {
                const float4 a = s_a[j + 1], b4 = s_b[j + 1];
                const float blue = s_c[j + 1];
#pragma unroll
                for (int s = 0; s < kSub; s++) shade_quad(quad[s], pxf[s], pyf[s], a, b4, blue);
            }
            float tmax = 0.0f;
#pragma unroll
            for (int s = 0; s < kSub; s++)
                tmax = fmaxf(tmax, fmaxf(fmaxf(quad[s].T[0][0], quad[s].T[0][1]), fmaxf(quad[s].T[1][0], quad[s].T[1][1])));
            if (ballot(!(tmax < 0.0001f)) == 0) { done = true; break; }
        }
    }

    // render.cu:59-73
#pragma unroll
    for (int s = 0; s < kSub; s++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int x = pix_x[s] + i, y = pix_y[s] + j;
                if (x < width && y < height) {
                    const size_t pid = (size_t)width * y + x;
                    float t = quad[s].T[j][i];
                    if (t < 0.0001f) t = 0.0f;
                    const float r = quad[s].r[j][i] + t * bg_r, g = quad[s].g[j][i] + t * bg_g, b = quad[s].b[j][i] + t * bg_b;
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
    // one workgroup per tile of the image padded to whole 8x8 blocks of tiles, blocks padded to a multiple of 8
    const long long blocks = (long long)((tiles_x + 7) / 8) * ((tiles_y + 7) / 8);
    const long long groups = (blocks + 7) / 8 * 8 * 64;
    if (groups > 0x7fffffffLL) return fail(FGS_E_INVALID, "%s: image too large", who);
    const dim3 grid((unsigned)groups);
#define FGS_LAUNCH_BLEND(SX, SY)                                                                        \
    hipLaunchKernelGGL((blend_kernel<SX, SY>), grid, dim3(kWave), 0, st,                                \
                       (const int2*)ranges, values_sorted, width, height, tiles_x, tiles_y,             \
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
