// Tile ranges and front-to-back alpha blending for gfx950 (wave64).
//
// Replaces FlashGS render<BX,BY> (csrc/cuda_rasterizer/render.cu:549-576): zero the ranges,
// identifyTileRanges (:9-31) and renderCUDA (:199-547).
//
// Blend layout: one wave64 owns one tile.  A tile is made of 16x16-pixel sub-tiles (1 for 16x16,
// 2 for 32x16, 4 for 32x32); lane l shades the 2x2 pixel quad at (2*(l%8), 2*(l/8)) of every
// sub-tile.  Gaussians are staged 32 at a time: the staging lanes tabulate the two one-dimensional
// parts of the exponent over the tile's columns and rows in LDS, while the loads of the following
// batch are already in flight; the wave then walks the batch, every lane reading the table
// entries of its own columns and rows.  After every second Gaussian one ballot tests whether all
// pixels of the tile have T < 1e-4, which is the reference's stop rule (render.cu:394-408).  A
// workgroup is a single wave, so no workgroup barrier is needed anywhere.
#include "fgs_internal.h"

namespace fgs {
namespace {


__global__ __launch_bounds__(256) void fill_i32_kernel(int* p, size_t n, int v)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

// render.cu:9-31, with the tile index checked against the number of tiles.  A thread looks at
// kRangesPerThread pairs, 256 apart so that the loads of a workgroup stay contiguous.
constexpr int kRangesPerThread = 8;

__global__ __launch_bounds__(256) void tile_ranges_kernel(int L, const uint64_t* __restrict__ keys,
                                                          int2* __restrict__ ranges, uint32_t num_tiles)
{
    const long long base = (long long)blockIdx.x * (256 * kRangesPerThread) + threadIdx.x;
    uint32_t cur[kRangesPerThread], prev[kRangesPerThread];
#pragma unroll
    for (int k = 0; k < kRangesPerThread; k++) {
        const long long idx = base + k * 256;
        cur[k] = 0; prev[k] = 0;
        if (idx < L) {
            cur[k] = (uint32_t)(keys[idx] >> 32);
            if (idx > 0) prev[k] = (uint32_t)(keys[idx - 1] >> 32);
        }
    }
#pragma unroll
    for (int k = 0; k < kRangesPerThread; k++) {
        const long long idx = base + k * 256;
        if (idx >= L) break;
        if (cur[k] >= num_tiles) continue;
        if (idx == 0) {
            ranges[cur[k]].x = 0;
        } else if (cur[k] != prev[k]) {
            if (prev[k] < num_tiles) ranges[prev[k]].y = (int)idx;
            ranges[cur[k]].x = (int)idx;
        }
        if (idx == L - 1) ranges[cur[k]].y = L;
    }
}

// render.cu:54-57
__device__ __forceinline__ uint8_t encode_u8(float x)
{
    float v = x * 255.0f;
    v = v > 0.0f ? v : 0.0f;       // also maps NaN to 0
    v = v < 255.0f ? v : 255.0f;
    return (uint8_t)v;
}

// The exponent of a Gaussian at a pixel, q = w + cx dx^2 + cz dy^2 + cy dx dy with (dx, dy) the
// offset of the pixel from the Gaussian's centre (render.cu:42-45), is split over the tile's own
// pixel grid.  With (X, Y) the pixel's integer offset from the tile centre and (ex, ey) the
// Gaussian centre's offset from the tile centre, dx = ex - X, dy = ey - Y and
//     q = F(X) + G(Y) + cy X Y,
//     F(X) = (w - cy ex ey) + dx (cx dx + cy ey),      G(Y) = dy (cz dy + cy ex).
// F and G depend on one coordinate only: for every staged Gaussian they are tabulated once per
// tile column and row (kFx + kGy values) by the staging lanes, and a lane gets the exponents of
// its 2x2 quad from two table reads, four additions and four FMAs with its own constants X*Y.
// All terms are of the magnitude of the exponent itself or of cy*|X|*|Y| with |X|, |Y| <= 16, so
// nothing is lost against the 2e-3 image tolerance.
struct Quad {
    float T[2][2], r[2][2], g[2][2], b[2][2];
};

constexpr int kBatch = 32;        // Gaussians staged per round: lanes 0-31 tabulate F, lanes 32-63 G

// A read that stays where it is written: the compiler neither sinks it to its first use nor drops
// it when the value turns out unused (volatile on the vector type keeps it one wide LDS read).
template <typename V>
__device__ __forceinline__ V lds_read(const char* p)
{
    typedef float Native __attribute__((ext_vector_type(sizeof(V) / sizeof(float))));
    const Native n = *(const volatile __attribute__((address_space(3))) Native*)p;
    V v;
    __builtin_memcpy(&v, &n, sizeof(V));
    return v;
}

// what a lane reads of one staged Gaussian: (cy, red, green, blue), F at its columns, G at its rows
template <int SX, int SY>
struct StagedT {
    float4 u;
    float2 f[SX], g[SY];
};

__device__ __forceinline__ void shade_quad(Quad& q, const float xy[2][2], const float2 f, const float2 g, const float4 u)
{
    // u = (cy, red, green, blue)
    const float fx[2] = {f.x, f.y}, gy[2] = {g.x, g.y};
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const float alpha = __builtin_amdgcn_exp2f(__builtin_fmaf(u.x, xy[j][i], fx[i] + gy[j]));
            const float at = alpha * q.T[j][i];
            q.r[j][i] += u.y * at;
            q.g[j][i] += u.z * at;
            q.b[j][i] += u.w * at;
            q.T[j][i] -= at;
        }
}

template <int SX, int SY>
__device__ __forceinline__ void blend_tile(
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
    using Staged = StagedT<SX, SY>;
    constexpr int kSub = SX * SY;              // 16x16 sub-tiles per tile = quads per lane
    constexpr int kFx = 16 * SX, kGy = 16 * SY;
    constexpr int kTab = kFx > kGy ? kFx : kGy;
    constexpr int kRec = kFx + kGy + 4;        // floats per staged Gaussian: F table, G table, (cy, r, g, b)
    __shared__ __align__(16) float s_rec[kBatch * kRec];

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
    // A launch ends when its longest list ends, and a wave that shares its SIMD equally with the
    // waves of short lists gets to its own end late: waves with long lists ask for a higher
    // issue priority.
    if (n > 1024) __builtin_amdgcn_s_setprio(3);
    else if (n > 512) __builtin_amdgcn_s_setprio(2);
    else if (n > 256) __builtin_amdgcn_s_setprio(1);

    // lane -> 2x2 quad of every 16x16 sub-tile
    const int qx = (lane & 7) * 2, qy = (lane >> 3) * 2;
    const float centre_x = (float)(tile_x * kFx + kFx / 2), centre_y = (float)(tile_y * kGy + kGy / 2);
    int pix_x[kSub], pix_y[kSub];
    float xy[kSub][2][2];                      // X*Y of the quad's pixels, offsets from the tile centre
    Quad quad[kSub];
#pragma unroll
    for (int s = 0; s < kSub; s++) {
        const int lx = (s % SX) * 16 + qx, ly = (s / SX) * 16 + qy;
        pix_x[s] = tile_x * kFx + lx;
        pix_y[s] = tile_y * kGy + ly;
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                xy[s][j][i] = (float)((lx + i - kFx / 2) * (ly + j - kGy / 2));
                quad[s].T[j][i] = 1.0f;
                quad[s].r[j][i] = 0.0f; quad[s].g[j][i] = 0.0f; quad[s].b[j][i] = 0.0f;
            }
    }

    // Byte offsets into a staged record.  They are held in vector registers (the empty asm hides
    // what the compiler could know about them) so that every LDS read of the unrolled batch is
    // "register + immediate": no address arithmetic in the loop.
    const char* const rec_bytes = reinterpret_cast<const char*>(s_rec);
    uint32_t off_f = 4u * (uint32_t)qx, off_g = 4u * (uint32_t)(kFx + qy), off_u = 4u * (uint32_t)(kFx + kGy);
    asm volatile("" : "+v"(off_f), "+v"(off_g), "+v"(off_u));

    // Staging role of this lane: Gaussian lane%32 of the batch; lanes 0-31 tabulate F, 32-63 G.
    const int stage_slot = lane & (kBatch - 1);
    const bool stage_g = lane >= kBatch;
    float* const stage_tab = s_rec + stage_slot * kRec + (stage_g ? kFx : 0);
    const int stage_len = stage_g ? kGy : kFx;

    // registers hold the batch that is staged next; loads for it overlap the shading of the current one
    float2 nxy = make_float2(0.f, 0.f);
    float4 nco = make_float4(0.f, 0.f, 0.f, 0.f), nrgb = make_float4(0.f, 0.f, 0.f, 0.f);
    // The list index is fetched two batches ahead and the attributes one batch ahead, so that no
    // wave waits for an index only to start the loads that depend on it.  Positions past the end
    // of the list are clamped to its last entry: those loads are valid and their result unused.
    uint32_t g_ahead = 0;
    if (n > 0) {
        const uint32_t g = point_list[min(range.x + stage_slot, range.y - 1)];
        g_ahead = point_list[min(range.x + kBatch + stage_slot, range.y - 1)];
        nxy = points_xy[g]; nco = conic_opacity[g]; nrgb = rgb_depth[g];
    }

    bool done = false;
    for (int base = 0; base < n && !done; base += kBatch) {
        const int cnt = min(kBatch, n - base);
        __builtin_amdgcn_wave_barrier();
        {
            // conic_opacity = (cx, cy, cz, w) in the units of the exponent (see fgs_preprocess).
            // With e the centre's offset from the first column (row) of the tile, the entry for
            // column k is con + d (curv d + lin) at d = e - k, evaluated as a polynomial in k.
            const float ex = nxy.x - centre_x, ey = nxy.y - centre_y;
            const float e = stage_g ? ey + (float)(kGy / 2) : ex + (float)(kFx / 2);
            const float curv = stage_g ? nco.z : nco.x;
            const float lin = nco.y * (stage_g ? ex : ey);
            const float con = stage_g ? 0.0f : nco.w - (nco.y * ex) * ey;
            const float c0 = con + e * (curv * e + lin);
            const float c1 = -(2.0f * curv * e + lin);
#pragma unroll
            for (int k = 0; k < kTab; k += 4) {
                float4 t;
                float* tv = &t.x;
#pragma unroll
                for (int c = 0; c < 4; c++) tv[c] = c0 + (float)(k + c) * (c1 + curv * (float)(k + c));
                if (k < stage_len) *reinterpret_cast<float4*>(stage_tab + k) = t;
            }
            if (stage_g) *reinterpret_cast<float4*>(s_rec + stage_slot * kRec + kFx + kGy) =
                make_float4(nco.y, nrgb.x, nrgb.y, nrgb.z);
        }
        __builtin_amdgcn_wave_barrier();
        nxy = points_xy[g_ahead]; nco = conic_opacity[g_ahead]; nrgb = rgb_depth[g_ahead];
        g_ahead = point_list[min(range.x + base + 2 * kBatch + stage_slot, range.y - 1)];
        // Gaussians go in pairs; the tile-wide stop is tested after each pair (render.cu:394-408)
        // The table reads of a Gaussian are issued before the Gaussian ahead of it is shaded, so
        // that a wave does not sit out the LDS latency once per Gaussian.
        auto fetch = [&](int j) {
            const int rec = j * kRec * 4;
            Staged r;
            r.u = lds_read<float4>(rec_bytes + off_u + rec);
#pragma unroll
            for (int c = 0; c < SX; c++) r.f[c] = lds_read<float2>(rec_bytes + off_f + rec + c * 64);
#pragma unroll
            for (int c = 0; c < SY; c++) r.g[c] = lds_read<float2>(rec_bytes + off_g + rec + c * 64);
            return r;
        };
        auto shade = [&](const Staged& r) {
#pragma unroll
            for (int s = 0; s < kSub; s++) shade_quad(quad[s], xy[s], r.f[s % SX], r.g[s / SX], r.u);
        };
        auto all_stopped = [&]() {
            bool live = false;                      // some pixel of this lane still has T >= 1e-4
#pragma unroll
            for (int s = 0; s < kSub; s++) {
                float m;
                asm("v_max3_f32 %0, %1, %2, %3" : "=v"(m) : "v"(quad[s].T[0][0]), "v"(quad[s].T[0][1]), "v"(quad[s].T[1][0]));
                live = live || !(m < 0.0001f) || !(quad[s].T[1][1] < 0.0001f);
            }
            return ballot(live) == 0;
        };
        // written out for the whole batch so that every record offset is an immediate
#define FGS_PAIR(J)                                                                   \
        if ((J) >= cnt) break;                                                        \
        second = fetch((J) + 1);                                                      \
        shade(first);                                                                 \
        if ((J) + 1 >= cnt) break;              /* odd tail (render.cu:486-487) */    \
        first = fetch(((J) + 2) % kBatch);      /* past the batch: read and dropped */\
        shade(second);                                                                \
        if (all_stopped()) { done = true; break; }
        static_assert(kBatch == 32, "the pairs below cover a batch of 32");
        Staged first = fetch(0), second;
        do {
            FGS_PAIR(0) FGS_PAIR(2) FGS_PAIR(4) FGS_PAIR(6) FGS_PAIR(8) FGS_PAIR(10) FGS_PAIR(12) FGS_PAIR(14)
            FGS_PAIR(16) FGS_PAIR(18) FGS_PAIR(20) FGS_PAIR(22) FGS_PAIR(24) FGS_PAIR(26) FGS_PAIR(28) FGS_PAIR(30)
        } while (0);
#undef FGS_PAIR
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

#define FGS_BLEND_PARAMS                                                                         \
    const int2* __restrict__ ranges, const uint32_t* __restrict__ point_list,                   \
    int width, int height, int tiles_x, int tiles_y,                                            \
    const float2* __restrict__ points_xy, const float4* __restrict__ rgb_depth,                 \
    const float4* __restrict__ conic_opacity, float bg_r, float bg_g, float bg_b,               \
    uint8_t* __restrict__ out_u8, float* __restrict__ out_f32
#define FGS_BLEND_ARGS                                                                           \
    ranges, point_list, width, height, tiles_x, tiles_y, points_xy, rgb_depth, conic_opacity,   \
    bg_r, bg_g, bg_b, out_u8, out_f32

template <int SX, int SY>
__global__ __launch_bounds__(kWave) void blend_kernel(FGS_BLEND_PARAMS)
{
    blend_tile<SX, SY>(FGS_BLEND_ARGS);
}

// The same kernel held to 4 resident waves per SIMD (16 per CU).  Every resident wave walks its
// own tile's list and the lists of the tiles in flight compete for the 4 MB L2 of their XCD: when
// there are more tiles than the chip holds at once, fewer resident waves mean fewer misses
// (measured on a 4K frame: -35 % fetched bytes and -8 % time against 8 waves per SIMD).
template <int SX, int SY>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(4, 4))) void blend_kernel_few_waves(FGS_BLEND_PARAMS)
{
    blend_tile<SX, SY>(FGS_BLEND_ARGS);
}
#undef FGS_BLEND_PARAMS
#undef FGS_BLEND_ARGS

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
        hipLaunchKernelGGL(tile_ranges_kernel,
                           dim3((unsigned)(((size_t)num_rendered + 256 * kRangesPerThread - 1) / (256 * kRangesPerThread))),
                           dim3(256), 0, st,
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
    // more tiles than the chip holds at 8 waves per SIMD: run the variant with fewer resident waves
    int dev = 0, cus = 0;
    FGS_HIP_TRY(hipGetDevice(&dev));
    FGS_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const bool few_waves = (long long)tiles_x * tiles_y > 32LL * cus;
#define FGS_LAUNCH_BLEND(SX, SY)                                                                        \
    do {                                                                                                \
        auto kernel = few_waves ? blend_kernel_few_waves<SX, SY> : blend_kernel<SX, SY>;                \
        hipLaunchKernelGGL(kernel, grid, dim3(kWave), 0, st,                                            \
                           (const int2*)ranges, values_sorted, width, height, tiles_x, tiles_y,         \
                           (const float2*)points_xy, (const float4*)rgb_depth, (const float4*)conic_opacity, \
                           bg[0], bg[1], bg[2], out_u8, out_f32);                                       \
    } while (0)
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
