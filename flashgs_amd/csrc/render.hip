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
// workgroup is a single wave, so no workgroup barrier is needed anywhere.  Every kernel exists in
// two forms: all fp32, operation for operation the reference's pixel shader (the default), and
// with the colour sums on the matrix unit four Gaussians at a time (f16 operands, fp32
// accumulation), which a caller asks for per call (FGS_BLEND_MATRIX_F16) or per process
// (fgs_set_colour_sums).
#include "fgs_internal.h"

#include <atomic>
#include <map>
#include <mutex>
#include <utility>

namespace fgs {
namespace {


__global__ __launch_bounds__(256) void fill_i32_kernel(int* p, size_t n, int v)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}


// Tiles of a small frame ranked by the length of their lists, longest first (in steps of 16;
// the order inside a step is whatever the atomics make it).  One workgroup.
// (Ranking in the last workgroup of tile_ranges_kernel instead costs more than this launch: every
// workgroup then has to push its ranges out of its XCD's L2 before it counts itself done.)
constexpr int kOrderCap = 8192;            // tiles
constexpr int kOrderBins = 128;            // everything from 2032 entries up shares the first bin
// The ranking is written by one launch and read by the next, so it needs memory of its own: one
// table per (device, stream), allocated on the first such blend on that stream (blends on one
// stream follow each other; blends on different streams may overlap and get a table each).  A
// stream that is being captured and has no table yet cannot allocate one and uses this
// per-device table instead, which captured blends on one device then share.
__device__ uint32_t g_tile_order[kOrderCap];
std::map<StreamKey, uint32_t*> g_order_tables;
std::mutex g_order_mutex;

int tile_order_table(hipStream_t stream, uint32_t** out)
{
    int device = 0;
    FGS_HIP_TRY(hipGetDevice(&device));
    std::lock_guard<std::mutex> lock(g_order_mutex);
    uint32_t*& table = g_order_tables[stream_key(device, stream)];
    if (!table) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        if (stream) FGS_HIP_TRY(hipStreamIsCapturing(stream, &capture));
        if (capture != hipStreamCaptureStatusNone) {
            void* shared = nullptr;
            FGS_HIP_TRY(hipGetSymbolAddress(&shared, HIP_SYMBOL(g_tile_order)));
            *out = (uint32_t*)shared;
            return FGS_OK;
        }
        if (hipMalloc((void**)&table, kOrderCap * sizeof(uint32_t)) != hipSuccess) {
            (void)hipGetLastError();
            table = nullptr;
            return fail(FGS_E_NOMEM, "cannot allocate the table of tile ranks");
        }
    }
    *out = table;
    return FGS_OK;
}

__global__ __launch_bounds__(1024) void tile_order_kernel(const int2* __restrict__ ranges, int num_tiles,
                                                          uint32_t* __restrict__ tile_order)
{
    constexpr int kPerThread = kOrderCap / 1024;
    __shared__ uint32_t s_count[kOrderBins];
    const int tid = threadIdx.x;
    if (tid < kOrderBins) s_count[tid] = 0;
    __syncthreads();
    uint32_t bin[kPerThread], slot[kPerThread];
#pragma unroll
    for (int k = 0; k < kPerThread; k++) {
        const int t = tid + k * 1024;
        bin[k] = 0; slot[k] = 0;
        if (t < num_tiles) {
            const int2 r = ranges[t];
            bin[k] = (uint32_t)(kOrderBins - 1 - max(0, min((r.y - r.x) >> 4, kOrderBins - 1)));
            slot[k] = atomicAdd(&s_count[bin[k]], 1u);
        }
    }
    __syncthreads();
    if (tid < kWave) {
        // exclusive prefix over the bins, two per lane
        const uint32_t a = s_count[2 * tid], b = s_count[2 * tid + 1];
        uint32_t incl = a + b;
#pragma unroll
        for (int o = 1; o < kWave; o <<= 1) {
            const uint32_t up = (uint32_t)__shfl_up((int)incl, o);
            if (tid >= o) incl += up;
        }
        const uint32_t excl = incl - (a + b);
        s_count[2 * tid] = excl;
        s_count[2 * tid + 1] = excl + a;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kPerThread; k++) {
        const int t = tid + k * 1024;
        if (t < num_tiles) tile_order[s_count[bin[k]] + slot[k]] = (uint32_t)t;
    }
}

// render.cu:9-31, with the tile index checked against the number of tiles.  A thread looks at
// kRangesPerThread pairs, 256 apart so that the loads of a workgroup stay contiguous.
// Also writes (0, 0) for the tiles without pairs (the reference clears the whole table first,
// render.cu:557): the pair that opens tile c clears the tiles between its predecessor's tile and
// c, the first pair those before it and the last pair those behind it.  A run of up to 4 tiles is
// cleared by the thread that found it, a longer one by its whole wave.
constexpr int kRangesPerThread = 4;

__global__ __launch_bounds__(256) void tile_ranges_kernel(int L, const uint64_t* __restrict__ keys,
                                                          int2* __restrict__ ranges, uint32_t num_tiles)
{
    const long long base = (long long)blockIdx.x * (256 * kRangesPerThread) + threadIdx.x;
    const int lane = threadIdx.x & (kWave - 1);
    uint32_t cur[kRangesPerThread], prev[kRangesPerThread];
#pragma unroll
    for (int k = 0; k < kRangesPerThread; k++) {
        const long long idx = base + k * 256;
        cur[k] = 0; prev[k] = 0;
        if (idx < L) {
            cur[k] = min((uint32_t)(keys[idx] >> 32), num_tiles);           // num_tiles: outside the image
            if (idx > 0) prev[k] = min((uint32_t)(keys[idx - 1] >> 32), num_tiles);
        }
    }
    auto clear_by_wave = [&](bool mine, uint32_t lo, uint32_t hi) {         // tiles [lo, hi)
        for (uint64_t todo = ballot(mine); todo; todo &= todo - 1) {
            const int src = __ffsll((long long)todo) - 1;
            const uint32_t from = (uint32_t)__shfl((int)lo, src), to = (uint32_t)__shfl((int)hi, src);
            for (uint32_t t = from + (uint32_t)lane; t < to; t += kWave) ranges[t] = make_int2(0, 0);
        }
    };
#pragma unroll
    for (int k = 0; k < kRangesPerThread; k++) {
        const long long idx = base + k * 256;
        const bool valid = idx < L;
        const bool opens = valid && (idx == 0 || cur[k] != prev[k]);
        if (opens) {
            if (idx > 0 && prev[k] < num_tiles) ranges[prev[k]].y = (int)idx;
            if (cur[k] < num_tiles) ranges[cur[k]].x = (int)idx;
        }
        if (valid && idx == L - 1 && cur[k] < num_tiles) ranges[cur[k]].y = L;
        // empty tiles in front of this pair's tile
        const uint32_t lo = idx == 0 ? 0u : min(prev[k] + 1u, num_tiles);
        const bool gap = opens && lo < cur[k];
        const bool wide = gap && cur[k] - lo > 4u;
        if (gap && !wide)
            for (uint32_t t = lo; t < cur[k]; t++) ranges[t] = make_int2(0, 0);
        clear_by_wave(wide, lo, cur[k]);
        clear_by_wave(valid && idx == L - 1 && cur[k] + 1u < num_tiles, cur[k] + 1u, num_tiles);
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
constexpr int kGroups = kBatch / 4;

// The colour sums C += (alpha T) c are a matrix product, pixels x Gaussians times Gaussians x
// channels, and go through v_mfma_f32_4x4x4_16b_f16: sixteen independent 4x4 products with an
// inner dimension of 4.  A block is four neighbouring lanes; row i of its A operand is lane i's
// pixel, its four f16 values that pixel's weights alpha T for four Gaussians; column j of B is
// channel j of those Gaussians' colours (the same in every block; column 3 is zero); lane j of the
// block accumulates, in fp32, channel j of the four lanes' pixels in its four result registers.
// A lane shades four pixels per sub-tile, so four Gaussians cost it four such instructions where
// the plain form costs 48 multiply-adds.  Weights and colours are rounded to f16 (to nearest),
// products and sums are fp32: the colour of a pixel differs from the all-fp32 sum by at most
// 2^-10 of itself.  The weights are scaled by 2^14 (added to the exponent when it is tabulated,
// taken out again with the result), which keeps them in f16's normal range down to 4e-9.
// T itself never leaves fp32.  This form is opt-in (FGS_BLEND_MATRIX_F16); walk_list_fp32 is the default.
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
constexpr float kWeightScaleLog2 = 14.0f;
constexpr float kWeightUnscale = 6.103515625e-05f;          // 2^-14
constexpr float kColourMax = 65504.0f;                      // largest f16: a colour beyond it is drawn as this

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

// A store to LDS that stays where it is written.
__device__ __forceinline__ void lds_write(char* p, float v)
{
    *(volatile __attribute__((address_space(3))) float*)p = v;
}

// what a lane reads of one staged Gaussian: F at its columns, G at its rows
template <int SX, int SY>
struct StagedT {
    float2 f[SX], g[SY];
};
// ... and of a group of four: their cy, and this lane's channel of their colours as four f16
struct StagedGroup {
    float4 cy;
    float2 colour;
};

// One Gaussian on one quad: the weights alpha T (scaled) of its four pixels, T updated.
__device__ __forceinline__ void shade_quad(Quad& q, const float xy[2][2], const float2 f, const float2 g, const float cy, float (&w)[4])
{
    const float fx[2] = {f.x, f.y}, gy[2] = {g.x, g.y};
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const float alpha = __builtin_amdgcn_exp2f(__builtin_fmaf(cy, xy[j][i], fx[i] + gy[j]));
            const float at = alpha * q.T[j][i];
            q.T[j][i] = __builtin_fmaf(at, -kWeightUnscale, q.T[j][i]);
            w[2 * j + i] = at;
        }
}

// The all-fp32 form (render.cu:40-52 operation for operation): colour sums by multiply-add.
__device__ __forceinline__ void shade_quad_fp32(Quad& q, const float xy[2][2], const float2 f, const float2 g, const float cy,
                                                const float4 rgb)
{
    const float fx[2] = {f.x, f.y}, gy[2] = {g.x, g.y};
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const float alpha = __builtin_amdgcn_exp2f(__builtin_fmaf(cy, xy[j][i], fx[i] + gy[j]));
            const float at = alpha * q.T[j][i];
            q.r[j][i] += rgb.x * at;
            q.g[j][i] += rgb.y * at;
            q.b[j][i] += rgb.z * at;
            q.T[j][i] -= at;
        }
}

__device__ __forceinline__ uint32_t pack_f16(float a, float b)
{
    const float2_t v = {a, b};
    const half2_t h = __builtin_convertvector(v, half2_t);       // v_cvt_pk_f16_f32, round to nearest
    return __builtin_bit_cast(uint32_t, h);
}

// Lane-constant part of the walk: where this lane reads the staged records, what it stages.
template <int SX, int SY>
struct LaneRole {
    static constexpr int kFx = 16 * SX, kGy = 16 * SY;
    static constexpr int kRec = kFx + kGy + 4;  // floats per staged Gaussian: F table, G table; padded so that the
                                                // staging lanes, one record apart, write to different LDS banks
    static constexpr int kGroupRec = 12;        // floats per group of four: cy x 4, 4 channels x 4 f16
    static constexpr int kStage = kBatch * kRec + kGroups * kGroupRec;      // floats of a wave's staging area
    uint32_t off_f, off_g, off_cy, off_colour;  // byte offsets into the staging area
    int stage_slot;                             // Gaussian lane%32 of the batch
    bool stage_g;                               // lanes 0-31 tabulate F, 32-63 G
    float xy[SX * SY][2][2];                    // X*Y of the quad's pixels, offsets from the tile centre

    __device__ __forceinline__ void init(int lane)
    {
        // lane -> 2x2 quad of every 16x16 sub-tile
        const int qx = (lane & 7) * 2, qy = (lane >> 3) * 2;
#pragma unroll
        for (int s = 0; s < SX * SY; s++) {
            const int lx = (s % SX) * 16 + qx, ly = (s / SX) * 16 + qy;
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int i = 0; i < 2; i++) xy[s][j][i] = (float)((lx + i - kFx / 2) * (ly + j - kGy / 2));
        }
        // The offsets are held in vector registers (the empty asm hides what the compiler could
        // know about them) so that every LDS read of the unrolled batch is "register +
        // immediate": no address arithmetic in the loop.
        off_f = 4u * (uint32_t)qx; off_g = 4u * (uint32_t)(kFx + qy);
        off_cy = 4u * (uint32_t)(kBatch * kRec); off_colour = off_cy + 16u + 8u * (uint32_t)(lane & 3);
        asm volatile("" : "+v"(off_f), "+v"(off_g), "+v"(off_cy), "+v"(off_colour));
        stage_slot = lane & (kBatch - 1);
        stage_g = lane >= kBatch;
    }
};

__device__ __forceinline__ void clear_quad(Quad& q)
{
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 2; i++) {
            q.T[j][i] = 1.0f;
            q.r[j][i] = 0.0f; q.g[j][i] = 0.0f; q.b[j][i] = 0.0f;
        }
}

// One wave blends entries [begin, begin + n) of the sorted list into the quads of the tile whose
// centre is given, front to back, starting from T = 1 and no colour; begin must be an even
// distance from the start of the tile's list, so that the pairs are the reference's pairs.
// Returns true when the walk ended at the tile-wide stop.  s_rec is this wave's staging area of
// LaneRole::kStage floats.
template <int SX, int SY>
__device__ __forceinline__ bool walk_list(
    const LaneRole<SX, SY>& role, float* s_rec,
    const uint32_t* __restrict__ point_list, int begin, int n,
    float centre_x, float centre_y,
    const float2* __restrict__ points_xy,
    const float4* __restrict__ rgb_depth,
    const float4* __restrict__ conic_opacity,
    Quad (&quad)[SX * SY])
{
    using Staged = StagedT<SX, SY>;
    using Role = LaneRole<SX, SY>;
    constexpr int kSub = SX * SY;
    constexpr int kFx = 16 * SX, kGy = 16 * SY;
    constexpr int kTab = kFx > kGy ? kFx : kGy;
    constexpr int kRec = Role::kRec, kGroupRec = Role::kGroupRec;
    const char* const rec_bytes = reinterpret_cast<const char*>(s_rec);
    const uint32_t off_f = role.off_f, off_g = role.off_g, off_cy = role.off_cy, off_colour = role.off_colour;
    const int stage_slot = role.stage_slot;
    const bool stage_g = role.stage_g;
    float* const stage_tab = s_rec + stage_slot * kRec + (stage_g ? kFx : 0);
    float* const stage_group = s_rec + kBatch * kRec + (stage_slot >> 2) * kGroupRec;
    const int stage_len = stage_g ? kGy : kFx;
    const int last = begin + n - 1;

#pragma unroll
    for (int s = 0; s < kSub; s++) clear_quad(quad[s]);
    float4_t acc[kSub][4];                  // colour sums in the layout of the matrix instruction
#pragma unroll
    for (int s = 0; s < kSub; s++)
#pragma unroll
        for (int p = 0; p < 4; p++) acc[s][p] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // registers hold the batch that is staged next; loads for it overlap the shading of the current one
    float2 nxy = make_float2(0.f, 0.f);
    float4 nco = make_float4(0.f, 0.f, 0.f, 0.f), nrgb = make_float4(0.f, 0.f, 0.f, 0.f);
    // The list index is fetched two batches ahead and the attributes one batch ahead, so that no
    // wave waits for an index only to start the loads that depend on it.  Positions past the end
    // of the list are clamped to its last entry: those loads are valid and their result unused.
    // (Attributes two batches ahead and indices four, in two alternating sets of registers, change
    // nothing: 4K frame 0.312 ms either way.)
    uint32_t g_ahead = 0;
    if (n > 0) {
        const uint32_t g = point_list[min(begin + stage_slot, last)];
        g_ahead = point_list[min(begin + kBatch + stage_slot, last)];
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
            // A slot past the end of the list gets an exponent that makes every weight zero.
            const bool unused = stage_slot >= cnt;
            const float ex = nxy.x - centre_x, ey = nxy.y - centre_y;
            const float e = stage_g ? ey + (float)(kGy / 2) : ex + (float)(kFx / 2);
            const float curv = unused ? 0.0f : (stage_g ? nco.z : nco.x);
            const float lin = unused ? 0.0f : nco.y * (stage_g ? ex : ey);
            // (log2 of the opacity is held below 2 so that no scaled weight leaves f16's range)
            const float w_log2 = (nco.w > 1.99f ? 1.99f : nco.w) + kWeightScaleLog2;
            const float con = stage_g ? 0.0f : (unused ? -1.0e30f : w_log2 - (nco.y * ex) * ey);
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
            if (stage_g) {
                stage_group[stage_slot & 3] = unused ? 0.0f : nco.y;
                _Float16* const colour = reinterpret_cast<_Float16*>(stage_group + 4) + (stage_slot & 3);
                auto in_range = [&](float c) {          // NaN stays NaN; a slot past the end of the list holds no colour
                    return unused ? 0.0f : (c > kColourMax ? kColourMax : (c < -kColourMax ? -kColourMax : c));
                };
                colour[0] = (_Float16)in_range(nrgb.x);
                colour[4] = (_Float16)in_range(nrgb.y);
                colour[8] = (_Float16)in_range(nrgb.z);
                colour[12] = (_Float16)0.0f;
            }
        }
        __builtin_amdgcn_wave_barrier();
        nxy = points_xy[g_ahead]; nco = conic_opacity[g_ahead]; nrgb = rgb_depth[g_ahead];
        g_ahead = point_list[min(begin + base + 2 * kBatch + stage_slot, last)];
        // Gaussians go in pairs; the tile-wide stop is tested after each pair (render.cu:394-408)
        // The table reads of a Gaussian are issued before the Gaussian ahead of it is shaded, so
        // that a wave does not sit out the LDS latency once per Gaussian.
        auto fetch = [&](int j) {
            const int rec = j * kRec * 4;
            Staged r;
#pragma unroll
            for (int c = 0; c < SX; c++) r.f[c] = lds_read<float2>(rec_bytes + off_f + rec + c * 64);
#pragma unroll
            for (int c = 0; c < SY; c++) r.g[c] = lds_read<float2>(rec_bytes + off_g + rec + c * 64);
            return r;
        };
        auto fetch_group = [&](int g) {
            StagedGroup r;
            r.cy = lds_read<float4>(rec_bytes + off_cy + g * kGroupRec * 4);
            r.colour = lds_read<float2>(rec_bytes + off_colour + g * kGroupRec * 4);
            return r;
        };
        uint32_t packed[kSub][4][2];        // f16 weights of the group's Gaussians 0-1 and 2-3, per pixel
        float w0[kSub][4], w1[kSub][4];
        auto shade = [&](const Staged& r, float cy, float (&w)[kSub][4]) {
#pragma unroll
            for (int s = 0; s < kSub; s++) shade_quad(quad[s], role.xy[s], r.f[s % SX], r.g[s / SX], cy, w[s]);
        };
        auto pack = [&](int half) {
#pragma unroll
            for (int s = 0; s < kSub; s++)
#pragma unroll
                for (int p = 0; p < 4; p++) packed[s][p][half] = pack_f16(w0[s][p], w1[s][p]);
        };
        auto accumulate = [&](const StagedGroup& grp) {
            const half4_t colour = __builtin_bit_cast(half4_t, grp.colour);
#pragma unroll
            for (int s = 0; s < kSub; s++)
#pragma unroll
                for (int p = 0; p < 4; p++) {
                    const uint2 a = make_uint2(packed[s][p][0], packed[s][p][1]);
                    acc[s][p] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, a), colour, acc[s][p], 0, 0, 0);
                }
        };
        auto all_stopped = [&]() {
            float live = quad[0].T[1][1];           // the largest T of this lane's pixels
#pragma unroll
            for (int s = 0; s < kSub; s++) {
                live = __builtin_fmaxf(__builtin_fmaxf(live, quad[s].T[0][0]), __builtin_fmaxf(quad[s].T[0][1], quad[s].T[1][0]));
                if (s > 0) live = __builtin_fmaxf(live, quad[s].T[1][1]);
            }
            return ballot(!(live < 0.0001f)) == 0;
        };
        // written out for the whole batch so that every record offset is an immediate
#define FGS_GROUP(G)                                                                         \
        if (4 * (G) >= cnt) break;                                                           \
        grp = next_grp;                                                                      \
        next_grp = fetch_group(((G) + 1) % kGroups);    /* past the batch: read and dropped */\
        second = fetch(4 * (G) + 1);                                                         \
        shade(first, grp.cy.x, w0);                                                          \
        first = fetch(4 * (G) + 2);                                                          \
        shade(second, grp.cy.y, w1);                                                         \
        pack(0);                                                                             \
        stop_mid = all_stopped();                                                            \
        if (!stop_mid) {                                                                     \
            second = fetch(4 * (G) + 3);                                                     \
            shade(first, grp.cy.z, w0);                                                      \
            first = fetch((4 * (G) + 4) % kBatch);                                           \
            shade(second, grp.cy.w, w1);                                                     \
            pack(1);                                                                         \
        } else {                                                                             \
            _Pragma("unroll") for (int s = 0; s < kSub; s++)                                 \
                _Pragma("unroll") for (int p = 0; p < 4; p++) packed[s][p][1] = 0u;          \
        }                                                                                    \
        accumulate(grp);                                                                     \
        if (stop_mid || all_stopped()) { done = true; break; }
        static_assert(kBatch == 32, "the groups below cover a batch of 32");
        Staged first = fetch(0), second;
        StagedGroup grp, next_grp = fetch_group(0);
        bool stop_mid = false;
        do {
            FGS_GROUP(0) FGS_GROUP(1) FGS_GROUP(2) FGS_GROUP(3) FGS_GROUP(4) FGS_GROUP(5) FGS_GROUP(6) FGS_GROUP(7)
        } while (0);
#undef FGS_GROUP
    }

    // Lane 4b+j holds channel j of the pixels of lanes 4b .. 4b+3: handed back through the
    // staging area (a block of 16 x 4 floats per four lanes, padded to 68 so that the stores of
    // the 32 lanes served together fall into different banks).
    static_assert(Role::kStage >= 16 * 68, "the staging area holds the 64 x 16 colour sums of a sub-tile");
    const int lane = lane_id();
#pragma unroll
    for (int s = 0; s < kSub; s++) {
        __builtin_amdgcn_wave_barrier();
        char* const out = reinterpret_cast<char*>(s_rec) + 4 * ((lane >> 2) * 68 + (lane & 3));
#pragma unroll
        for (int p = 0; p < 4; p++)
#pragma unroll
            for (int r = 0; r < 4; r++) lds_write(out + 4 * (r * 16 + p * 4), acc[s][p][r]);
        __builtin_amdgcn_wave_barrier();
        const char* const in = rec_bytes + 4 * ((lane >> 2) * 68 + (lane & 3) * 16);
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const float4 c = lds_read<float4>(in + 16 * p);
            quad[s].r[p >> 1][p & 1] = c.x * kWeightUnscale;
            quad[s].g[p >> 1][p & 1] = c.y * kWeightUnscale;
            quad[s].b[p >> 1][p & 1] = c.z * kWeightUnscale;
        }
    }
    __builtin_amdgcn_wave_barrier();
    return done;
}

// The same walk with every operation in fp32 (render.cu:40-52 operation for operation): the colour
// sums are three multiply-adds per pixel, and a staged Gaussian is one record - F table, G table,
// (cy, red, green, blue) - so a lane reads all it needs of a Gaussian with three LDS reads and
// nothing is converted, packed or handed between lanes.  Same arguments and result as walk_list.
template <int SX, int SY>
__device__ __forceinline__ bool walk_list_fp32(
    const LaneRole<SX, SY>& role, float* s_rec,
    const uint32_t* __restrict__ point_list, int begin, int n,
    float centre_x, float centre_y,
    const float2* __restrict__ points_xy,
    const float4* __restrict__ rgb_depth,
    const float4* __restrict__ conic_opacity,
    Quad (&quad)[SX * SY])
{
    constexpr int kSub = SX * SY;
    constexpr int kFx = 16 * SX, kGy = 16 * SY;
    constexpr int kTab = kFx > kGy ? kFx : kGy;
    constexpr int kRec = LaneRole<SX, SY>::kRec;        // kFx + kGy + 4: the tables, then (cy, r, g, b)
    struct Staged {
        float4 u;
        float2 f[SX], g[SY];
    };
    const char* const rec_bytes = reinterpret_cast<const char*>(s_rec);
    const uint32_t off_f = role.off_f, off_g = role.off_g;
    uint32_t off_u = 4u * (uint32_t)(kFx + kGy);
    asm volatile("" : "+v"(off_u));                     // kept in a vector register: reads are "register + immediate"
    const int stage_slot = role.stage_slot;
    const bool stage_g = role.stage_g;
    float* const stage_tab = s_rec + stage_slot * kRec + (stage_g ? kFx : 0);
    const int stage_len = stage_g ? kGy : kFx;
    const int last = begin + n - 1;

#pragma unroll
    for (int s = 0; s < kSub; s++) clear_quad(quad[s]);

    // registers hold the batch that is staged next; the list index is fetched two batches ahead
    // and the attributes one batch ahead (see walk_list)
    float2 nxy = make_float2(0.f, 0.f);
    float4 nco = make_float4(0.f, 0.f, 0.f, 0.f), nrgb = make_float4(0.f, 0.f, 0.f, 0.f);
    uint32_t g_ahead = 0;
    if (n > 0) {
        const uint32_t g = point_list[min(begin + stage_slot, last)];
        g_ahead = point_list[min(begin + kBatch + stage_slot, last)];
        nxy = points_xy[g]; nco = conic_opacity[g]; nrgb = rgb_depth[g];
    }

    bool done = false;
    for (int base = 0; base < n && !done; base += kBatch) {
        const int cnt = min(kBatch, n - base);
        __builtin_amdgcn_wave_barrier();
        {
            // the entry for column (row) k is con + d (curv d + lin) at d = e - k, as a polynomial in k
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
        g_ahead = point_list[min(begin + base + 2 * kBatch + stage_slot, last)];
        // the reads of a Gaussian are issued before the Gaussian ahead of it is shaded
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
            for (int s = 0; s < kSub; s++)
                shade_quad_fp32(quad[s], role.xy[s], r.f[s % SX], r.g[s / SX], r.u.x, make_float4(r.u.y, r.u.z, r.u.w, 0.f));
        };
        auto all_stopped = [&]() {
            float live = quad[0].T[1][1];           // the largest T of this lane's pixels
#pragma unroll
            for (int s = 0; s < kSub; s++) {
                live = __builtin_fmaxf(__builtin_fmaxf(live, quad[s].T[0][0]), __builtin_fmaxf(quad[s].T[0][1], quad[s].T[1][0]));
                if (s > 0) live = __builtin_fmaxf(live, quad[s].T[1][1]);
            }
            return ballot(!(live < 0.0001f)) == 0;
        };
        // Gaussians go in pairs, the tile-wide stop is tested after each pair (render.cu:394-408);
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
    __builtin_amdgcn_wave_barrier();
    return done;
}

template <int SX, int SY, bool kFp32, typename... Args>
__device__ __forceinline__ bool walk(Args&&... args)
{
    if constexpr (kFp32) return walk_list_fp32<SX, SY>(args...);
    else return walk_list<SX, SY>(args...);
}

// render.cu:59-73
template <int SX, int SY>
__device__ __forceinline__ void write_tile(
    int lane, int tile_x, int tile_y, int width, int height, const Quad (&quad)[SX * SY],
    float bg_r, float bg_g, float bg_b, uint8_t* __restrict__ out_u8, float* __restrict__ out_f32)
{
    const int qx = (lane & 7) * 2, qy = (lane >> 3) * 2;
#pragma unroll
    for (int s = 0; s < SX * SY; s++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int x = tile_x * 16 * SX + (s % SX) * 16 + qx + i, y = tile_y * 16 * SY + (s / SX) * 16 + qy + j;
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

// Position in the launch -> tile.  The hardware deals consecutive workgroups out to the 8 XCDs in
// turn, and every XCD has its own L2.  Neighbouring tiles share most of their Gaussians, so each
// XCD is given whole 8x8 blocks of tiles (its positions g = 8*slot + xcd walk blocks xcd, xcd+8,
// ... 64 tiles at a time): a Gaussian's attribute lines are then fetched into one L2 once instead
// of into several L2s once per tile.  False for the padding positions.
__device__ __forceinline__ bool tile_of_position(int group, int tiles_x, int tiles_y, int* tile_x, int* tile_y)
{
    const int xcd = group & 7, slot = group >> 3;
    const int blocks_x = (tiles_x + 7) >> 3;
    const int block = (slot >> 6) * 8 + xcd, inner = slot & 63;
    *tile_x = (block % blocks_x) * 8 + (inner & 7);
    *tile_y = (block / blocks_x) * 8 + (inner >> 3);
    return *tile_x < tiles_x && *tile_y < tiles_y;
}

template <int SX, int SY, bool kFp32>
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
    constexpr int kSub = SX * SY;              // 16x16 sub-tiles per tile = quads per lane
    constexpr int kFx = 16 * SX, kGy = 16 * SY;
    __shared__ __align__(16) float s_rec[LaneRole<SX, SY>::kStage];

    const int lane = threadIdx.x;
    int tile_x, tile_y;
    if (!tile_of_position((int)blockIdx.x, tiles_x, tiles_y, &tile_x, &tile_y)) return;
    const int2 range = ranges[tile_y * tiles_x + tile_x];
    const int n = range.y - range.x;
    // A launch ends when its longest list ends, and a wave that shares its SIMD equally with the
    // waves of short lists gets to its own end late: waves with long lists ask for a higher
    // issue priority.
    if (n > 1024) __builtin_amdgcn_s_setprio(3);
    else if (n > 512) __builtin_amdgcn_s_setprio(2);
    else if (n > 256) __builtin_amdgcn_s_setprio(1);

    LaneRole<SX, SY> role;
    role.init(lane);
    Quad quad[kSub];
#pragma unroll
    for (int s = 0; s < kSub; s++) clear_quad(quad[s]);
    const float centre_x = (float)(tile_x * kFx + kFx / 2), centre_y = (float)(tile_y * kGy + kGy / 2);
    walk<SX, SY, kFp32>(role, s_rec, point_list, range.x, n, centre_x, centre_y, points_xy, rgb_depth, conic_opacity, quad);
    write_tile<SX, SY>(lane, tile_x, tile_y, width, height, quad, bg_r, bg_g, bg_b, out_u8, out_f32);
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

// Registers are budgeted for 6 resident waves per SIMD on 16x16 tiles, 3 and 2 on the wider ones
// (their colour sums take 32 and 64 registers).
template <int SX, int SY>
constexpr int kFewWaves = SX * SY == 1 ? 4 : SX * SY == 2 ? 3 : 2;
template <int SX, int SY>
constexpr int kPlainWaves = SX * SY == 1 ? 6 : kFewWaves<SX, SY>;

template <int SX, int SY, bool kFp32>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(kPlainWaves<SX, SY>))) void blend_kernel(FGS_BLEND_PARAMS)
{
    blend_tile<SX, SY, kFp32>(FGS_BLEND_ARGS);
}

// The same kernel held to 4 resident waves per SIMD (16 per CU; 3 and 2 for the wider tiles,
// whose colour sums need more registers).  Every resident wave walks its own tile's list and the
// lists of the tiles in flight compete for the 4 MB L2 of their XCD: when there are more tiles
// than the chip holds at once, fewer resident waves mean fewer misses (a 4K frame takes the same
// time at 4, 5 and 6 waves per SIMD and half as long again at 8).
template <int SX, int SY, bool kFp32>
__global__ __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(kFewWaves<SX, SY>, kFewWaves<SX, SY>))) void blend_kernel_few_waves(FGS_BLEND_PARAMS)
{
    blend_tile<SX, SY, kFp32>(FGS_BLEND_ARGS);
}

// A frame of few tiles is placed on the chip almost at once, one wave per tile: the launch then
// lasts as long as the busiest SIMD (the sum of the lists placed on it) and at least as long as
// the longest list walked by one wave.  Here the tiles are ranked by list length
// (tile_order_kernel) and a workgroup of four waves takes one tile from each quarter of the
// ranking: the workgroups with the longest lists are dispatched first, the short ones fill in
// behind them, and a long list has three shorter ones beside it.  Every wave blends the first
// kOwnShare entries of its own tile; what is left of a list of more than kOwnShare + kMinRest
// entries after that is cut into four runs of pairs, one per wave.  A run is blended from T = 1, C = 0 and the owner folds the runs in front-to-back order,
// C += T C_run, T *= T_run, which is the same sum in another order of additions.  A run stops
// when its own T is below the threshold everywhere, so a tile can be walked a little further than
// the reference walks it: what that adds is below 1e-4 of a colour.
constexpr int kOwnShare = 256;
constexpr int kMinRest = 512;               // a shorter rest is not worth two barriers: the owner walks it
constexpr int kSharedWaves = 4;

template <bool kFp32>
__global__ __launch_bounds__(kSharedWaves * kWave) __attribute__((amdgpu_waves_per_eu(6, 6))) void blend_kernel_shared(FGS_BLEND_PARAMS, const uint32_t* __restrict__ tile_order)
{
    using Role = LaneRole<1, 1>;
    __shared__ __align__(16) float s_rec[kSharedWaves][Role::kStage];
    __shared__ int s_rest[kSharedWaves], s_from[kSharedWaves], s_tile_x[kSharedWaves], s_tile_y[kSharedWaves];
    static_assert(Role::kStage >= 4 * 4 * kWave, "a run's result (4 pixels x 4 floats per lane) is handed over in the staging area");

    const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // Wave w takes rank g of quarter w of the tiles ranked by list length: the workgroups with
    // the longest lists come first in the launch, and a long list has three shorter ones beside it.
    const int rank = wave * (int)gridDim.x + (int)blockIdx.x;
    const bool active = rank < tiles_x * tiles_y;
    int tile_x = 0, tile_y = 0;
    if (active) {
        const int tile = (int)tile_order[rank];
        tile_x = tile % tiles_x;
        tile_y = tile / tiles_x;
    }
    int2 range = make_int2(0, 0);
    if (active) range = ranges[tile_y * tiles_x + tile_x];
    const int n = range.y - range.x;
    if (n > 256) __builtin_amdgcn_s_setprio(1);

    Role role;
    role.init(lane);
    if (lane == 0) {
        s_rest[wave] = n;               // job 0 of wave w: the head of its own list, in one run
        s_from[wave] = range.x;
        s_tile_x[wave] = tile_x;
        s_tile_y[wave] = tile_y;
    }
    __builtin_amdgcn_wave_barrier();    // job 0 reads these back in the same wave; the others after the barrier below
    // job 0: own head; job 1 + v: this wave's run of what is left of tile v.  While a wave blends
    // runs, the result of its own head waits in its private memory, not in registers.
    Quad part[1];
    volatile float kept[16];
    bool shared_out = false;
    for (int job = 0; job <= kSharedWaves; job++) {
        const int v = job == 0 ? wave : job - 1;
        const int rest = __builtin_amdgcn_readfirstlane(s_rest[v]);
        if (job != 0 && rest == 0) continue;
        int skip = 0, count = rest > kOwnShare + kMinRest ? kOwnShare : rest;
        if (job != 0) {
            const int run = (((rest + kSharedWaves - 1) / kSharedWaves) + 1) & ~1;      // whole pairs
            skip = min(wave * run, rest);
            count = min(run, rest - skip);
        }
        clear_quad(part[0]);
        const bool stopped = walk<1, 1, kFp32>(role, s_rec[wave], point_list, __builtin_amdgcn_readfirstlane(s_from[v]) + skip, count,
                                             (float)(__builtin_amdgcn_readfirstlane(s_tile_x[v]) * 16 + 8),
                                             (float)(__builtin_amdgcn_readfirstlane(s_tile_y[v]) * 16 + 8),
                                             points_xy, rgb_depth, conic_opacity, part);
        if (job == 0) {
            if (lane == 0) {
                s_rest[wave] = (!stopped && n > kOwnShare + kMinRest) ? n - kOwnShare : 0;
                s_from[wave] = range.x + kOwnShare;
            }
            __syncthreads();
            shared_out = (s_rest[0] | s_rest[1] | s_rest[2] | s_rest[3]) != 0;
            if (!shared_out) break;
            __builtin_amdgcn_s_setprio(3);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                kept[4 * k + 0] = part[0].r[k >> 1][k & 1]; kept[4 * k + 1] = part[0].g[k >> 1][k & 1];
                kept[4 * k + 2] = part[0].b[k >> 1][k & 1]; kept[4 * k + 3] = part[0].T[k >> 1][k & 1];
            }
            continue;
        }
        float4* const mine = reinterpret_cast<float4*>(s_rec[wave]);
#pragma unroll
        for (int k = 0; k < 4; k++)
            mine[k * kWave + lane] = make_float4(part[0].r[k >> 1][k & 1], part[0].g[k >> 1][k & 1],
                                                 part[0].b[k >> 1][k & 1], part[0].T[k >> 1][k & 1]);
        __syncthreads();
        if (wave == v) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float r = kept[4 * k + 0], g = kept[4 * k + 1], b = kept[4 * k + 2], t = kept[4 * k + 3];
#pragma unroll
                for (int w = 0; w < kSharedWaves; w++) {
                    const float4 p = reinterpret_cast<const float4*>(s_rec[w])[k * kWave + lane];
                    r += t * p.x; g += t * p.y; b += t * p.z;
                    t *= p.w;
                }
                kept[4 * k + 0] = r; kept[4 * k + 1] = g; kept[4 * k + 2] = b; kept[4 * k + 3] = t;
            }
        }
        __syncthreads();
    }
    if (shared_out) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            part[0].r[k >> 1][k & 1] = kept[4 * k + 0]; part[0].g[k >> 1][k & 1] = kept[4 * k + 1];
            part[0].b[k >> 1][k & 1] = kept[4 * k + 2]; part[0].T[k >> 1][k & 1] = kept[4 * k + 3];
        }
    }
    if (active) write_tile<1, 1>(lane, tile_x, tile_y, width, height, part, bg_r, bg_g, bg_b, out_u8, out_f32);
}
#undef FGS_BLEND_PARAMS
#undef FGS_BLEND_ARGS

// How the colour sums are formed by the entry points that do not say (see fgs_set_colour_sums).
std::atomic<int> g_colour_sums{FGS_COLOUR_SUMS_FP32};

// The mode of one call: what its flags ask for, else the process default.
int colour_mode(int flags, int* mode, const char* who)
{
    if (flags & ~(FGS_BLEND_FP32 | FGS_BLEND_MATRIX_F16)) return fail(FGS_E_INVALID, "%s: unknown flags 0x%x", who, flags);
    if ((flags & FGS_BLEND_FP32) && (flags & FGS_BLEND_MATRIX_F16))
        return fail(FGS_E_INVALID, "%s: FGS_BLEND_FP32 and FGS_BLEND_MATRIX_F16 exclude each other", who);
    *mode = (flags & FGS_BLEND_FP32) ? FGS_COLOUR_SUMS_FP32
          : (flags & FGS_BLEND_MATRIX_F16) ? FGS_COLOUR_SUMS_MATRIX_F16 : g_colour_sums.load();
    return FGS_OK;
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

// How a frame is blended.  More tiles than the chip holds at 8 waves per SIMD: the variant with
// fewer resident waves.  A frame of 16x16 tiles that is resident at once: workgroups of four tiles
// that share out their long lists, which needs the tiles ranked by list length.
struct BlendShape {
    int cus;
    bool few_waves, shared;
};

int blend_shape(int block_x, int block_y, int tiles_x, int tiles_y, BlendShape* shape)
{
    int dev = 0;
    FGS_HIP_TRY(hipGetDevice(&dev));
    FGS_HIP_TRY(hipDeviceGetAttribute(&shape->cus, hipDeviceAttributeMultiprocessorCount, dev));
    const long long num_tiles = (long long)tiles_x * tiles_y;
    shape->few_waves = num_tiles > 32LL * shape->cus;
    shape->shared = !shape->few_waves && block_x == 16 && block_y == 16 && num_tiles <= kOrderCap && shape->cus > 0;
    return FGS_OK;
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
    if (num_rendered == 0)
        hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)fill_blocks), dim3(256), 0, st, ranges, words, 0);
    else
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
               uint8_t* out_u8, float* out_f32, int flags, void* stream, const char* who)
{
    int sx = 0, sy = 0, mode = 0;
    int rc = check_tile(block_x, block_y, &sx, &sy, who);
    if (rc != FGS_OK) return rc;
    rc = colour_mode(flags, &mode, who);
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
    BlendShape shape;
    rc = blend_shape(block_x, block_y, tiles_x, tiles_y, &shape);
    if (rc != FGS_OK) return rc;
    const bool few_waves = shape.few_waves;
    const bool fp32 = mode == FGS_COLOUR_SUMS_FP32;
#define FGS_LAUNCH_BLEND(SX, SY)                                                                        \
    do {                                                                                                \
        auto kernel = fp32 ? (few_waves ? blend_kernel_few_waves<SX, SY, true> : blend_kernel<SX, SY, true>) \
                           : (few_waves ? blend_kernel_few_waves<SX, SY, false> : blend_kernel<SX, SY, false>); \
        hipLaunchKernelGGL(kernel, grid, dim3(kWave), 0, st,                                            \
                           (const int2*)ranges, values_sorted, width, height, tiles_x, tiles_y,         \
                           (const float2*)points_xy, (const float4*)rgb_depth, (const float4*)conic_opacity, \
                           bg[0], bg[1], bg[2], out_u8, out_f32);                                       \
    } while (0)
    if (shape.shared) {
        const int num_tiles = tiles_x * tiles_y;
        uint32_t* tile_order = nullptr;
        rc = tile_order_table(st, &tile_order);
        if (rc != FGS_OK) return rc;
        hipLaunchKernelGGL(tile_order_kernel, dim3(1), dim3(1024), 0, st, (const int2*)ranges, num_tiles, tile_order);
        hipLaunchKernelGGL(fp32 ? blend_kernel_shared<true> : blend_kernel_shared<false>, dim3((unsigned)((num_tiles + kSharedWaves - 1) / kSharedWaves)), dim3(kSharedWaves * kWave), 0, st,
                           (const int2*)ranges, values_sorted, width, height, tiles_x, tiles_y,
                           (const float2*)points_xy, (const float4*)rgb_depth, (const float4*)conic_opacity,
                           bg[0], bg[1], bg[2], out_u8, out_f32, (const uint32_t*)tile_order);
    } else if (sx == 1 && sy == 1) FGS_LAUNCH_BLEND(1, 1);
    else if (sx == 2 && sy == 1) FGS_LAUNCH_BLEND(2, 1);
    else FGS_LAUNCH_BLEND(2, 2);
#undef FGS_LAUNCH_BLEND
    return check_hip(hipGetLastError(), who);
}

int render_impl(int block_x, int block_y, int num_rendered, int width, int height,
                const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                const uint64_t* keys_sorted, const uint32_t* values_sorted,
                int* ranges, const float bg[3], uint8_t* out_u8, float* out_f32, int flags, void* stream, const char* who)
{
    int sx = 0, sy = 0, mode = 0;
    int rc = check_tile(block_x, block_y, &sx, &sy, who);
    if (rc != FGS_OK) return rc;
    rc = colour_mode(flags, &mode, who);        // before anything is launched
    if (rc != FGS_OK) return rc;
    if (num_rendered > 0 && (!points_xy || !rgb_depth || !conic_opacity || !keys_sorted || !values_sorted))
        return fail(FGS_E_INVALID, "%s: null buffer", who);
    rc = ranges_impl(block_x, block_y, num_rendered, width, height, keys_sorted, ranges, stream, who);
    if (rc != FGS_OK) return rc;
    return blend_impl(block_x, block_y, width, height, points_xy, rgb_depth, conic_opacity, values_sorted, ranges,
                      bg, out_u8, out_f32, flags, stream, who);
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
                                nullptr, 0, stream, #NAME);                                                  \
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
                            out_color_u8, out_color_f32, 0, stream, "fgs_render_f32");
}

extern "C" int fgs_render_ex(int block_x, int block_y, int num_rendered, int width, int height,
                             const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                             const uint64_t* gaussian_keys_sorted, const uint32_t* gaussian_values_sorted,
                             int* ranges, const float bg_color[3], uint8_t* out_color_u8, float* out_color_f32,
                             int flags, void* stream)
{
    return fgs::render_impl(block_x, block_y, num_rendered, width, height, points_xy, rgb_depth,
                            conic_opacity, gaussian_keys_sorted, gaussian_values_sorted, ranges, bg_color,
                            out_color_u8, out_color_f32, flags, stream, "fgs_render_ex");
}

extern "C" int fgs_set_colour_sums(int mode)
{
    if (mode != FGS_COLOUR_SUMS_MATRIX_F16 && mode != FGS_COLOUR_SUMS_FP32) {
        fgs::fail(FGS_E_INVALID, "fgs_set_colour_sums: mode %d unknown", mode);
        return -1;
    }
    return fgs::g_colour_sums.exchange(mode);
}

extern "C" const char* fgs_blend_kernel_name(int block_x, int block_y, int width, int height, int flags)
{
    using namespace fgs;
    int sx = 0, sy = 0, mode = 0;
    if (check_tile(block_x, block_y, &sx, &sy, "fgs_blend_kernel_name") != FGS_OK || width <= 0 || height <= 0) return "";
    if (colour_mode(flags, &mode, "fgs_blend_kernel_name") != FGS_OK) return "";
    BlendShape shape;
    if (blend_shape(block_x, block_y, (width + block_x - 1) / block_x, (height + block_y - 1) / block_y, &shape) != FGS_OK) return "";
    const bool fp32 = mode == FGS_COLOUR_SUMS_FP32;
#define FGS_NAME(few, plain) (shape.few_waves ? (fp32 ? few ", true>" : few ", false>") : (fp32 ? plain ", true>" : plain ", false>"))
    if (shape.shared) return fp32 ? "tile_order_kernel + blend_kernel_shared<true>" : "tile_order_kernel + blend_kernel_shared<false>";
    if (sx == 1 && sy == 1) return FGS_NAME("blend_kernel_few_waves<1, 1", "blend_kernel<1, 1");
    if (sx == 2 && sy == 1) return FGS_NAME("blend_kernel_few_waves<2, 1", "blend_kernel<2, 1");
    return FGS_NAME("blend_kernel_few_waves<2, 2", "blend_kernel<2, 2");
#undef FGS_NAME
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
                           gaussian_values_sorted, ranges, bg_color, out_color_u8, out_color_f32, 0, stream, "fgs_blend");
}

extern "C" int fgs_blend_ex(int block_x, int block_y, int width, int height,
                            const float* points_xy, const float* rgb_depth, const float* conic_opacity,
                            const uint32_t* gaussian_values_sorted, const int* ranges, const float bg_color[3],
                            uint8_t* out_color_u8, float* out_color_f32, int flags, void* stream)
{
    return fgs::blend_impl(block_x, block_y, width, height, points_xy, rgb_depth, conic_opacity,
                           gaussian_values_sorted, ranges, bg_color, out_color_u8, out_color_f32, flags, stream, "fgs_blend_ex");
}

