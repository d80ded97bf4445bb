// Preprocess + key emission for gfx950 (wave64).
//
// One launch does what FlashGS preprocessCUDA (csrc/cuda_rasterizer/preprocess.cu:243-418)
// does: near/opacity cull, projection, 2D covariance, conic, opacity-aware radius, exact
// ellipse/tile test, (tile << 32 | depth) key emission, and - only for Gaussians that emitted a
// key - SH colour and the 40-byte attribute record.
//
// Differences in mechanism (not in results):
//  * Key slots come from a count -> wave scan -> block scan -> scan over workgroups by one
//    dedicated wave of the launch instead of atomics on one counter, so the unsorted list has a
//    fixed order: ascending Gaussian index, then row-major tiles.  A stable sort then fixes tie
//    order too.
//  * The candidate tiles of all Gaussians of a wave with rectangles of at most 64 tiles are laid
//    end to end and tested one per lane per step, so lanes stay busy whatever the mix of sizes;
//    larger rectangles are tested by the whole wave, 64 tiles a step, and rectangles of more than
//    1024 tiles by the whole workgroup, which gets the passing tiles of every column and row as
//    an interval found by bisection with the reference's own edge predicates: the tiles are
//    counted from the intervals alone and visited only to write their keys.
//
// THIS FILE MUST BE COMPILED WITH -ffp-contract=off.  Every fp32 expression that feeds a key is
// written in the operand order of the reference and has to be evaluated one IEEE operation at a
// time, so that a scalar CPU evaluation of the same expressions gives the same bits.
#include "fgs_internal.h"

#include <atomic>
#include <chrono>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

namespace fgs {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kStashCap = 1024;         // flat candidates (and so stashed hits) per wave
constexpr int kHugeMin = 1024;          // rectangles with more tiles than this are tested by the whole workgroup
// such rectangles per workgroup: as many as the LDS of 7 workgroups per CU leaves room for (a
// rectangle beyond the list stays with its wave, 64 tiles a step, and everything behind this
// workgroup waits for that count)
constexpr int kHugeCap = 27;
constexpr int kSpanWords = kWavesPerBlock * kStashCap / 4;   // column + row spans of one listed rectangle
static_assert(kSpanWords / kWave <= kWave, "one lane per group of 64 columns");
constexpr unsigned kSpinLimit = 1u << 22;   // polls before a wait on the scan over workgroups gives up

struct Camera {
    float view[16];
    float proj[16];
    float campos[3];
    int W, H, bx, by, gx, gy;
    float tan_fovx, tan_fovy, fx, fy;
};

// ---- scalar numerics ---------------------------------------------------------------------------

// min / max of preprocess.cu:116-117 and max.f32 of :36-41: a NaN operand yields the other one
__device__ __forceinline__ float min_f(float a, float b)
{
    if (!(a == a)) return b;
    if (!(b == b)) return a;
    return a < b ? a : b;
}
__device__ __forceinline__ float max_f(float a, float b)
{
    if (!(a == a)) return b;
    if (!(b == b)) return a;
    return a > b ? a : b;
}

// Saturating float -> int: NaN -> 0, out-of-range clamps (the behaviour preprocess.cu:93-98 and
// :309-310 get from the device conversion instruction).
__device__ __forceinline__ int to_int_sat(float f)
{
    if (!(f == f)) return 0;
    if (f >= 2147483648.0f) return 2147483647;
    if (f <= -2147483648.0f) return -2147483647 - 1;
    return (int)f;
}

// log2 of a positive normal float from its exponent plus an odd series in
// s = (m-1)/(m+1); stands in for the approximate instruction of preprocess.cu:57-62.
__device__ __forceinline__ float log2_det(float x)
{
    uint32_t bits = __float_as_uint(x);
    int e = (int)(bits >> 23) - 127;
    float m = __uint_as_float((bits & 0x007fffffu) | 0x3f800000u);
    if (m > 1.41421354f) { m = m * 0.5f; e += 1; }
    float s = (m - 1.0f) / (m + 1.0f);
    float s2 = s * s;
    float p = 0.111111111f;
    p = p * s2 + 0.142857143f;
    p = p * s2 + 0.2f;
    p = p * s2 + 0.333333333f;
    p = p * s2 + 1.0f;
    float r = (s * 2.88539008f) * p;
    return (float)e + r;
}

// preprocess.cu:64-67 - the reference's literals make this double precision.
__device__ __forceinline__ float ndc_to_pix(float v, int S)
{
    return (float)((((double)v + 1.0) * (double)S - 1.0) * 0.5);
}

// 3x3 product with GLM's [col][row] storage and summation order (type_mat3x3.inl:486-519).
struct Mat3 { float c[3][3]; };

__device__ __forceinline__ Mat3 mul(const Mat3& a, const Mat3& b)
{
    Mat3 r;
#pragma unroll
    for (int col = 0; col < 3; col++)
#pragma unroll
        for (int row = 0; row < 3; row++)
            r.c[col][row] = a.c[0][row] * b.c[col][0] + a.c[1][row] * b.c[col][1] + a.c[2][row] * b.c[col][2];
    return r;
}

__device__ __forceinline__ Mat3 transposed(const Mat3& m)
{
    Mat3 r;
#pragma unroll
    for (int col = 0; col < 3; col++)
#pragma unroll
        for (int row = 0; row < 3; row++)
            r.c[col][row] = m.c[row][col];
    return r;
}

// preprocess.cu:103-143
__device__ __forceinline__ void cov2d(const float t_in[3], const Camera& cam, const float s[6], float& c00, float& c01, float& c11)
{
    const float* vm = cam.view;
    float tx = t_in[0], ty = t_in[1], tz = t_in[2];
    const float limx = 1.3f * cam.tan_fovx;
    const float limy = 1.3f * cam.tan_fovy;
    const float txtz = tx / tz;
    const float tytz = ty / tz;
    tx = min_f(limx, max_f(-limx, txtz)) * tz;
    ty = min_f(limy, max_f(-limy, tytz)) * tz;

    Mat3 J;
    J.c[0][0] = cam.fx / tz; J.c[0][1] = 0.0f;        J.c[0][2] = -(cam.fx * tx) / (tz * tz);
    J.c[1][0] = 0.0f;        J.c[1][1] = cam.fy / tz; J.c[1][2] = -(cam.fy * ty) / (tz * tz);
    J.c[2][0] = 0.0f;        J.c[2][1] = 0.0f;        J.c[2][2] = 0.0f;
    Mat3 Wm;
    Wm.c[0][0] = vm[0]; Wm.c[0][1] = vm[4]; Wm.c[0][2] = vm[8];
    Wm.c[1][0] = vm[1]; Wm.c[1][1] = vm[5]; Wm.c[1][2] = vm[9];
    Wm.c[2][0] = vm[2]; Wm.c[2][1] = vm[6]; Wm.c[2][2] = vm[10];
    Mat3 T = mul(Wm, J);
    Mat3 V;
    V.c[0][0] = s[0]; V.c[0][1] = s[1]; V.c[0][2] = s[2];
    V.c[1][0] = s[1]; V.c[1][1] = s[3]; V.c[1][2] = s[4];
    V.c[2][0] = s[2]; V.c[2][1] = s[4]; V.c[2][2] = s[5];
    Mat3 cov = mul(mul(transposed(T), transposed(V)), T);
    c00 = cov.c[0][0] + 0.3f;
    c01 = cov.c[0][1];
    c11 = cov.c[1][1] + 0.3f;
}

// The ellipse/tile test of the reference (preprocess.cu:187-241), cut into the pieces that depend
// on one tile coordinate only.  For the test against the nearer vertical edge of tile column x
// (preprocess.cu:196-215 with the segment test :187-194): a = conic z, b = -2 conic_y dx,
// c = conic_x dx^2 - w, delta = b^2 - 4ac depend on x alone, and tile row y enters through
//   t1 = (top - cy) 2a + b,     near_ok = t1 <= 0 || t1^2 <= delta,
//   t2 = (bottom - cy) 2a + b,  far_ok  = t2 >= 0 || t2^2 <= delta.
// The test against the nearer horizontal edge is the same with the axes exchanged.  Every
// expression is evaluated exactly as the reference writes it, one IEEE operation at a time.
struct EdgeTest {
    float two_a, b, delta;
};

// centre: the Gaussian's coordinate across the edge; lo, hi: first and last pixel of the tile
// across the edge; a: conic entry along the edge, c_across: conic entry across it
__device__ __forceinline__ EdgeTest edge_test(float a, float cony, float c_across, float centre, int lo, int hi, float w)
{
    const float d = (centre * 2.0f < (float)(lo + hi)) ? centre - (float)lo : centre - (float)hi;
    EdgeTest e;
    e.b = -2.0f * cony * d;
    const float c = c_across * d * d - w;
    e.delta = e.b * e.b - 4.0f * a * c;
    e.two_a = 2.0f * a;
    return e;
}

__device__ __forceinline__ bool near_ok(const EdgeTest& e, float first_px, float centre_along)
{
    const float t1 = (first_px - centre_along) * e.two_a + e.b;
    return t1 <= 0.0f || t1 * t1 <= e.delta;
}

__device__ __forceinline__ bool far_ok(const EdgeTest& e, float last_px, float centre_along)
{
    const float t2 = (last_px - centre_along) * e.two_a + e.b;
    return t2 >= 0.0f || t2 * t2 <= e.delta;
}

// preprocess.cu:238-241 || :196-236 for tile (x, y)
__device__ __forceinline__ bool tile_hit(int x, int y, int bx, int by, float cx, float cy,
                                         float conx, float cony, float conz, float power)
{
    const int minx = x * bx, miny = y * by;
    const int maxx = minx + bx - 1, maxy = miny + by - 1;
    const float fminx = (float)minx, fminy = (float)miny, fmaxx = (float)maxx, fmaxy = (float)maxy;
    if (cx >= fminx && cx <= fmaxx && cy >= fminy && cy <= fmaxy) return true;

    const float w = 2.0f * power;
    const EdgeTest v = edge_test(conz, cony, conx, cx, minx, maxx, w);
    if (v.delta >= 0.0f && near_ok(v, fminy, cy) && far_ok(v, fmaxy, cy)) return true;
    const EdgeTest h = edge_test(conx, cony, conz, cy, miny, maxy, w);
    return h.delta >= 0.0f && near_ok(h, fminx, cx) && far_ok(h, fmaxx, cx);
}

// For one tile column (or row) of a rectangle: which of the `count` tiles along it pass the edge
// test.  near_ok can only turn from true to false and far_ok from false to true as the tile index
// grows (both t1 and t2 are non-decreasing in it when 2a > 0: every operation that leads to them
// is monotone, rounding included), so the tiles that pass are the interval between two points
// that bisection finds with the very predicates of the per-tile test.  Packed as
// first | last << 15 | centre-inside-this-column << 30; an empty interval is first 1, last 0.
__device__ __forceinline__ uint32_t edge_span(float a, float cony, float c_across, float centre, float centre_along,
                                              int tile, int block, int first_tile_along, int block_along, int count, float w)
{
    const int lo_px = tile * block, hi_px = lo_px + block - 1;
    const uint32_t inside = (centre >= (float)lo_px && centre <= (float)hi_px) ? 1u << 30 : 0u;
    const EdgeTest e = edge_test(a, cony, c_across, centre, lo_px, hi_px, w);
    if (!(e.delta >= 0.0f)) return inside | 1u;
    // Two bisections side by side, so that their dependent chains overlap: near_ok holds for
    // tiles [0, n_lo) and fails from n_hi on; far_ok fails for tiles [0, f_lo), holds from f_hi on.
    int n_lo = 0, n_hi = count, f_lo = 0, f_hi = count;
    while (n_lo < n_hi || f_lo < f_hi) {
        const int n_mid = (n_lo + n_hi) >> 1, f_mid = (f_lo + f_hi) >> 1;
        const bool n_ok = near_ok(e, (float)((first_tile_along + n_mid) * block_along), centre_along);
        const bool f_ok = far_ok(e, (float)((first_tile_along + f_mid) * block_along + block_along - 1), centre_along);
        if (n_lo < n_hi) { if (n_ok) n_lo = n_mid + 1; else n_hi = n_mid; }
        if (f_lo < f_hi) { if (f_ok) f_hi = f_mid; else f_lo = f_mid + 1; }
    }
    const int last = n_lo - 1;
    const int first = f_lo;
    if (first > last) return inside | 1u;
    return inside | (uint32_t)first | ((uint32_t)last << 15);
}

// j / w and j % w for 0 <= j, 1 <= w.  Below 2^20 the quotient comes from a reciprocal estimate
// (off by less than 1/4 there) corrected by one step either way.
__device__ __forceinline__ void div_mod(int j, int w, int& q, int& r)
{
    if (j >= (1 << 20)) { q = j / w; r = j - q * w; return; }
    q = (int)(((float)j + 0.5f) * __builtin_amdgcn_rcpf((float)w));
    r = j - q * w;
    if (r < 0) { q--; r += w; }
    else if (r >= w) { q++; r -= w; }
}

// preprocess.cu:13-34, :145-185
__device__ __forceinline__ void sh_to_rgb(const float* __restrict__ sh, float px, float py, float pz,
                                          const Camera& cam, float rgb[3])
{
    constexpr float C0 = 0.28209479177387814f;
    constexpr float C1 = 0.4886025119029199f;
    constexpr float C2_0 = 1.0925484305920792f, C2_1 = -1.0925484305920792f, C2_2 = 0.31539156525252005f,
                    C2_3 = -1.0925484305920792f, C2_4 = 0.5462742152960396f;
    constexpr float C3_0 = -0.5900435899266435f, C3_1 = 2.890611442640554f, C3_2 = -0.4570457994644658f,
                    C3_3 = 0.3731763325901154f, C3_4 = -0.4570457994644658f, C3_5 = 1.445305721320277f,
                    C3_6 = -0.5900435899266435f;

    // 48 floats = 12 aligned 16-byte loads (the record is 192 bytes), taken in four groups of
    // four coefficients per channel so that only 12 of them are live at a time: the sums below
    // run in coefficient order, so splitting them changes no result.
    const float4* src = reinterpret_cast<const float4*>(sh);
    float v[12];
    auto load_group = [&](int g) {
#pragma unroll
        for (int q = 0; q < 3; q++) {
            float4 f = src[3 * g + q];
            v[4 * q + 0] = f.x; v[4 * q + 1] = f.y; v[4 * q + 2] = f.z; v[4 * q + 3] = f.w;
        }
    };
    load_group(0);
    float dx = px - cam.campos[0], dy = py - cam.campos[1], dz = pz - cam.campos[2];
    float l2 = dx * dx + dy * dy + dz * dz;
    float inv = 1.0f / __builtin_sqrtf(l2);
    float x = dx * inv, y = dy * inv, z = dz * inv;
    float xx = x * x, yy = y * y, zz = z * z;
    float xy = x * y, yz = y * z, xz = x * z;
    float res[3];
#pragma unroll
    for (int ch = 0; ch < 3; ch++) {        // coefficients 0-3
        float r = C0 * v[ch] + 0.5f;
        res[ch] = r - C1 * y * v[3 + ch] + C1 * z * v[6 + ch] - C1 * x * v[9 + ch];
    }
    __builtin_amdgcn_sched_barrier(0);
    load_group(1);
#pragma unroll
    for (int ch = 0; ch < 3; ch++)          // coefficients 4-7
        res[ch] = res[ch] +
                  C2_0 * xy * v[0 + ch] +
                  C2_1 * yz * v[3 + ch] +
                  C2_2 * (2.0f * zz - xx - yy) * v[6 + ch] +
                  C2_3 * xz * v[9 + ch];
    __builtin_amdgcn_sched_barrier(0);
    load_group(2);
#pragma unroll
    for (int ch = 0; ch < 3; ch++) {        // coefficients 8-11
        float r = res[ch] + C2_4 * (xx - yy) * v[0 + ch];
        res[ch] = r +
                  C3_0 * y * (3.0f * xx - yy) * v[3 + ch] +
                  C3_1 * xy * z * v[6 + ch] +
                  C3_2 * y * (4.0f * zz - xx - yy) * v[9 + ch];
    }
    __builtin_amdgcn_sched_barrier(0);
    load_group(3);
#pragma unroll
    for (int ch = 0; ch < 3; ch++) {        // coefficients 12-15
        float r = res[ch] +
                  C3_3 * z * (2.0f * zz - 3.0f * xx - 3.0f * yy) * v[0 + ch] +
                  C3_4 * x * (4.0f * zz - xx - yy) * v[3 + ch] +
                  C3_5 * z * (xx - yy) * v[6 + ch] +
                  C3_6 * x * (xx - 3.0f * yy) * v[9 + ch];
        rgb[ch] = max_f(r, 0.0f);
    }
}

// ---- scan over workgroups ------------------------------------------------------------------------
//
// Key slots are handed out in workgroup order.  Every workgroup publishes its key count as soon
// as it knows it; one wave of the launch (the scanner: the first wave of workgroup 0, which does
// nothing else) reads the counts in order, 128 per trip to memory, and publishes for every
// workgroup the number of keys in front of it; a workgroup picks that number up after its colour
// work, when it has long been written.  Nobody but the scanner reads other workgroups' counts, so
// the wait of a workgroup is one read of one word, whatever else loads the memory system.
//
// status word: [33:32] state, [31:0] value; 0 = nothing published yet.
// The scan words hold a control word and two generations of (counts, offsets) arrays.  A launch
// works in the generation the control word names and clears the other one, which the launch
// after it will use; the scanner flips the control word when it has read the last count, i.e.
// after every workgroup of this launch has read the control word, so no workgroup of this launch
// can see the flipped value; the next launch (same stream, or otherwise ordered after this one)
// starts from it.  Nothing on the host changes from launch to launch, so a captured launch can be
// replayed.
//
// Every wait is bounded by spin_limit polls.  A wait that gives up makes the launch report a
// negative pair count: the scanner marks all offsets it can no longer compute as poisoned, a
// workgroup that gave up on its offset (or found it poisoned) writes its keys from slot 0 and
// lowers *curr_offset to INT_MIN, and the scanner's own final write of the total is a
// compare-and-swap against the starting value, so INT_MIN stays whichever comes first.
//
// A scanner that gives up does so before it has seen every count, i.e. possibly before every
// workgroup of the launch has been dispatched, so it must not hand the other generation on: a
// workgroup dispatched after a flip would take the wrong generation, clear the arrays the others
// publish in and leave words behind that the next launch would take for its own.  Instead it
// sets the "aborted" bit of the control word and leaves the generation alone.  The bit is sticky:
// every workgroup that finds it - the rest of this launch and every later launch on these scan
// words - does nothing but lower *curr_offset to INT_MIN, until the host clears the words
// (fgs_reset_scan), which is the one way back to a state in which all status words are zero.
constexpr int kControlWords = 8;          // control word + padding in front of the arrays
constexpr uint64_t kControlGeneration = 1;  // control word: which generation this launch works in ...
constexpr uint64_t kControlAborted = 2;     // ... and whether a scanner on these words has given up
constexpr uint64_t kStateCount = 1;       // key count of one workgroup
constexpr uint64_t kStateOffset = 2;      // number of keys in front of a workgroup
constexpr uint64_t kStatePoison = 3;      // the offset could not be computed
constexpr int kIntMin = -2147483647 - 1;

__device__ __forceinline__ uint64_t pack_status(uint64_t state, uint32_t value)
{
    return (state << 32) | (uint64_t)value;
}

__device__ __forceinline__ void publish(uint64_t* slot, uint64_t word)
{
    __hip_atomic_store(slot, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ uint64_t peek(const uint64_t* slot)
{
    return __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The pair count (or INT_MIN) for a host that polls for it: `mirror` is pinned host memory.
__device__ __forceinline__ void report_count(int* mirror, int value)
{
    if (mirror) __hip_atomic_store(mirror, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// The scanner: one wave.  Reads the workgroups' counts in order, kScanPerLane consecutive ones
// per lane and trip, and writes the exclusive running sum of every count that is there and has no
// gap in front of it; then goes on from the first gap.  What counts is how soon after a count an
// offset follows, i.e. the time of one trip: 128 counts per trip measured fastest on a 3M-Gaussian
// frame (0.203 ms for the launch against 0.207 with 256, 0.219 with 512 and 0.256 with 1024).
constexpr int kScanPerLane = 2;

__device__ __forceinline__ bool scan_counts(const uint64_t* counts, uint64_t* offsets, int num_blocks,
                                            int* curr_offset, int* count_mirror, unsigned spin_limit)
{
    const int lane = lane_id();
    const uint32_t start = (uint32_t)*curr_offset;      // the caller's starting offset (example.py:69 zeroes it)
    uint32_t running = start;
    unsigned spins = 0;
    int base = 0;
    bool gave_up = false;
    while (base < num_blocks) {
        const int first = base + lane * kScanPerLane;
        uint64_t w[kScanPerLane];
#pragma unroll
        for (int k = 0; k < kScanPerLane; k++) w[k] = first + k < num_blocks ? peek(counts + first + k) : 0;
        // this lane's entries that exist, and how many of them are there without a gap
        const int valid = max(0, min(kScanPerLane, num_blocks - first));
        int ready = 0;
#pragma unroll
        for (int k = 0; k < kScanPerLane; k++)
            if (ready == k && k < valid && (uint32_t)(w[k] >> 32) != 0u) ready = k + 1;
        const uint64_t gaps = ballot(ready < valid);
        const int gap_lane = gaps ? __ffsll((long long)gaps) - 1 : kWave;
        const int take = lane < gap_lane ? valid : (lane == gap_lane ? ready : 0);
        uint32_t before[kScanPerLane], lane_sum = 0;
#pragma unroll
        for (int k = 0; k < kScanPerLane; k++) {
            before[k] = lane_sum;
            if (k < take) lane_sum += (uint32_t)w[k];
        }
        const uint32_t incl = wave_inclusive_sum(lane_sum);
        const uint32_t lane_base = running + incl - lane_sum;
#pragma unroll
        for (int k = 0; k < kScanPerLane; k++)
            if (k < take) publish(offsets + first + k, pack_status(kStateOffset, lane_base + before[k]));
        running += (uint32_t)bcast_i((int)incl, kWave - 1);
        const int taken = bcast_i((int)wave_inclusive_sum((uint32_t)take), kWave - 1);
        base += taken;
        if (taken != 0) spins = 0;
        else if (++spins > spin_limit) { gave_up = true; break; }
        else __builtin_amdgcn_s_sleep(1);
    }
    if (gave_up) {
        for (int j = base + lane; j < num_blocks; j += kWave) publish(offsets + j, pack_status(kStatePoison, 0u));
        if (lane == 0) { atomicMin(curr_offset, kIntMin); report_count(count_mirror, kIntMin); }
    } else if (lane == 0) {
        // the total is known here, while workgroups are still writing their keys: a host that polls
        // the mirror can launch the sort behind this launch that much earlier
        const int found = atomicCAS(curr_offset, (int)start, (int)running);
        report_count(count_mirror, found == (int)start ? (int)running : kIntMin);
    }
    return gave_up;
}

// Executed by one lane of a workgroup: the number of keys in front of the workgroup, once the
// scanner has written it.  *failed is set when it did not come within spin_limit polls or is
// poisoned.
__device__ __forceinline__ uint32_t wait_for_offset(const uint64_t* slot, unsigned spin_limit, bool* failed)
{
    unsigned spins = 0;
    for (;;) {
        const uint64_t word = peek(slot);
        const uint32_t state = (uint32_t)(word >> 32) & 3u;
        if (state == kStateOffset) return (uint32_t)word;
        if (state == kStatePoison || ++spins > spin_limit) { *failed = true; return 0u; }
        __builtin_amdgcn_s_sleep(2);
    }
}

__global__ __launch_bounds__(kBlock) void preprocess_kernel(
    int P,
    const float* __restrict__ positions,
    const float* __restrict__ shs,
    const float* __restrict__ opacities,
    const float* __restrict__ cov3ds,
    Camera cam,
    float* __restrict__ points_xy,
    float* __restrict__ rgb_depth,
    float* __restrict__ conic_opacity,
    uint64_t* __restrict__ keys,
    uint32_t* __restrict__ values,
    int* __restrict__ curr_offset,
    int64_t capacity,            // <= 0: unchecked
    uint64_t* __restrict__ scan_words,     // control word, then two generations of (counts, offsets), status_capacity words each
    int status_capacity,
    int num_blocks,                        // workgroups that hold Gaussians; the grid has one more, the scanner's
    unsigned spin_limit,
    int* __restrict__ count_mirror)        // pinned host memory that also receives the pair count, or null
{
    __shared__ uint32_t s_wave_total[kWavesPerBlock];
    __shared__ uint32_t s_block_base;
    __shared__ uint32_t s_stash[kWavesPerBlock][kStashCap];     // hits of the flat candidates, in emission order
    __shared__ uint64_t s_hits[kWavesPerBlock][kStashCap / kWave + 1];
    // flat candidate -> lane that owns it; free again after the flat tile tests, when the listed
    // rectangles use it for their column and row spans
    __shared__ __align__(4) uint8_t s_owner[kWavesPerBlock][kStashCap];
    // rectangles too big for one wave: parameters, per-wave hit counts, first key slot
    __shared__ float s_huge_f[kHugeCap][6];
    __shared__ int s_huge_i[kHugeCap][4];
    __shared__ uint32_t s_huge_u[kHugeCap][3];                  // depth bits, Gaussian index, first slot
    __shared__ uint32_t s_huge_cnt[kHugeCap][kWavesPerBlock];
    __shared__ int s_huge_spans[kHugeCap];                      // 1: the tiles that pass are found from column and row spans
    __shared__ int s_nhuge;
    __shared__ int s_centre[2];                                 // column and row of a listed rectangle that hold its centre
    __shared__ uint32_t s_control;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    if (tid == 0) {
        s_nhuge = 0;
        s_control = (uint32_t)peek(scan_words);     // one read per workgroup: all its threads must agree on it
    }
    __syncthreads();
    const uint32_t control = s_control;
    if (control & kControlAborted) {
        // a scanner on these words gave up (in this launch or an earlier one): touch nothing
        if (tid == 0) { atomicMin(curr_offset, kIntMin); if (blockIdx.x == 0) report_count(count_mirror, kIntMin); }
        return;
    }

    // this launch's generation of the scan words; the other one is cleared for the launch that follows
    const uint32_t which = control & (uint32_t)kControlGeneration;
    uint64_t* const counts = scan_words + kControlWords + (size_t)which * 2 * status_capacity;
    uint64_t* const offsets = counts + status_capacity;
    {
        uint64_t* const other = scan_words + kControlWords + (size_t)(which ^ 1u) * 2 * status_capacity;
        const long long words = 2LL * status_capacity, threads = (long long)kBlock * (num_blocks + 1);
        for (long long w = (long long)blockIdx.x * kBlock + tid; w < words; w += threads) other[w] = 0;
    }
    // Workgroup 0 is the scanner.  The hardware dispatches workgroups in index order, so it runs
    // from the start, and every workgroup whose count it waits for is running or finished when a
    // later one waits for its offset (and every wait is bounded in any case).
    if (blockIdx.x == 0) {
        if (wave == 0) {
            const bool gave_up = scan_counts(counts, offsets, num_blocks, curr_offset, count_mirror, spin_limit);
            // Read every count: every workgroup has read the control word by now, so the other
            // generation can be handed to the next launch.  Gave up: workgroups may still be
            // dispatched; the generation stays and the words are marked unusable.
            if (lane == 0) publish(scan_words, gave_up ? (uint64_t)which | kControlAborted : (uint64_t)(which ^ 1u));
        }
        return;
    }
    const int ticket = (int)blockIdx.x - 1;
    // Every later workgroup's offset waits for this one's count: until the count is published the
    // waves ask for a higher issue priority than the waves that are past that point.
    __builtin_amdgcn_s_setprio(2);
    const int idx = ticket * kBlock + tid;
    // tile coordinates travel in 12 bits each and tile indices in 26 when candidates are laid flat
    const bool pack_ok = cam.gx <= 4096 && cam.gy <= 4096 && (long long)cam.gx * cam.gy <= (1 << 26);

    // ---- per-Gaussian state (preprocess.cu:282-316) ----
    bool cand = false;           // passed both culls and has a non-empty candidate rectangle
    float px = 0.f, py = 0.f, pz = 0.f;
    float depth = 0.f;
    float cx = 0.f, cy = 0.f;
    float conx = 0.f, cony = 0.f, conz = 0.f;
    float power = 0.f, log2_op = 0.f;
    int rminx = 0, rminy = 0, rw = 0, rh = 0;

    if (idx < P) {
        px = positions[3 * (size_t)idx + 0];
        py = positions[3 * (size_t)idx + 1];
        pz = positions[3 * (size_t)idx + 2];
        // all per-Gaussian inputs are requested up front so that their latencies overlap
        const float opacity = opacities[idx];
        const float2* cv = reinterpret_cast<const float2*>(cov3ds + 6 * (size_t)idx);
        const float2 s01 = cv[0], s23 = cv[1], s45 = cv[2];
        const float* m = cam.view;
        float t[3];
        t[0] = m[0] * px + m[4] * py + m[8] * pz + m[12];
        t[1] = m[1] * px + m[5] * py + m[9] * pz + m[13];
        t[2] = m[2] * px + m[6] * py + m[10] * pz + m[14];
        depth = t[2];
        if (t[2] > 0.2f) {
            if (!(255.0f * opacity < 1.0f)) {
                const float* q = cam.proj;
                float hx = q[0] * px + q[4] * py + q[8] * pz + q[12];
                float hy = q[1] * px + q[5] * py + q[9] * pz + q[13];
                float hw = q[3] * px + q[7] * py + q[11] * pz + q[15];
                float p_w = 1.0f / (hw + 0.0000001f);
                float projx = hx * p_w, projy = hy * p_w;

                float s[6];
                s[0] = s01.x; s[1] = s01.y; s[2] = s23.x; s[3] = s23.y; s[4] = s45.x; s[5] = s45.y;
                float c00, c01, c11;
                cov2d(t, cam, s, c00, c01, c11);

                float det = c00 * c11 - c01 * c01;
                float det_inv = 1.0f / det;
                conx = c11 * det_inv;
                cony = -c01 * det_inv;
                conz = c00 * det_inv;

                log2_op = log2_det(opacity);
                power = 0.69314718055f * 8.0f + 0.69314718055f * log2_op;
                int ext_x = to_int_sat(1.414214f * __builtin_sqrtf(c00 * power) + 1.0f);
                int ext_y = to_int_sat(1.414214f * __builtin_sqrtf(c11 * power) + 1.0f);

                cx = ndc_to_pix(projx, cam.W);
                cy = ndc_to_pix(projy, cam.H);
                // preprocess.cu:90-100
                rminx = min(cam.gx, max(0, to_int_sat((cx - (float)ext_x) / (float)cam.bx)));
                rminy = min(cam.gy, max(0, to_int_sat((cy - (float)ext_y) / (float)cam.by)));
                // (the "+ 1" wraps at INT_MAX, as the integer add of the reference's device does: written out, not left to overflow)
                int rmaxx = min(cam.gx, max(0, (int)((uint32_t)to_int_sat((cx + (float)ext_x) / (float)cam.bx) + 1u)));
                int rmaxy = min(cam.gy, max(0, (int)((uint32_t)to_int_sat((cy + (float)ext_y) / (float)cam.by) + 1u)));
                rw = rmaxx - rminx;
                rh = rmaxy - rminy;
                cand = rw * rh > 0;
            }
        }
    }
    // a rectangle with both extents negative has a positive product but no tiles
    const bool has_tiles = cand && rw > 0;
    const int area = has_tiles ? rw * rh : 0;

    // ---- count keys ----
    // Rectangles of up to 64 tiles are "flat": their candidates are laid end to end over the wave
    // (Gaussian-major, row-major inside a Gaussian - the order keys are emitted in), so every lane
    // tests one candidate per step whatever the mix of rectangle sizes.  Hits are compacted into
    // an LDS stash as (tile << 6 | owner lane) and written out once the slots are known.  A wave
    // stashes at most kStashCap candidates; what does not fit, and every larger rectangle, is
    // tested by the whole wave, 64 tiles a step, once to count and once more to emit.
    const bool flat_ok = has_tiles && area <= kWave && pack_ok;
    uint32_t cand_incl = wave_inclusive_sum(flat_ok ? (uint32_t)area : 0u);
    const bool flat = flat_ok && cand_incl <= (uint32_t)kStashCap;
    // A rectangle of thousands of tiles would keep one wave busy for a long time while every later
    // workgroup waits for this workgroup's count: such rectangles are put on a list and all waves
    // of the workgroup share the testing, a contiguous quarter of the tiles each.
    int huge_slot = -1;
    if (has_tiles && area > kHugeMin && area < (1 << 26)) {
        const int e = atomicAdd(&s_nhuge, 1);
        if (e < kHugeCap) {
            huge_slot = e;
            s_huge_f[e][0] = cx; s_huge_f[e][1] = cy; s_huge_f[e][2] = conx;
            s_huge_f[e][3] = cony; s_huge_f[e][4] = conz; s_huge_f[e][5] = power;
            s_huge_i[e][0] = rminx; s_huge_i[e][1] = rminy; s_huge_i[e][2] = rw; s_huge_i[e][3] = area;
            s_huge_u[e][0] = __float_as_uint(depth); s_huge_u[e][1] = (uint32_t)idx;
            // Spans need 2a > 0 for both edge directions and values that cannot overflow on the
            // way to t1, t2 (the monotonicity argument assumes no NaN), and room for one word
            // per column and row; everything else is tested tile by tile.
            const float big = 1e30f;
            s_huge_spans[e] = conx > 0.0f && conz > 0.0f && conx < big && conz < big && fabsf(cony) < big &&
                              fabsf(cx) < 1e9f && fabsf(cy) < 1e9f && fabsf(power) < big &&
                              rw + rh <= kSpanWords;
        }
    }
    const bool large = has_tiles && !flat && huge_slot < 0;
    // lanes that drop out are at the end of the scan order, so the prefix of the others is unchanged
    const uint32_t cand_excl = cand_incl - (uint32_t)area;
    const uint64_t flat_lanes = ballot(flat);
    const int last_flat = flat_lanes ? 63 - __builtin_clzll(flat_lanes) : 0;
    const int n_cand = flat_lanes ? bcast_i((int)cand_incl, last_flat) : 0;

    uint8_t* owner_of = s_owner[wave];
    uint32_t* stash = s_stash[wave];
    uint64_t* hit_words = s_hits[wave];
    if (flat)
        for (int k = 0; k < area; k++) owner_of[cand_excl + k] = (uint8_t)lane;
    __builtin_amdgcn_wave_barrier();

    const uint32_t rect_pack = (uint32_t)rminx | ((uint32_t)rminy << 12) | ((uint32_t)(rw - 1) << 24);
    int n_stash = 0;
    for (int c0 = 0; c0 < n_cand; c0 += kWave) {
        const int c = c0 + lane;
        const bool live = c < n_cand;
        const int own = live ? (int)owner_of[c] : lane;
        const float gcx = __shfl(cx, own), gcy = __shfl(cy, own);
        const float gconx = __shfl(conx, own), gcony = __shfl(cony, own), gconz = __shfl(conz, own);
        const float gpower = __shfl(power, own);
        const uint32_t grect = (uint32_t)__shfl((int)rect_pack, own);
        const int k = c - __shfl((int)cand_excl, own);
        const int gminx = (int)(grect & 0xfffu), gminy = (int)((grect >> 12) & 0xfffu), grw = (int)(grect >> 24) + 1;
        // k / grw for 0 <= k < 64, 1 <= grw <= 64: (k + 0.5) / grw is at least 1/128 away from an
        // integer, far more than the error of the approximate reciprocal
        const int ty = (int)(((float)k + 0.5f) * __builtin_amdgcn_rcpf((float)grw));
        const int tx = k - ty * grw;
        const bool hit = live && tile_hit(gminx + tx, gminy + ty, cam.bx, cam.by, gcx, gcy, gconx, gcony, gconz, gpower);
        const uint64_t hits = ballot(hit);
        if (hit) stash[n_stash + popc_below(hits)] = ((uint32_t)((gminy + ty) * cam.gx + gminx + tx) << 6) | (uint32_t)own;
        if (lane == 0) hit_words[c0 / kWave] = hits;
        n_stash += __popcll(hits);
    }
    __builtin_amdgcn_wave_barrier();

    uint32_t count = 0;
    if (flat) {      // hits among this lane's candidates [cand_excl, cand_excl + area)
        const int w0 = (int)(cand_excl >> 6), b0 = (int)(cand_excl & 63u);
        uint64_t m = hit_words[w0] >> b0;
        if (b0 + area > kWave) m |= hit_words[w0 + 1] << (kWave - b0);
        if (area < kWave) m &= (1ull << area) - 1ull;
        count = (uint32_t)__popcll(m);
    }
    const uint32_t flat_count = count;
    const uint64_t large_lanes = ballot(large);
    for (uint64_t todo = large_lanes; todo; todo &= todo - 1) {
        const int src = __ffsll((long long)todo) - 1;
        const float gcx = bcast_f(cx, src), gcy = bcast_f(cy, src);
        const float gconx = bcast_f(conx, src), gcony = bcast_f(cony, src), gconz = bcast_f(conz, src);
        const float gpower = bcast_f(power, src);
        const int gminx = bcast_i(rminx, src), gminy = bcast_i(rminy, src);
        const int grw = bcast_i(rw, src), garea = bcast_i(area, src);
        uint32_t total = 0;
        for (int base = 0; base < garea; base += kWave) {
            const int j = base + lane;
            bool ok = false;
            if (j < garea) {
                int tx, ty;
                div_mod(j, grw, ty, tx);
                ok = tile_hit(gminx + tx, gminy + ty, cam.bx, cam.by, gcx, gcy, gconx, gcony, gconz, gpower);
            }
            total += (uint32_t)__popcll(ballot(ok));
        }
        if (lane == src) count = total;
    }

    // the listed rectangles: wave w counts tiles [w*part, (w+1)*part) of each
    __syncthreads();
    const int n_huge = min(s_nhuge, kHugeCap);
    uint32_t* const spans = reinterpret_cast<uint32_t*>(&s_owner[0][0]);
    // Fills spans[0, rw) with the rows that pass the vertical-edge test in each column of the
    // rectangle and spans[rw, rw + rh) with the columns that pass the horizontal-edge test in
    // each row.  All threads of the workgroup call it; barriers before and after.
    auto fill_spans = [&](int e) {
        const float gcx = s_huge_f[e][0], gcy = s_huge_f[e][1];
        const float gconx = s_huge_f[e][2], gcony = s_huge_f[e][3], gconz = s_huge_f[e][4];
        const float w = 2.0f * s_huge_f[e][5];
        const int gminx = s_huge_i[e][0], gminy = s_huge_i[e][1], grw = s_huge_i[e][2];
        const int grh = s_huge_i[e][3] / grw;
        __syncthreads();
        for (int i = tid; i < grw + grh; i += kBlock)
            spans[i] = i < grw ? edge_span(gconz, gcony, gconx, gcx, gcy, gminx + i, cam.bx, gminy, cam.by, grh, w)
                               : edge_span(gconx, gcony, gconz, gcy, gcx, gminy + i - grw, cam.by, gminx, cam.bx, grw, w);
        __syncthreads();
    };
    // Walks the tiles of listed rectangle e that are this wave's share, in row-major order, and
    // calls visit(tx, ty, passes) once per step of 64 tiles with every lane's own tile.
    //  * With spans the share is a quarter of the rows.  A step covers 64 columns of one row;
    //    it is skipped when neither the column spans of those columns reach the row (their
    //    union is kept per 64 columns) nor the row's own span reaches the columns.
    //  * Without spans the share is a quarter of the tiles, each tested in full.
    auto walk_listed = [&](int e, bool from_spans, auto&& visit) {
        const int gminx = s_huge_i[e][0], gminy = s_huge_i[e][1], grw = s_huge_i[e][2], garea = s_huge_i[e][3];
        if (from_spans) {
            const int grh = garea / grw;
            const int chunks = (grw + kWave - 1) / kWave;
            // lane c keeps the union of the column spans of columns 64c .. 64c + 63 (first row, last row)
            uint32_t chunk_lo = 0x7fffu, chunk_hi = 0;
            for (int c = 0; c < chunks; c++) {
                const int x = c * kWave + lane;
                const uint32_t col = x < grw ? spans[x] : 1u;
                uint32_t lo = col & 0x7fffu, hi = (col >> 15) & 0x7fffu;
                if (lo > hi) { lo = 0x7fffu; hi = 0; }
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) {
                    lo = min(lo, (uint32_t)__shfl_xor((int)lo, o));
                    hi = max(hi, (uint32_t)__shfl_xor((int)hi, o));
                }
                if (lane == c) { chunk_lo = lo; chunk_hi = hi; }
            }
            const int rows = (grh + kWavesPerBlock - 1) / kWavesPerBlock;
            const int y_lo = min(grh, wave * rows), y_hi = min(grh, y_lo + rows);
            for (int ty = y_lo; ty < y_hi; ty++) {
                const uint32_t row = spans[grw + ty];
                const uint32_t rlo = row & 0x7fffu, rhi = (row >> 15) & 0x7fffu;
                // one lane per chunk decides whether the step is needed; the wave walks the needed ones
                const bool columns_reach = (uint32_t)ty >= chunk_lo && (uint32_t)ty <= chunk_hi;
                const bool row_reaches = rlo <= rhi && rlo <= (uint32_t)(lane * kWave + kWave - 1) && rhi >= (uint32_t)(lane * kWave);
                uint64_t needed = ballot(lane < chunks && (columns_reach || row_reaches || (row >> 30) != 0));
                for (; needed; needed &= needed - 1) {
                    const int c = __ffsll((long long)needed) - 1;
                    const int tx = c * kWave + lane;
                    bool ok = false;
                    if (tx < grw) {
                        const uint32_t col = spans[tx];
                        const bool by_column = (uint32_t)ty >= (col & 0x7fffu) && (uint32_t)ty <= ((col >> 15) & 0x7fffu);
                        const bool by_row = (uint32_t)tx >= rlo && (uint32_t)tx <= rhi;
                        ok = by_column || by_row || ((col & row) >> 30) != 0;
                    }
                    visit(tx, ty, ok);
                }
            }
        } else {
            const int part = ((garea + kWavesPerBlock - 1) / kWavesPerBlock + kWave - 1) / kWave * kWave;
            const int j_lo = min(garea, wave * part), j_hi = min(garea, j_lo + part);
            for (int base = j_lo; base < j_hi; base += kWave) {
                const int j = base + lane;
                bool ok = false;
                int tx = 0, ty = 0;
                if (j < j_hi) {
                    div_mod(j, grw, ty, tx);
                    ok = tile_hit(gminx + tx, gminy + ty, cam.bx, cam.by, s_huge_f[e][0], s_huge_f[e][1],
                                  s_huge_f[e][2], s_huge_f[e][3], s_huge_f[e][4], s_huge_f[e][5]);
                }
                visit(tx, ty, ok);
            }
        }
    };
    // How many tiles of listed rectangle e pass, per quarter of its rows (the quarters are the
    // waves' shares when the keys are written).  From the spans no tile has to be visited: a tile
    // passes if its row's span holds its column, or its column's span holds its row, or it is
    // the tile of the centre.  The rows add up their spans; every column goes down its own span
    // and counts the rows whose span does not hold it already.
    auto count_from_spans = [&](int e) {
        const int grw = s_huge_i[e][2];
        const int grh = s_huge_i[e][3] / grw;
        const int rows = (grh + kWavesPerBlock - 1) / kWavesPerBlock;
        auto add = [&](int ty, uint32_t v) {
            int q = 0;
#pragma unroll
            for (int k = 1; k < kWavesPerBlock; k++) q += ty >= k * rows ? 1 : 0;
            atomicAdd(&s_huge_cnt[e][q], v);
        };
        for (int ty = tid; ty < grh; ty += kBlock) {
            const uint32_t row = spans[grw + ty];
            const uint32_t rlo = row & 0x7fffu, rhi = (row >> 15) & 0x7fffu;
            if (rlo <= rhi) add(ty, rhi - rlo + 1u);
            if (row >> 30) s_centre[1] = ty;
        }
        for (int tx = tid; tx < grw; tx += kBlock) {
            const uint32_t col = spans[tx];
            const uint32_t clo = col & 0x7fffu, chi = (col >> 15) & 0x7fffu;
            if (col >> 30) s_centre[0] = tx;
            for (uint32_t ty = clo; ty <= chi; ty++) {          // an empty span is 1 .. 0
                const uint32_t row = spans[grw + (int)ty];
                const uint32_t rlo = row & 0x7fffu, rhi = (row >> 15) & 0x7fffu;
                if (!(rlo <= rhi && (uint32_t)tx >= rlo && (uint32_t)tx <= rhi)) add((int)ty, 1u);
            }
        }
        __syncthreads();
        if (tid == 0 && s_centre[0] >= 0 && s_centre[1] >= 0) {
            // the tile of the centre, unless a span has counted it
            const int tx = s_centre[0], ty = s_centre[1];
            const uint32_t col = spans[tx], row = spans[grw + ty];
            const bool by_column = (uint32_t)ty >= (col & 0x7fffu) && (uint32_t)ty <= ((col >> 15) & 0x7fffu);
            const bool by_row = (uint32_t)tx >= (row & 0x7fffu) && (uint32_t)tx <= ((row >> 15) & 0x7fffu);
            if (!by_column && !by_row) {
                int q = 0;
                while (ty >= (q + 1) * rows) q++;
                atomicAdd(&s_huge_cnt[e][q], 1u);
            }
        }
    };
    for (int e = 0; e < n_huge; e++) {
        if (s_huge_spans[e] != 0) {
            if (tid < kWavesPerBlock) s_huge_cnt[e][tid] = 0;
            if (tid == 0) { s_centre[0] = -1; s_centre[1] = -1; }
            fill_spans(e);
            count_from_spans(e);
            continue;
        }
        uint32_t total = 0;
        walk_listed(e, false, [&](int, int, bool ok) { total += (uint32_t)__popcll(ballot(ok)); });
        if (lane == 0) s_huge_cnt[e][wave] = total;
    }
    if (n_huge > 0) {
        __syncthreads();
        if (huge_slot >= 0) {
            count = 0;
            for (int w = 0; w < kWavesPerBlock; w++) count += s_huge_cnt[huge_slot][w];
        }
    }

    // ---- slots: wave scan, block scan, scan over workgroups ----
    uint32_t incl = wave_inclusive_sum(count);
    const uint32_t wave_total = (uint32_t)bcast_i((int)incl, kWave - 1);
    if (lane == 0) s_wave_total[wave] = wave_total;
    __syncthreads();

    uint32_t wave_base = 0, block_total = 0;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; w++) {
        uint32_t t = s_wave_total[w];
        if (w < wave) wave_base += t;
        block_total += t;
    }

    // The workgroup's count is published right away; its offset is picked up after the colour
    // work below, when the scanner has long written it.
    if (tid == 0) publish(counts + ticket, pack_status(kStateCount, block_total));
    __builtin_amdgcn_s_setprio(0);

    // ---- attributes of Gaussians that emit a key, and of every Gaussian whose rectangle is a
    // single tile, hit or not (preprocess.cu:317, 411-417: vertex_valid starts as single_tile) ----
    if (count > 0 || area == 1) {
        constexpr float log2e = 1.4426950216293334961f;
        reinterpret_cast<float2*>(points_xy)[idx] = make_float2(cx, cy);
        reinterpret_cast<float4*>(conic_opacity)[idx] =
            make_float4((-0.5f * log2e) * conx, -log2e * cony, (-0.5f * log2e) * conz, log2_op);
        float rgb[3];
        sh_to_rgb(shs + 48 * (size_t)idx, px, py, pz, cam, rgb);
        reinterpret_cast<float4*>(rgb_depth)[idx] = make_float4(rgb[0], rgb[1], rgb[2], depth);
    }

    if (tid == 0) {
        bool failed = false;
        s_block_base = wait_for_offset(offsets + ticket, spin_limit, &failed);
        if (failed) { atomicMin(curr_offset, kIntMin); report_count(count_mirror, kIntMin); }
    }
    __syncthreads();
    const uint32_t my_slot = s_block_base + wave_base + (incl - count);

    // ---- emit ----
    const uint64_t cap = capacity > 0 ? (uint64_t)capacity : ~0ull;
    const uint32_t depth_bits = __float_as_uint(depth);
    if (n_huge > 0) {
        if (huge_slot >= 0) s_huge_u[huge_slot][2] = my_slot;
        __syncthreads();
        for (int e = 0; e < n_huge; e++) {
            const bool from_spans = s_huge_spans[e] != 0;
            if (from_spans) fill_spans(e);
            const int gminx = s_huge_i[e][0], gminy = s_huge_i[e][1];
            const uint32_t gdepth = s_huge_u[e][0], gidx = s_huge_u[e][1];
            uint64_t slot = s_huge_u[e][2];
            for (int w = 0; w < wave; w++) slot += s_huge_cnt[e][w];
            if (s_huge_cnt[e][wave] == 0) continue;
            walk_listed(e, from_spans, [&](int tx, int ty, bool ok) {
                const uint64_t hits = ballot(ok);
                if (ok) {
                    const uint64_t dst = slot + (uint64_t)popc_below(hits);
                    if (dst < cap) {
                        keys[dst] = ((uint64_t)(uint32_t)((gminy + ty) * cam.gx + gminx + tx) << 32) | gdepth;
                        values[dst] = gidx;
                    }
                }
                slot += (uint64_t)__popcll(hits);
            });
        }
    }
    {
        // stash entry e of owner o goes to slot(o) + (e - entries before o's first)
        uint32_t before = wave_inclusive_sum(flat_count);
        const uint32_t delta = my_slot - (before - flat_count);
        const uint32_t gidx_base = (uint32_t)(ticket * kBlock + wave * kWave);
        for (int e0 = 0; e0 < n_stash; e0 += kWave) {
            const int e = e0 + lane;
            const bool live = e < n_stash;
            const uint32_t entry = live ? stash[e] : (uint32_t)lane;
            const int own = (int)(entry & 63u);
            const uint32_t odelta = (uint32_t)__shfl((int)delta, own);
            const uint32_t odepth = (uint32_t)__shfl((int)depth_bits, own);
            const uint64_t dst = (uint64_t)(odelta + (uint32_t)e);
            if (live && dst < cap) {
                keys[dst] = ((uint64_t)(entry >> 6) << 32) | odepth;
                values[dst] = gidx_base + (uint32_t)own;
            }
        }
    }
    for (uint64_t todo = large_lanes; todo; todo &= todo - 1) {
        const int src = __ffsll((long long)todo) - 1;
        if (bcast_i((int)count, src) == 0) continue;
        const float gcx = bcast_f(cx, src), gcy = bcast_f(cy, src);
        const float gconx = bcast_f(conx, src), gcony = bcast_f(cony, src), gconz = bcast_f(conz, src);
        const float gpower = bcast_f(power, src);
        const int gminx = bcast_i(rminx, src), gminy = bcast_i(rminy, src);
        const int grw = bcast_i(rw, src), garea = bcast_i(area, src);
        const uint32_t gdepth = (uint32_t)bcast_i((int)depth_bits, src);
        const uint32_t gidx = (uint32_t)(ticket * kBlock + wave * kWave + src);
        uint64_t slot = (uint32_t)bcast_i((int)my_slot, src);
        for (int base = 0; base < garea; base += kWave) {
            const int j = base + lane;
            bool ok = false;
            int tx = 0, ty = 0;
            if (j < garea) {
                div_mod(j, grw, ty, tx);
                ok = tile_hit(gminx + tx, gminy + ty, cam.bx, cam.by, gcx, gcy, gconx, gcony, gconz, gpower);
            }
            const uint64_t hits = ballot(ok);
            if (ok) {
                const uint64_t dst = slot + (uint64_t)popc_below(hits);
                if (dst < cap) {
                    keys[dst] = ((uint64_t)(uint32_t)((gminy + ty) * cam.gx + gminx + tx) << 32) | gdepth;
                    values[dst] = gidx;
                }
            }
            slot += (uint64_t)__popcll(hits);
        }
    }

}

// ---- scan words, one set per (device, stream) -------------------------------------------------------
//
// Launches on one stream follow each other, so they can share one set of scan words; launches on
// different streams of a device may overlap in time and get a set each.  A set is allocated on
// the first call on its stream; when a larger P arrives a larger set is allocated and the stream
// uses that one from then on.  No set is ever freed: a HIP graph captured on the stream holds the
// address of the set its launch used in its kernel node, and replaying it after a free would make
// every workgroup read and write freed memory.  A retired set costs 32 bytes per 256 Gaussians of
// the P it was sized for and keeps serving the graphs that know it (its own control word and
// generations stay consistent: launches on one stream, replayed or not, follow each other).

struct Scratch {
    uint64_t* words = nullptr;      // control word (+ padding), then two generations of (counts, offsets)
    size_t capacity = 0;            // workgroups each of the four arrays holds
};

__global__ __launch_bounds__(256) void clear_words_kernel(uint64_t* words, size_t n)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) words[i] = 0;
}

// Zeroes n words on the stream with a kernel (not a memset node, so that it may be captured).
int clear_words(uint64_t* words, size_t n, hipStream_t stream)
{
    size_t blocks = (n + 255) / 256;
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(clear_words_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, words, n);
    return check_hip(hipGetLastError(), "clear_words_kernel launch");
}

constexpr int kMaxDevices = 64;
std::map<StreamKey, Scratch> g_scratch;
std::vector<uint64_t*> g_retired;   // sets replaced by larger ones: kept, since captured graphs may hold their addresses
std::mutex g_mutex;
std::atomic<unsigned> g_spin_limit{kSpinLimit};

// *out stays null when the stream is being captured and has no (large enough) set yet: nothing
// can be allocated then, and the caller falls back to the words inside the library's image.
int acquire_scratch(int device, int num_blocks, hipStream_t stream, Scratch** out)
{
    *out = nullptr;
    Scratch& s = g_scratch[stream_key(device, stream)];
    if (s.capacity < (size_t)num_blocks) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        if (stream) FGS_HIP_TRY(hipStreamIsCapturing(stream, &capture));
        if (capture != hipStreamCaptureStatusNone) return FGS_OK;
        size_t cap = 4096;
        while (cap < (size_t)num_blocks) cap <<= 1;
        const size_t words = kControlWords + 4 * cap;
        uint64_t* fresh = nullptr;
        if (hipMalloc((void**)&fresh, words * sizeof(uint64_t)) != hipSuccess) {
            (void)hipGetLastError();
            return fail(FGS_E_NOMEM, "cannot allocate %zu bytes of scan status", words * sizeof(uint64_t));
        }
        // cleared on the stream itself, in front of the launch that uses it first; the set in use
        // so far (if any) is left alone and alive for the launches and graphs that hold its address
        int rc = clear_words(fresh, words, stream);
        if (rc != FGS_OK) return rc;
        if (s.words) g_retired.push_back(s.words);
        s.words = fresh;
        s.capacity = cap;
    }
    *out = &s;
    return FGS_OK;
}

} // namespace

void camera_matrices(const float pos[3], const float rot[9], int width, int height,
                     float fx, float fy, float zFar, float zNear, float view[16], float proj[16])
{
    // View matrix (preprocess.cu:420-427).  The nine rotation floats fill GLM columns
    // (pybind.cpp:140-143), so column c of the upper 3x3 is rot[3c..3c+2]; the translation column
    // is rotation * (-position) with GLM's mat3 * vec3 order (type_mat3x3.inl:468-474).
    const float nx = -pos[0], ny = -pos[1], nz = -pos[2];
    for (int c = 0; c < 3; c++) {
        view[4 * c + 0] = rot[3 * c + 0];
        view[4 * c + 1] = rot[3 * c + 1];
        view[4 * c + 2] = rot[3 * c + 2];
        view[4 * c + 3] = 0.0f;
    }
    for (int r = 0; r < 3; r++) view[12 + r] = rot[r] * nx + rot[3 + r] * ny + rot[6 + r] * nz;
    view[15] = 1.0f;

    // Projection (preprocess.cu:429-448): proj = transpose(P) * view, GLM mat4 product order
    // (type_mat4x4.inl:630-648).  A[c][r] below is transpose(P) in [col][row] storage.
    const float top = (float)height / (2.0f * fy) * zNear;
    const float bottom = -top;
    const float right = (float)width / (2.0f * fx) * zNear;
    const float left = -right;
    float A[4][4] = {};
    A[0][0] = 2.0f * zNear / (right - left);
    A[1][1] = 2.0f * zNear / (top - bottom);
    A[2][0] = (right + left) / (right - left);
    A[2][1] = (top + bottom) / (top - bottom);
    A[2][3] = 1.0f;
    A[2][2] = 1.0f * zFar / (zFar - zNear);
    A[3][2] = -(zFar * zNear) / (zFar - zNear);
    for (int c = 0; c < 4; c++)
        for (int r = 0; r < 4; r++)
            proj[4 * c + r] = A[0][r] * view[4 * c + 0] + A[1][r] * view[4 * c + 1] +
                              A[2][r] * view[4 * c + 2] + A[3][r] * view[4 * c + 3];
}

} // namespace fgs

extern "C" void fgs_camera_matrices(const float cam_position[3], const float cam_rotation[9],
                                    int width, int height, float focal_x, float focal_y, float zFar, float zNear,
                                    float view[16], float proj[16])
{
    fgs::camera_matrices(cam_position, cam_rotation, width, height, focal_x, focal_y, zFar, zNear, view, proj);
}

namespace fgs {
namespace {

// ---- scan status held in the library's own image, for callers that cannot allocate ----------------
//
// The same scan words as the allocated ones, as a file-scope device array: one copy per
// GPU that loads the library, zero when the code object is loaded, kept until the process ends.
// In host code the array's name is only a handle; the device address comes from
// hipGetSymbolAddress, once per device with that device current.
constexpr int kStaticBlocks = 1 << 16;                        // workgroups each of the four arrays holds
constexpr int kStaticMaxP = kStaticBlocks * kBlock;           // 16 777 216 Gaussians
static __device__ __align__(256) uint64_t scratch[kControlWords + 4 * kStaticBlocks];
uint64_t* g_static_words[kMaxDevices];                        // device address of `scratch`, per device

int static_scratch(int device, uint64_t** out)
{
    if (!g_static_words[device]) {
        void* ptr = nullptr;
        FGS_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return fail(FGS_E_HIP, "hipGetSymbolAddress returned a null address for the scan status");
        g_static_words[device] = (uint64_t*)ptr;
    }
    *out = g_static_words[device];
    return FGS_OK;
}

__global__ void mirror_count_kernel(const int* curr_offset, int* count_mirror)
{
    report_count(count_mirror, *curr_offset);
}

int preprocess_impl(bool allocate, const char* who, int P,
                    const float* positions, const float* shs, const float* opacities, const float* cov3Ds,
                    int width, int height, int block_x, int block_y,
                    const float cam_position[3], const float cam_rotation[9],
                    float focal_x, float focal_y, float zFar, float zNear,
                    float* points_xy, float* rgb_depth, float* conic_opacity,
                    uint64_t* gaussian_keys_unsorted, uint32_t* gaussian_values_unsorted,
                    int* curr_offset, int64_t key_capacity, int* count_mirror, void* stream)
{
    if (P < 0) return fail(FGS_E_INVALID, "%s: P = %d is negative", who, P);
    if (width <= 0 || height <= 0 || block_x <= 0 || block_y <= 0)
        return fail(FGS_E_INVALID, "%s: width/height/block must be positive (got %d x %d, block %d x %d)",
                    who, width, height, block_x, block_y);
    if (!cam_position || !cam_rotation) return fail(FGS_E_INVALID, "%s: null camera", who);
    if (!curr_offset) return fail(FGS_E_INVALID, "%s: null curr_offset", who);
    if (P > 0 && (!positions || !shs || !opacities || !cov3Ds || !points_xy || !rgb_depth || !conic_opacity ||
                  !gaussian_keys_unsorted || !gaussian_values_unsorted))
        return fail(FGS_E_INVALID, "%s: null buffer", who);
    if (!allocate && P > kStaticMaxP)
        return fail(FGS_E_INVALID, "%s: P = %d exceeds the %d Gaussians the built-in scan status holds "
                                   "(fgs_preprocess has no such limit)", who, P, kStaticMaxP);
    int* mirror_on_device = nullptr;
    if (count_mirror) {
        void* mapped = nullptr;
        if (hipHostGetDevicePointer(&mapped, count_mirror, 0) != hipSuccess || !mapped) {
            (void)hipGetLastError();
            return fail(FGS_E_INVALID, "%s: count_mirror must be pinned host memory (hipHostMalloc)", who);
        }
        mirror_on_device = (int*)mapped;
        *(volatile int*)count_mirror = FGS_COUNT_PENDING;      // whatever an earlier frame left there is not this launch's count
    }
    if (P == 0) {
        if (mirror_on_device) {
            hipLaunchKernelGGL(mirror_count_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, (const int*)curr_offset, mirror_on_device);
            return check_hip(hipGetLastError(), "mirror_count_kernel launch");
        }
        return FGS_OK;
    }
    if (((uintptr_t)shs | (uintptr_t)rgb_depth | (uintptr_t)conic_opacity) % 16 != 0 ||
        ((uintptr_t)cov3Ds | (uintptr_t)points_xy | (uintptr_t)gaussian_keys_unsorted) % 8 != 0)
        return fail(FGS_E_INVALID, "%s: shs/rgb_depth/conic_opacity must be 16-byte aligned, "
                                   "cov3Ds/points_xy/keys 8-byte aligned", who);
    if ((long long)P + kBlock > 2147483647LL) return fail(FGS_E_INVALID, "%s: P = %d too large", who, P);

    Camera cam;
    camera_matrices(cam_position, cam_rotation, width, height, focal_x, focal_y, zFar, zNear, cam.view, cam.proj);
    cam.campos[0] = cam_position[0]; cam.campos[1] = cam_position[1]; cam.campos[2] = cam_position[2];
    cam.W = width; cam.H = height; cam.bx = block_x; cam.by = block_y;
    cam.gx = (width + block_x - 1) / block_x;      // preprocess.cu:461
    cam.gy = (height + block_y - 1) / block_y;
    cam.tan_fovx = (float)width / (2.0f * focal_x);   // preprocess.cu:465-466
    cam.tan_fovy = (float)height / (2.0f * focal_y);
    cam.fx = focal_x; cam.fy = focal_y;

    int device = 0;
    FGS_HIP_TRY(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return fail(FGS_E_INVALID, "%s: device %d unsupported", who, device);
    const int num_blocks = (P + kBlock - 1) / kBlock;
    hipStream_t st = (hipStream_t)stream;

    std::lock_guard<std::mutex> lock(g_mutex);
    uint64_t* words = nullptr;
    int status_capacity = 0;
    Scratch* own = nullptr;
    if (allocate) {
        int rc = acquire_scratch(device, num_blocks, st, &own);
        if (rc != FGS_OK) return rc;
        if (!own && P > kStaticMaxP)
            return fail(FGS_E_INVALID, "%s: the stream is being captured and no call with P >= %d has run on it "
                                       "before, so nothing can be allocated; run one such call first", who, P);
    }
    if (own) {
        words = own->words;
        status_capacity = (int)own->capacity;
    } else {
        int rc = static_scratch(device, &words);
        if (rc != FGS_OK) return rc;
        status_capacity = kStaticBlocks;
    }

    hipLaunchKernelGGL(preprocess_kernel, dim3(num_blocks + 1), dim3(kBlock), 0, st,
                       P, positions, shs, opacities, cov3Ds, cam, points_xy, rgb_depth, conic_opacity,
                       gaussian_keys_unsorted, gaussian_values_unsorted, curr_offset, key_capacity,
                       words, status_capacity, num_blocks, g_spin_limit.load(), mirror_on_device);
    return check_hip(hipGetLastError(), "preprocess_kernel launch");
}

} // namespace
} // namespace fgs

extern "C" unsigned fgs_set_scan_spin_limit(unsigned polls)
{
    return fgs::g_spin_limit.exchange(polls);
}

extern "C" int fgs_reset_scan(void* stream)
{
    using namespace fgs;
    int device = 0;
    FGS_HIP_TRY(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return fail(FGS_E_INVALID, "fgs_reset_scan: device %d unsupported", device);
    hipStream_t st = (hipStream_t)stream;
    std::lock_guard<std::mutex> lock(g_mutex);
    // the stream's own scan words, if it has any, and the built-in ones of the device
    auto it = g_scratch.find(stream_key(device, st));
    if (it != g_scratch.end() && it->second.words) {
        int rc = clear_words(it->second.words, kControlWords + 4 * it->second.capacity, st);
        if (rc != FGS_OK) return rc;
    }
    uint64_t* words = nullptr;
    int rc = static_scratch(device, &words);
    if (rc != FGS_OK) return rc;
    return clear_words(words, kControlWords + 4 * (size_t)kStaticBlocks, st);
}

extern "C" int fgs_preprocess(int P,
                              const float* positions, const float* shs, const float* opacities, const float* cov3Ds,
                              int width, int height, int block_x, int block_y,
                              const float cam_position[3], const float cam_rotation[9],
                              float focal_x, float focal_y, float zFar, float zNear,
                              float* points_xy, float* rgb_depth, float* conic_opacity,
                              uint64_t* gaussian_keys_unsorted, uint32_t* gaussian_values_unsorted,
                              int* curr_offset, int64_t key_capacity, void* stream)
{
    return fgs::preprocess_impl(true, "fgs_preprocess", P, positions, shs, opacities, cov3Ds, width, height, block_x, block_y,
                                cam_position, cam_rotation, focal_x, focal_y, zFar, zNear, points_xy, rgb_depth,
                                conic_opacity, gaussian_keys_unsorted, gaussian_values_unsorted, curr_offset,
                                key_capacity, nullptr, stream);
}

extern "C" int fgs_preprocess_static(int P,
                                     const float* positions, const float* shs, const float* opacities, const float* cov3Ds,
                                     int width, int height, int block_x, int block_y,
                                     const float cam_position[3], const float cam_rotation[9],
                                     float focal_x, float focal_y, float zFar, float zNear,
                                     float* points_xy, float* rgb_depth, float* conic_opacity,
                                     uint64_t* gaussian_keys_unsorted, uint32_t* gaussian_values_unsorted,
                                     int* curr_offset, int64_t key_capacity, void* stream)
{
    return fgs::preprocess_impl(false, "fgs_preprocess_static", P, positions, shs, opacities, cov3Ds, width, height,
                                block_x, block_y, cam_position, cam_rotation, focal_x, focal_y, zFar, zNear, points_xy,
                                rgb_depth, conic_opacity, gaussian_keys_unsorted, gaussian_values_unsorted, curr_offset,
                                key_capacity, nullptr, stream);
}

extern "C" int fgs_preprocess_mirrored(int P,
                                       const float* positions, const float* shs, const float* opacities, const float* cov3Ds,
                                       int width, int height, int block_x, int block_y,
                                       const float cam_position[3], const float cam_rotation[9],
                                       float focal_x, float focal_y, float zFar, float zNear,
                                       float* points_xy, float* rgb_depth, float* conic_opacity,
                                       uint64_t* gaussian_keys_unsorted, uint32_t* gaussian_values_unsorted,
                                       int* curr_offset, int64_t key_capacity, int* count_mirror, void* stream)
{
    if (!count_mirror) return fgs::fail(FGS_E_INVALID, "fgs_preprocess_mirrored: null count_mirror");
    return fgs::preprocess_impl(true, "fgs_preprocess_mirrored", P, positions, shs, opacities, cov3Ds, width, height,
                                block_x, block_y, cam_position, cam_rotation, focal_x, focal_y, zFar, zNear, points_xy,
                                rgb_depth, conic_opacity, gaussian_keys_unsorted, gaussian_values_unsorted, curr_offset,
                                key_capacity, count_mirror, stream);
}

extern "C" int fgs_wait_count(const int* count_mirror, double timeout_seconds, int* count)
{
    if (!count_mirror || !count) return fgs::fail(FGS_E_INVALID, "fgs_wait_count: null argument");
    const volatile int* const word = count_mirror;
    const auto start = std::chrono::steady_clock::now();
    for (unsigned polls = 0;; polls++) {
        const int seen = *word;
        if (seen != FGS_COUNT_PENDING) {
            *count = seen;
            return FGS_OK;
        }
        if ((polls & 1023u) == 1023u &&
            std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count() > timeout_seconds)
            return fgs::fail(FGS_E_TIMEOUT, "fgs_wait_count: no pair count within %.3f s", timeout_seconds);
        __builtin_ia32_pause();
    }
}
