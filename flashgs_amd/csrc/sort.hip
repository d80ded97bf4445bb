// Device-wide stable sort of (u64 key, u32 value) pairs for gfx950 (wave64).
//
// Stands in for the cub::DeviceRadixSort::SortPairs call of FlashGS
// (csrc/cuda_rasterizer/sort.cu:28-44): ascending, stable, on key bits [0, 32 + tile_bits).
//
// The key is (tile id << 32 | depth bits), and what the renderer needs is every tile's pairs,
// contiguous and ordered by depth.  So the sort runs most-significant part first:
//
//  1. Partition by tile id: one stable counting pass per 8 bits of tile id (two passes for up to
//     65536 tiles; above that digits of 9 bits, so an 8K frame of 129 600 tiles still takes two).
//     A pass is count -> offsets -> scatter: `count_chunk_kernel` builds one digit histogram per
//     block of 4096 pairs (3840 with 9-bit digits) and the sums of every chunk of blocks,
//     `offsets_kernel` turns them into the exclusive start of every (block, digit) run, and
//     `scatter_kernel` ranks its block in LDS (wave64 ballot matching, so equal digits keep
//     their input order) and writes each run to its start.  A list of up to 64 blocks takes
//     count -> scatter.  No workgroup ever waits for another one.
//  2. Sort every tile's segment by the 32 depth bits without touching memory in between: the
//     last scatter pass also tabulates where each tile id's segment begins (with more than two
//     passes `segment_starts_kernel` does, from the sorted keys), then segments are handled by
//     size class.  Up to 1024 pairs one wave holds the segment in registers as 64-bit
//     words depth << 32 | value (| position where the values of a segment do not ascend) and runs
//     a bitonic network on them (the result is that of a stable sort by depth); lane exchanges inside a row of 16 lanes are
//     data-parallel-primitive moves.  Up to 4096 (8 waves) and 8192 pairs (16 waves) a workgroup
//     runs up to four stable 8-bit counting passes in LDS (in place: the pairs wait in registers
//     while they are counted), skipping a pass in which all pairs share the digit.  Longer segments, and segments whose keys differ above the sorted bit
//     range, go through the same passes with the ping-pong copy in HBM instead of LDS.
//
// Bytes moved per pair: 8 (count) + 24 (scatter) per partition pass, 24 for the segment sort:
// 88 for two partition passes, against 8 + 6 * 24 = 152 for a six-pass LSD sort of 47 bits.
#include "fgs_internal.h"

namespace fgs {
namespace {

constexpr int kBins = 256;                      // counters of a counting pass inside a segment (8-bit digits)
constexpr int kSortBlock = 256;
constexpr int kSortWaves = kSortBlock / kWave;
constexpr int kXcds = 8;                        // accelerator dies of the device, workgroup i of a launch runs on die i % 8

// Shape of a partition pass: digits of kBitsT bits, kItemsT pairs per thread.  Up to 65 536 tiles
// two passes of 8 bits do; above that (an 8K frame has 129 600) digits of 9 bits keep it at two
// passes up to 262 144 tiles, with 15 pairs per thread so that the workgroup's LDS still lets
// three workgroups share a CU.
template <int kBitsT, int kItemsT>
struct PassShape {
    static constexpr int kBits = kBitsT;
    static constexpr int kBinsP = 1 << kBitsT;
    static constexpr int kItems = kItemsT;                  // pairs per thread in count/scatter
    static constexpr int kTile = kSortBlock * kItemsT;      // pairs per count/scatter workgroup
    static constexpr int kPerThread = kBinsP / kSortBlock;  // digits per thread where a thread stands for digits
    static_assert(kBinsP % kSortBlock == 0 && kTile <= 65535, "16-bit counts per wave and digit");
};
using Narrow = PassShape<8, 16>;
using Wide = PassShape<9, 15>;
constexpr int kNarrowMaxTileBits = 16;
// A short list (the 0.2M pairs of a 720p frame are 49 blocks of 4096) leaves most CUs without a
// block and every block ranking 16 rounds: there four pairs per thread, four times the blocks.
using Short = PassShape<8, 4>;


// A list of at most kSmallRows blocks needs no launch that turns the histogram rows into starts:
// the scatter workgroups add the rows up themselves.
constexpr int kSmallRows = 64;
constexpr int kShortPairs = kSmallRows * Narrow::kTile;     // up to this many pairs: blocks of Short::kTile, still without that launch

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Tile ids up to this count get a table of segment starts in the workspace; beyond it every
// segment workgroup searches for its own bounds.
constexpr uint32_t kMaxTableIds = 1u << 20;

// The ids of the longer segments are listed per size class in kListShards separate lists (each
// with its own counter, a workgroup appends to the list of its index modulo kListShards): one
// shared counter would serialise thousands of atomic additions on one address.
constexpr int kListShards = 32;
constexpr int kListClasses = 4;
static_assert(kListClasses * kListShards * 4 <= 512, "the list counters fit in the 512 bytes in front of the lists");

struct Workspace {
    size_t alt_keys, alt_values, hist, chunk_sums, seg_start, seg_flags, seg_lists, total;
};

struct PassGrid {
    int tiles, chunk, chunks;       // workgroups of a count/scatter launch; chunks of `chunk` histogram rows each
};

PassGrid pass_grid(int n, int tile)
{
    PassGrid g;
    g.tiles = (n + tile - 1) / tile;
    g.chunk = g.tiles > 256 ? (g.tiles + 255) / 256 : 1;     // at most 256 chunks, one count workgroup each: about one per CU
    g.chunks = (g.tiles + g.chunk - 1) / g.chunk;
    return g;
}

// Sized for whichever pass shape the frame turns out to need (the tile count is not known here).
Workspace workspace_for(int n)
{
    Workspace w;
    const PassGrid a = pass_grid(n, Narrow::kTile), b = pass_grid(n, Wide::kTile);
    size_t hist = (size_t)a.tiles * Narrow::kBinsP > (size_t)b.tiles * Wide::kBinsP ? (size_t)a.tiles * Narrow::kBinsP
                                                                                     : (size_t)b.tiles * Wide::kBinsP;
    if (n <= kShortPairs && (size_t)pass_grid(n, Short::kTile).tiles * Short::kBinsP > hist)
        hist = (size_t)pass_grid(n, Short::kTile).tiles * Short::kBinsP;
    const size_t sums = (size_t)a.chunks * Narrow::kBinsP > (size_t)b.chunks * Wide::kBinsP ? (size_t)a.chunks * Narrow::kBinsP
                                                                                             : (size_t)b.chunks * Wide::kBinsP;
    w.alt_keys = 0;
    w.alt_values = align_up((size_t)n * 8, 256);
    w.hist = w.alt_values + align_up((size_t)n * 4, 256);
    w.chunk_sums = w.hist + hist * 4;
    w.seg_start = align_up(w.chunk_sums + sums * 4, 256);
    w.seg_flags = w.seg_start + align_up(((size_t)kMaxTableIds + 1) * 4, 256);
    w.seg_lists = w.seg_flags + kMaxTableIds / 8;
    // counters (kListClasses * kListShards words), then per class kListShards lists, each able to
    // hold every segment of its class
    w.total = w.seg_lists + 512 + (size_t)kListShards * (((size_t)n / 512 + 2) + ((size_t)n / 1024 + 2) + ((size_t)n / 4096 + 2) +
                                                         ((size_t)n / 8192 + 2)) * 4;
    return w;
}

__device__ __forceinline__ uint32_t digit_of(uint64_t key, int shift, uint32_t mask)
{
    return (uint32_t)(key >> shift) & mask;
}

// ---- partition pass, step 1: hist[block][digit] ---------------------------------------------------

template <class Shape>
__global__ __launch_bounds__(kSortBlock) void count_kernel(const uint64_t* __restrict__ keys, int n,
                                                           int shift, int nbits, uint32_t* __restrict__ hist,
                                                           uint32_t* __restrict__ seg_flags, uint32_t flag_words,
                                                           uint32_t* __restrict__ seg_counts)
{
    constexpr int kB = Shape::kBinsP;
    __shared__ uint32_t h[kB];
    const int tid = threadIdx.x;
    if (seg_flags) {        // the last pass also clears what the segment launches append to
        const uint32_t gid = blockIdx.x * kSortBlock + tid;
        for (uint32_t w = gid; w < flag_words; w += gridDim.x * kSortBlock) seg_flags[w] = 0;
        if (gid < (uint32_t)(kListClasses * kListShards)) seg_counts[gid] = 0;
    }
#pragma unroll
    for (int q = 0; q < Shape::kPerThread; q++) h[q * kSortBlock + tid] = 0;
    __syncthreads();
    const uint32_t mask = (1u << nbits) - 1u;
    const int base = blockIdx.x * Shape::kTile;
#pragma unroll
    for (int i = 0; i < Shape::kItems; i++) {
        const int idx = base + i * kSortBlock + tid;
        if (idx < n) atomicAdd(&h[digit_of(keys[idx], shift, mask)], 1u);
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < Shape::kPerThread; q++)
        hist[(size_t)blockIdx.x * kB + q * kSortBlock + tid] = h[q * kSortBlock + tid];
}

// The same for a list of more than kSmallRows blocks: one workgroup counts a whole chunk of
// `chunk` consecutive blocks, blockDim.x / kSortBlock of them at a time, and so also has the
// chunk's digit sums, which the offsets launch needs (a launch of their own would read the rows
// back just to add them up).
constexpr int kCountGroups = 4;

template <class Shape>
__global__ __launch_bounds__(kCountGroups * kSortBlock) void count_chunk_kernel(
    const uint64_t* __restrict__ keys, int n, int shift, int nbits, uint32_t* __restrict__ hist,
    int tiles, int chunk, uint32_t* __restrict__ chunk_sums,
    uint32_t* __restrict__ seg_flags, uint32_t flag_words, uint32_t* __restrict__ seg_counts)
{
    constexpr int kB = Shape::kBinsP, kPer = Shape::kPerThread;
    __shared__ uint32_t h[kCountGroups][kB];
    const int tid = threadIdx.x % kSortBlock, group = threadIdx.x / kSortBlock;
    const int groups = (int)blockDim.x / kSortBlock;
    if (seg_flags) {        // the last pass also clears what the segment launches append to
        const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
        for (uint32_t w = gid; w < flag_words; w += gridDim.x * blockDim.x) seg_flags[w] = 0;
        if (gid < (uint32_t)(kListClasses * kListShards)) seg_counts[gid] = 0;
    }
    const uint32_t mask = (1u << nbits) - 1u;
    const int t0 = blockIdx.x * chunk, t1 = min(tiles, t0 + chunk);
    uint32_t sum[kPer];
#pragma unroll
    for (int q = 0; q < kPer; q++) { sum[q] = 0; h[group][q * kSortBlock + tid] = 0; }
    __syncthreads();
    for (int first = t0; first < t1; first += groups) {      // the same trips for every group
        const int row = first + group;
        if (row < t1) {
            const int base = row * Shape::kTile;
            uint64_t k[Shape::kItems];
#pragma unroll
            for (int i = 0; i < Shape::kItems; i++) {
                const int idx = base + i * kSortBlock + tid;
                k[i] = idx < n ? keys[idx] : 0ull;
            }
#pragma unroll
            for (int i = 0; i < Shape::kItems; i++)
                if (base + i * kSortBlock + tid < n) atomicAdd(&h[group][digit_of(k[i], shift, mask)], 1u);
        }
        __syncthreads();
        if (row < t1) {
#pragma unroll
            for (int q = 0; q < kPer; q++) {
                const uint32_t c = h[group][q * kSortBlock + tid];
                h[group][q * kSortBlock + tid] = 0;          // read and cleared by the same thread
                hist[(size_t)row * kB + q * kSortBlock + tid] = c;
                sum[q] += c;
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int q = 0; q < kPer; q++) h[group][q * kSortBlock + tid] = sum[q];
    __syncthreads();
    if (group == 0) {
#pragma unroll
        for (int q = 0; q < kPer; q++) {
            uint32_t total = 0;
            for (int g = 0; g < groups; g++) total += h[g][q * kSortBlock + tid];
            chunk_sums[(size_t)blockIdx.x * kB + q * kSortBlock + tid] = total;
        }
    }
}

// ---- step 2: exclusive start of every (block, digit) run ----------------------------------------
// start[b][d] = sum of hist[*][d' < d] + sum of hist[b' < b][d]   (digit-major, then block)

// One workgroup per chunk, up to 1024 / bins threads per digit (blockDim.x / bins of them): the
// chunk sums are few and the loop over them is latency-bound, so each group of `bins` threads
// takes every groups-th batch of 16 independent loads.
constexpr int kOffsetThreads = 1024;

template <class Shape>
__global__ __launch_bounds__(kOffsetThreads) void offsets_kernel(uint32_t* __restrict__ hist, int tiles, int chunk,
                                                                 const uint32_t* __restrict__ chunk_sums, int chunks)
{
    constexpr int kB = Shape::kBinsP;
    constexpr int kMaxGroups = kOffsetThreads / kB;
    __shared__ uint32_t s_total[kMaxGroups][kB], s_before[kMaxGroups][kB];
    __shared__ uint32_t s_wave[kB / kWave];
    const int d = threadIdx.x & (kB - 1), group = threadIdx.x / kB;
    const int lane = d & (kWave - 1), wave = d / kWave;
    const int mine = (int)blockIdx.x;
    const int groups = (int)blockDim.x / kB;
    uint32_t total = 0, before = 0;
    for (int c0 = group * 16; c0 < chunks; c0 += 16 * groups) {
        uint32_t v[16];
#pragma unroll
        for (int j = 0; j < 16; j++) v[j] = c0 + j < chunks ? chunk_sums[(size_t)(c0 + j) * kB + d] : 0u;
#pragma unroll
        for (int j = 0; j < 16; j++) {
            if (c0 + j < mine) before += v[j];
            total += v[j];
        }
    }
    s_total[group][d] = total;
    s_before[group][d] = before;
    __syncthreads();
    total = 0; before = 0;
#pragma unroll
    for (int g = 0; g < kMaxGroups; g++)
        if (g < groups) { total += s_total[g][d]; before += s_before[g][d]; }
    // exclusive scan of the digit totals over the digits (every group does the same sums)
    uint32_t incl = wave_inclusive_sum(total);
    if (group == 0 && lane == kWave - 1) s_wave[wave] = incl;
    __syncthreads();
    if (group != 0) return;
    uint32_t digit_base = incl - total;
    for (int w = 0; w < wave; w++) digit_base += s_wave[w];

    uint32_t run = digit_base + before;
    const int t0 = mine * chunk, t1 = min(tiles, t0 + chunk);
    for (int tb = t0; tb < t1; tb += 16) {
        uint32_t c[16];
#pragma unroll
        for (int j = 0; j < 16; j++) c[j] = tb + j < t1 ? hist[(size_t)(tb + j) * kB + d] : 0u;
#pragma unroll
        for (int j = 0; j < 16; j++) {
            if (tb + j < t1) hist[(size_t)(tb + j) * kB + d] = run;
            run += c[j];
        }
    }
}


// ---- step 3: stable scatter ---------------------------------------------------------------------------

// With kTable (the last pass of at most two) the launch also writes the table of segment starts,
// seg_start[v] = first index of the output whose tile field is >= v, v in [0, ids], ids = 2^(bits of
// the tile field).  The input of that pass is ordered by the low part of the tile field (the bits
// below this pass's digit), so the first pair with low part >= L lies in exactly one workgroup's
// block, and that workgroup writes the entries (d, L) of every digit d: the destination of its
// first pair with digit d and low part >= L, or, if it has none, the end of its run of digit d,
// which is where the next workgroup's run of d begins.  Every entry has one writer, empty ids
// included, and no launch has to read the keys again.
template <class Shape, bool kTable>
__global__ __launch_bounds__(kSortBlock) void scatter_kernel(
    const uint64_t* __restrict__ keys_in, const uint32_t* __restrict__ values_in,
    uint64_t* __restrict__ keys_out, uint32_t* __restrict__ values_out,
    int n, int shift, int nbits,
    const uint32_t* __restrict__ start,          // [blocks][bins] from offsets_kernel, or ...
    int raw_rows,                                // ... if > 0, the raw_rows histogram rows themselves (a short list)
    int* __restrict__ seg_start)                 // kTable: [2^(shift - 32 + nbits) + 1]
{
    constexpr int kB = Shape::kBinsP, kItems = Shape::kItems, kTile = Shape::kTile, kPer = Shape::kPerThread;
    // per-wave digit counts, then per-wave digit offsets: at most kTile, so 16 bits do, and with
    // them the workgroup's LDS stays under a third of the CU's (three resident workgroups, not two)
    __shared__ uint16_t s_count[kSortWaves][kB];
    __shared__ uint16_t s_bin_start[kB];              // where each digit starts in the ranked block
    __shared__ uint32_t s_global[kB];                 // destination of ranked slot p with digit d: s_global[d] + p
    __shared__ uint32_t s_wave_sum[kPer * kSortWaves];
    __shared__ uint64_t s_keys[kTile];
    __shared__ uint32_t s_values[kTile];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const uint32_t mask = (1u << nbits) - 1u;
    // Workgroups go round-robin to the 8 XCDs, each with an L2 of its own.  Every XCD takes a
    // contiguous range of blocks: the runs that neighbouring blocks write for one digit are
    // neighbours in memory, and the cache line where two of them meet is then completed in one
    // L2 instead of being written out in parts by two (first pass at 4K: 62 -> 51 us).
    const int xcd = (int)blockIdx.x % kXcds, per = (int)gridDim.x / kXcds, rest = (int)gridDim.x % kXcds;
    const int tile = xcd * per + min(xcd, rest) + (int)blockIdx.x / kXcds;
    const int tile_base = tile * kTile;
    const int in_tile = min(kTile, n - tile_base);

    // The low parts L whose first pair (the first of the input with low part >= L) lies in this
    // block: those above the low part of the pair in front of the block, up to that of the
    // block's last pair; the last block also takes the ones no pair reaches.
    const int low_bits = shift - 32;
    const uint32_t low_mask = (1u << low_bits) - 1u;
    __shared__ int s_own[2];
    uint64_t edge_key = 0;          // thread 0: the pair in front of the block, thread 1: the block's last pair
    if (kTable && tid < 2 && (tid == 1 || tile > 0)) edge_key = keys_in[tid == 0 ? tile_base - 1 : tile_base + in_tile - 1];

    // wave w owns slots [w*64*kItems, (w+1)*64*kItems) of the block, item-major; everything is
    // requested before the first use so the latencies overlap
    uint64_t key[kItems];
    uint32_t val[kItems];
    uint32_t slot[kItems];
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int off = wave * (kWave * kItems) + i * kWave + lane;
        key[i] = off < in_tile ? keys_in[tile_base + off] : ~0ull;
    }
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int off = wave * (kWave * kItems) + i * kWave + lane;
        val[i] = off < in_tile ? values_in[tile_base + off] : 0u;
    }
    uint32_t my_start[kPer];
    if (raw_rows == 0) {
#pragma unroll
        for (int q = 0; q < kPer; q++) my_start[q] = start[(size_t)tile * kB + q * kSortBlock + tid];
    } else {
        // A list of at most kSmallRows blocks: every workgroup adds up the histogram rows itself
        // (the digit totals, and what the blocks in front of it hold of each digit), which
        // saves the launch that would do it.
        uint32_t total[kPer], before[kPer], incl[kPer];
#pragma unroll
        for (int q = 0; q < kPer; q++) {
            const int d = q * kSortBlock + tid;
            total[q] = 0; before[q] = 0;
#pragma unroll 16
            for (int b = 0; b < raw_rows; b++) {
                const uint32_t c = start[(size_t)b * kB + d];
                total[q] += c;
                before[q] += b < tile ? c : 0u;
            }
            incl[q] = wave_inclusive_sum(total[q]);
            if (lane == kWave - 1) s_wave_sum[q * kSortWaves + wave] = incl[q];
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < kPer; q++) {
            uint32_t digit_base = incl[q] - total[q];
#pragma unroll
            for (int w = 0; w < kPer * kSortWaves; w++)
                if (w < q * kSortWaves + wave) digit_base += s_wave_sum[w];
            my_start[q] = digit_base + before[q];
        }
    }
#pragma unroll
    for (int w = 0; w < kSortWaves; w++)
#pragma unroll
        for (int q = 0; q < kPer; q++) s_count[w][q * kSortBlock + tid] = 0;
    if (kTable && tid < 2) {
        const int low = (int)((uint32_t)(edge_key >> 32) & low_mask);
        s_own[tid] = tid == 0 ? (tile > 0 ? low + 1 : 0) : (tile == (int)gridDim.x - 1 ? (int)low_mask : low);
    }
    __syncthreads();

    // rank inside the wave: lanes with equal digits find each other with one ballot per digit bit
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int off = wave * (kWave * kItems) + i * kWave + lane;
        const bool valid = off < in_tile;
        const uint32_t d = digit_of(key[i], shift, mask);
        uint64_t peers = ballot(valid);
#pragma unroll
        for (int b = 0; b < Shape::kBits; b++) {
            const bool bit = (d >> b) & 1u;
            const uint64_t with_bit = ballot(bit);
            peers &= bit ? with_bit : ~with_bit;
        }
        const int below = popc_below(peers);
        uint32_t before = 0;
        if (valid && below == 0) {      // lowest lane of each group updates the wave's counter
            before = s_count[wave][d];
            s_count[wave][d] = (uint16_t)(before + (uint32_t)__popcll(peers));
        }
        const int leader = valid ? __ffsll((long long)peers) - 1 : lane;
        before = (uint32_t)__shfl((int)before, leader);
        slot[i] = before + (uint32_t)below;
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();

    // digit totals of the block; per-wave offsets inside each digit.  A thread stands for the
    // digits tid, tid + 256, ...; the scan runs over the digits in their order.
    uint32_t total[kPer], incl[kPer];
#pragma unroll
    for (int q = 0; q < kPer; q++) {
        const int d = q * kSortBlock + tid;
        total[q] = 0;
#pragma unroll
        for (int w = 0; w < kSortWaves; w++) {
            const uint32_t c = s_count[w][d];
            s_count[w][d] = (uint16_t)total[q];
            total[q] += c;
        }
        incl[q] = wave_inclusive_sum(total[q]);
        if (lane == kWave - 1) s_wave_sum[q * kSortWaves + wave] = incl[q];
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < kPer; q++) {
        const int d = q * kSortBlock + tid;
        uint32_t before_wave = 0;
#pragma unroll
        for (int w = 0; w < kPer * kSortWaves; w++)
            if (w < q * kSortWaves + wave) before_wave += s_wave_sum[w];
        const uint32_t bin_start = before_wave + incl[q] - total[q];
        s_bin_start[d] = (uint16_t)bin_start;
        s_global[d] = my_start[q] - bin_start;
    }
    __syncthreads();

    // move the pairs to their ranked slots in LDS
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int off = wave * (kWave * kItems) + i * kWave + lane;
        if (off < in_tile) {
            const uint32_t dg = digit_of(key[i], shift, mask);
            const uint32_t p = (uint32_t)s_bin_start[dg] + s_count[wave][dg] + slot[i];
            s_keys[p] = key[i];
            s_values[p] = val[i];
        }
    }
    __syncthreads();

    const int own_lo = kTable ? s_own[0] : 0, own_hi = kTable ? s_own[1] : -1;

    // write out: neighbouring threads hold neighbouring ranked slots.  All LDS reads first (a slot
    // past the end reads the last pair and stores nothing), so their latencies overlap.
    {
        uint64_t out_key[kItems];
        uint32_t out_value[kItems], out_at[kItems];
#pragma unroll
        for (int i = 0; i < kItems; i++) {
            const int p = min(i * kSortBlock + tid, in_tile - 1);
            out_key[i] = s_keys[p];
            out_value[i] = s_values[p];
        }
#pragma unroll
        for (int i = 0; i < kItems; i++)
            out_at[i] = s_global[digit_of(out_key[i], shift, mask)] + (uint32_t)(i * kSortBlock + tid);
#pragma unroll
        for (int i = 0; i < kItems; i++) {
            if (i * kSortBlock + tid < in_tile) {
                keys_out[out_at[i]] = out_key[i];
                values_out[out_at[i]] = out_value[i];
            }
        }
    }
    if (kTable) {
        if (own_lo <= own_hi) {
            // the first pair of digit d with a low part >= L, for every owned L up to its own
            // (a loop of its own: in the one above the LDS reads of all slots are in flight together)
#pragma unroll 4
            for (int i = 0; i < kItems; i++) {
                const int p = i * kSortBlock + tid;
                if (p >= in_tile) break;
                const uint32_t field = (uint32_t)(s_keys[p] >> 32);
                const uint32_t d = (field >> low_bits) & mask;
                const int low = (int)(field & low_mask);
                int prev = own_lo - 1;
                if (p > (int)s_bin_start[d]) prev = (int)((uint32_t)(s_keys[p - 1] >> 32) & low_mask);
                for (int l = max(prev + 1, own_lo); l <= low; l++)
                    seg_start[(d << low_bits) | (uint32_t)l] = (int)(s_global[d] + (uint32_t)p);
            }
            // owned low parts above the last pair of a digit's run: the end of the run
#pragma unroll
            for (int q = 0; q < kPer; q++) {
                const uint32_t d = (uint32_t)(q * kSortBlock + tid);
                if (d > mask) continue;
                int last = own_lo - 1;
                if (total[q]) last = (int)((uint32_t)(s_keys[(uint32_t)s_bin_start[d] + total[q] - 1u] >> 32) & low_mask);
                const int end = (int)(my_start[q] + total[q]);
                for (int l = max(last + 1, own_lo); l <= own_hi; l++) seg_start[(d << low_bits) | (uint32_t)l] = end;
            }
        }
        if (tile == 0 && tid == 0) seg_start[(size_t)1 << (low_bits + nbits)] = n;
    }
}

// ---- per-tile segment sort on the 32 depth bits ----------------------------------------------------

// size classes of the segments: pairs per segment
constexpr int kCapTiny = 512, kCapSmall = 1024, kCapMedium = 4096, kCapLarge = 8192;
constexpr int kMergedLargeMax = 1 << 24;     // up to this many pairs the last launch also takes the class of 4097 .. 8192 pairs
constexpr int kMergedTailMax = 1 << 19;      // up to this many pairs the last launch also takes the classes of 1025 .. 8192 pairs
constexpr uint32_t kOneLaunchIds = 262144;   // up to this many tile ids one launch sorts every segment of up to kCapSmall pairs

// First index in [0, n) whose tile field is >= v (n if none), found by the whole wave probing 64
// evenly spaced positions per step.  `keys` is ordered by tile field.  All lanes return the same.
__device__ __forceinline__ int wave_lower_bound(const uint64_t* __restrict__ keys, int n, uint32_t v, uint32_t tile_mask)
{
    const int lane = lane_id();
    int lo = 0, hi = n;                 // the answer lies in [lo, hi]; every index < lo is < v, index hi (if < n) is >= v
    while (hi > lo) {
        const int span = hi - lo;
        const int step = (span + kWave - 1) / kWave;        // >= 1
        const int pos = lo + lane * step;                    // probes at lo, lo+step, ...
        bool ge = true;                                      // a probe at or past hi counts as ">= v"
        if (pos < hi) ge = ((uint32_t)(keys[pos] >> 32) & tile_mask) >= v;
        const uint64_t m = ballot(ge);
        const int first = m ? __ffsll((long long)m) - 1 : kWave;     // first probe that is >= v
        if (first == 0) return lo;
        const int new_hi = first < kWave ? min(hi, lo + first * step) : hi;
        lo = lo + (first - 1) * step + 1;                    // the probe before `first` is < v
        hi = new_hi;
    }
    return lo;
}

// seg_start[v] = first index whose tile field is >= v, for v in [0, ids]; seg_start[ids] = n.
// A thread looks at kStartsPerThread pairs, 256 apart so that the loads of a workgroup stay
// contiguous: where the tile field changes, it fills the entries of the ids in between (empty ids
// get the same start as the next non-empty one).  Also clears the flag words and list counters.
constexpr int kStartsPerThread = 8;

__global__ __launch_bounds__(256) void segment_starts_kernel(const uint64_t* __restrict__ keys, int n, uint32_t tile_mask,
                                                             uint32_t ids, int* __restrict__ seg_start,
                                                             uint32_t* __restrict__ seg_flags, uint32_t flag_words,
                                                             uint32_t* __restrict__ seg_counts)
{
    const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
    for (uint32_t w = gid; w < flag_words; w += gridDim.x * blockDim.x) seg_flags[w] = 0;
    if (gid < (uint32_t)(kListClasses * kListShards)) seg_counts[gid] = 0;
    const long long base = (long long)blockIdx.x * (256 * kStartsPerThread) + threadIdx.x;
    uint32_t cur[kStartsPerThread], before[kStartsPerThread];
#pragma unroll
    for (int k = 0; k < kStartsPerThread; k++) {
        const long long i = base + k * 256;
        cur[k] = 0; before[k] = 0;
        if (i < n) {
            cur[k] = (uint32_t)(keys[i] >> 32) & tile_mask;
            before[k] = i == 0 ? 0u : ((uint32_t)(keys[i - 1] >> 32) & tile_mask) + 1u;
        }
    }
    // A run of up to kOwnFill entries is written by the thread that found it; a longer one (a band
    // of empty tiles, and the ids behind the last pair) by the whole wave, 64 entries per step.
    constexpr uint32_t kOwnFill = 4;
    const int lane = threadIdx.x & (kWave - 1);
    auto fill_by_wave = [&](bool mine, uint32_t lo, uint32_t hi, int value) {
        for (uint64_t todo = ballot(mine); todo; todo &= todo - 1) {
            const int src = __ffsll((long long)todo) - 1;
            const uint32_t from = (uint32_t)__shfl((int)lo, src), to = (uint32_t)__shfl((int)hi, src);
            const int what = __shfl(value, src);
            for (uint32_t v = from + (uint32_t)lane; v <= to; v += kWave) seg_start[v] = what;
        }
    };
#pragma unroll
    for (int k = 0; k < kStartsPerThread; k++) {
        const long long i = base + k * 256;
        const bool valid = i < n;
        // ids before[k]..cur[k] start at pair i: nothing to do when the field repeats
        const bool some = valid && before[k] <= cur[k];
        const bool longer = some && cur[k] - before[k] >= kOwnFill;
        if (some && !longer)
            for (uint32_t v = before[k]; v <= cur[k]; v++) seg_start[v] = (int)i;
        fill_by_wave(longer, before[k], cur[k], (int)i);
        fill_by_wave(valid && i == n - 1 && cur[k] < ids, cur[k] + 1, ids, n);
    }
}

// One stable counting pass of a segment over bits shift..shift+7 of the sort word, by the kWaves
// waves of one workgroup.  Wave w owns the contiguous part [w*per, (w+1)*per) of the segment.
// Returns false (and moves nothing) when every pair has the same digit.  All threads of the
// workgroup must call it.  KeyT is uint32_t for depth words in LDS, uint64_t for whole keys in HBM.
template <int kWaves, typename KeyT>
__device__ __forceinline__ bool counting_pass(const KeyT* src_k, const uint32_t* src_v, KeyT* dst_k, uint32_t* dst_v,
                                              int n, int shift, uint32_t (*cnt)[kBins], uint32_t* wave_sum, int* flag)
{
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int per = ((n + kWaves - 1) / kWaves + kWave - 1) / kWave * kWave;   // a multiple of 64
    const int w_lo = min(n, wave * per), w_hi = min(n, w_lo + per);

    for (int d = lane; d < kBins; d += kWave) cnt[wave][d] = 0;
    if (kWaves > 1) { if (tid == 0) *flag = 0; __syncthreads(); } else __builtin_amdgcn_wave_barrier();
    for (int i = w_lo + lane; i < w_hi; i += kWave)
        atomicAdd(&cnt[wave][(uint32_t)(src_k[i] >> shift) & 255u], 1u);
    if (kWaves > 1) __syncthreads(); else __builtin_amdgcn_wave_barrier();

    bool uniform;
    if (kWaves == 1) {
        // lane handles digits lane, lane+64, lane+128, lane+192; scan in digit order
        uint32_t base = 0;
        bool any_full = false;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t c = cnt[0][q * kWave + lane];
            any_full = any_full || c == (uint32_t)n;
            uint32_t incl = wave_inclusive_sum(c);
            cnt[0][q * kWave + lane] = base + incl - c;
            base += (uint32_t)bcast_i((int)incl, kWave - 1);
        }
        uniform = ballot(any_full) != 0;
        __builtin_amdgcn_wave_barrier();
    } else {
        // thread t < 256 handles digit t
        uint32_t total = 0;
        if (tid < kBins) {
            for (int w = 0; w < kWaves; w++) {
                const uint32_t c = cnt[w][tid];
                cnt[w][tid] = total;          // offset of wave w inside digit tid
                total += c;
            }
            if (total == (uint32_t)n) *flag = 1;
            uint32_t incl = wave_inclusive_sum(total);
            if (lane == kWave - 1) wave_sum[wave] = incl;
            total = incl - total;             // exclusive inside this wave's 64 digits
        }
        __syncthreads();
        if (tid < kBins) {
            uint32_t base = total;
            for (int w = 0; w < wave; w++) base += wave_sum[w];
            for (int w = 0; w < kWaves; w++) cnt[w][tid] += base;     // absolute start of (wave, digit)
        }
        __syncthreads();
        uniform = *flag != 0;
    }
    if (uniform) return false;

    // stable ranking, 64 pairs at a time in segment order
    for (int base = w_lo; base < w_hi; base += kWave) {
        const int i = base + lane;
        const bool valid = i < w_hi;
        KeyT k = 0;
        uint32_t v = 0;
        if (valid) { k = src_k[i]; v = src_v[i]; }
        const uint32_t d = (uint32_t)(k >> shift) & 255u;
        uint64_t peers = ballot(valid);
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const bool bit = (d >> b) & 1u;
            const uint64_t with_bit = ballot(bit);
            peers &= bit ? with_bit : ~with_bit;
        }
        const int below = popc_below(peers);
        uint32_t before = 0;
        if (valid && below == 0) {
            before = cnt[wave][d];
            cnt[wave][d] = before + (uint32_t)__popcll(peers);
        }
        const int leader = valid ? __ffsll((long long)peers) - 1 : lane;
        before = (uint32_t)__shfl((int)before, leader);
        if (valid) {
            dst_k[before + (uint32_t)below] = k;
            dst_v[before + (uint32_t)below] = v;
        }
        __builtin_amdgcn_wave_barrier();
    }
    return true;
}

// The same pass over a segment of depth words and values held in LDS, in place: every thread takes
// its kPer pairs into registers (pair w_lo + it*64 + lane for it < kPer, so a wave still ranks its
// contiguous part 64 pairs at a time in segment order), and once all of them are counted nobody
// needs the arrays any more and the ranked pairs go back into them.  Half the LDS of a ping-pong
// copy, and one read of every pair instead of two.  The counters are 16 bits wide (positions stay
// below 65536), two to a word, counted with 32-bit atomic additions on the half that is meant.
template <int kWaves, int kPer>
__device__ __forceinline__ bool counting_pass_lds(uint32_t* s_k, uint32_t* s_v, int n, int shift,
                                                  uint16_t (*cnt)[kBins], uint32_t* wave_sum, int* flag)
{
    static_assert(kWaves * kWave >= kBins, "one thread per digit in the scan");
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int per = ((n + kWaves - 1) / kWaves + kWave - 1) / kWave * kWave;   // a multiple of 64, at most 64 * kPer
    const int w_lo = min(n, wave * per), w_hi = min(n, w_lo + per);

    uint32_t* const cnt_words = (uint32_t*)cnt[wave];
    cnt_words[lane] = 0;
    cnt_words[lane + kWave] = 0;
    if (tid == 0) *flag = 0;
    __syncthreads();
    uint32_t k[kPer], v[kPer];
#pragma unroll
    for (int it = 0; it < kPer; it++) {
        const int i = w_lo + it * kWave + lane;
        k[it] = 0; v[it] = 0;
        if (i < w_hi) {
            k[it] = s_k[i];
            v[it] = s_v[i];
            const uint32_t d = (k[it] >> shift) & 255u;
            atomicAdd(&cnt_words[d >> 1], (d & 1u) ? 0x10000u : 1u);
        }
    }
    __syncthreads();

    uint32_t total = 0;
    if (tid < kBins) {                   // thread t handles digit t
        for (int w = 0; w < kWaves; w++) {
            const uint32_t c = cnt[w][tid];
            cnt[w][tid] = (uint16_t)total;          // offset of wave w inside digit tid
            total += c;
        }
        if (total == (uint32_t)n) *flag = 1;
        const uint32_t incl = wave_inclusive_sum(total);
        if (lane == kWave - 1) wave_sum[wave] = incl;
        total = incl - total;             // exclusive inside this wave's 64 digits
    }
    __syncthreads();
    if (tid < kBins) {
        uint32_t base = total;
        for (int w = 0; w < wave; w++) base += wave_sum[w];
        for (int w = 0; w < kWaves; w++) cnt[w][tid] = (uint16_t)(cnt[w][tid] + base);     // absolute start of (wave, digit)
    }
    __syncthreads();
    if (*flag != 0) return false;        // every pair has the same digit: nothing to move

    // stable ranking, 64 pairs at a time in segment order
#pragma unroll
    for (int it = 0; it < kPer; it++) {
        if (w_lo + it * kWave >= w_hi) break;
        const bool valid = w_lo + it * kWave + lane < w_hi;
        const uint32_t d = (k[it] >> shift) & 255u;
        uint64_t peers = ballot(valid);
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const bool bit = (d >> b) & 1u;
            const uint64_t with_bit = ballot(bit);
            peers &= bit ? with_bit : ~with_bit;
        }
        const int below = popc_below(peers);
        uint32_t before = 0;
        if (valid && below == 0) {
            before = cnt[wave][d];
            cnt[wave][d] = (uint16_t)(before + (uint32_t)__popcll(peers));
        }
        const int leader = valid ? __ffsll((long long)peers) - 1 : lane;
        before = (uint32_t)__shfl((int)before, leader);
        if (valid) {
            s_k[before + (uint32_t)below] = k[it];
            s_v[before + (uint32_t)below] = v[it];
        }
        __builtin_amdgcn_wave_barrier();
    }
    return true;
}

// Sorts the segment [lo, hi) of tile id v in LDS.  Called by all kWaves waves of a workgroup
// with the same arguments; hi - lo <= kCap.  A segment whose keys differ above the depth word
// cannot be rebuilt from depth words: it is flagged (or, without a flag array, left alone) for
// the general kernel.
// Returns true when that was the case (nothing is moved then).
template <int kWaves, int kCap>
__device__ __forceinline__ bool sort_segment_lds(uint64_t* __restrict__ keys, uint32_t* __restrict__ values,
                                                 uint32_t v, int lo, int hi, uint32_t* __restrict__ seg_flags,
                                                 uint32_t* s_k, uint32_t* s_v,
                                                 uint16_t (*s_cnt)[kBins], uint32_t* s_wave_sum, int* s_flag)
{
    static_assert(kCap % (kWaves * kWave) == 0, "every thread holds the same number of pairs");
    const int tid = threadIdx.x;
    const int len = hi - lo;
    const uint32_t upper = (uint32_t)(keys[lo] >> 32);
    bool mixed = false;
    if (tid == 0) *s_flag = 0;
    __syncthreads();
    for (int i = tid; i < len; i += kWaves * kWave) {
        const uint64_t k = keys[lo + i];
        s_k[i] = (uint32_t)k;
        s_v[i] = values[lo + i];
        mixed = mixed || (uint32_t)(k >> 32) != upper;
    }
    if (mixed) *s_flag = 1;
    __syncthreads();
    const bool any_mixed = *s_flag != 0;
    __syncthreads();                             // the passes reuse the flag
    if (any_mixed) {
        if (seg_flags && tid == 0) atomicOr(&seg_flags[v >> 5], 1u << (v & 31));
        return true;
    }

#pragma unroll 1
    for (int shift = 0; shift < 32; shift += 8) {
        counting_pass_lds<kWaves, kCap / (kWaves * kWave)>(s_k, s_v, len, shift, s_cnt, s_wave_sum, s_flag);
        __syncthreads();
    }
    for (int i = tid; i < len; i += kWaves * kWave) {
        keys[lo + i] = ((uint64_t)upper << 32) | s_k[i];
        values[lo + i] = s_v[i];
    }
    __syncthreads();
    return false;
}

// Segment sort in LDS for one size class: segments with min_len < length <= kCap.
// With a table of segment starts, workgroup w looks at the kIds tile ids [w*kIds, (w+1)*kIds),
// one per lane, and sorts those of its class one after the other.  Without a table (more tile ids
// than the table holds) the grid has one workgroup per tile id and each searches for its bounds.
template <int kWaves, int kCap, int kIds>
__global__ __launch_bounds__(kWaves * kWave) void segment_sort_kernel(
    uint64_t* __restrict__ keys, uint32_t* __restrict__ values, int n, uint32_t tile_mask, int min_len, uint32_t ids,
    const int* __restrict__ seg_start, uint32_t* __restrict__ seg_flags,
    const uint32_t* __restrict__ list, const uint32_t* __restrict__ list_count, uint32_t list_cap)
{
    __shared__ uint32_t s_k[kCap];
    __shared__ uint32_t s_v[kCap];
    __shared__ __align__(4) uint16_t s_cnt[kWaves][kBins];
    __shared__ uint32_t s_wave_sum[kWaves];
    __shared__ int s_bounds[2];
    __shared__ int s_flag;
    __shared__ uint64_t s_match;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);

    if (!seg_start) {
        const uint32_t v = blockIdx.x;
        if (tid < kWave) {
            const int a = wave_lower_bound(keys, n, v, tile_mask);
            const int b = v == tile_mask ? n : wave_lower_bound(keys, n, v + 1, tile_mask);
            if (lane == 0) { s_bounds[0] = a; s_bounds[1] = b; }
        }
        __syncthreads();
        const int lo = s_bounds[0], hi = s_bounds[1];
        if (hi - lo <= min_len || hi - lo > kCap) return;
        sort_segment_lds<kWaves, kCap>(keys, values, v, lo, hi, seg_flags, s_k, s_v, s_cnt, s_wave_sum, &s_flag);
        return;
    }

    if (list) {      // the segments of this class were listed: deal them out round-robin, shard by shard
        const uint32_t shard = blockIdx.x % kListShards;
        const uint32_t count = list_count[shard];
        for (uint32_t i = blockIdx.x / kListShards; i < count; i += gridDim.x / kListShards) {
            const uint32_t v = list[(size_t)shard * list_cap + i];
            sort_segment_lds<kWaves, kCap>(keys, values, v, seg_start[v], seg_start[v + 1], seg_flags,
                                           s_k, s_v, s_cnt, s_wave_sum, &s_flag);
        }
        return;
    }

    const uint32_t first_id = blockIdx.x * (uint32_t)kIds;
    if (tid < kWave) {
        const uint32_t v = first_id + (uint32_t)lane;
        int len = 0;
        if (lane < kIds && v < ids) len = seg_start[v + 1] - seg_start[v];
        const uint64_t m = ballot(len > min_len && len <= kCap);
        if (lane == 0) s_match = m;
    }
    __syncthreads();
    for (uint64_t todo = s_match; todo; todo &= todo - 1) {
        const uint32_t v = first_id + (uint32_t)(__ffsll((long long)todo) - 1);
        sort_segment_lds<kWaves, kCap>(keys, values, v, seg_start[v], seg_start[v + 1], seg_flags,
                                       s_k, s_v, s_cnt, s_wave_sum, &s_flag);
    }
}

// x of lane (l ^ kJ).  Within a row of 16 lanes the exchange is a data-parallel-primitive move
// (no LDS traffic); across rows it goes through the lane crossbar.
template <int kJ>
__device__ __forceinline__ uint32_t from_lane_xor(uint32_t x)
{
    constexpr int kQuadXor1 = 0xB1, kQuadXor2 = 0x4E, kQuadReverse = 0x1B, kRowHalfMirror = 0x141, kRowRor8 = 0x128;
    if (kJ == 1) return (uint32_t)__builtin_amdgcn_mov_dpp((int)x, kQuadXor1, 0xf, 0xf, true);
    if (kJ == 2) return (uint32_t)__builtin_amdgcn_mov_dpp((int)x, kQuadXor2, 0xf, 0xf, true);
    if (kJ == 4) {      // reverse the 8 lanes, then each quad: lane l reads lane l ^ 4
        const int t = __builtin_amdgcn_mov_dpp((int)x, kRowHalfMirror, 0xf, 0xf, true);
        return (uint32_t)__builtin_amdgcn_mov_dpp(t, kQuadReverse, 0xf, 0xf, true);
    }
    if (kJ == 8) return (uint32_t)__builtin_amdgcn_mov_dpp((int)x, kRowRor8, 0xf, 0xf, true);
    return (uint32_t)__shfl_xor((int)x, kJ);
}

template <int kJ>
__device__ __forceinline__ uint64_t from_lane_xor64(uint64_t x)
{
    return ((uint64_t)from_lane_xor<kJ>((uint32_t)(x >> 32)) << 32) | from_lane_xor<kJ>((uint32_t)x);
}

// The network over kT register slots of every lane, 64 * kT elements, element i in slot i % kT of
// lane i / kT.  A compare distance below kT pairs two slots of one lane (registers only); a
// larger one pairs the same slot of two lanes: 21 of the (log n)(log n + 1)/2 exchange steps
// cross lanes whatever kT is, where the slot-major layout (element i in lane i % 64) makes it
// 33 of 36 for 256 elements and 45 of 55 for 1024.  The merge width k runs in a loop; the compare
// distances j are written out, so the code holds every exchange pattern once whatever the number
// of stages.
template <int kT>
__device__ __forceinline__ void bitonic_network(uint64_t (&c)[kT], int lane)
{
    constexpr int n = kT * kWave;
#pragma unroll 1
    for (int k = 2; k <= n; k <<= 1) {
        // element lane*kT + t sits in an ascending run of width k: a matter of t alone while the
        // runs are shorter than a lane's slots, of the lane alone from there on
        bool ascending[kT];
        const bool lane_ascending = (lane & (k / kT)) == 0;
#pragma unroll
        for (int t = 0; t < kT; t++) ascending[t] = k < kT ? (t & k) == 0 : lane_ascending;
#pragma unroll
        for (int j = n / 2; j > 0; j >>= 1) {
            if (j >= k) continue;
            if (j < kT) {
#pragma unroll
                for (int t = 0; t < kT; t++) {
                    if ((t & j) != 0) continue;
                    const int t2 = t | j;
                    const bool swap = (c[t] > c[t2]) == ascending[t];
                    const uint64_t a = swap ? c[t2] : c[t], b = swap ? c[t] : c[t2];
                    c[t] = a; c[t2] = b;
                }
            } else {
                constexpr int kLanesMax = kWave / 2;
                const int jl = j / kT;                                   // 1, 2, ... 32
                const bool lower = (lane & jl) == 0;
#pragma unroll
                for (int t = 0; t < kT; t++) {
                    const uint64_t mine = c[t];
                    const uint64_t other = jl == 1 ? from_lane_xor64<1>(mine) : jl == 2 ? from_lane_xor64<2>(mine)
                                         : jl == 4 ? from_lane_xor64<4>(mine) : jl == 8 ? from_lane_xor64<8>(mine)
                                         : jl == 16 ? from_lane_xor64<16>(mine) : from_lane_xor64<kLanesMax>(mine);
                    const bool keep_min = lower == ascending[t];
                    const bool take = (other < mine) == keep_min;       // the words are never equal
                    c[t] = take ? other : mine;
                }
            }
        }
    }
}

// Words of LDS a wave needs to sort up to n pairs with the network: one 64-bit word for every
// second pair (the sorted pairs go through it in two halves), one word of padding after every 16 (lane l puts its kUse consecutive ranks down at once; without
// the padding the lanes of a wave would all start in the same bank).
__host__ __device__ constexpr int staging_words(int n) { return n <= 64 ? n + n / 16 : n / 2 + n / 32; }
__device__ __forceinline__ int staged(int i) { return i + (i >> 4); }

// Sorts the segment [lo, hi) of tile id v with the network over kUse slots per lane, 64 * kUse >= hi - lo.
// The network orders 64-bit words, depth above and a tie-break below, and it does not matter
// which slot a word starts in: the loads are the contiguous ones (element t*64 + lane in slot t),
// the network leaves rank lane*kUse + t in slot t, and the sorted words go through LDS to be
// stored contiguously again.  Equal depths have to stay in input order.  The pairs of one tile
// come out of the preprocess in ascending order of their values (Gaussian indices): then the value
// itself is the tie-break and the sorted word is the pair.  A segment whose values do not ascend
// carries positions instead and looks its values up afterwards.
template <int kUse>
__device__ __forceinline__ void sort_segment_bitonic_of(uint64_t* __restrict__ keys, uint32_t* __restrict__ values,
                                                        uint32_t v, int lo, int hi, uint32_t* __restrict__ seg_flags,
                                                        uint64_t* s_w)
{
    // The lane number is made opaque here and again behind the network: otherwise every index and
    // address derived from it, for every width of the network, is computed once in front of the loop
    // over the segments and kept in registers through all of it (80 registers of a 16-slot network).
    int lane = threadIdx.x & (kWave - 1);
    asm volatile("" : "+v"(lane));
    const int len = hi - lo;
    uint64_t c[kUse];
    uint32_t val[kUse];
    // Every load is issued before the first one is looked at (nothing but the load stands under
    // the condition: a use in there would be waited for before the next slot's load goes out).  A
    // slot past the end of the segment keeps all ones and sorts behind every pair.
    const uint64_t* const key_at = keys + lo + lane;
    const uint32_t* const value_at = values + lo + lane;
#pragma unroll
    for (int t = 0; t < kUse; t++) {
        c[t] = ~0ull;
        val[t] = ~0u;
        if (t * kWave + lane < len) {
            c[t] = key_at[t * kWave];
            val[t] = value_at[t * kWave];
        }
    }
    const uint32_t upper = (uint32_t)bcast_i((int)(uint32_t)(c[0] >> 32), 0);
    bool mixed = false;
#pragma unroll
    for (int t = 0; t < kUse; t++) {
        mixed = mixed || (t * kWave + lane < len && (uint32_t)(c[t] >> 32) != upper);
        c[t] <<= 32;                                                // the padding: depth of all ones
    }
    bool descends = false;   // position i + 1 holds a smaller value than position i
#pragma unroll
    for (int t = 0; t < kUse; t++) {
        uint32_t next = (uint32_t)__shfl_down((int)val[t], 1);
        if (t + 1 < kUse) {
            const uint32_t wrap = (uint32_t)bcast_i((int)val[t + 1 < kUse ? t + 1 : t], 0);
            if (lane == kWave - 1) next = wrap;
        }
        descends = descends || (t * kWave + lane + 1 < len && next < val[t]);
    }
    // (looked at behind the values on purpose: in front of them, their loads would wait for it)
    if (ballot(mixed)) {     // keys differ above the depth word: left to the general kernel
        if (seg_flags && lane == 0) atomicOr(&seg_flags[v >> 5], 1u << (v & 31));
        return;
    }
    const bool by_value = ballot(descends) == 0;
    // (no branches around the slots: where two paths meet, the sixteen words are copied from the
    // registers one path left them in to those of the other)
    uint32_t* const s_val = (uint32_t*)s_w;
#pragma unroll
    for (int t = 0; t < kUse; t++) {
        const int i = t * kWave + lane;
        if (!by_value && i < len) s_val[i] = val[t];
        c[t] |= by_value || i >= len ? val[t] : (uint32_t)i;     // the padding stays all ones
    }
    bitonic_network<kUse>(c, lane);
    asm volatile("" : "+v"(lane));
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int t = 0; t < kUse; t++) {
        const uint32_t low = (uint32_t)c[t];
        const uint32_t looked_up = s_val[by_value ? 0u : min(low, (uint32_t)(kUse * kWave - 1))];
        c[t] = (c[t] & 0xffffffff00000000ull) | (by_value ? low : looked_up);
    }
    // back to contiguous stores through LDS, the lower half of the ranks (lanes 0..31) first, then
    // the upper half through the same words: half the LDS, twice the waves per CU
    constexpr int kRounds = kUse >= 2 ? 2 : 1, kPart = kUse * kWave / kRounds;
    uint64_t* const key_to = keys + lo + lane;
    uint32_t* const value_to = values + lo + lane;
#pragma unroll
    for (int h = 0; h < kRounds; h++) {
        __builtin_amdgcn_wave_barrier();
        if (lane / (kWave / kRounds) == h) {
#pragma unroll
            for (int t = 0; t < kUse; t++) {
                const int r = lane * kUse + t;
                if (r < len) s_w[staged(r - h * kPart)] = c[t];
            }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int t = h * (kUse / kRounds); t < (h + 1) * (kUse / kRounds); t++) {
            const int i = t * kWave + lane;
            if (i < len) {
                const uint64_t w = s_w[staged(i - h * kPart)];
                key_to[t * kWave] = ((uint64_t)upper << 32) | (w >> 32);
                value_to[t * kWave] = (uint32_t)w;
            }
        }
    }
    __builtin_amdgcn_wave_barrier();
}

// The network over the smallest power of two of register slots (at most kT) that holds the segment.
// s_w: staging_words(64 * kT) 64-bit words.
template <int kT>
__device__ __forceinline__ void sort_segment_bitonic(uint64_t* __restrict__ keys, uint32_t* __restrict__ values,
                                                     uint32_t v, int lo, int hi, uint32_t* __restrict__ seg_flags,
                                                     uint64_t* s_w)
{
    const int len = hi - lo;
    if (len <= kWave) sort_segment_bitonic_of<1>(keys, values, v, lo, hi, seg_flags, s_w);
    else if (kT >= 2 && len <= 2 * kWave) sort_segment_bitonic_of<(kT >= 2 ? 2 : 1)>(keys, values, v, lo, hi, seg_flags, s_w);
    else if (kT >= 4 && len <= 4 * kWave) sort_segment_bitonic_of<(kT >= 4 ? 4 : 1)>(keys, values, v, lo, hi, seg_flags, s_w);
    else if (kT >= 8 && len <= 8 * kWave) sort_segment_bitonic_of<(kT >= 8 ? 8 : 1)>(keys, values, v, lo, hi, seg_flags, s_w);
    else sort_segment_bitonic_of<kT>(keys, values, v, lo, hi, seg_flags, s_w);
}

// One wave per workgroup; with a table of segment starts the workgroup looks at kIds tile ids
// (one per lane) and sorts those with min_len < length <= 64*kT one after the other; without a
// table the grid has one workgroup per tile id and each searches for its bounds.
template <int kT, int kIds>
__global__ __launch_bounds__(kWave) void segment_sort_wave_kernel(
    uint64_t* __restrict__ keys, uint32_t* __restrict__ values, int n, uint32_t tile_mask, int min_len, uint32_t ids,
    const int* __restrict__ seg_start, uint32_t* __restrict__ seg_flags,
    int list_max0, int list_max1, int list_max2,
    uint32_t* __restrict__ seg_counts, uint32_t* __restrict__ list0, uint32_t* __restrict__ list1,
    uint32_t* __restrict__ list2, uint32_t* __restrict__ list3,
    uint32_t list_cap0, uint32_t list_cap1, uint32_t list_cap2, uint32_t list_cap3)
{
    __shared__ uint64_t s_w[staging_words(kT * kWave)];
    const int lane = threadIdx.x;
    uint32_t first_id = blockIdx.x;
    uint64_t todo = 0;
    int lo_found = 0, hi_found = 0;
    if (!seg_start) {
        lo_found = wave_lower_bound(keys, n, first_id, tile_mask);
        hi_found = first_id == tile_mask ? n : wave_lower_bound(keys, n, first_id + 1, tile_mask);
        todo = hi_found - lo_found > min_len && hi_found - lo_found <= kT * kWave ? 1u : 0u;
    } else {
        first_id = blockIdx.x * (uint32_t)kIds;
        const uint32_t mine = first_id + (uint32_t)lane;
        int len = 0;
        if (lane < kIds && mine < ids) len = seg_start[mine + 1] - seg_start[mine];
        // This launch sees every tile id once: it also lists the ids of the longer segments by class
        // (lengths up to list_max0, list_max1, list_max2, and everything longer), so that those
        // fewer, longer-running segments can be dealt out evenly by the launches that follow.
        if (list0) {
            // neighbouring tiles tend to be equally busy: mix the index so that every list gets its share
            const uint32_t shard = (blockIdx.x ^ (blockIdx.x >> 5) ^ (blockIdx.x >> 10) ^ (blockIdx.x >> 15)) % kListShards;
            if (len > kT * kWave && len <= list_max0)
                list0[(size_t)shard * list_cap0 + atomicAdd(&seg_counts[0 * kListShards + shard], 1u)] = mine;
            else if (len > list_max0 && len <= list_max1)
                list1[(size_t)shard * list_cap1 + atomicAdd(&seg_counts[1 * kListShards + shard], 1u)] = mine;
            else if (len > list_max1 && len <= list_max2)
                list2[(size_t)shard * list_cap2 + atomicAdd(&seg_counts[2 * kListShards + shard], 1u)] = mine;
            else if (len > list_max2)
                list3[(size_t)shard * list_cap3 + atomicAdd(&seg_counts[3 * kListShards + shard], 1u)] = mine;
        }
        todo = ballot(len > min_len && len <= kT * kWave);
    }
    for (; todo; todo &= todo - 1) {
        const uint32_t v = first_id + (uint32_t)(__ffsll((long long)todo) - 1);
        const int lo = seg_start ? seg_start[v] : lo_found, hi = seg_start ? seg_start[v + 1] : hi_found;
        sort_segment_bitonic<kT>(keys, values, v, lo, hi, seg_flags, s_w);
        __builtin_amdgcn_wave_barrier();
    }
}

// The listed segments of one class (at most 64*kT pairs each), dealt out round-robin to
// single-wave workgroups.
template <int kT>
__global__ __launch_bounds__(kWave) void segment_sort_wave_list_kernel(
    uint64_t* __restrict__ keys, uint32_t* __restrict__ values, const int* __restrict__ seg_start,
    uint32_t* __restrict__ seg_flags, const uint32_t* __restrict__ list, const uint32_t* __restrict__ list_count,
    uint32_t list_cap)
{
    __shared__ uint64_t s_w[staging_words(kT * kWave)];
    const uint32_t shard = blockIdx.x % kListShards;
    const uint32_t count = list_count[shard];
    for (uint32_t i = blockIdx.x / kListShards; i < count; i += gridDim.x / kListShards) {
        const uint32_t v = list[(size_t)shard * list_cap + i];
        sort_segment_bitonic<kT>(keys, values, v, seg_start[v], seg_start[v + 1], seg_flags, s_w);
        __builtin_amdgcn_wave_barrier();
    }
}

// The same passes with whole keys and the ping-pong copy in HBM: for segments longer than
// min_len and for shorter segments whose keys differ above the depth word.  General and slow;
// inputs produced by fgs_preprocess only reach it with more than min_len pairs in one tile.
// Sixteen waves per workgroup: such a segment has thousands of pairs, every pass reads them from
// memory 64 per wave and step, and the workgroup has the CU almost to itself (a frame of 109M
// pairs with 534 such segments: 0.55 ms for the launch with four waves).
constexpr int kGeneralWaves = 16;

__device__ __forceinline__ void sort_segment_general(uint64_t* __restrict__ keys, uint32_t* __restrict__ values,
                                                     uint64_t* __restrict__ alt_keys, uint32_t* __restrict__ alt_values,
                                                     int lo, int hi, uint32_t (*s_cnt)[kBins], uint32_t* s_wave_sum, int* s_flag)
{
    const int tid = threadIdx.x;
    const int len = hi - lo;
    uint64_t* kbuf[2] = { keys + lo, alt_keys + lo };
    uint32_t* vbuf[2] = { values + lo, alt_values + lo };
    int cur = 0;
#pragma unroll 1
    for (int shift = 0; shift < 32; shift += 8) {
        const bool moved = counting_pass<kGeneralWaves, uint64_t>(kbuf[cur], vbuf[cur], kbuf[cur ^ 1], vbuf[cur ^ 1], len,
                                                                  shift, s_cnt, s_wave_sum, s_flag);
        __threadfence_block();
        __syncthreads();
        if (moved) cur ^= 1;
    }
    if (cur == 1)
        for (int i = tid; i < len; i += kGeneralWaves * kWave) { kbuf[0][i] = kbuf[1][i]; vbuf[0][i] = vbuf[1][i]; }
    __threadfence_block();
    __syncthreads();
}

// With a table of segment starts the first list_blocks workgroups take the listed segments (the
// ones longer than min_len: neighbouring tiles tend to be equally crowded, so they are dealt out
// one segment at a time, round-robin), the workgroups behind them look at 64 tile ids each for
// shorter segments that were flagged.
// With a table (kLds) a listed segment of up to kCapHuge pairs is sorted in LDS like the classes
// below it, sixteen pairs per thread in registers during a pass (a workgroup then has the LDS of
// its CU to itself): the passes through memory take 7 us each for 12 000 pairs, those in LDS 2.
// The listed blocks first sort the listed segments of the classes below (first_class 1:
// 1025 .. kCapLarge pairs, 2: only those above kCapMedium, 3: none; shard by shard like the
// launches of those classes): a frame with a short list of pairs has few such segments or none,
// and one launch instead of three is what counts there; up to kMergedLargeMax pairs the class
// above kCapMedium still has few.
constexpr int kCapHuge = 16384;

template <bool kLds>
__global__ __launch_bounds__(kGeneralWaves * kWave) void segment_sort_general_kernel(
    uint64_t* __restrict__ keys, uint32_t* __restrict__ values,
    uint64_t* __restrict__ alt_keys, uint32_t* __restrict__ alt_values,
    int n, uint32_t tile_mask, int min_len, uint32_t ids,
    const int* __restrict__ seg_start, const uint32_t* __restrict__ seg_flags,
    const uint32_t* __restrict__ list, const uint32_t* __restrict__ list_count, uint32_t list_cap, uint32_t list_blocks,
    const uint32_t* __restrict__ list_medium, uint32_t cap_medium, const uint32_t* __restrict__ list_large, uint32_t cap_large,
    int first_class)
{
    constexpr int kLdsCap = kLds ? kCapHuge : 1;
    __shared__ uint32_t s_k[kLdsCap];
    __shared__ uint32_t s_v[kLdsCap];
    __shared__ uint32_t s_cnt[kGeneralWaves][kBins];      // the passes in LDS use it as 16-bit counters
    __shared__ uint32_t s_wave_sum[kGeneralWaves];
    __shared__ int s_bounds[2];
    __shared__ int s_flag;
    __shared__ uint64_t s_match;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);

    if (!seg_start) {
        const uint32_t v = blockIdx.x;
        if (tid < kWave) {
            const int a = wave_lower_bound(keys, n, v, tile_mask);
            const int b = v == tile_mask ? n : wave_lower_bound(keys, n, v + 1, tile_mask);
            if (lane == 0) { s_bounds[0] = a; s_bounds[1] = b; s_flag = 0; }
        }
        __syncthreads();
        const int lo = s_bounds[0], hi = s_bounds[1];
        const int len = hi - lo;
        if (len < 2) return;
        if (len <= min_len) {       // without flags the shorter segments are re-examined here
            const uint32_t upper = (uint32_t)(keys[lo] >> 32);
            bool mixed = false;
            for (int i = tid; i < len; i += kGeneralWaves * kWave) mixed = mixed || (uint32_t)(keys[lo + i] >> 32) != upper;
            if (mixed) s_flag = 1;
            __syncthreads();
            const bool any_mixed = s_flag != 0;
            __syncthreads();
            if (!any_mixed) return;
        }
        sort_segment_general(keys, values, alt_keys, alt_values, lo, hi, s_cnt, s_wave_sum, &s_flag);
        return;
    }

    if (blockIdx.x < list_blocks) {
        const uint32_t shard = blockIdx.x % kListShards;
        // list_count: the counters of all classes, class c at c * kListShards (1: medium, 2: large, 3: long)
        for (int c = first_class; c <= 3; c++) {
            const uint32_t* const ids_of = c == 1 ? list_medium : c == 2 ? list_large : list;
            const uint32_t cap = c == 1 ? cap_medium : c == 2 ? cap_large : list_cap;
            const uint32_t count = list_count[c * kListShards + shard];
            for (uint32_t i = blockIdx.x / kListShards; i < count; i += list_blocks / kListShards) {
                const uint32_t v = ids_of[(size_t)shard * cap + i];
                const int lo = seg_start[v], hi = seg_start[v + 1];
                bool through_memory = true;
                if constexpr (kLds) {
                    // keys that differ above the depth word: through memory right away (no flag: the
                    // workgroups that look at the flags run beside this one)
                    if (hi - lo <= kCapHuge)
                        through_memory = sort_segment_lds<kGeneralWaves, kCapHuge>(keys, values, v, lo, hi, nullptr, s_k, s_v,
                                                                                   (uint16_t (*)[kBins])s_cnt, s_wave_sum, &s_flag);
                }
                if (through_memory) sort_segment_general(keys, values, alt_keys, alt_values, lo, hi, s_cnt, s_wave_sum, &s_flag);
            }
        }
        return;
    }
    const uint32_t first_id = (blockIdx.x - list_blocks) * (uint32_t)kWave;
    if (tid < kWave) {
        const uint32_t v = first_id + (uint32_t)lane;
        bool take = false;
        if (v < ids) {
            const int len = seg_start[v + 1] - seg_start[v];
            take = len > 1 && len <= min_len && ((seg_flags[v >> 5] >> (v & 31)) & 1u);
        }
        const uint64_t m = ballot(take);
        if (lane == 0) s_match = m;
    }
    __syncthreads();
    for (uint64_t todo = s_match; todo; todo &= todo - 1) {
        const uint32_t v = first_id + (uint32_t)(__ffsll((long long)todo) - 1);
        sort_segment_general(keys, values, alt_keys, alt_values, seg_start[v], seg_start[v + 1], s_cnt, s_wave_sum, &s_flag);
    }
}



} // namespace
} // namespace fgs

extern "C" size_t fgs_get_sort_buffer_size(int num_rendered)
{
    if (num_rendered < 0 || num_rendered > FGS_MAX_RENDERED) return 0;
    return fgs::workspace_for(num_rendered).total;
}

extern "C" int fgs_sort_gaussian(int num_rendered,
                                 int width, int height, int block_x, int block_y,
                                 char* list_sorting_space, size_t sorting_size,
                                 const uint64_t* gaussian_keys_unsorted, const uint32_t* gaussian_values_unsorted,
                                 uint64_t* gaussian_keys_sorted, uint32_t* gaussian_values_sorted, void* stream)
{
    using namespace fgs;
    if (num_rendered < 0)
        return fail(FGS_E_INVALID, "fgs_sort_gaussian: num_rendered = %d is negative "
                                   "(a negative count is what a failed preprocess leaves behind)", num_rendered);
    if (num_rendered > FGS_MAX_RENDERED)
        return fail(FGS_E_INVALID, "fgs_sort_gaussian: num_rendered = %d exceeds %d", num_rendered, FGS_MAX_RENDERED);
    if (width <= 0 || height <= 0 || block_x <= 0 || block_y <= 0)
        return fail(FGS_E_INVALID, "fgs_sort_gaussian: width/height/block must be positive");
    if (num_rendered == 0) return FGS_OK;
    if (!list_sorting_space || !gaussian_keys_unsorted || !gaussian_values_unsorted ||
        !gaussian_keys_sorted || !gaussian_values_sorted)
        return fail(FGS_E_INVALID, "fgs_sort_gaussian: null buffer");
    if ((uintptr_t)list_sorting_space % 256 != 0)
        return fail(FGS_E_INVALID, "fgs_sort_gaussian: list_sorting_space must be 256-byte aligned");
    if (((uintptr_t)gaussian_keys_unsorted | (uintptr_t)gaussian_keys_sorted) % 8 != 0)
        return fail(FGS_E_INVALID, "fgs_sort_gaussian: key buffers must be 8-byte aligned");

    const int n = num_rendered;
    const Workspace ws = workspace_for(n);
    if (sorting_size < ws.total)
        return fail(FGS_E_WORKSPACE, "fgs_sort_gaussian: list_sorting_space holds %zu bytes, %zu needed for %d pairs",
                    sorting_size, ws.total, n);

    const long long tiles_xy = (long long)((width + block_x - 1) / block_x) * ((height + block_y - 1) / block_y);
    if (tiles_xy >= (1LL << 30)) return fail(FGS_E_INVALID, "fgs_sort_gaussian: too many tiles");
    const int tile_bits = bit_length((uint32_t)tiles_xy);         // sort.cu:34-39: bits [0, 32 + tile_bits)
    const uint32_t tile_mask = (1u << tile_bits) - 1u;

    hipStream_t st = (hipStream_t)stream;
    uint64_t* alt_keys = (uint64_t*)(list_sorting_space + ws.alt_keys);
    uint32_t* alt_values = (uint32_t*)(list_sorting_space + ws.alt_values);
    uint32_t* hist = (uint32_t*)(list_sorting_space + ws.hist);
    uint32_t* chunk_sums = (uint32_t*)(list_sorting_space + ws.chunk_sums);

    // The table of segment starts (with it the flag words and the lists of the longer segments)
    // exists up to kMaxTableIds tile ids.  The last partition pass writes it when there are at
    // most two passes: with more, one workgroup could own 2^18 and more entries of a sparse frame.
    const uint32_t ids = 1u << tile_bits;
    int* seg_start = nullptr;
    uint32_t* seg_flags = nullptr;
    uint32_t* seg_counts = nullptr;
    if (n > 1 && ids <= kMaxTableIds) {
        seg_start = (int*)(list_sorting_space + ws.seg_start);
        seg_flags = (uint32_t*)(list_sorting_space + ws.seg_flags);
        seg_counts = (uint32_t*)(list_sorting_space + ws.seg_lists);
    }
    bool table_by_scatter = false;
    const bool one_wave_launch = seg_start && ids <= kOneLaunchIds;
    const uint32_t flag_words = (ids + 31) / 32;

    // 1. stable partition by tile id, least significant tile digit first
    auto partition = [&](auto shape) {
        using Shape = decltype(shape);
        const PassGrid g = pass_grid(n, Shape::kTile);
        const bool small = n <= kShortPairs;         // the scatter workgroups add up the histogram rows themselves
        const int passes = (tile_bits + Shape::kBits - 1) / Shape::kBits;
        table_by_scatter = seg_start && passes <= 2;
        const uint64_t* src_k = gaussian_keys_unsorted;
        const uint32_t* src_v = gaussian_values_unsorted;
        for (int p = 0; p < passes; p++) {
            const bool to_sorted = ((passes - p) & 1) != 0;      // the last pass lands in the caller's sorted buffers
            uint64_t* dst_k = to_sorted ? gaussian_keys_sorted : alt_keys;
            uint32_t* dst_v = to_sorted ? gaussian_values_sorted : alt_values;
            const int shift = 32 + Shape::kBits * p;
            const int nbits = tile_bits - Shape::kBits * p < Shape::kBits ? tile_bits - Shape::kBits * p : Shape::kBits;
            const bool last = p == passes - 1;
            if (small) {
                hipLaunchKernelGGL((count_kernel<Shape>), dim3(g.tiles), dim3(kSortBlock), 0, st, src_k, n, shift, nbits, hist,
                                   last ? seg_flags : nullptr, flag_words, seg_counts);
            } else {
                const int groups = g.chunk < kCountGroups ? g.chunk : kCountGroups;
                hipLaunchKernelGGL((count_chunk_kernel<Shape>), dim3(g.chunks), dim3(groups * kSortBlock), 0, st,
                                   src_k, n, shift, nbits, hist, g.tiles, g.chunk, chunk_sums,
                                   last ? seg_flags : nullptr, flag_words, seg_counts);
                hipLaunchKernelGGL((offsets_kernel<Shape>), dim3(g.chunks), dim3(g.chunks > 16 ? kOffsetThreads : Shape::kBinsP), 0, st,
                                   hist, g.tiles, g.chunk, chunk_sums, g.chunks);
            }
            if (last && table_by_scatter)
                hipLaunchKernelGGL((scatter_kernel<Shape, true>), dim3(g.tiles), dim3(kSortBlock), 0, st,
                                   src_k, src_v, dst_k, dst_v, n, shift, nbits, hist, small ? g.tiles : 0, seg_start);
            else
                hipLaunchKernelGGL((scatter_kernel<Shape, false>), dim3(g.tiles), dim3(kSortBlock), 0, st,
                                   src_k, src_v, dst_k, dst_v, n, shift, nbits, hist, small ? g.tiles : 0, (int*)nullptr);
            src_k = dst_k;
            src_v = dst_v;
        }
    };
    if (tile_bits <= kNarrowMaxTileBits) {
        if (n <= kShortPairs) partition(Short());
        else partition(Narrow());
    } else {
        partition(Wide());
    }

    // 2. every tile id's segment by depth, in place in the sorted buffers
    if (n > 1) {
        if (seg_start && !table_by_scatter) {
            const unsigned blocks = (unsigned)(((size_t)n + 256 * kStartsPerThread - 1) / (256 * kStartsPerThread));
            hipLaunchKernelGGL(segment_starts_kernel, dim3(blocks), dim3(256), 0, st,
                               (const uint64_t*)gaussian_keys_sorted, n, tile_mask, ids, seg_start, seg_flags, flag_words, seg_counts);
        }
        uint64_t* ks = gaussian_keys_sorted;
        uint32_t* vs = gaussian_values_sorted;
        seg_counts = (uint32_t*)(list_sorting_space + ws.seg_lists);
        const uint32_t cap_small = (uint32_t)(n / 512 + 2), cap_medium = (uint32_t)(n / 1024 + 2), cap_large = (uint32_t)(n / 4096 + 2),
                       cap_long = (uint32_t)(n / 8192 + 2);
        uint32_t* list_small = seg_counts + 128;
        uint32_t* list_medium = list_small + (size_t)kListShards * cap_small;
        uint32_t* list_large = list_medium + (size_t)kListShards * cap_medium;
        uint32_t* list_long = list_large + (size_t)kListShards * cap_large;
        const uint32_t* no_list = nullptr;
        // grids of the list-driven launches: a multiple of kListShards, enough for every listed segment
        // (the limits are several times what is resident at once: a workgroup takes every
        // (grid / kListShards)-th segment of its shard, and the shards are not equally long)
        auto list_grid = [](unsigned most, unsigned limit) {
            const unsigned g = most < limit ? most : limit;
            return (g + kListShards - 1) / kListShards * kListShards;
        };
#define FGS_SEGMENT_CLASS(WAVES, CAP, IDS, MINLEN, GRID, LIST, COUNT, LISTCAP)                                \
        hipLaunchKernelGGL((segment_sort_kernel<WAVES, CAP, IDS>), dim3(GRID), dim3((WAVES) * kWave), 0, st,  \
                           ks, vs, n, tile_mask, MINLEN, ids, (const int*)seg_start, seg_flags,               \
                           (const uint32_t*)(LIST), (const uint32_t*)(COUNT), LISTCAP)
        // Up to 512 pairs: one wave, bitonic network in registers; one tile id per wave (neighbouring
        // tiles tend to be equally busy, so a wave that took several of them would become the tail
        // of the launch).  With a table the launch also lists the longer segments.
        // Up to kOneLaunchIds tile ids the first launch takes the segments of 513..1024 pairs too,
        // with 16 register slots: on a frame of few tiles there are few of them, about one wave per
        // SIMD, and a launch of their own lasts as long as one such sort (1080p: -15 us, 4K: -8 us).
        // While the 16-slot code needed 145 registers, the launch over the 131 072 ids of an 8K
        // frame, most of them under 128 pairs, lost more to the three waves per SIMD than the
        // second launch cost (+40 us); at 75 registers it wins there as well (-12 us, and -0.28 ms
        // on the 8K frame of 109M pairs).
        if (one_wave_launch)
            hipLaunchKernelGGL((segment_sort_wave_kernel<kCapSmall / kWave, 1>), dim3(ids), dim3(kWave),
                               0, st, ks, vs, n, tile_mask, 1, ids, (const int*)seg_start, seg_flags,
                               kCapSmall, kCapMedium, kCapLarge, seg_counts, list_small, list_medium,
                               list_large, list_long, cap_small, cap_medium, cap_large, cap_long);
        else
            hipLaunchKernelGGL((segment_sort_wave_kernel<kCapTiny / kWave, 1>), dim3(ids), dim3(kWave),
                               0, st, ks, vs, n, tile_mask, 1, ids, (const int*)seg_start, seg_flags,
                               kCapSmall, kCapMedium, kCapLarge, seg_counts, seg_start ? list_small : nullptr, list_medium,
                               list_large, list_long, cap_small, cap_medium, cap_large, cap_long);
        // A short list of pairs has few segments of more than 1024 pairs, or none: there the one
        // launch below takes those classes too (720p, 0.2M pairs: two launches less).
        const bool merged_tail = seg_start && n <= kMergedTailMax;
        const bool merged_large = seg_start && !merged_tail && n <= kMergedLargeMax;
        if (seg_start) {
            if (n > kCapTiny && !one_wave_launch)       // 513..1024: the same network over 16 register slots, from the lists
                hipLaunchKernelGGL((segment_sort_wave_list_kernel<kCapSmall / kWave>),
                                   dim3(list_grid((unsigned)(n / (kCapTiny + 1) + 1), 8192u)),
                                   dim3(kWave), 0, st, ks, vs, (const int*)seg_start, seg_flags,
                                   (const uint32_t*)list_small, (const uint32_t*)seg_counts, cap_small);
            if (n > kCapSmall && !merged_tail) {
                FGS_SEGMENT_CLASS(8, kCapMedium, 64, kCapSmall, list_grid((unsigned)(n / (kCapSmall + 1) + 1), 4096u),
                                  list_medium, seg_counts + kListShards, cap_medium);
                if (n > kCapMedium && !merged_large)
                    FGS_SEGMENT_CLASS(16, kCapLarge, 64, kCapMedium, list_grid((unsigned)(n / (kCapMedium + 1) + 1), 1024u),
                                      list_large, seg_counts + 2 * kListShards, cap_large);
            }
        } else {
            if (n > kCapTiny) FGS_SEGMENT_CLASS(4, kCapSmall, 1, kCapTiny, ids, no_list, no_list, 0u);
            if (n > kCapSmall) FGS_SEGMENT_CLASS(8, kCapMedium, 64, kCapSmall, ids, no_list, no_list, 0u);
            if (n > kCapMedium) FGS_SEGMENT_CLASS(16, kCapLarge, 64, kCapMedium, ids, no_list, no_list, 0u);
        }
#undef FGS_SEGMENT_CLASS
        // longer segments from their list, one workgroup per segment; behind them the shorter ones that were flagged
        if (seg_start) {
            const int smallest = merged_tail ? kCapSmall : merged_large ? kCapMedium : kCapLarge;
            const unsigned blocks = n > smallest ? list_grid((unsigned)(n / (smallest + 1) + 1), n > kMergedLargeMax ? 2048u : 256u) : 0u;
            hipLaunchKernelGGL(segment_sort_general_kernel<true>, dim3(blocks + (ids + kWave - 1) / kWave),
                               dim3(kGeneralWaves * kWave), 0, st, ks, vs, alt_keys, alt_values, n, tile_mask, kCapLarge, ids,
                               (const int*)seg_start, (const uint32_t*)seg_flags,
                               (const uint32_t*)list_long, (const uint32_t*)seg_counts, cap_long, blocks,
                               (const uint32_t*)list_medium, cap_medium, (const uint32_t*)list_large, cap_large,
                               merged_tail ? 1 : merged_large ? 2 : 3);
        } else {
            hipLaunchKernelGGL(segment_sort_general_kernel<false>, dim3(ids),
                               dim3(kGeneralWaves * kWave), 0, st, ks, vs, alt_keys, alt_values, n, tile_mask, kCapLarge, ids,
                               (const int*)seg_start, (const uint32_t*)seg_flags,
                               no_list, no_list, 0u, 0u, no_list, 0u, no_list, 0u, 0);
        }
    }
    return check_hip(hipGetLastError(), "sort launch");
}
