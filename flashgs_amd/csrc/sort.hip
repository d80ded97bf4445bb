// Device-wide stable LSD radix sort of (u64 key, u32 value) pairs for gfx950 (wave64).
//
// Stands in for the cub::DeviceRadixSort::SortPairs call of FlashGS
// (csrc/cuda_rasterizer/sort.cu:28-44): ascending, stable, on key bits [0, end_bit).
//
// Structure: one histogram launch counts all 8-bit digits of all passes, one small launch turns
// the counts into exclusive digit bases, then one launch per digit reorders the pairs.  A
// reorder workgroup ranks its tile of pairs in LDS (per-wave digit counters, wave64 ballot
// matching, so equal digits keep their input order), publishes the tile's digit counts and
// obtains the counts of all earlier tiles by walking back through their published words
// (chained scan with decoupled look-back; tiles are numbered by an atomic ticket so a tile only
// ever waits for tiles that already run).
#include "fgs_internal.h"

namespace fgs {
namespace {

constexpr int kBins = 256;
constexpr int kMaxPasses = 8;
constexpr int kSortBlock = 256;
constexpr int kSortWaves = kSortBlock / kWave;
constexpr int kItems = 8;                       // pairs per thread
constexpr int kTile = kSortBlock * kItems;      // pairs per workgroup
constexpr int kHistBlock = 256;
constexpr unsigned kSpinLimit = 1u << 22;

// status word of one (tile, digit): [31:30] state, [29:0] count
constexpr uint32_t kAggregate = 1u << 30;
constexpr uint32_t kPrefix = 2u << 30;
constexpr uint32_t kValueMask = (1u << 30) - 1;

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct Workspace {
    size_t alt_keys, alt_values, counters, status, total;
    int tiles;
};

// counters block: kMaxPasses*kBins digit counts/bases, then kMaxPasses tile tickets (padded)
constexpr size_t kCounterWords = kMaxPasses * kBins + 64;

Workspace workspace_for(int n)
{
    Workspace w;
    w.tiles = (n + kTile - 1) / kTile;
    w.alt_keys = 0;
    w.alt_values = align_up((size_t)n * 8, 256);
    w.counters = w.alt_values + align_up((size_t)n * 4, 256);
    w.status = w.counters + kCounterWords * 4;
    w.total = w.status + (size_t)kMaxPasses * w.tiles * kBins * 4;
    return w;
}

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* p, size_t n, uint32_t v)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

// counts[pass][digit] += number of keys whose digit `pass` equals `digit`
__global__ __launch_bounds__(kHistBlock) void histogram_kernel(const uint64_t* __restrict__ keys, int n,
                                                               int passes, int end_bit, uint32_t* __restrict__ counts)
{
    __shared__ uint32_t h[kMaxPasses * kBins];
    for (int j = threadIdx.x; j < passes * kBins; j += kHistBlock) h[j] = 0;
    __syncthreads();
    const int stride = gridDim.x * kHistBlock;
    for (int i = blockIdx.x * kHistBlock + threadIdx.x; i < n; i += stride) {
        const uint64_t k = keys[i];
        for (int p = 0; p < passes; p++) {
            const int shift = 8 * p;
            const int nbits = min(8, end_bit - shift);
            const uint32_t d = (uint32_t)(k >> shift) & ((1u << nbits) - 1u);
            atomicAdd(&h[p * kBins + d], 1u);
        }
    }
    __syncthreads();
    for (int j = threadIdx.x; j < passes * kBins; j += kHistBlock) {
        const uint32_t c = h[j];
        if (c) atomicAdd(&counts[j], c);
    }
}

// one workgroup per pass: counts[pass][*] -> exclusive prefix over digits, in place
__global__ __launch_bounds__(kBins) void digit_base_kernel(uint32_t* __restrict__ counts)
{
    __shared__ uint32_t s[kBins];
    uint32_t* c = counts + blockIdx.x * kBins;
    const int d = threadIdx.x;
    const uint32_t mine = c[d];
    s[d] = mine;
    __syncthreads();
    for (int o = 1; o < kBins; o <<= 1) {
        uint32_t add = d >= o ? s[d - o] : 0u;
        __syncthreads();
        s[d] += add;
        __syncthreads();
    }
    c[d] = s[d] - mine;
}

__device__ __forceinline__ uint32_t digit_of(uint64_t key, int shift, uint32_t mask)
{
    return (uint32_t)(key >> shift) & mask;
}

__global__ __launch_bounds__(kSortBlock) void reorder_kernel(
    const uint64_t* __restrict__ keys_in, const uint32_t* __restrict__ values_in,
    uint64_t* __restrict__ keys_out, uint32_t* __restrict__ values_out,
    int n, int shift, int nbits,
    const uint32_t* __restrict__ digit_base,     // [kBins] exclusive digit bases of this pass
    uint32_t* __restrict__ status,               // [tiles][kBins], zero before the launch
    uint32_t* __restrict__ ticket)               // zero before the launch
{
    __shared__ uint32_t s_count[kSortWaves][kBins];   // per-wave digit counts, then per-wave digit offsets
    __shared__ uint32_t s_bin_start[kBins];           // where each digit starts in the ranked tile
    __shared__ uint32_t s_global[kBins];              // destination of ranked slot p with digit d: s_global[d] + p
    __shared__ uint32_t s_wave_sum[kSortWaves];
    __shared__ uint64_t s_keys[kTile];
    __shared__ uint32_t s_values[kTile];
    __shared__ int s_tile;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const uint32_t mask = (1u << nbits) - 1u;

    if (tid == 0) s_tile = (int)atomicAdd(ticket, 1u);
#pragma unroll
    for (int w = 0; w < kSortWaves; w++) s_count[w][tid] = 0;
    __syncthreads();
    const int tile = s_tile;
    const int tile_base = tile * kTile;
    const int in_tile = min(kTile, n - tile_base);

    // ---- load: wave w owns slots [w*64*kItems, (w+1)*64*kItems) of the tile, item-major ----
    uint64_t key[kItems];
    uint32_t slot[kItems];
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int off = wave * (kWave * kItems) + i * kWave + lane;
        key[i] = off < in_tile ? keys_in[tile_base + off] : ~0ull;
    }

    // ---- rank inside the wave: lanes with equal digits find each other with 8 ballots ----
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int off = wave * (kWave * kItems) + i * kWave + lane;
        const bool valid = off < in_tile;
        const uint32_t d = digit_of(key[i], shift, mask);
        uint64_t peers = ballot(valid);
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const bool bit = (d >> b) & 1u;
            const uint64_t with_bit = ballot(bit);
            peers &= bit ? with_bit : ~with_bit;
        }
        const int below = popc_below(peers);
        uint32_t before = 0;
        if (valid && below == 0) {      // lowest lane of each group updates the wave's counter
            before = s_count[wave][d];
            s_count[wave][d] = before + (uint32_t)__popcll(peers);
        }
        const int leader = valid ? __ffsll((long long)peers) - 1 : lane;
        before = (uint32_t)__shfl((int)before, leader);
        slot[i] = before + (uint32_t)below;
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();

    // ---- digit totals of the tile; per-wave offsets inside each digit ----
    const int d = tid;      // one thread per digit from here on
    uint32_t total = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; w++) {
        const uint32_t c = s_count[w][d];
        s_count[w][d] = total;
        total += c;
    }
    if (tile == 0)
        __hip_atomic_store(status + d, kPrefix | total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        __hip_atomic_store(status + (size_t)tile * kBins + d, kAggregate | total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // exclusive scan of the totals over the 256 digits
    uint32_t incl = total;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        uint32_t up = (uint32_t)__shfl_up((int)incl, o);
        if (lane >= o) incl += up;
    }
    if (lane == kWave - 1) s_wave_sum[wave] = incl;
    __syncthreads();
    uint32_t before_wave = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; w++)
        if (w < wave) before_wave += s_wave_sum[w];
    const uint32_t bin_start = before_wave + incl - total;
    s_bin_start[d] = bin_start;
    __syncthreads();

    // ---- move the pairs to their ranked slots in LDS ----
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int off = wave * (kWave * kItems) + i * kWave + lane;
        if (off < in_tile) {
            const uint32_t dg = digit_of(key[i], shift, mask);
            const uint32_t p = s_bin_start[dg] + s_count[wave][dg] + slot[i];
            s_keys[p] = key[i];
            s_values[p] = values_in[tile_base + off];
        }
    }

    // ---- counts of all earlier tiles for digit d ----
    uint32_t earlier = 0;
    if (tile > 0) {
        unsigned spins = 0;
        int j = tile - 1;
        while (j >= 0) {
            const uint32_t w = __hip_atomic_load(status + (size_t)j * kBins + d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t st = w & ~kValueMask;
            if (st == 0) {
                if (++spins > kSpinLimit) break;        // bounded wait: give up rather than hang
                __builtin_amdgcn_s_sleep(1);
                continue;
            }
            earlier += w & kValueMask;
            if (st == kPrefix) break;
            j--;
        }
        __hip_atomic_store(status + (size_t)tile * kBins + d, kPrefix | ((earlier + total) & kValueMask),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    s_global[d] = digit_base[d] + earlier - bin_start;
    __syncthreads();

    // ---- write out: neighbouring threads hold neighbouring ranked slots ----
#pragma unroll
    for (int i = 0; i < kItems; i++) {
        const int p = i * kSortBlock + tid;
        if (p < in_tile) {
            const uint64_t k = s_keys[p];
            const uint32_t dst = s_global[digit_of(k, shift, mask)] + (uint32_t)p;
            keys_out[dst] = k;
            values_out[dst] = s_values[p];
        }
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

    const Workspace ws = workspace_for(num_rendered);
    if (sorting_size < ws.total)
        return fail(FGS_E_WORKSPACE, "fgs_sort_gaussian: list_sorting_space holds %zu bytes, %zu needed for %d pairs",
                    sorting_size, ws.total, num_rendered);

    const long long tiles_xy = (long long)((width + block_x - 1) / block_x) * ((height + block_y - 1) / block_y);
    if (tiles_xy > 0xffffffffLL) return fail(FGS_E_INVALID, "fgs_sort_gaussian: too many tiles");
    const int end_bit = 32 + bit_length((uint32_t)tiles_xy);     // sort.cu:34-39
    const int passes = (end_bit + 7) / 8;

    hipStream_t st = (hipStream_t)stream;
    uint64_t* alt_keys = (uint64_t*)(list_sorting_space + ws.alt_keys);
    uint32_t* alt_values = (uint32_t*)(list_sorting_space + ws.alt_values);
    uint32_t* counters = (uint32_t*)(list_sorting_space + ws.counters);
    uint32_t* tickets = counters + kMaxPasses * kBins;
    uint32_t* status = (uint32_t*)(list_sorting_space + ws.status);

    // counters, tickets and the status words of the passes that run are contiguous
    const size_t zero_words = kCounterWords + (size_t)passes * ws.tiles * kBins;
    size_t fill_blocks = (zero_words + 2047) / 2048;
    if (fill_blocks > 2048) fill_blocks = 2048;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)fill_blocks), dim3(256), 0, st, counters, zero_words, 0u);

    const int hist_blocks = ws.tiles < 1024 ? ws.tiles : 1024;
    hipLaunchKernelGGL(histogram_kernel, dim3(hist_blocks), dim3(kHistBlock), 0, st,
                       gaussian_keys_unsorted, num_rendered, passes, end_bit, counters);
    hipLaunchKernelGGL(digit_base_kernel, dim3(passes), dim3(kBins), 0, st, counters);

    const uint64_t* src_k = gaussian_keys_unsorted;
    const uint32_t* src_v = gaussian_values_unsorted;
    for (int p = 0; p < passes; p++) {
        const bool to_sorted = ((passes - p) & 1) != 0;      // the last pass lands in the caller's sorted buffers
        uint64_t* dst_k = to_sorted ? gaussian_keys_sorted : alt_keys;
        uint32_t* dst_v = to_sorted ? gaussian_values_sorted : alt_values;
        const int shift = 8 * p;
        const int nbits = end_bit - shift < 8 ? end_bit - shift : 8;
        hipLaunchKernelGGL(reorder_kernel, dim3(ws.tiles), dim3(kSortBlock), 0, st,
                           src_k, src_v, dst_k, dst_v, num_rendered, shift, nbits,
                           counters + p * kBins, status + (size_t)p * ws.tiles * kBins, tickets + p);
        src_k = dst_k;
        src_v = dst_v;
    }
    return check_hip(hipGetLastError(), "radix sort launch");
}
