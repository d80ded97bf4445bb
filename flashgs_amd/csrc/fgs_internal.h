// Internal declarations shared by the HIP translation units of libflashgs_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include <thread>
#include <tuple>

#include "../../include/flashgs_hip.h"

namespace fgs {

// Records `msg` as this thread's last error and returns `code`.
int fail(int code, const char* fmt, ...);

// Maps a HIP status to FGS_OK / FGS_E_HIP (recording the HIP error text).
int check_hip(hipError_t st, const char* what);

#define FGS_HIP_TRY(expr)                                  \
    do {                                                   \
        int _rc = ::fgs::check_hip((expr), #expr);         \
        if (_rc != FGS_OK) return _rc;                     \
    } while (0)

// Host camera set-up (FlashGS preprocess.cu:420-448): column-major view and projection.
void camera_matrices(const float pos[3], const float rot[9], int width, int height,
                     float fx, float fy, float zFar, float zNear, float view[16], float proj[16]);

// bit_length(n) - what FlashGS sort.cu:9-24 (getHigherMsb) evaluates to.
inline int bit_length(uint32_t n)
{
    int b = 0;
    while (n) { b++; n >>= 1; }
    return b;
}

// What the library's per-stream memory is keyed by.  hipStreamPerThread is one handle that names a
// different stream in every host thread, so there the thread is part of the key.
typedef std::tuple<int, hipStream_t, std::thread::id> StreamKey;
inline StreamKey stream_key(int device, hipStream_t stream)
{
    return StreamKey(device, stream, stream == hipStreamPerThread ? std::this_thread::get_id() : std::thread::id());
}

constexpr int kWave = 64;

// ---- device-side wave helpers (wave64) --------------------------------------------------------

__device__ __forceinline__ int lane_id()
{
    return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// number of set bits of `m` strictly below this lane
__device__ __forceinline__ int popc_below(uint64_t m)
{
    return (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
}

__device__ __forceinline__ uint64_t ballot(bool p) { return __builtin_amdgcn_ballot_w64(p); }

__device__ __forceinline__ int bcast_i(int v, int src_lane) { return __builtin_amdgcn_readlane(v, src_lane); }
__device__ __forceinline__ float bcast_f(float v, int src_lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src_lane));
}

// Inclusive prefix sum over the 64 lanes of a wave with data-parallel-primitive moves (VALU only):
// shifts by 1, 2, 4, 8 inside each row of 16 lanes, then the last lane of rows 0 and 2 is added
// to rows 1 and 3, then lane 31 to rows 2 and 3.  Lanes without a source add 0.
__device__ __forceinline__ uint32_t wave_inclusive_sum(uint32_t x)
{
    constexpr int kRowShr1 = 0x111, kRowShr2 = 0x112, kRowShr4 = 0x114, kRowShr8 = 0x118;
    constexpr int kRowBcast15 = 0x142, kRowBcast31 = 0x143;
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kRowShr1, 0xf, 0xf, false);
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kRowShr2, 0xf, 0xf, false);
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kRowShr4, 0xf, 0xf, false);
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kRowShr8, 0xf, 0xf, false);
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kRowBcast15, 0xa, 0xf, false);
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kRowBcast31, 0xc, 0xf, false);
    return x;
}

} // namespace fgs
