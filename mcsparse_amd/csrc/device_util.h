// Wave64 building blocks shared by the gfx950 kernels.
#ifndef MCSPARSE_AMD_DEVICE_UTIL_H_
#define MCSPARSE_AMD_DEVICE_UTIL_H_

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

namespace mcsp {

constexpr int kWave = 64;

// DPP controls (gfx9 encoding)
constexpr int kDppQuadXor1 = 0xB1;      // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;      // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
template <int CTRL>
__device__ __forceinline__ double dpp_mov(double v) {
    const long long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_update_dpp(0, static_cast<int>(b), CTRL, 0xF, 0xF, false);
    const int hi = __builtin_amdgcn_update_dpp(0, static_cast<int>(b >> 32), CTRL, 0xF, 0xF, false);
    return __longlong_as_double((static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo));
}

// Sum over aligned groups of L consecutive lanes (L a power of two, 1..64); every lane of a
// group ends with the group's total.  Steps inside a row of 16 lanes are DPP moves; the
// 32- and 64-lane steps go through the LDS crossbar (ds_bpermute), which needs no LDS storage.
template <int L, typename T>
__device__ __forceinline__ T group_sum(T v) {
    if constexpr (L >= 2) v += dpp_mov<kDppQuadXor1>(v);
    if constexpr (L >= 4) v += dpp_mov<kDppQuadXor2>(v);
    if constexpr (L >= 8) v += dpp_mov<kDppRowHalfMirror>(v);
    if constexpr (L >= 16) v += dpp_mov<kDppRowMirror>(v);
    if constexpr (L >= 32) v += __shfl_xor(v, 16, kWave);
    if constexpr (L >= 64) v += __shfl_xor(v, 32, kWave);
    return v;
}

__device__ __forceinline__ unsigned lane_id() { return __lane_id(); }

// Streaming loads: data read once, kept from displacing the gathered operand in cache.
template <typename T>
__device__ __forceinline__ T load_stream(const T* p) {
    return __builtin_nontemporal_load(p);
}

}  // namespace mcsp

#endif  // MCSPARSE_AMD_DEVICE_UTIL_H_
