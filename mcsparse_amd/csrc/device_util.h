// Wave64 building blocks shared by the gfx950 kernels.
#ifndef MCSPARSE_AMD_DEVICE_UTIL_H_
#define MCSPARSE_AMD_DEVICE_UTIL_H_

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>
#include <utility>

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

// Value held by lane U of every aligned group of L consecutive lanes (L = 4..64, U < L), with
// no trip through memory: a quad permute for L = 4, row broadcasts (one per half row for L = 8)
// inside the 16-lane DPP rows, lane reads into scalar registers beyond that.
template <int L, int U>
__device__ __forceinline__ int group_bcast_bits(int v) {
    static_assert(L >= 4 && L <= kWave && (L & (L - 1)) == 0 && U >= 0 && U < L, "group shape");
    // mov_dpp leaves the previous contents of the destination undefined, which is fine where
    // every lane receives a value and lets the compiler fold the move into the instruction
    // that uses it.
    if constexpr (L == 4) {
        return __builtin_amdgcn_mov_dpp(v, U | (U << 2) | (U << 4) | (U << 6), 0xF, 0xF, true);
    } else if constexpr (L == 8) {
        constexpr int kRowBcast = 0x150;  // row_newbcast:0
        const int lower = __builtin_amdgcn_mov_dpp(v, kRowBcast + U, 0xF, 0xF, true);
        return __builtin_amdgcn_update_dpp(lower, v, kRowBcast + 8 + U, 0xF, 0xC, false);
    } else if constexpr (L == 16) {
        return __builtin_amdgcn_mov_dpp(v, 0x150 + U, 0xF, 0xF, true);
    } else if constexpr (L == 32) {
        const int lower = __builtin_amdgcn_readlane(v, U);
        const int upper = __builtin_amdgcn_readlane(v, 32 + U);
        return __lane_id() < 32 ? lower : upper;
    } else {
        return __builtin_amdgcn_readlane(v, U);
    }
}
template <int L, int U>
__device__ __forceinline__ uint32_t group_bcast(uint32_t v) {
    return static_cast<uint32_t>(group_bcast_bits<L, U>(static_cast<int>(v)));
}
template <int L, int U>
__device__ __forceinline__ uint64_t group_bcast(uint64_t v) {
    const int lo = group_bcast_bits<L, U>(static_cast<int>(v));
    const int hi = group_bcast_bits<L, U>(static_cast<int>(v >> 32));
    return (static_cast<uint64_t>(static_cast<uint32_t>(hi)) << 32) | static_cast<uint32_t>(lo);
}
template <int L, int U>
__device__ __forceinline__ float group_bcast(float v) {
    return __int_as_float(group_bcast_bits<L, U>(__float_as_int(v)));
}
template <int L, int U>
__device__ __forceinline__ double group_bcast(double v) {
    const long long b = __double_as_longlong(v);
    const int lo = group_bcast_bits<L, U>(static_cast<int>(b));
    const int hi = group_bcast_bits<L, U>(static_cast<int>(b >> 32));
    return __longlong_as_double((static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo));
}

// f(std::integral_constant<int, 0>{}) ... f(std::integral_constant<int, N-1>{}): a loop whose
// counter is a constant expression inside the body.
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

__device__ __forceinline__ unsigned lane_id() { return __lane_id(); }

// Streaming loads: data read once, kept from displacing the gathered operand in cache.
template <typename T>
__device__ __forceinline__ T load_stream(const T* p) {
    return __builtin_nontemporal_load(p);
}

}  // namespace mcsp

#endif  // MCSPARSE_AMD_DEVICE_UTIL_H_
