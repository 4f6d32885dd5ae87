// Device helpers shared by the SpMM kernels (spmm.hip, spmm_blocks.hip): 128-bit row accesses of op(B) and C,
// the XCD-aware workgroup order, and one row of A times op(B) for a lane group.
#ifndef MCSPARSE_AMD_SPMM_DEVICE_H_
#define MCSPARSE_AMD_SPMM_DEVICE_H_

#include "device_util.h"
#include "internal.h"

namespace mcsp {
namespace spmm_detail {

constexpr int kBlock = 256;

template <typename T, int V>
struct Vec {
    T v[V];
};

template <typename T, int V>
__device__ __forceinline__ Vec<T, V> load_vec(const T* p) {
    Vec<T, V> r;
    if constexpr (V == 1) {
        r.v[0] = p[0];
    } else if constexpr (sizeof(T) * V == 16) {
        typedef T Native __attribute__((ext_vector_type(V)));
        const Native n = *reinterpret_cast<const Native*>(p);
#pragma unroll
        for (int i = 0; i < V; ++i) r.v[i] = n[i];
    } else {
        static_assert(sizeof(T) * V == 8, "unsupported vector width");
        typedef T Native __attribute__((ext_vector_type(V)));
        const Native n = *reinterpret_cast<const Native*>(p);
#pragma unroll
        for (int i = 0; i < V; ++i) r.v[i] = n[i];
    }
    return r;
}

// Stores of C: written once and not read again by the call, so they are marked as streaming, which keeps the
// rows of op(B) in cache and lets the lines leave as they fill (N = 64: 552 -> 535 us, N = 256: 1.90 -> 1.82 ms).
template <typename T, int V>
__device__ __forceinline__ void store_vec(T* p, const Vec<T, V>& r) {
    if constexpr (V == 1) {
        __builtin_nontemporal_store(r.v[0], p);
    } else {
        typedef T Native __attribute__((ext_vector_type(V)));
        Native n;
#pragma unroll
        for (int i = 0; i < V; ++i) n[i] = r.v[i];
        __builtin_nontemporal_store(n, reinterpret_cast<Native*>(p));
    }
}

// Byte offsets into op(B) are 32-bit when the whole operand lies within 4 GiB of its first
// element (WIDE = false): a row's offset then travels between lanes in one register and the
// load takes it next to the scalar base address, which leaves one vector instruction of address
// arithmetic per row of op(B).
template <bool WIDE>
struct ByteOffset { typedef uint32_t type; };
template <>
struct ByteOffset<true> { typedef uint64_t type; };

// Workgroups are handed to the XCDs of a device in turn (workgroup h runs on XCD h % xcds), each XCD with
// an L2 of its own.  Rows that are close in the matrix tend to read the same rows of op(B), so
// an XCD should work on a contiguous stretch of rows: this maps the hardware's workgroup number
// to a position such that every XCD takes `chunk` consecutive positions at a time.  chunk = 1 (or one XCD)
// is the identity; positions past `count` (the grid is padded to whole rounds) do no work.
__device__ __forceinline__ uint64_t xcd_position(uint32_t hw_block, uint32_t chunk, uint32_t xcds) {
    const uint32_t per_round = xcds * chunk;
    const uint32_t round = hw_block / per_round;
    const uint32_t rem = hw_block % per_round;
    return static_cast<uint64_t>(round) * per_round + (rem % xcds) * chunk + rem / xcds;
}
inline uint32_t xcd_padded_grid(uint64_t count, uint32_t chunk, uint32_t xcds) {
    const uint64_t per_round = static_cast<uint64_t>(xcds) * chunk;
    return static_cast<uint32_t>((count + per_round - 1) / per_round * per_round);
}

// acc += sum over the nonzeros [begin, end) of one row of A of value * (V columns of the row of
// op(B) the nonzero names), for a group of LR >= 4 lanes that all pass the same range.
// B_bytes is the operand's first element, lane_off the byte offset of this lane's columns.
//
// What bounds these kernels is the return path of the vector memory unit, and a load in which
// all lanes of a group ask for the same word still returns a word per lane.  So the lanes fetch
// LR nonzeros of the row at once, one each, turn them into row offsets, and pass offsets and
// values round in registers; the loop then loads rows of op(B) and nothing else.
template <typename T, int LR, int V, bool WIDE>
__device__ __forceinline__ void row_times_b(idx_t begin, idx_t end, idx_t lane, idx_t base,
                                            const idx_t* __restrict__ col, const T* __restrict__ val,
                                            const char* __restrict__ B_bytes,
                                            typename ByteOffset<WIDE>::type lane_off,
                                            typename ByteOffset<WIDE>::type ldb_bytes, T (&acc)[V]) {
    typedef typename ByteOffset<WIDE>::type off_t;
    constexpr int kBatch = LR < 8 ? LR : 8;  // rows of op(B) in flight per lane
    for (idx_t j = begin; j < end; j += LR) {
        const bool has = j + lane < end;
        const off_t roff = has ? static_cast<off_t>(col[j + lane] - base) * ldb_bytes : off_t(0);
        const T aa = has ? val[j + lane] : T(0);
        const idx_t left = end - j;
        auto chunk = [&](auto checked) {
            constexpr bool kChecked = decltype(checked)::value;
            static_for<LR / kBatch>([&](auto g) {
                constexpr int u0 = decltype(g)::value * kBatch;
                if (!kChecked || u0 < left) {
                    Vec<T, V> b[kBatch];
                    static_for<kBatch>([&](auto u) {
                        constexpr int k = u0 + decltype(u)::value;
                        if (!kChecked || k < left) {  // the same for all lanes of the group
                            const off_t off = group_bcast<LR, k>(roff) + lane_off;
                            b[decltype(u)::value] = load_vec<T, V>(reinterpret_cast<const T*>(B_bytes + off));
                        }
                    });
                    static_for<kBatch>([&](auto u) {
                        constexpr int k = u0 + decltype(u)::value;
                        if (!kChecked || k < left) {
                            const T a = group_bcast<LR, k>(aa);
#pragma unroll
                            for (int i = 0; i < V; ++i) acc[i] += a * b[decltype(u)::value].v[i];
                        }
                    });
                }
            });
        };
        if (left >= LR) chunk(std::false_type{});
        else chunk(std::true_type{});
    }
}

// Writes V adjacent columns of one row of C: beta*C + alpha*acc, C untouched by reads if beta == 0.
template <typename T, int V>
__device__ __forceinline__ void store_c(T* __restrict__ C, int64_t ldc, bool c_row_major, uint64_t row, uint64_t c0,
                                        const T (&acc)[V], T alpha, T beta) {
    const bool beta0 = beta == T(0);
    if (c_row_major) {
        T* Cp = C + static_cast<int64_t>(row) * ldc + c0;
        Vec<T, V> out;
        if (beta0) {
#pragma unroll
            for (int i = 0; i < V; ++i) out.v[i] = alpha * acc[i];
        } else {
            const Vec<T, V> old = load_vec<T, V>(Cp);
#pragma unroll
            for (int i = 0; i < V; ++i) out.v[i] = beta * old.v[i] + alpha * acc[i];
        }
        store_vec<T, V>(Cp, out);
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) {
            T* Cp = C + static_cast<int64_t>(c0 + i) * ldc + row;
            *Cp = beta0 ? alpha * acc[i] : beta * *Cp + alpha * acc[i];
        }
    }
}

// Four consecutive rows of one column of a column-major C (16-byte aligned): beta*C + alpha*acc with
// 128-bit accesses, C untouched by reads if beta == 0.
template <typename T>
__device__ __forceinline__ void store_c_four_rows(T* __restrict__ Cp, T a0, T a1, T a2, T a3, T alpha, T beta) {
    constexpr int W = 16 / sizeof(T);  // elements per 128-bit access: 4 floats, 2 doubles
    const T acc[4] = {a0, a1, a2, a3};
    const bool beta0 = beta == T(0);
#pragma unroll
    for (int h = 0; h < 4 / W; ++h) {
        Vec<T, W> out;
        if (beta0) {
#pragma unroll
            for (int i = 0; i < W; ++i) out.v[i] = alpha * acc[h * W + i];
        } else {
            const Vec<T, W> old = load_vec<T, W>(Cp + h * W);
#pragma unroll
            for (int i = 0; i < W; ++i) out.v[i] = beta * old.v[i] + alpha * acc[h * W + i];
        }
        store_vec<T, W>(Cp + h * W, out);
    }
}

// op(B) lies within 4 GiB of its first element: byte offsets into it fit 32 bits
inline bool narrow_offsets(const SpmmArgs& a, size_t value_bytes) {
    const uint64_t last = (a.k == 0 ? 0 : static_cast<uint64_t>(a.k) - 1) * static_cast<uint64_t>(a.ldb) + a.n;
    return last * value_bytes <= 0xffffffffull;
}

}  // namespace spmm_detail
}  // namespace mcsp

#endif  // MCSPARSE_AMD_SPMM_DEVICE_H_
