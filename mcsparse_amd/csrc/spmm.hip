// CSR SpMM for gfx950: C = alpha*A*op(B) + beta*C, A is m x k CSR, op(B) is k x n dense.
//
// The reference (src/kernels/level3/spmm/csr_spmm_device.hpp:91-167) runs one wavefront per
// (row, output column) and therefore re-reads the CSR row n times, after transposing a
// row-major B into a freshly allocated column-major copy (mcsp_spmm_gpu.cpp:119-133).  Here a
// row-major op(B) is read in place: a lane group owns one row of A and each lane a few adjacent
// columns of C, so every nonzero pulls one contiguous stretch of a row of B with wide loads and
// A is read once per column panel.  When consecutive rows of A share columns (stencils, banded
// and finite-element matrices) the same rows of B would be pulled through L1 again and again, so
// the main kernel first de-duplicates the column indices of its block of rows with a hash table in
// LDS, stages every distinct row of B in LDS once, and accumulates from there.  A column-major
// op(B) is handled by a gather kernel with the lanes spread over the nonzeros of the row.  With
// beta == 0, C is never read.
#include <cstdlib>

#include "device_util.h"
#include "internal.h"

namespace mcsp {

namespace {

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

template <typename T, int V>
__device__ __forceinline__ void store_vec(T* p, const Vec<T, V>& r) {
    if constexpr (V == 1) {
        p[0] = r.v[0];
    } else {
        typedef T Native __attribute__((ext_vector_type(V)));
        Native n;
#pragma unroll
        for (int i = 0; i < V; ++i) n[i] = r.v[i];
        *reinterpret_cast<Native*>(p) = n;
    }
}

// op(B) row-major.  LR lanes per row of A, V adjacent columns per lane; blockIdx.y walks the
// column panels of LR*V columns.  V > 1 requires n, ldb (and ldc when C is row-major) to be
// multiples of V and 16-byte aligned base pointers, which the launcher checks.
template <typename T, int LR, int V, bool BETA0, bool C_ROW>
__global__ __launch_bounds__(kBlock) void spmm_rowb_kernel(idx_t m, idx_t n, idx_t base,
                                                           const idx_t* __restrict__ row_ptr,
                                                           const idx_t* __restrict__ col, const T* __restrict__ val,
                                                           const T* __restrict__ B, int64_t ldb, T* __restrict__ C,
                                                           int64_t ldc, T alpha, T beta) {
    constexpr int kRowsPerBlock = kBlock / LR;
    const idx_t lane = threadIdx.x % LR;
    const uint64_t row = static_cast<uint64_t>(blockIdx.x) * kRowsPerBlock + threadIdx.x / LR;
    const uint64_t c0 = (static_cast<uint64_t>(blockIdx.y) * LR + lane) * V;
    if (row >= m || c0 >= n) return;

    const idx_t start = row_ptr[row] - base;
    const idx_t end = row_ptr[row + 1] - base;
    T acc[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = T(0);

    constexpr int kUnroll = 8;
    const T* Bc = B + c0;
    idx_t j = start;
    for (; j + kUnroll <= end; j += kUnroll) {
        idx_t c[kUnroll];
        T a[kUnroll];
        Vec<T, V> b[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            c[u] = col[j + u] - base;
            a[u] = val[j + u];
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) b[u] = load_vec<T, V>(Bc + static_cast<int64_t>(c[u]) * ldb);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i] += a[u] * b[u].v[i];
        }
    }
    for (; j < end; ++j) {
        const idx_t c = col[j] - base;
        const T a = val[j];
        const Vec<T, V> b = load_vec<T, V>(Bc + static_cast<int64_t>(c) * ldb);
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] += a * b.v[i];
    }

    if constexpr (C_ROW) {
        T* Cp = C + static_cast<int64_t>(row) * ldc + c0;
        Vec<T, V> out;
        if constexpr (BETA0) {
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
            if constexpr (BETA0) {
                *Cp = alpha * acc[i];
            } else {
                *Cp = beta * *Cp + alpha * acc[i];
            }
        }
    }
}

// Row-major op(B) and C with LDS staging.  A workgroup owns R consecutive rows of A, one lane
// group of LR lanes per row, V adjacent columns per lane, and walks the columns of C in panels
// of LR*V.  Per workgroup:
//   1. the column indices of all its nonzeros go into an open-addressing hash table in LDS
//      (atomicCAS, linear probing), which leaves every distinct column in exactly one slot;
//   2. a scan over the slots numbers the distinct columns 0..D-1;
//   3. per panel, the D rows of B are copied to LDS once (128-bit coalesced loads), then every
//      lane group accumulates its row of C from LDS.
// A block whose nonzeros (CNT_CAP) or distinct columns (D_CAP) do not fit falls back to reading B
// from global memory, so any matrix is handled; the result does not depend on which path ran
// beyond the usual rounding, because both add the products of a row in column order.
constexpr idx_t kEmptySlot = 0xFFFFFFFFu;

template <typename T, int LR, int V, int R, int CNT_CAP, int D_CAP, int HASH, bool BETA0>
__global__ __launch_bounds__(R* LR) void spmm_rowb_lds_kernel(idx_t m, idx_t n, idx_t base,
                                                              const idx_t* __restrict__ row_ptr,
                                                              const idx_t* __restrict__ col,
                                                              const T* __restrict__ val, const T* __restrict__ B,
                                                              int64_t ldb, T* __restrict__ C, int64_t ldc, T alpha,
                                                              T beta) {
    constexpr int NT = R * LR;
    constexpr int PANEL = LR * V;
    constexpr int SPT = HASH / NT;  // hash slots per thread in the numbering pass
    static_assert(HASH % NT == 0 && (HASH & (HASH - 1)) == 0, "hash size");
    static_assert(NT % kWave == 0 && NT <= 1024, "workgroup size");
    static_assert(D_CAP <= 65535 && HASH <= 65536, "ids are 16 bit");
    constexpr int kHashShift = 32 - __builtin_ctz(HASH);

    __shared__ idx_t s_tab[HASH];
    __shared__ uint16_t s_idmap[HASH];
    __shared__ uint16_t s_slot[CNT_CAP];
    __shared__ T s_val[CNT_CAP];
    __shared__ idx_t s_keys[D_CAP];
    __shared__ T s_tile[D_CAP * PANEL];
    __shared__ idx_t s_ptr[R + 1];
    __shared__ uint32_t s_wave[NT / kWave];

    const uint32_t tid = threadIdx.x;
    const uint64_t r0 = static_cast<uint64_t>(blockIdx.x) * R;
    if (tid <= R) {
        const uint64_t r = r0 + tid < m ? r0 + tid : m;
        s_ptr[tid] = row_ptr[r] - base;
    }
    for (uint32_t i = tid; i < HASH; i += NT) s_tab[i] = kEmptySlot;
    __syncthreads();
    const idx_t start = s_ptr[0];
    const idx_t cnt = s_ptr[R] - start;
    bool staged = cnt <= CNT_CAP;  // uniform over the workgroup
    uint32_t distinct = 0;
    if (staged) {
        for (idx_t k = tid; k < cnt; k += NT) {
            const idx_t c = col[start + k] - base;
            s_val[k] = val[start + k];
            uint32_t h = (c * 0x9E3779B1u) >> kHashShift;
            while (true) {
                const idx_t old = atomicCAS(&s_tab[h], kEmptySlot, c);
                if (old == kEmptySlot || old == c) break;
                h = (h + 1) & (HASH - 1);
            }
            s_slot[k] = static_cast<uint16_t>(h);
        }
        __syncthreads();
        // number the occupied slots
        uint32_t mine = 0;
#pragma unroll
        for (int i = 0; i < SPT; ++i) mine += s_tab[tid * SPT + i] != kEmptySlot;
        // block-wide exclusive scan of `mine`
        const unsigned lane64 = tid % kWave, wave = tid / kWave;
        uint32_t inc = mine;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const uint32_t up = __shfl_up(inc, off, kWave);
            if (lane64 >= static_cast<unsigned>(off)) inc += up;
        }
        if (lane64 == kWave - 1) s_wave[wave] = inc;
        __syncthreads();
        uint32_t id = inc - mine;
#pragma unroll
        for (unsigned w = 0; w < NT / kWave; ++w) {
            const uint32_t t = s_wave[w];
            if (w < wave) id += t;
            distinct += t;
        }
        staged = distinct <= D_CAP;
        if (staged) {
#pragma unroll
            for (int i = 0; i < SPT; ++i) {
                const idx_t key = s_tab[tid * SPT + i];
                if (key != kEmptySlot) {
                    s_idmap[tid * SPT + i] = static_cast<uint16_t>(id);
                    s_keys[id] = key;
                    ++id;
                }
            }
        }
        __syncthreads();
        if (staged) {
            for (idx_t k = tid; k < cnt; k += NT) s_slot[k] = s_idmap[s_slot[k]];
        }
    }

    const uint32_t lane = tid % LR;
    const uint32_t group = tid / LR;
    const uint64_t row = r0 + group;
    const bool row_ok = row < m;
    const idx_t k_begin = s_ptr[group] - start;
    const idx_t k_end = s_ptr[group + 1] - start;

    for (uint64_t p0 = 0; p0 < n; p0 += PANEL) {
        const uint64_t c0 = p0 + static_cast<uint64_t>(lane) * V;
        const bool col_ok = c0 < n;
        if (staged) {
            // copy the distinct rows of B for this panel: lane group g takes rows g, g+R, ...
            constexpr int kBatch = 4;
            for (uint32_t d0 = group; d0 < distinct; d0 += R * kBatch) {
                Vec<T, V> tmp[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const uint32_t d = d0 + u * R;
                    if (d < distinct && col_ok) tmp[u] = load_vec<T, V>(B + static_cast<int64_t>(s_keys[d]) * ldb + c0);
                }
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const uint32_t d = d0 + u * R;
                    if (d < distinct && col_ok) store_vec<T, V>(&s_tile[d * PANEL + lane * V], tmp[u]);
                }
            }
            __syncthreads();
        }
        if (row_ok && col_ok) {
            T acc[V];
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i] = T(0);
            if (staged) {
                for (idx_t k = k_begin; k < k_end; ++k) {
                    const uint32_t id = s_slot[k];
                    const T a = s_val[k];
                    const Vec<T, V> b = load_vec<T, V>(&s_tile[id * PANEL + lane * V]);
#pragma unroll
                    for (int i = 0; i < V; ++i) acc[i] += a * b.v[i];
                }
            } else {
                const T* Bc = B + c0;
                for (idx_t j = start + k_begin; j < start + k_end; ++j) {
                    const idx_t c = col[j] - base;
                    const T a = val[j];
                    const Vec<T, V> b = load_vec<T, V>(Bc + static_cast<int64_t>(c) * ldb);
#pragma unroll
                    for (int i = 0; i < V; ++i) acc[i] += a * b.v[i];
                }
            }
            T* Cp = C + static_cast<int64_t>(row) * ldc + c0;
            Vec<T, V> out;
            if constexpr (BETA0) {
#pragma unroll
                for (int i = 0; i < V; ++i) out.v[i] = alpha * acc[i];
            } else {
                const Vec<T, V> old = load_vec<T, V>(Cp);
#pragma unroll
                for (int i = 0; i < V; ++i) out.v[i] = beta * old.v[i] + alpha * acc[i];
            }
            store_vec<T, V>(Cp, out);
        }
        if (staged) __syncthreads();  // the tile is overwritten by the next panel
    }
}

// Row-major op(B) and C, wide C (a panel of 64 columns per wavefront, lane = column).
// A wavefront walks kRowsPerWave consecutive rows of A and keeps the last W rows of B it loaded in
// a private LDS ring.  The ring's tags (column indices) live one per lane in a VGPR, so looking a
// column up is one compare across the wave plus a ballot -- a fully associative cache with FIFO
// replacement, no workgroup barrier and no atomics.  Consecutive rows of stencil-like matrices
// share most of their columns, so about two thirds of the B rows come from LDS instead of L2.
// Per round of up to 32 nonzeros: phase 1 looks every nonzero up and loads its B value through a
// generic pointer that is either the ring slot (hit) or the row of B in global memory (miss), so
// the code is straight-line and all loads of the round are in flight together; phase 2 stores
// the missed rows into the ring and accumulates.
constexpr int kCacheBatch = 32;     // nonzeros looked up per round (= registers holding B values)
constexpr int kRowsPerWave = 32;

template <typename T>
__device__ __forceinline__ T readlane_value(T v, int lane_index) {
    if constexpr (sizeof(T) == 4) {
        return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane_index));
    } else {
        const long long bits = __double_as_longlong(v);
        const int lo = __builtin_amdgcn_readlane(static_cast<int>(bits), lane_index);
        const int hi = __builtin_amdgcn_readlane(static_cast<int>(bits >> 32), lane_index);
        return __longlong_as_double((static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo));
    }
}

template <typename T, int W, bool BETA0>
__global__ __launch_bounds__(kBlock) void spmm_rowb_wcache_kernel(idx_t m, idx_t n, idx_t base,
                                                                  const idx_t* __restrict__ row_ptr,
                                                                  const idx_t* __restrict__ col,
                                                                  const T* __restrict__ val,
                                                                  const T* __restrict__ B, int64_t ldb,
                                                                  T* __restrict__ C, int64_t ldc, T alpha, T beta) {
    static_assert(W >= kCacheBatch && W < kWave, "ring size");
    // W ring rows plus one spare row that absorbs the stores of nonzeros that were hits
    __shared__ T s_ring[kBlock / kWave][(W + 1) * kWave];
    const unsigned lane = threadIdx.x % kWave;
    // readfirstlane tells the compiler what it cannot see: these values are the same in all 64
    // lanes, so the bookkeeping below stays in scalar registers.
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    T* ring = s_ring[wave];
    const uint64_t gwave = static_cast<uint64_t>(blockIdx.x) * (kBlock / kWave) + wave;
    const uint64_t row_begin = gwave * kRowsPerWave;
    if (row_begin >= m) return;  // whole wave leaves together
    const uint64_t row_end = row_begin + kRowsPerWave < m ? row_begin + kRowsPerWave : m;
    const uint64_t ccol = static_cast<uint64_t>(blockIdx.y) * kWave + lane;
    const bool col_ok = ccol < n;
    const T* Bc = B + ccol;

    idx_t tags = 0xFFFFFFFFu;  // lane s holds the column cached in ring slot s
    uint32_t next = 0;         // FIFO insertion point (same in every lane)

    for (uint64_t row = row_begin; row < row_end; ++row) {
        const idx_t start = __builtin_amdgcn_readfirstlane(row_ptr[row]) - base;
        const idx_t end = __builtin_amdgcn_readfirstlane(row_ptr[row + 1]) - base;
        T acc = T(0);
        for (idx_t j0 = start; j0 < end; j0 += kCacheBatch) {
            const uint32_t cnt = end - j0 < kCacheBatch ? end - j0 : kCacheBatch;
            const idx_t my_c = lane < cnt ? col[j0 + lane] - base : 0u;
            const T my_a = lane < cnt ? val[j0 + lane] : T(0);
            T b[kCacheBatch];
            uint32_t store_slot[kCacheBatch];
            uint64_t pending = 0;  // ring slots handed out in this round (their data is not stored yet)
#pragma unroll
            for (int j = 0; j < kCacheBatch; ++j) {
                const bool live = static_cast<uint32_t>(j) < cnt;
                const idx_t c = __builtin_amdgcn_readlane(my_c, j);
                const uint64_t match = __ballot(tags == c);
                const uint32_t hit_slot = match != 0 ? __ffsll(static_cast<long long>(match)) - 1 : 0u;
                // a slot handed out earlier in this round has no data yet (a column repeated in the row)
                const bool usable = match != 0 && ((pending >> hit_slot) & 1ull) == 0;
                const bool insert = live && match == 0;
                const uint32_t slot = next;
                next = insert ? (next + 1 == W ? 0u : next + 1) : next;
                tags = (insert && lane == slot) ? c : tags;
                pending |= insert ? (1ull << slot) : 0ull;
                store_slot[j] = insert ? slot : static_cast<uint32_t>(W);
                const T* from_ring = ring + (usable ? hit_slot : static_cast<uint32_t>(W)) * kWave + lane;
                const T* from_b = Bc + static_cast<int64_t>(c) * ldb;
                // lanes past the last column of C and dead nonzeros read the spare row instead
                const T* src = (live && !usable && col_ok) ? from_b : from_ring;
                b[j] = *src;
            }
#pragma unroll
            for (int j = 0; j < kCacheBatch; ++j) ring[store_slot[j] * kWave + lane] = b[j];
#pragma unroll
            for (int j = 0; j < kCacheBatch; ++j) {
                const T a = readlane_value(my_a, j);  // zero for dead nonzeros
                const T bj = static_cast<uint32_t>(j) < cnt ? b[j] : T(0);
                acc += a * bj;
            }
        }
        if (col_ok) {
            T* Cp = C + static_cast<int64_t>(row) * ldc + ccol;
            if constexpr (BETA0) {
                *Cp = alpha * acc;
            } else {
                *Cp = beta * *Cp + alpha * acc;
            }
        }
    }
}

// op(B) column-major: element (kk, j) at j*ldb + kk.  One wavefront per row of A, lanes strided
// over its nonzeros, JB output columns accumulated at once so the row of A is re-read only
// n/JB times.
template <typename T, int JB, bool BETA0>
__global__ __launch_bounds__(kBlock) void spmm_colb_kernel(idx_t m, idx_t n, idx_t base,
                                                           const idx_t* __restrict__ row_ptr,
                                                           const idx_t* __restrict__ col, const T* __restrict__ val,
                                                           const T* __restrict__ B, int64_t ldb, T* __restrict__ C,
                                                           int64_t c_row_stride, int64_t c_col_stride, T alpha,
                                                           T beta) {
    const unsigned lane = threadIdx.x % kWave;
    const uint64_t row = static_cast<uint64_t>(blockIdx.x) * (kBlock / kWave) + threadIdx.x / kWave;
    const bool live = row < m;  // dead waves still run the reductions with zero work
    const idx_t start = live ? row_ptr[row] - base : 0;
    const idx_t end = live ? row_ptr[row + 1] - base : 0;

    for (idx_t j0 = 0; j0 < n; j0 += JB) {
        T s[JB];
#pragma unroll
        for (int jj = 0; jj < JB; ++jj) s[jj] = T(0);
        for (idx_t e = start + lane; e < end; e += kWave) {
            const idx_t c = col[e] - base;
            const T a = val[e];
#pragma unroll
            for (int jj = 0; jj < JB; ++jj) {
                if (j0 + jj < n) s[jj] += a * B[static_cast<int64_t>(j0 + jj) * ldb + c];
            }
        }
#pragma unroll
        for (int jj = 0; jj < JB; ++jj) s[jj] = group_sum<kWave>(s[jj]);
        if (live && lane == 0) {
#pragma unroll
            for (int jj = 0; jj < JB; ++jj) {
                if (j0 + jj < n) {
                    T* Cp = C + static_cast<int64_t>(row) * c_row_stride + static_cast<int64_t>(j0 + jj) * c_col_stride;
                    if constexpr (BETA0) {
                        *Cp = alpha * s[jj];
                    } else {
                        *Cp = beta * *Cp + alpha * s[jj];
                    }
                }
            }
        }
    }
}

template <typename T, int LR, int V>
void launch_rowb(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    const uint64_t row_blocks = (static_cast<uint64_t>(a.m) + (kBlock / LR) - 1) / (kBlock / LR);
    const uint64_t panels = (static_cast<uint64_t>(a.n) + LR * V - 1) / (LR * V);
    const dim3 grid(static_cast<uint32_t>(row_blocks), static_cast<uint32_t>(panels));
    const T* val = static_cast<const T*>(a.val);
    const T* B = static_cast<const T*>(a.B);
    T* C = static_cast<T*>(a.C);
    const bool beta0 = beta == T(0);
#define MCSP_LAUNCH_ROWB(B0, CR)                                                                                   \
    hipLaunchKernelGGL((spmm_rowb_kernel<T, LR, V, B0, CR>), grid, dim3(kBlock), 0, stream, a.m, a.n, a.base,       \
                       a.row_ptr, a.col, val, B, a.ldb, C, a.ldc, alpha, beta)
    if (beta0 && a.c_row_major) MCSP_LAUNCH_ROWB(true, true);
    else if (beta0) MCSP_LAUNCH_ROWB(true, false);
    else if (a.c_row_major) MCSP_LAUNCH_ROWB(false, true);
    else MCSP_LAUNCH_ROWB(false, false);
#undef MCSP_LAUNCH_ROWB
}

template <typename T, int V>
void launch_rowb_v(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    const uint64_t lanes_needed = (static_cast<uint64_t>(a.n) + V - 1) / V;
    if (lanes_needed <= 1) launch_rowb<T, 1, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 2) launch_rowb<T, 2, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 4) launch_rowb<T, 4, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 8) launch_rowb<T, 8, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 16) launch_rowb<T, 16, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 32) launch_rowb<T, 32, V>(stream, a, alpha, beta);
    else launch_rowb<T, 64, V>(stream, a, alpha, beta);
}


// Shapes of the LDS-staged kernel: lanes per row follow the width of C (up to 16 lanes x 128
// bits = one 256-byte stretch of a row of B); R rows per workgroup keep the workgroup at 256
// threads.  CNT_CAP / D_CAP are sized for ~32 nonzeros per row with about 2.5x column reuse;
// anything beyond falls back inside the kernel.
template <typename T, int LR, int R, int CNT_CAP, int D_CAP, int HASH>
void launch_rowb_lds_shape(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    constexpr int V = 16 / sizeof(T);
    const uint64_t blocks = (static_cast<uint64_t>(a.m) + R - 1) / R;
    const T* val = static_cast<const T*>(a.val);
    const T* B = static_cast<const T*>(a.B);
    T* C = static_cast<T*>(a.C);
    if (beta == T(0)) {
        hipLaunchKernelGGL((spmm_rowb_lds_kernel<T, LR, V, R, CNT_CAP, D_CAP, HASH, true>),
                           dim3(static_cast<uint32_t>(blocks)), dim3(R * LR), 0, stream, a.m, a.n, a.base, a.row_ptr,
                           a.col, val, B, a.ldb, C, a.ldc, alpha, beta);
    } else {
        hipLaunchKernelGGL((spmm_rowb_lds_kernel<T, LR, V, R, CNT_CAP, D_CAP, HASH, false>),
                           dim3(static_cast<uint32_t>(blocks)), dim3(R * LR), 0, stream, a.m, a.n, a.base, a.row_ptr,
                           a.col, val, B, a.ldb, C, a.ldc, alpha, beta);
    }
}

template <typename T>
void launch_rowb_lds(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    constexpr int V = 16 / sizeof(T);
    const uint64_t lanes_needed = (static_cast<uint64_t>(a.n) + V - 1) / V;
    //                                     LR   R   CNT   D   HASH
    if (lanes_needed <= 2) launch_rowb_lds_shape<T, 2, 128, 4608, 1536, 8192>(stream, a, alpha, beta);
    else if (lanes_needed <= 4) launch_rowb_lds_shape<T, 4, 64, 2304, 768, 4096>(stream, a, alpha, beta);
    else if (lanes_needed <= 8) launch_rowb_lds_shape<T, 8, 32, 1152, 384, 2048>(stream, a, alpha, beta);
    else launch_rowb_lds_shape<T, 16, 16, 576, 164, 1024>(stream, a, alpha, beta);
}

template <typename T>
void launch_rowb_wcache(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    constexpr int W = 32;
    const uint64_t waves = (static_cast<uint64_t>(a.m) + kRowsPerWave - 1) / kRowsPerWave;
    const uint64_t blocks = (waves + (kBlock / kWave) - 1) / (kBlock / kWave);
    const uint64_t panels = (static_cast<uint64_t>(a.n) + kWave - 1) / kWave;
    const dim3 grid(static_cast<uint32_t>(blocks), static_cast<uint32_t>(panels));
    const T* val = static_cast<const T*>(a.val);
    const T* B = static_cast<const T*>(a.B);
    T* C = static_cast<T*>(a.C);
    if (beta == T(0)) {
        hipLaunchKernelGGL((spmm_rowb_wcache_kernel<T, W, true>), grid, dim3(kBlock), 0, stream, a.m, a.n, a.base,
                           a.row_ptr, a.col, val, B, a.ldb, C, a.ldc, alpha, beta);
    } else {
        hipLaunchKernelGGL((spmm_rowb_wcache_kernel<T, W, false>), grid, dim3(kBlock), 0, stream, a.m, a.n, a.base,
                           a.row_ptr, a.col, val, B, a.ldb, C, a.ldc, alpha, beta);
    }
}
}  // namespace

template <typename T>
void launch_spmm(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    if (a.m == 0 || a.n == 0) return;
    if (a.b_row_major) {
        constexpr int kWide = 16 / sizeof(T);  // elements per 128-bit access
        const bool aligned = (reinterpret_cast<uintptr_t>(a.B) % 16 == 0) && (a.ldb % kWide == 0) &&
                             (a.n % kWide == 0) &&
                             (!a.c_row_major || ((reinterpret_cast<uintptr_t>(a.C) % 16 == 0) && (a.ldc % kWide == 0)));
        static const bool use_lds = getenv("MCSPARSE_SPMM_LDS") != nullptr;  // experiment switch
        static const bool use_wcache = getenv("MCSPARSE_SPMM_WCACHE") != nullptr;  // experiment switch
        if (a.c_row_major && a.n >= 48 && use_wcache) launch_rowb_wcache<T>(stream, a, alpha, beta);
        else if (aligned && a.c_row_major && use_lds) launch_rowb_lds<T>(stream, a, alpha, beta);
        else if (aligned) launch_rowb_v<T, kWide>(stream, a, alpha, beta);
        else launch_rowb_v<T, 1>(stream, a, alpha, beta);
    } else {
        constexpr int kJB = 4;
        const uint64_t blocks = (static_cast<uint64_t>(a.m) + (kBlock / kWave) - 1) / (kBlock / kWave);
        const int64_t rs = a.c_row_major ? a.ldc : 1;
        const int64_t cs = a.c_row_major ? 1 : a.ldc;
        const T* val = static_cast<const T*>(a.val);
        const T* B = static_cast<const T*>(a.B);
        T* C = static_cast<T*>(a.C);
        if (beta == T(0)) {
            hipLaunchKernelGGL((spmm_colb_kernel<T, kJB, true>), dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0,
                               stream, a.m, a.n, a.base, a.row_ptr, a.col, val, B, a.ldb, C, rs, cs, alpha, beta);
        } else {
            hipLaunchKernelGGL((spmm_colb_kernel<T, kJB, false>), dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0,
                               stream, a.m, a.n, a.base, a.row_ptr, a.col, val, B, a.ldb, C, rs, cs, alpha, beta);
        }
    }
}

template void launch_spmm<float>(hipStream_t, const SpmmArgs&, float, float);
template void launch_spmm<double>(hipStream_t, const SpmmArgs&, double, double);

}  // namespace mcsp
