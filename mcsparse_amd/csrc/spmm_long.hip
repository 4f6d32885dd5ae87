// Long rows of a CSR SpMM.  The row kernels (spmm.hip) give a row of A to one lane group, which walks its
// nonzeros with a handful of loads in flight: a row of 50,000 nonzeros keeps that one group busy for
// milliseconds after every other row is done (1 M power-law rows, N = 16: 7.3 ms, of which the longest row is 7).
// The reference has the same shape (one wavefront per row and output column,
// src/kernels/level3/spmm/csr_spmm_device.hpp:121-137).  Here rows longer than kSpmmLongRow are left out by the
// row kernels and taken in pieces of kSpmmLongChunk nonzeros, a workgroup each:
//   1. spmm_long_find_kernel lists the pieces (row, piece) and, for rows of several pieces, the rows;
//   2. spmm_long_chunk_kernel forms the sums of a piece, all 256 threads on its nonzeros, and writes the row of C
//      (one piece) or a row of partial sums (several);
//   3. spmm_long_reduce_kernel adds the partial sums of a row in the order of the pieces and writes the row of C.
// Every sum is formed in a fixed order, so results repeat bit for bit; where the pieces and partial sums of a row
// lie in the scratch area depends on the order in which the rows were found, which nothing else depends on.
#include "spmm_device.h"

namespace mcsp {

namespace {

using namespace spmm_detail;

struct LongCounters {
    uint32_t items, rows, slots, pad;
};

__global__ void spmm_long_zero_kernel(LongCounters* c) {
    c->items = 0;
    c->rows = 0;
    c->slots = 0;
    c->pad = 0;
}

// item: {row, piece, pieces of the row, first row of partial sums of the row (unused for one piece)}
//
// The places in the three lists come off three counters, and atomic adds to one address take their turns (3.4 ns
// each: 12,000 long rows among 4 M, found by a thread each, 195 us).  So a workgroup looks at kFindRows rows,
// collects its long ones in LDS with places relative to the workgroup, and takes its share of the lists with one
// add per counter (the same matrix: 36 us).
constexpr uint32_t kFindRows = 8192;   // rows a workgroup looks at
constexpr uint32_t kFindList = 2048;   // long rows it can collect; further ones take their places one by one

__device__ __forceinline__ void write_long_row(uint32_t row, uint32_t pieces, uint32_t first, uint32_t slot, uint32_t at,
                                               uint4* __restrict__ items, uint4* __restrict__ rows, uint32_t cap_items,
                                               uint32_t cap_rows, uint32_t cap_slots) {
    // (the capacities hold for every structure whose offsets add up to nnz; for one that does not, nothing is
    // written out of bounds, and the rows that found no room are missing from the product)
    bool fits = first + pieces <= cap_items && first + pieces >= first;
    if (pieces > 1) {
        fits = fits && slot + pieces <= cap_slots && slot + pieces >= slot && at < cap_rows;
        if (at < cap_rows) rows[at] = fits ? make_uint4(row, slot, pieces, 0u) : make_uint4(row, 0u, 0u, 0u);
    }
    for (uint32_t j = 0; j < pieces && first + j < cap_items; ++j)
        items[first + j] = make_uint4(row, j, fits ? pieces : 0u, slot);
}

__global__ __launch_bounds__(kBlock) void spmm_long_find_kernel(idx_t m, const idx_t* __restrict__ row_ptr,
                                                                LongCounters* __restrict__ c, uint4* __restrict__ items,
                                                                uint4* __restrict__ rows, uint32_t cap_items,
                                                                uint32_t cap_rows, uint32_t cap_slots) {
    __shared__ uint4 s_list[kFindList];      // {row, pieces, first item, first slot}, relative to the workgroup
    __shared__ uint32_t s_list_row[kFindList];  // place in the list of rows of several pieces
    __shared__ uint32_t s_count, s_items, s_slots, s_rows;
    __shared__ uint32_t s_base[3];
    const uint32_t tid = threadIdx.x;
    if (tid == 0) {
        s_count = 0;
        s_items = 0;
        s_slots = 0;
        s_rows = 0;
    }
    __syncthreads();
    const uint64_t row0 = static_cast<uint64_t>(blockIdx.x) * kFindRows;
    constexpr uint32_t kAtOnce = 8;  // rows a thread asks for before it looks at any: one trip to memory for the lot
    static_assert(kFindRows % (kBlock * kAtOnce) == 0, "whole rounds");
    for (uint32_t k0 = tid; k0 < kFindRows; k0 += kBlock * kAtOnce) {
        idx_t lens[kAtOnce];
#pragma unroll
        for (uint32_t u = 0; u < kAtOnce; ++u) {
            const uint64_t row = row0 + k0 + u * kBlock;
            const uint64_t r = row < m ? row : m - 1;  // m != 0 here
            lens[u] = row < m ? row_ptr[r + 1] - row_ptr[r] : 0;
        }
#pragma unroll
        for (uint32_t u = 0; u < kAtOnce; ++u) {
            const uint64_t row = row0 + k0 + u * kBlock;
            const idx_t len = lens[u];
            if (len <= kSpmmLongRow) continue;
            const uint32_t pieces = (len + kSpmmLongChunk - 1) / kSpmmLongChunk;
            const uint32_t at = atomicAdd(&s_count, 1u);
            if (at < kFindList) {
                const uint32_t first = atomicAdd(&s_items, pieces);
                const uint32_t slot = pieces > 1 ? atomicAdd(&s_slots, pieces) : 0u;
                s_list_row[at] = pieces > 1 ? atomicAdd(&s_rows, 1u) : 0u;
                s_list[at] = make_uint4(static_cast<uint32_t>(row), pieces, first, slot);
            } else {  // no room in the workgroup's list: places straight off the counters
                const uint32_t first = atomicAdd(&c->items, pieces);
                const uint32_t slot = pieces > 1 ? atomicAdd(&c->slots, pieces) : 0u;
                const uint32_t place = pieces > 1 ? atomicAdd(&c->rows, 1u) : 0u;
                write_long_row(static_cast<uint32_t>(row), pieces, first, slot, place, items, rows, cap_items, cap_rows,
                               cap_slots);
            }
        }
    }
    __syncthreads();
    const uint32_t listed = min(s_count, kFindList);
    if (listed == 0) return;  // whole workgroup
    if (tid == 0) {
        s_base[0] = atomicAdd(&c->items, s_items);
        s_base[1] = s_slots != 0 ? atomicAdd(&c->slots, s_slots) : 0u;
        s_base[2] = s_rows != 0 ? atomicAdd(&c->rows, s_rows) : 0u;
    }
    __syncthreads();
    for (uint32_t k = tid; k < listed; k += kBlock) {
        const uint4 e = s_list[k];
        write_long_row(e.x, e.y, s_base[0] + e.z, s_base[1] + e.w, s_base[2] + s_list_row[k], items, rows, cap_items,
                       cap_rows, cap_slots);
    }
}

// lanes: lane groups of `lanes` threads (a power of two up to 64) hold the columns of a panel of lanes * V columns
// (blockIdx.y walks the panels); the kBlock / lanes groups take the nonzeros of the piece in turn, kAhead rows of
// op(B) in flight each, and their sums meet in LDS, added in the order of the groups.
// op(B)(kk, j) lies at kk * b_rs + j * b_cs; V > 1 needs b_cs == 1 and 16-byte aligned rows (the launcher checks).
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void spmm_long_chunk_kernel(idx_t n, idx_t base, uint32_t lanes,
                                                                 const idx_t* __restrict__ row_ptr,
                                                                 const idx_t* __restrict__ col, const T* __restrict__ val,
                                                                 const T* __restrict__ B, int64_t b_rs, int64_t b_cs,
                                                                 T* __restrict__ C, int64_t ldc, bool c_row_major,
                                                                 T alpha, T beta, const LongCounters* __restrict__ c,
                                                                 const uint4* __restrict__ items, uint32_t cap_items,
                                                                 T* __restrict__ partials, int64_t ld_partials, idx_t nnz) {
    constexpr int kAhead = 4;
    __shared__ T s_sum[kBlock * V];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid % lanes;
    const uint32_t group = tid / lanes;
    const uint32_t groups = kBlock / lanes;
    const uint64_t c_own = (static_cast<uint64_t>(blockIdx.y) * lanes + lane) * V;
    const bool stores = c_own < n;
    const uint64_t c0 = stores ? c_own : 0;
    const uint32_t count = min(c->items, cap_items);
    const idx_t last_nonzero = nnz - 1;  // nnz != 0 where a row is long
    for (uint32_t it = blockIdx.x; it < count; it += gridDim.x) {
        const uint4 item = items[it];
        const uint32_t row = item.x, piece = item.y, pieces = item.z;
        if (pieces == 0) continue;  // whole workgroup: a row that found no room
        const idx_t row_start = row_ptr[row] - base;
        const idx_t row_end = min(row_ptr[row + 1] - base, nnz);
        const idx_t start = row_start + piece * kSpmmLongChunk;
        const idx_t end = min(start + static_cast<idx_t>(kSpmmLongChunk), row_end);
        T acc[V];
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] = T(0);
        for (idx_t e = start + group; e < end; e += groups * kAhead) {
            idx_t cc[kAhead];
            T aa[kAhead];
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const idx_t j = min(e + u * groups, last_nonzero);
                cc[u] = col[j] - base;
                aa[u] = val[j];
            }
            Vec<T, V> b[kAhead];
#pragma unroll
            for (int u = 0; u < kAhead; ++u)
                b[u] = load_vec<T, V>(B + static_cast<int64_t>(cc[u]) * b_rs + static_cast<int64_t>(c0) * b_cs);
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                if (e + u * groups < end) {  // a lane without a nonzero stays out: 0 * inf would be NaN
#pragma unroll
                    for (int i = 0; i < V; ++i) acc[i] += aa[u] * b[u].v[i];
                }
            }
        }
#pragma unroll
        for (int i = 0; i < V; ++i) s_sum[tid * V + i] = acc[i];
        __syncthreads();
        if (group == 0) {
            T sum[V];
#pragma unroll
            for (int i = 0; i < V; ++i) sum[i] = T(0);
            for (uint32_t g = 0; g < groups; ++g) {
#pragma unroll
                for (int i = 0; i < V; ++i) sum[i] += s_sum[(g * lanes + lane) * V + i];
            }
            if (stores) {
                if (pieces == 1) {
                    store_c<T, V>(C, ldc, c_row_major, row, c0, sum, alpha, beta);
                } else {
                    T* out = partials + static_cast<int64_t>(item.w + piece) * ld_partials + c0;
#pragma unroll
                    for (int i = 0; i < V; ++i) out[i] = sum[i];
                }
            }
        }
        __syncthreads();  // the sums are read before the next piece writes them
    }
}

// One thread per (row of several pieces, V columns): the partial sums of the pieces in their order.
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void spmm_long_reduce_kernel(idx_t n, T* __restrict__ C, int64_t ldc,
                                                                  bool c_row_major, T alpha, T beta,
                                                                  const LongCounters* __restrict__ c,
                                                                  const uint4* __restrict__ rows, uint32_t cap_rows,
                                                                  const T* __restrict__ partials, int64_t ld_partials) {
    const uint64_t per_row = (static_cast<uint64_t>(n) + V - 1) / V;
    const uint64_t work = static_cast<uint64_t>(min(c->rows, cap_rows)) * per_row;
    for (uint64_t w = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; w < work;
         w += static_cast<uint64_t>(gridDim.x) * kBlock) {
        const uint4 entry = rows[w / per_row];
        const uint64_t c0 = (w % per_row) * V;
        if (entry.z == 0) continue;
        T sum[V];
#pragma unroll
        for (int i = 0; i < V; ++i) sum[i] = T(0);
        for (uint32_t j = 0; j < entry.z; ++j) {
            const T* in = partials + static_cast<int64_t>(entry.y + j) * ld_partials + c0;
#pragma unroll
            for (int i = 0; i < V; ++i) sum[i] += in[i];
        }
        store_c<T, V>(C, ldc, c_row_major, entry.x, c0, sum, alpha, beta);
    }
}

struct LongLayout {
    size_t counters, items, rows, partials, total;
    uint32_t cap_items, cap_rows, cap_slots;
    int64_t ld_partials;
};

// A row of several pieces is longer than a piece, so there are at most nnz / piece such rows, with at most
// 2 * nnz / piece pieces (ceil(len / piece) <= 2 * len / piece); rows of one piece number at most nnz / kSpmmLongRow.
LongLayout long_layout(idx_t nnz, int64_t n, size_t value_bytes) {
    LongLayout l;
    const uint64_t per_piece = static_cast<uint64_t>(nnz) / kSpmmLongChunk;
    l.cap_rows = static_cast<uint32_t>(per_piece + 1);
    l.cap_slots = static_cast<uint32_t>(2 * per_piece + 2);
    l.cap_items = static_cast<uint32_t>(static_cast<uint64_t>(nnz) / kSpmmLongRow + 2 * per_piece + 2);
    l.ld_partials = (n + 3) / 4 * 4;
    size_t off = 0;
    // the first kAlign bytes are left to the row-length analysis of the call (34 counters)
    off += 2 * kAlign;
    l.counters = off; off += kAlign;
    l.items = off; off += align_up(static_cast<size_t>(l.cap_items) * sizeof(uint4));
    l.rows = off; off += align_up(static_cast<size_t>(l.cap_rows) * sizeof(uint4));
    l.partials = off; off += align_up(static_cast<size_t>(l.cap_slots) * l.ld_partials * value_bytes);
    l.total = off;
    return l;
}

}  // namespace

size_t spmm_long_rows_bytes(idx_t nnz, int64_t n, size_t value_bytes) { return long_layout(nnz, n, value_bytes).total; }

void launch_spmm_long_find(hipStream_t stream, const SpmmArgs& a, size_t value_bytes) {
    const LongLayout l = long_layout(a.nnz, a.long_n, value_bytes);
    char* w = static_cast<char*>(a.long_ws);
    LongCounters* c = reinterpret_cast<LongCounters*>(w + l.counters);
    hipLaunchKernelGGL(spmm_long_zero_kernel, dim3(1), dim3(1), 0, stream, c);
    hipLaunchKernelGGL(spmm_long_find_kernel, dim3((a.m + kFindRows - 1) / kFindRows), dim3(kBlock), 0, stream, a.m, a.row_ptr,
                       c, reinterpret_cast<uint4*>(w + l.items), reinterpret_cast<uint4*>(w + l.rows), l.cap_items,
                       l.cap_rows, l.cap_slots);
}

template <typename T>
void launch_spmm_long_rows(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    const LongLayout l = long_layout(a.nnz, a.long_n, sizeof(T));
    char* w = static_cast<char*>(a.long_ws);
    const LongCounters* c = reinterpret_cast<const LongCounters*>(w + l.counters);
    const uint4* items = reinterpret_cast<const uint4*>(w + l.items);
    const uint4* rows = reinterpret_cast<const uint4*>(w + l.rows);
    T* partials = reinterpret_cast<T*>(w + l.partials);
    const T* val = static_cast<const T*>(a.val);
    const T* B = static_cast<const T*>(a.B);
    T* C = static_cast<T*>(a.C);
    const int64_t b_rs = a.b_row_major ? a.ldb : 1;
    const int64_t b_cs = a.b_row_major ? 1 : a.ldb;
    constexpr int kWide = 16 / sizeof(T);
    const bool wide = a.b_row_major && (reinterpret_cast<uintptr_t>(a.B) % 16 == 0) && (a.ldb % kWide == 0) &&
                      (a.n % kWide == 0) &&
                      (!a.c_row_major || ((reinterpret_cast<uintptr_t>(a.C) % 16 == 0) && (a.ldc % kWide == 0)));
    const uint32_t v = wide ? kWide : 1;
    const uint64_t lanes_needed = (static_cast<uint64_t>(a.n) + v - 1) / v;
    uint32_t lanes = 1;
    while (lanes < kWave && lanes < lanes_needed) lanes *= 2;
    const uint32_t panels = static_cast<uint32_t>((lanes_needed + lanes - 1) / lanes);
    // pieces are few (a 2048th of the nonzeros at most): a grid that lets every compute unit hold several
    const dim3 grid(2048, panels);
    const uint32_t reduce_blocks = 1024;
    if (wide) {
        hipLaunchKernelGGL((spmm_long_chunk_kernel<T, kWide>), grid, dim3(kBlock), 0, stream, a.n, a.base, lanes,
                           a.row_ptr, a.col, val, B, b_rs, b_cs, C, a.ldc, a.c_row_major, alpha, beta, c, items,
                           l.cap_items, partials, l.ld_partials, a.nnz);
        hipLaunchKernelGGL((spmm_long_reduce_kernel<T, kWide>), dim3(reduce_blocks), dim3(kBlock), 0, stream, a.n, C,
                           a.ldc, a.c_row_major, alpha, beta, c, rows, l.cap_rows, partials, l.ld_partials);
    } else {
        hipLaunchKernelGGL((spmm_long_chunk_kernel<T, 1>), grid, dim3(kBlock), 0, stream, a.n, a.base, lanes, a.row_ptr,
                           a.col, val, B, b_rs, b_cs, C, a.ldc, a.c_row_major, alpha, beta, c, items, l.cap_items,
                           partials, l.ld_partials, a.nnz);
        hipLaunchKernelGGL((spmm_long_reduce_kernel<T, 1>), dim3(reduce_blocks), dim3(kBlock), 0, stream, a.n, C, a.ldc,
                           a.c_row_major, alpha, beta, c, rows, l.cap_rows, partials, l.ld_partials);
    }
}

template void launch_spmm_long_rows<float>(hipStream_t, const SpmmArgs&, float, float);
template void launch_spmm_long_rows<double>(hipStream_t, const SpmmArgs&, double, double);

}  // namespace mcsp
