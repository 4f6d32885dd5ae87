// CSR SpMM for gfx950: C = alpha*A*op(B) + beta*C, A is m x k CSR, op(B) is k x n dense.
//
// The reference (src/kernels/level3/spmm/csr_spmm_device.hpp:91-167) runs one wavefront per
// (row, output column) and therefore re-reads the CSR row n times, after transposing a
// row-major B into a freshly allocated column-major copy (mcsp_spmm_gpu.cpp:119-133).  Here a
// row-major op(B) is read in place: a lane group owns one row of A and each lane a few adjacent
// columns of C, so every nonzero pulls one contiguous stretch of a row of B with wide loads and
// A is read once per column panel.  A column-major op(B) is handled by a gather kernel with the
// lanes spread over the nonzeros of the row.  With beta == 0, C is never read.
#include "spmm_device.h"

namespace mcsp {

namespace {

using namespace spmm_detail;

// op(B) row-major.  LR lanes per row of A, V adjacent columns per lane; blockIdx.y walks the
// column panels of LR*V columns.  V > 1 requires n, ldb (and ldc when C is row-major) to be
// multiples of V and 16-byte aligned base pointers, which the launcher checks.
template <typename T, int LR, int V, bool WIDE>
__global__ __launch_bounds__(kBlock) void spmm_rowb_kernel(idx_t m, idx_t n, idx_t base,
                                                           const idx_t* __restrict__ row_ptr,
                                                           const idx_t* __restrict__ col, const T* __restrict__ val,
                                                           const T* __restrict__ B, int64_t ldb, T* __restrict__ C,
                                                           int64_t ldc, bool c_row_major, T alpha, T beta,
                                                           idx_t long_row) {
    typedef typename ByteOffset<WIDE>::type off_t;
    constexpr int kRowsPerBlock = kBlock / LR;
    const idx_t lane = threadIdx.x % LR;
    const uint64_t row = static_cast<uint64_t>(blockIdx.x) * kRowsPerBlock + threadIdx.x / LR;
    const uint64_t c_own = (static_cast<uint64_t>(blockIdx.y) * LR + lane) * V;
    if (row >= m) return;  // whole lane groups
    // Lanes past the last column still fetch their share of the row's nonzeros for the group;
    // they compute on column 0 and store nothing.
    const bool stores = c_own < n;
    const uint64_t c0 = stores ? c_own : 0;

    const idx_t start = row_ptr[row] - base;
    const idx_t end = row_ptr[row + 1] - base;
    // long_row != 0: rows with more nonzeros are the work of the kernels in spmm_long.hip, C included
    if (long_row != 0 && end - start > long_row) return;  // whole lane groups
    T acc[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = T(0);

    static_assert(LR >= 4, "narrower operands take spmm_narrow_kernel");
    row_times_b<T, LR, V, WIDE>(start, end, lane, base, col, val, reinterpret_cast<const char*>(B),
                                static_cast<off_t>(c0 * sizeof(T)), static_cast<off_t>(ldb * sizeof(T)), acc);

    if (stores) store_c<T, V>(C, ldc, c_row_major, row, c0, acc, alpha, beta);
}

// op(B) row-major with few columns (n <= 2 vectors of V).  A row of op(B) then takes only
// C = 1 or 2 lanes, and what a row of A costs is the chain of dependent loads (offsets,
// nonzeros, rows of op(B)) rather than bytes.  So 16 lanes share a row of A as P = 16 / C
// phases x C column lanes: phase p takes the nonzeros p, p + P, ... of the row, kSteps of them in
// flight at once, and the P partial sums are added up across the lanes at the end.  A lane group
// works through kNarrowRowsPerGroup rows one after the other and asks for the offsets of the row
// after next and the nonzeros of the next row while the rows of op(B) of the current one are on
// their way, so that a row costs one trip to memory instead of three.  Measured on a 27-point
// stencil, n = 8: 1 row per group (no reading ahead) 213 us, 2 rows 183, 3 rows 191, 4 rows 188,
// 8 rows 203, 16 rows 207: more rows per group are fewer lane groups to hide the rest behind.
constexpr int kNarrowRowsPerGroup = 2;
template <typename T, int V, int C>
__global__ __launch_bounds__(kBlock) void spmm_narrow_kernel(idx_t m, idx_t n, idx_t nnz, idx_t base,
                                                             const idx_t* __restrict__ row_ptr,
                                                             const idx_t* __restrict__ col,
                                                             const T* __restrict__ val, const T* __restrict__ B,
                                                             int64_t ldb, T* __restrict__ Cm, int64_t ldc,
                                                             bool c_row_major, T alpha, T beta, idx_t long_row) {
    constexpr int kLanes = 16;
    constexpr int P = kLanes / C;
    constexpr int kSteps = 4;  // measured on a 27-point stencil, n = 8: 1, 2, 4, 8 steps -> 305, 280, 260, 291 us
    constexpr int kGroups = kBlock / kLanes;
    const idx_t sub = threadIdx.x % kLanes;
    const idx_t phase = sub / C;
    const uint64_t c_own = static_cast<uint64_t>(sub % C) * V;
    const bool in_panel = c_own < n;
    const uint64_t c0 = in_panel ? c_own : 0;
    // the groups of a workgroup take neighbouring rows in every round
    const uint64_t first_row = static_cast<uint64_t>(blockIdx.x) * (kGroups * kNarrowRowsPerGroup) + threadIdx.x / kLanes;
    const uint64_t last_row = static_cast<uint64_t>(m) - 1;  // m != 0 here

    if (nnz == 0) {  // nothing to read, only C to scale
        T zero[V];
#pragma unroll
        for (int i = 0; i < V; ++i) zero[i] = T(0);
        for (int it = 0; it < kNarrowRowsPerGroup; ++it) {
            const uint64_t row = first_row + static_cast<uint64_t>(it) * kGroups;
            if (row < m && phase == 0 && in_panel) store_c<T, V>(Cm, ldc, c_row_major, row, c0, zero, alpha, beta);
        }
        return;
    }
    // Loads that sit under a test of their own are waited for one by one; so offsets are read from a
    // row clamped to the last one and nonzeros from an index clamped to the last nonzero, and whether
    // a row or a nonzero is really there is only asked where its product would be added.
    const idx_t last_nonzero = nnz - 1;
    // left: the row is not this kernel's to write (past the end, or longer than long_row != 0: such rows are the
    // work of the kernels in spmm_long.hip, C included)
    auto range_of = [&](uint64_t row, idx_t& at, idx_t& end, bool& left) {
        const uint64_t r = row < last_row ? row : last_row;
        const idx_t b = row_ptr[r] - base;
        const idx_t e = row_ptr[r + 1] - base;
        left = row >= m || (long_row != 0 && e - b > long_row);
        at = b + phase;
        end = left ? b : e;  // and counts as empty
    };
    idx_t at, end, at_next, end_next;
    bool left, left_next;
    range_of(first_row, at, end, left);
    range_of(first_row + kGroups, at_next, end_next, left_next);
    idx_t cc[kSteps];
    T aa[kSteps];
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
        const idx_t j = min(at + u * P, last_nonzero);
        cc[u] = col[j];
        aa[u] = val[j];
    }
    for (int it = 0; it < kNarrowRowsPerGroup; ++it) {
        const uint64_t row = first_row + static_cast<uint64_t>(it) * kGroups;
        if (__all(row >= m)) break;  // the same for all lanes of the wavefront from here on
        T acc[V];
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] = T(0);
        Vec<T, V> b[kSteps];
#pragma unroll
        for (int u = 0; u < kSteps; ++u) b[u] = load_vec<T, V>(B + static_cast<int64_t>(cc[u] - base) * ldb + c0);
        // the next row's nonzeros and the offsets of the row after it, while those are on their way
        idx_t cc_next[kSteps];
        T aa_next[kSteps];
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            const idx_t j = min(at_next + u * P, last_nonzero);
            cc_next[u] = col[j];
            aa_next[u] = val[j];
        }
        idx_t at_after, end_after;
        bool left_after;
        range_of(row + 2 * kGroups, at_after, end_after, left_after);
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            if (at + u * P < end) {  // a lane without a nonzero stays out: 0 * inf would be NaN
#pragma unroll
                for (int i = 0; i < V; ++i) acc[i] += aa[u] * b[u].v[i];
            }
        }
        // a row with more than kSteps * P nonzeros: the rest, kSteps * P at a time
        at += kSteps * P;
        while (__any(at < end)) {
            idx_t c2[kSteps];
            T a2[kSteps];
#pragma unroll
            for (int u = 0; u < kSteps; ++u) {
                const idx_t j = min(at + u * P, last_nonzero);
                c2[u] = col[j];
                a2[u] = val[j];
            }
            Vec<T, V> b2[kSteps];
#pragma unroll
            for (int u = 0; u < kSteps; ++u) b2[u] = load_vec<T, V>(B + static_cast<int64_t>(c2[u] - base) * ldb + c0);
#pragma unroll
            for (int u = 0; u < kSteps; ++u) {
                if (at + u * P < end) {
#pragma unroll
                    for (int i = 0; i < V; ++i) acc[i] += a2[u] * b2[u].v[i];
                }
            }
            at += kSteps * P;
        }
        // sum over the nonzero phases: the lanes of a 16-lane DPP row that serve the same columns
#pragma unroll
        for (int i = 0; i < V; ++i) {
            if constexpr (C == 1) {
                acc[i] = group_sum<kLanes>(acc[i]);
            } else {
                static_assert(C == 2, "column lanes per row");
                constexpr int kQuadXor2 = 0x4E, kRowRor4 = 0x124, kRowRor8 = 0x128;  // lanes 2, 4 and 8 away
                acc[i] += dpp_mov<kQuadXor2>(acc[i]);
                acc[i] += dpp_mov<kRowRor4>(acc[i]);
                acc[i] += dpp_mov<kRowRor8>(acc[i]);
            }
        }
        if (!left && phase == 0 && in_panel) store_c<T, V>(Cm, ldc, c_row_major, row, c0, acc, alpha, beta);
        at = at_next;
        end = end_next;
        left = left_next;
        at_next = at_after;
        end_next = end_after;
        left_next = left_after;
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            cc[u] = cc_next[u];
            aa[u] = aa_next[u];
        }
    }
}

template <typename T, int V, int C>
void launch_narrow(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    constexpr int kRowsPerBlock = kBlock / 16 * kNarrowRowsPerGroup;
    const uint64_t blocks = (static_cast<uint64_t>(a.m) + kRowsPerBlock - 1) / kRowsPerBlock;
    hipLaunchKernelGGL((spmm_narrow_kernel<T, V, C>), dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0, stream, a.m,
                       a.n, a.nnz, a.base, a.row_ptr, a.col, static_cast<const T*>(a.val),
                       static_cast<const T*>(a.B), a.ldb, static_cast<T*>(a.C), a.ldc, a.c_row_major, alpha, beta,
                       a.long_row);
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
                                                           T beta, idx_t long_row) {
    const unsigned lane = threadIdx.x % kWave;
    const uint64_t row = static_cast<uint64_t>(blockIdx.x) * (kBlock / kWave) + threadIdx.x / kWave;
    bool live = row < m;  // dead waves still run the reductions with zero work
    // long_row != 0: rows with more nonzeros are the work of the kernels in spmm_long.hip, C included
    if (live && long_row != 0 && row_ptr[row + 1] - row_ptr[row] > long_row) live = false;
    const idx_t start = live ? row_ptr[row] - base : 0;
    const idx_t end = live ? row_ptr[row + 1] - base : 0;

    for (idx_t j0 = 0; j0 < n; j0 += JB) {
        T s[JB];
#pragma unroll
        for (int jj = 0; jj < JB; ++jj) s[jj] = T(0);
        for (idx_t e = start + lane; e < end; e += kWave) {
            const idx_t c = col[e] - base;
            const T a = val[e];
            // the JB gathers without a test per load (a column past n reads column n - 1 again), so that
            // they are on their way together; the test comes where the product is added
            T b[JB];
#pragma unroll
            for (int jj = 0; jj < JB; ++jj) b[jj] = B[static_cast<int64_t>(min(j0 + jj, n - 1)) * ldb + c];
#pragma unroll
            for (int jj = 0; jj < JB; ++jj) {
                if (j0 + jj < n) s[jj] += a * b[jj];
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

// ---- dense transposes for column-major operands ---------------------------------------------
// dst (cols x rows_padded, row-major, leading dimension ldd) <- transpose of src (rows x cols,
// row-major, leading dimension lds), 64 x 64 elements per workgroup through LDS so that both sides
// move whole cache lines.  Columns [rows, rows_padded) of dst are filled with zeros.  ACCUMULATE:
// dst = beta * dst + transpose(src) (beta == 0 does not read dst) and nothing is padded.
// Stands in for mcspDenseTransposeKernel (src/common/mcsp_dense_transpose_device.hpp:8-38).
constexpr int kTransTile = 64;
template <typename T, bool ACCUMULATE>
__global__ __launch_bounds__(kBlock) void transpose_kernel(uint32_t rows, uint32_t cols, uint32_t rows_padded,
                                                           const T* __restrict__ src, int64_t lds,
                                                           T* __restrict__ dst, int64_t ldd, T beta) {
    __shared__ T tile[kTransTile][kTransTile + 1];
    const uint32_t tx = threadIdx.x % kTransTile;
    const uint32_t ty = threadIdx.x / kTransTile;  // 0..3
    const uint32_t r0 = blockIdx.x * kTransTile;   // along rows of src
    const uint32_t c0 = blockIdx.y * kTransTile;   // along cols of src
    T got[kTransTile / 4];
#pragma unroll
    for (int k = 0; k < kTransTile / 4; ++k) {
        const uint32_t r = r0 + ty + 4 * k;
        const uint32_t c = c0 + tx;
        // clamped position, so that the sixteen loads are on their way together
        const uint32_t rr = r < rows ? r : rows - 1;
        const uint32_t cc = c < cols ? c : cols - 1;
        got[k] = src[static_cast<int64_t>(rr) * lds + cc];
    }
#pragma unroll
    for (int k = 0; k < kTransTile / 4; ++k) {
        const uint32_t r = r0 + ty + 4 * k;
        tile[ty + 4 * k][tx] = r < rows ? got[k] : T(0);
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kTransTile / 4; ++k) {
        const uint32_t c = c0 + ty + 4 * k;  // row of dst
        const uint32_t r = r0 + tx;          // column of dst
        if (c < cols && r < (ACCUMULATE ? rows : rows_padded)) {
            T* out = dst + static_cast<int64_t>(c) * ldd + r;
            const T v = tile[tx][ty + 4 * k];
            if constexpr (ACCUMULATE) {
                *out = beta == T(0) ? v : beta * *out + v;
            } else {
                __builtin_nontemporal_store(v, out);  // a copy larger than the caches, read back from the start
            }
        }
    }
}

// ---- row groups -------------------------------------------------------------------------
// Neighbouring rows of a matrix from a mesh or a stencil share most of their columns.  A lane
// group that owns kSpmmGroupRows consecutive rows walks the merged column list of the group
// (built once per structure by launch_spmm_schedule) and feeds every row of op(B) it loads to
// the accumulators of all rows that have the column, so the bytes pulled through the vector
// memory path -- what bounds this kernel -- shrink by the overlap of the rows.  Values are read
// from the CSR array on every call: entry k of a row is its k-th nonzero in storage order,
// whatever the order is, so unsorted rows only lose sharing, never correctness.
constexpr uint32_t kNoColumn = 0xffffffffu;
constexpr int R = kSpmmGroupRows;

// Offsets of the rows of one group; rows past the end of the matrix are empty.
__device__ __forceinline__ void group_row_ranges(idx_t m, idx_t base, const idx_t* __restrict__ row_ptr, uint64_t r0,
                                                 idx_t (&begin)[R], idx_t (&end)[R]) {
    idx_t next = row_ptr[r0] - base;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        begin[r] = next;
        if (r0 + r < static_cast<uint64_t>(m)) next = row_ptr[r0 + r + 1] - base;
        end[r] = next;
    }
}

// One thread merges the rows of one group.  The column indices of the 64 groups of a wavefront
// are one contiguous stretch of the CSR array, and so are their merged lists; read or written
// thread by thread they would cost a cache line per element, so the wavefront first copies the
// stretch into LDS and collects the lists there before it writes them out (when they fit).
constexpr uint32_t kMergeStage = 8192;  // column indices a wavefront keeps in LDS
constexpr uint32_t kMergeOut = 4096;    // merged entries a wavefront collects in LDS
template <bool FILL>
__global__ __launch_bounds__(kWave) void group_merge_kernel(idx_t m, idx_t base, const idx_t* __restrict__ row_ptr,
                                                            const idx_t* __restrict__ col,
                                                            uint32_t* __restrict__ group_ptr,
                                                            uint32_t* __restrict__ entries,
                                                            unsigned long long* __restrict__ span_sum) {
    __shared__ idx_t s_col[kMergeStage];
    __shared__ uint32_t s_out[FILL ? kMergeOut : 1];
    const uint64_t groups = spmm_groups(m);
    const uint64_t first_group = static_cast<uint64_t>(blockIdx.x) * kWave;
    const uint64_t group = first_group + threadIdx.x;
    const uint64_t first_row = first_group * R < m ? first_group * R : m;
    const uint64_t end_row = (first_group + kWave) * R < m ? (first_group + kWave) * R : m;
    const idx_t stretch_begin = row_ptr[first_row] - base;
    const idx_t stretch_end = row_ptr[end_row] - base;
    const bool staged = stretch_end - stretch_begin <= kMergeStage;
    if (staged) {
        // sixteen loads on their way before the first is parked: the copy is bound by latency otherwise
        constexpr int kAhead = 16;
        const idx_t length = stretch_end - stretch_begin;
        for (idx_t t0 = 0; t0 < length; t0 += kAhead * kWave) {
            idx_t got[kAhead];
#pragma unroll
            for (int a = 0; a < kAhead; ++a) {
                const idx_t t = t0 + a * kWave + threadIdx.x;
                got[a] = t < length ? col[stretch_begin + t] : 0;
            }
#pragma unroll
            for (int a = 0; a < kAhead; ++a) {
                const idx_t t = t0 + a * kWave + threadIdx.x;
                if (t < length) s_col[t] = got[a];
            }
        }
    }
    // FILL: the lists of this wavefront's groups occupy entries[out_begin, out_end)
    uint32_t out_begin = 0, out_end = 0;
    if (FILL) {
        out_begin = group_ptr[first_group < groups ? first_group : groups];
        out_end = group_ptr[first_group + kWave < groups ? first_group + kWave : groups];
    }
    const bool collected = FILL && out_end - out_begin <= kMergeOut;
    __syncthreads();
    // slot `groups` receives the total after the scan; threads past it only take part in the
    // wavefront's sum below
    uint32_t count = 0;
    uint32_t first = kNoColumn, last = 0;
    if (group < groups) {
        idx_t i[R], e[R];
        group_row_ranges(m, base, row_ptr, group * R, i, e);
        if (e[R - 1] - i[0] <= kSpmmMaxMergedGroup) {
            const uint32_t out = FILL ? group_ptr[group] : 0;
            // the head of every row stays in a register and is read again only when the row moves on
            auto merge = [&](auto staged_c, auto collected_c) {
                constexpr bool kStaged = decltype(staged_c)::value;
                constexpr bool kCollected = decltype(collected_c)::value;
                auto head_of = [&](int r) -> uint32_t {
                    if (i[r] >= e[r]) return kNoColumn;
                    return static_cast<uint32_t>((kStaged ? s_col[i[r] - stretch_begin] : col[i[r]]) - base);
                };
                uint32_t head[R];
#pragma unroll
                for (int r = 0; r < R; ++r) head[r] = head_of(r);
                while (true) {
                    uint32_t lo = kNoColumn;
#pragma unroll
                    for (int r = 0; r < R; ++r) lo = head[r] < lo ? head[r] : lo;
                    if (lo == kNoColumn) break;
                    if (first == kNoColumn) first = lo;
                    last = lo > last ? lo : last;
                    uint32_t flags = 0;
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        if (head[r] == lo) {
                            flags |= 1u << r;
                            ++i[r];
                            head[r] = head_of(r);
                        }
                    }
                    if (FILL) {
                        if (kCollected) s_out[out - out_begin + count] = (lo << R) | flags;
                        else entries[out + count] = (lo << R) | flags;
                    }
                    ++count;
                }
            };
            if (staged) {
                if (collected) merge(std::true_type{}, std::true_type{});
                else merge(std::true_type{}, std::false_type{});
            } else {
                merge(std::false_type{}, std::false_type{});
            }
        }
    }
    if (FILL) {
        __syncthreads();
        if (collected && staged) {
            for (uint32_t t = threadIdx.x; t < out_end - out_begin; t += kWave) entries[out_begin + t] = s_out[t];
        }
    }
    if (!FILL) {
        if (group <= groups) group_ptr[group] = count;
        // how far apart the columns of a group lie, summed over the wavefront before it is added
        unsigned long long span = count != 0 ? last - first : 0;
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) span += __shfl_xor(span, off, kWave);
        if (lane_id() == 0 && span != 0) atomicAdd(span_sum, span);
    }
}

__global__ void zero_u64_kernel(unsigned long long* p) { *p = 0; }

// Returns the top bit of w and shifts w left by one: an add whose carry is the answer.
__device__ __forceinline__ bool shift_out_top(uint32_t& w) {
    unsigned doubled;
    const bool top = __builtin_uadd_overflow(w, w, &doubled);
    w = doubled;
    return top;
}

// LR lanes (4..64) per row group, V = 16 B / sizeof(T) adjacent columns per lane; blockIdx.y walks
// panels of LR*V columns.  The lanes of a group fetch LR entries of the merged list at once, one
// each, work out from the flag bits which value of which row belongs to their entry, fetch
// those, and pass row offsets, flags and values round in registers.
// The register allocation of this kernel sits at the edge between six and four wavefronts per SIMD:
// clamping the column of an entry (one instruction) made the compiler's scheduler settle on 118
// registers instead of 79 and the kernel 13 % slower at 64 columns.  The occupancy the narrow groups
// run best at is therefore asked for outright (six; the wider groups measured 6 % slower when held to
// it and keep five).
template <typename T, int LR, bool WIDE>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(LR <= 16 ? 6 : 5))) void spmm_group_kernel(idx_t m, idx_t n, idx_t base,
                                                            const idx_t* __restrict__ row_ptr,
                                                            const idx_t* __restrict__ col, const T* __restrict__ val,
                                                            const uint32_t* __restrict__ group_ptr,
                                                            const uint32_t* __restrict__ entries,
                                                            const T* __restrict__ B, int64_t ldb, T* __restrict__ C,
                                                            int64_t ldc, bool c_row_major, T alpha, T beta,
                                                            uint32_t xcd_chunk, uint32_t xcds, idx_t k, idx_t nnz,
                                                            uint32_t total_entries) {
    typedef typename ByteOffset<WIDE>::type off_t;
    constexpr int V = 16 / sizeof(T);
    constexpr int kGroupsPerBlock = kBlock / LR;
    // rows of op(B) a lane asks for at a time: pairs that alternate with the arithmetic of the pair
    // before (measured best below a wavefront per group), eight at once for one group per wavefront
    constexpr bool kAlternate = LR < kWave;
    constexpr int kBatch = kAlternate ? 2 : 8;
    const idx_t lane = threadIdx.x % LR;
    const uint64_t group = xcd_position(blockIdx.x, xcd_chunk, xcds) * kGroupsPerBlock + threadIdx.x / LR;
    const uint64_t r0 = group * R;
    if (r0 >= static_cast<uint64_t>(m)) return;  // whole lane groups
    const uint64_t c_own = (static_cast<uint64_t>(blockIdx.y) * LR + lane) * V;
    const bool stores = c_own < static_cast<uint64_t>(n);  // lanes past the last column only help fetching
    const uint64_t c0 = stores ? c_own : 0;

    idx_t i[R], e[R];
    group_row_ranges(m, base, row_ptr, r0, i, e);

    T acc[R][V];
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int c = 0; c < V; ++c) acc[r][c] = T(0);
    }
    const char* B_bytes = reinterpret_cast<const char*>(B);
    const off_t lane_off = static_cast<off_t>(c0 * sizeof(T));
    const off_t ldb_bytes = static_cast<off_t>(ldb * sizeof(T));

    if (e[R - 1] - i[0] <= kSpmmMaxMergedGroup) {
        // The schedule lives in the caller's buffer.  Whatever it holds, nothing is read outside the
        // arrays: list bounds are held to the list, columns to the k rows of op(B), value positions to
        // the nonzeros.  (An overwritten schedule gives wrong numbers, never a fault.)
        const uint32_t s_end = min(group_ptr[group + 1], total_entries);
        const uint32_t s_begin = min(group_ptr[group], s_end);
        const idx_t last_value = nnz - 1;  // nnz != 0: the group has nonzeros
        const off_t roff_limit = static_cast<off_t>(k - 1) * ldb_bytes;
        const unsigned group_first = (__lane_id() / LR) * LR;
        const uint64_t group_bits = LR == kWave ? ~0ull : ((1ull << (LR % kWave)) - 1ull);
        const uint64_t below = (1ull << lane) - 1ull;
        // The entries of the next chunk are asked for a chunk ahead (one register; their latency was one of the two
        // dependent ones of a chunk: 495 -> 485 us at 64 columns, no change at 256), without a test of their own:
        // the place is held inside the list, and what lies past the group's end is not used.
        const uint32_t last_entry = total_entries - 1;  // inside the loop s < s_end <= total_entries
        uint32_t ent_next = s_begin < s_end ? entries[min(s_begin + lane, last_entry)] : 0u;
        for (uint32_t s = s_begin; s < s_end; s += LR) {
            const uint32_t ent = s + lane < s_end ? ent_next : 0u;
            ent_next = entries[min(s + LR + lane, last_entry)];
            // this lane's entry is the p-th of the chunk that row r takes part in: the p-th value of
            // the row from where the row stands.  take[r] holds which entries of the chunk row r
            // takes part in, one bit per entry with entry 0 in the top bit: doubling the word moves
            // the next entry's bit into the carry, which is then the lane mask the multiply-adds of
            // that entry run under.
            T v[R];
            uint32_t take[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const bool mine = (ent >> r) & 1u;
                const uint64_t in = (__ballot(mine) >> group_first) & group_bits;
                // loaded whether or not it is wanted (the place is clamped anyway): a select costs less than a branch
                const T loaded = val[min(i[r] + static_cast<idx_t>(__popcll(in & below)), last_value)];
                v[r] = mine ? loaded : T(0);
                i[r] += __popcll(in);
                take[r] = __brev(static_cast<uint32_t>(in));
            }
            const off_t roff = min(static_cast<off_t>(ent >> R) * ldb_bytes, roff_limit);
            const uint32_t flags = ent & ((1u << R) - 1u);
            const uint32_t left = s_end - s;
            // With kAlternate two batches of rows of op(B) take turns: the loads of one are on their
            // way while the multiply-adds of the other run, so a wavefront's arithmetic hides part
            // of its own loads.
            auto chunk = [&](auto checked) {
                constexpr bool kChecked = decltype(checked)::value;
                constexpr int kBatches = LR / kBatch;
                Vec<T, V> b[kAlternate ? 2 : 1][kBatch];
                auto load_batch = [&](auto g) {
                    constexpr int u0 = decltype(g)::value * kBatch;
                    static_for<kBatch>([&](auto u) {
                        constexpr int k = u0 + decltype(u)::value;
                        if (!kChecked || k < left) {
                            const off_t off = group_bcast<LR, k>(roff) + lane_off;
                            b[kAlternate ? decltype(g)::value & 1 : 0][decltype(u)::value] =
                                load_vec<T, V>(reinterpret_cast<const T*>(B_bytes + off));
                        }
                    });
                };
                auto use_batch = [&](auto g) {
                    constexpr int u0 = decltype(g)::value * kBatch;
                    static_for<kBatch>([&](auto u) {
                        constexpr int k = u0 + decltype(u)::value;
                        if (!kChecked || k < left) {
                            // a row that lacks the column must not see it at all (0 * inf would be NaN)
                            uint32_t fk = 0;
                            if constexpr (LR == kWave) fk = group_bcast<LR, k>(flags);  // one group per wavefront: scalar
                            static_for<R>([&](auto rc) {
                                constexpr int r = decltype(rc)::value;
                                bool has;
                                if constexpr (LR == kWave) has = (fk >> r) & 1u;
                                else has = shift_out_top(take[r]);
                                if (has) {
                                    const T a = group_bcast<LR, k>(v[r]);
#pragma unroll
                                    for (int c = 0; c < V; ++c) acc[r][c] += a * b[kAlternate ? decltype(g)::value & 1 : 0][decltype(u)::value].v[c];
                                }
                            });
                        }
                    });
                };
                if constexpr (kAlternate) load_batch(std::integral_constant<int, 0>{});
                static_for<kBatches>([&](auto g) {
                    constexpr int next = decltype(g)::value + 1;
                    if constexpr (!kAlternate) {
                        if (!kChecked || decltype(g)::value * kBatch < left) load_batch(g);
                    } else if constexpr (next < kBatches) {
                        if (!kChecked || next * kBatch < left) load_batch(std::integral_constant<int, next>{});
                    }
                    if (!kChecked || decltype(g)::value * kBatch < left) use_batch(g);
                });
            };
            // A chunk that is at least three quarters full runs the code of a full one: a lane whose
            // entry lies past the end of the list holds 0, reads row 0 of op(B) and adds nothing,
            // which costs less than the tests that would skip it.
            if (left * 4 >= LR * 3) chunk(std::false_type{});
            else chunk(std::true_type{});
        }
    } else {
        // a group too long to be worth merging: one row after the other
#pragma unroll
        for (int r = 0; r < R; ++r)
            row_times_b<T, LR, V, WIDE>(i[r], e[r], lane, base, col, val, B_bytes, lane_off, ldb_bytes, acc[r]);
    }

    if (!stores) return;
    // A column-major C holds the four rows of the group next to each other in every column: 16 or 32
    // bytes per column and lane, which the lane groups of a workgroup (64 consecutive rows) complete to
    // whole lines.
    static_assert(R == 4, "four rows per 128-bit (fp32) or two 128-bit (fp64) accesses");
    const bool whole_columns = !c_row_major && r0 + R <= static_cast<uint64_t>(m) &&
                               ((reinterpret_cast<uintptr_t>(C) | static_cast<uintptr_t>(ldc * sizeof(T))) & 15u) == 0;
    if (whole_columns) {
#pragma unroll
        for (int c = 0; c < V; ++c)
            store_c_four_rows<T>(C + static_cast<int64_t>(c0 + c) * ldc + r0, acc[0][c], acc[1][c], acc[2][c], acc[3][c], alpha,
                                 beta);
        return;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (r0 + r < static_cast<uint64_t>(m)) store_c<T, V>(C, ldc, c_row_major, r0 + r, c0, acc[r], alpha, beta);
    }
}

template <typename T, int LR>
void launch_group(hipStream_t stream, const SpmmArgs& a, const uint32_t* group_ptr, const uint32_t* entries,
                  uint32_t total_entries, T alpha, T beta, uint64_t mean_span) {
    constexpr int V = 16 / sizeof(T);
    const uint64_t groups = spmm_groups(a.m);
    const uint64_t group_blocks = (groups + (kBlock / LR) - 1) / (kBlock / LR);
    const uint64_t panels = (static_cast<uint64_t>(a.n) + LR * V - 1) / (LR * V);
    // Rows whose columns lie `mean_span` apart read rows of op(B) from a window of that many rows
    // around them.  An XCD that works through mean_span / 16 consecutive rows at a time keeps the
    // rows of op(B) it shares with the stretches before and after (the neighbouring grid lines of
    // a stencil) in its own L2 -- as long as such a stretch of op(B) is small against the 4 MB of
    // an L2; beyond that the plain round-robin does as well.
    constexpr uint64_t kRowsPerBlock = static_cast<uint64_t>(kBlock / LR) * R;
    const uint32_t xcds = device_topology().xcds;
    uint32_t xcd_chunk = 1;
    const uint64_t stretch_rows = mean_span / 16;
    if (stretch_rows * a.n * sizeof(T) <= (1u << 20)) {
        while (static_cast<uint64_t>(xcd_chunk) * 2 * kRowsPerBlock <= stretch_rows) xcd_chunk *= 2;
    }
    const dim3 grid(xcd_padded_grid(group_blocks, xcd_chunk, xcds), static_cast<uint32_t>(panels));
    const T* val = static_cast<const T*>(a.val);
    const T* B = static_cast<const T*>(a.B);
    T* C = static_cast<T*>(a.C);
    if (narrow_offsets(a, sizeof(T))) {
        hipLaunchKernelGGL((spmm_group_kernel<T, LR, false>), grid, dim3(kBlock), 0, stream, a.m, a.n, a.base, a.row_ptr,
                           a.col, val, group_ptr, entries, B, a.ldb, C, a.ldc, a.c_row_major, alpha, beta, xcd_chunk, xcds, a.k,
                           a.nnz, total_entries);
    } else {
        hipLaunchKernelGGL((spmm_group_kernel<T, LR, true>), grid, dim3(kBlock), 0, stream, a.m, a.n, a.base, a.row_ptr,
                           a.col, val, group_ptr, entries, B, a.ldb, C, a.ldc, a.c_row_major, alpha, beta, xcd_chunk, xcds, a.k,
                           a.nnz, total_entries);
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
    if (narrow_offsets(a, sizeof(T))) {
        hipLaunchKernelGGL((spmm_rowb_kernel<T, LR, V, false>), grid, dim3(kBlock), 0, stream, a.m, a.n, a.base,
                           a.row_ptr, a.col, val, B, a.ldb, C, a.ldc, a.c_row_major, alpha, beta, a.long_row);
    } else {
        hipLaunchKernelGGL((spmm_rowb_kernel<T, LR, V, true>), grid, dim3(kBlock), 0, stream, a.m, a.n, a.base,
                           a.row_ptr, a.col, val, B, a.ldb, C, a.ldc, a.c_row_major, alpha, beta, a.long_row);
    }
}

template <typename T, int V>
void launch_rowb_v(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    const uint64_t lanes_needed = (static_cast<uint64_t>(a.n) + V - 1) / V;
    if (lanes_needed <= 1) launch_narrow<T, V, 1>(stream, a, alpha, beta);
    else if (lanes_needed <= 2) launch_narrow<T, V, 2>(stream, a, alpha, beta);
    else if (lanes_needed <= 4) launch_rowb<T, 4, V>(stream, a, alpha, beta);  // measured faster than four column lanes above
    else if (lanes_needed <= 8) launch_rowb<T, 8, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 16) launch_rowb<T, 16, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 32) launch_rowb<T, 32, V>(stream, a, alpha, beta);
    else launch_rowb<T, 64, V>(stream, a, alpha, beta);
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
        if (aligned) launch_rowb_v<T, kWide>(stream, a, alpha, beta);
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
                               stream, a.m, a.n, a.base, a.row_ptr, a.col, val, B, a.ldb, C, rs, cs, alpha, beta,
                               a.long_row);
        } else {
            hipLaunchKernelGGL((spmm_colb_kernel<T, kJB, false>), dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0,
                               stream, a.m, a.n, a.base, a.row_ptr, a.col, val, B, a.ldb, C, rs, cs, alpha, beta,
                               a.long_row);
        }
    }
    if (a.long_row != 0) {
        launch_spmm_long_find(stream, a, sizeof(T));
        launch_spmm_long_rows<T>(stream, a, alpha, beta);
    }
}

SpmmScheduleLayout spmm_schedule_layout(idx_t m, idx_t nnz) {
    SpmmScheduleLayout l;
    const uint64_t slots = spmm_groups(m) + 1;
    size_t off = 0;
    l.group_ptr = off; off += align_up(slots * sizeof(uint32_t));
    l.span_sum = off; off += kAlign;
    l.entries = off; off += align_up(static_cast<size_t>(nnz) * sizeof(uint32_t));
    l.scan_ws = off; off += exclusive_scan_workspace_bytes(slots);
    l.total = off;
    return l;
}

void launch_spmm_schedule(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, const idx_t* row_ptr, const idx_t* col,
                          void* schedule) {
    const SpmmScheduleLayout l = spmm_schedule_layout(m, nnz);
    char* w = static_cast<char*>(schedule);
    uint32_t* group_ptr = reinterpret_cast<uint32_t*>(w + l.group_ptr);
    uint32_t* entries = reinterpret_cast<uint32_t*>(w + l.entries);
    const uint64_t slots = spmm_groups(m) + 1;
    const dim3 grid(static_cast<uint32_t>((slots + kWave - 1) / kWave));
    unsigned long long* span_sum = reinterpret_cast<unsigned long long*>(w + l.span_sum);
    // a fill kernel rather than a memset node, so that the sequence can be captured in a HIP graph
    hipLaunchKernelGGL(zero_u64_kernel, dim3(1), dim3(1), 0, stream, span_sum);
    hipLaunchKernelGGL((group_merge_kernel<false>), grid, dim3(kWave), 0, stream, m, base, row_ptr, col, group_ptr,
                       entries, span_sum);
    launch_exclusive_scan_u32(stream, group_ptr, slots, w + l.scan_ws);
    hipLaunchKernelGGL((group_merge_kernel<true>), grid, dim3(kWave), 0, stream, m, base, row_ptr, col, group_ptr,
                       entries, span_sum);
}

bool spmm_schedule_usable(const SpmmArgs& a, size_t value_bytes) {
    const int64_t wide = static_cast<int64_t>(16 / value_bytes);
    // Few 128-bit vectors per row are too few lanes per group to share the fetching.  Against the kernel without a
    // schedule, on a 27-point stencil, rows of three degrees of freedom per node and a 5-point Laplacian: four lanes
    // (16 fp32 columns) half as fast; five and eight lanes (20 and 32 fp32 columns) 8 to 25 % slower or level; nine
    // and more lanes of fp32 6 to 28 % faster; ten to sixteen lanes of fp64 between 9 % slower and 13 % faster, more
    // lanes level or faster (up to 56 %).
    const int64_t lanes_at_least = value_bytes == 4 ? 9 : 17;
    return a.b_row_major && a.n > (lanes_at_least - 1) * wide && a.k <= kSpmmMaxScheduledColumns &&
           reinterpret_cast<uintptr_t>(a.B) % 16 == 0 &&
           a.ldb % wide == 0 && a.n % wide == 0 &&
           (!a.c_row_major || (reinterpret_cast<uintptr_t>(a.C) % 16 == 0 && a.ldc % wide == 0));
}

template <typename T>
void launch_spmm_scheduled(hipStream_t stream, const SpmmArgs& a, const void* schedule, uint32_t total_entries,
                           uint64_t mean_span, T alpha, T beta) {
    if (a.m == 0 || a.n == 0) return;
    constexpr int V = 16 / sizeof(T);
    const SpmmScheduleLayout l = spmm_schedule_layout(a.m, a.nnz);
    const char* w = static_cast<const char*>(schedule);
    const uint32_t* group_ptr = reinterpret_cast<const uint32_t*>(w + l.group_ptr);
    const uint32_t* entries = reinterpret_cast<const uint32_t*>(w + l.entries);
    const uint64_t lanes_needed = (static_cast<uint64_t>(a.n) + V - 1) / V;
    if (lanes_needed <= 4) launch_group<T, 4>(stream, a, group_ptr, entries, total_entries, alpha, beta, mean_span);
    else if (lanes_needed <= 8) launch_group<T, 8>(stream, a, group_ptr, entries, total_entries, alpha, beta, mean_span);
    else if (lanes_needed <= 16) launch_group<T, 16>(stream, a, group_ptr, entries, total_entries, alpha, beta, mean_span);
    else if (lanes_needed <= 32) launch_group<T, 32>(stream, a, group_ptr, entries, total_entries, alpha, beta, mean_span);
    else launch_group<T, 64>(stream, a, group_ptr, entries, total_entries, alpha, beta, mean_span);
}

template <typename T>
void launch_transpose(hipStream_t stream, idx_t rows, idx_t cols, idx_t rows_padded, const T* src, int64_t lds, T* dst,
                      int64_t ldd) {
    if (rows == 0 || cols == 0) return;
    const dim3 grid((rows_padded + kTransTile - 1) / kTransTile, (cols + kTransTile - 1) / kTransTile);
    hipLaunchKernelGGL((transpose_kernel<T, false>), grid, dim3(kBlock), 0, stream, rows, cols, rows_padded, src, lds,
                       dst, ldd, T(0));
}

template <typename T>
void launch_transpose_accumulate(hipStream_t stream, idx_t rows, idx_t cols, const T* src, int64_t lds, T* dst,
                                 int64_t ldd, T beta) {
    if (rows == 0 || cols == 0) return;
    const dim3 grid((rows + kTransTile - 1) / kTransTile, (cols + kTransTile - 1) / kTransTile);
    hipLaunchKernelGGL((transpose_kernel<T, true>), grid, dim3(kBlock), 0, stream, rows, cols, rows, src, lds, dst, ldd,
                       beta);
}

template void launch_transpose<float>(hipStream_t, idx_t, idx_t, idx_t, const float*, int64_t, float*, int64_t);
template void launch_transpose<double>(hipStream_t, idx_t, idx_t, idx_t, const double*, int64_t, double*, int64_t);
template void launch_transpose_accumulate<float>(hipStream_t, idx_t, idx_t, const float*, int64_t, float*, int64_t, float);
template void launch_transpose_accumulate<double>(hipStream_t, idx_t, idx_t, const double*, int64_t, double*, int64_t,
                                                  double);
template void launch_spmm_scheduled<float>(hipStream_t, const SpmmArgs&, const void*, uint32_t, uint64_t, float, float);
template void launch_spmm_scheduled<double>(hipStream_t, const SpmmArgs&, const void*, uint32_t, uint64_t, double, double);
template void launch_spmm<float>(hipStream_t, const SpmmArgs&, float, float);
template void launch_spmm<double>(hipStream_t, const SpmmArgs&, double, double);

}  // namespace mcsp
