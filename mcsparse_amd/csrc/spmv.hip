// CSR SpMV for gfx950: y = alpha*A*x + beta*y.
//
// Two kernel families, picked from the row-length analysis of the structure:
//  * vector : L consecutive lanes of a wavefront own one row (L = 1..64, chosen from the mean
//             row length); U rows per lane group are kept in flight at once so that a wave has
//             enough bytes outstanding to cover HBM latency.  Best for regular matrices.
//  * merge  : the rows' end offsets and the nonzero indices are merged into one path of m+nnz
//             items that is cut into equal tiles, one per workgroup, so a 200k-nonzero row and
//             a million 1-nonzero rows cost the same per item.  Rows that straddle tiles leave a
//             (row, partial sum) carry that a second kernel adds in a fixed order, so results do
//             not depend on scheduling.
// Both families are correct for any CSR structure.  With beta == 0, y is never read.
//
// Stands in for mcspSpmvCsrVectorKernel of the reference
// (src/kernels/level2/spmv/csr_vector_device.hpp:22-79), which runs one wavefront per row.
#include "device_util.h"
#include "internal.h"

namespace mcsp {

namespace {

constexpr int kBlock = 256;

// ------------------------------------------------------------------------------------------
// vector family
// ------------------------------------------------------------------------------------------
// What a kernel does with a finished row sum s.
enum YUpdate : int { kYSet = 0, kYScale = 1 };  // y = alpha*s | y = beta*y + alpha*s

template <typename T, int L, int U, int UPDATE>
__global__ __launch_bounds__(kBlock) void spmv_vector_kernel(idx_t m, idx_t base, const idx_t* __restrict__ row_ptr,
                                                             const idx_t* __restrict__ col,
                                                             const T* __restrict__ val, const T* __restrict__ x,
                                                             T* __restrict__ y, T alpha, T beta) {
    constexpr int kGroups = kBlock / L;  // lane groups (= rows per pass) in a workgroup
    const idx_t lane = threadIdx.x % L;
    const idx_t group = threadIdx.x / L;
    const uint64_t row0 = static_cast<uint64_t>(blockIdx.x) * (kGroups * U) + group;

    // A load that sits under a test of its own, or whose only use does, is waited for on the spot,
    // one latency after the other.  So the loads of the U rows are written without tests (from
    // clamped indices), each kind back to back, and the tests come where the values are used.
    idx_t j[U], e[U];
    T s[U];
    {
        idx_t begin_raw[U], end_raw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t row = row0 + static_cast<uint64_t>(u) * kGroups;
            const uint64_t r = row < m ? row : m - 1;  // m != 0 here
            begin_raw[u] = row_ptr[r];
            end_raw[u] = row_ptr[r + 1];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t row = row0 + static_cast<uint64_t>(u) * kGroups;
            j[u] = row < m ? begin_raw[u] - base + lane : 0;
            e[u] = row < m ? end_raw[u] - base : 0;
            s[u] = T(0);
        }
    }

    // All lanes stay in the loop until every row of the wave is done, so that the loads of the
    // U rows are issued back to back and the DPP reduction below sees 64 active lanes.
    bool more;
    do {
        idx_t c[U];
        T v[U];
        bool act[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            act[u] = j[u] < e[u];
            c[u] = act[u] ? load_stream(col + j[u]) : base;
            v[u] = act[u] ? load_stream(val + j[u]) : T(0);
        }
        T xv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) xv[u] = x[c[u] - base];
        // every gather is asked for before the first one is needed
#pragma unroll
        for (int u = 0; u < U; ++u) asm volatile("" : "+v"(xv[u]));
        more = false;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            // a lane without a nonzero must not touch the sum at all: 0 * x[..] is NaN for an infinite x
            if (act[u]) s[u] += v[u] * xv[u];
            j[u] += L;
            more |= j[u] < e[u];
        }
    } while (__any(more));

#pragma unroll
    for (int u = 0; u < U; ++u) s[u] = group_sum<L>(s[u]);

    if (lane == 0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t row = row0 + static_cast<uint64_t>(u) * kGroups;
            if (row < m) {
                if constexpr (UPDATE == kYSet) {
                    y[row] = alpha * s[u];
                } else {
                    y[row] = beta * y[row] + alpha * s[u];
                }
            }
        }
    }
}

template <typename T, int L, int U>
void launch_vector_lu(hipStream_t stream, const SpmvArgs& a, T alpha, T beta) {
    constexpr int rows_per_block = (kBlock / L) * U;
    const uint64_t blocks = (static_cast<uint64_t>(a.m) + rows_per_block - 1) / rows_per_block;
    const dim3 grid(static_cast<uint32_t>(blocks));
    const T* val = static_cast<const T*>(a.val);
    const T* x = static_cast<const T*>(a.x);
    T* y = static_cast<T*>(a.y);
    if (beta == T(0)) {
        hipLaunchKernelGGL((spmv_vector_kernel<T, L, U, kYSet>), grid, dim3(kBlock), 0, stream, a.m, a.base, a.row_ptr,
                           a.col, val, x, y, alpha, beta);
    } else {
        hipLaunchKernelGGL((spmv_vector_kernel<T, L, U, kYScale>), grid, dim3(kBlock), 0, stream, a.m, a.base,
                           a.row_ptr, a.col, val, x, y, alpha, beta);
    }
}

// ------------------------------------------------------------------------------------------
// merge family
// ------------------------------------------------------------------------------------------
// Path items per thread, IPT, times kBlock threads make a tile, the share of one workgroup.  Tiles that
// run in storage order take 8 items per thread.  Tiles that run in the order of their first column
// take 4: the shorter a tile, the narrower the window of x it reads inside a long row, so rows from
// half the length on keep their gathers within the band in flight (measured on a power-law matrix
// of 4 M rows: 1.09 ms with 8 items, 1.00 ms with 4, 1.01 ms with 2).
constexpr int kItemsInOrder = 8;
constexpr int kItemsByColumn = 4;
static_assert(kBlock * kItemsByColumn == static_cast<int>(kMergeTileItems),
              "the analysis compares row lengths with the size of a tile that runs in column order");

// Path coordinate of diagonal d: how many row ends (x) precede it; nonzeros consumed = d - x.
// A row end is consumed before a nonzero whenever row_end <= nonzero index.
__device__ __forceinline__ idx_t merge_search_global(uint64_t d, idx_t m, idx_t nnz, idx_t base,
                                                     const idx_t* __restrict__ row_ptr) {
    uint64_t lo = d > nnz ? d - nnz : 0;
    uint64_t hi = d < m ? d : m;
    while (lo < hi) {
        const uint64_t mid = (lo + hi) >> 1;
        const uint64_t row_end = row_ptr[mid + 1] - base;
        if (row_end <= d - mid - 1) {
            lo = mid + 1;
        } else {
            hi = mid;
        }
    }
    return static_cast<idx_t>(lo);
}

// Tiles that lie inside long rows read x through a window that moves up with the tile's position in
// the row.  Run in storage order, the tiles in flight at any moment belong to a few rows and their
// windows are scattered over all of x; run in the order of their first column, all of them read
// the same band of x, which then stays in L2 while the band moves once across the vector.  A coarse
// order is enough: tiles are dropped into kOrderBuckets buckets by their first column and the
// buckets run one after the other, in whatever order the tiles arrived inside them.  The result
// does not depend on the order the tiles run in (carries are indexed by tile).
constexpr int kOrderBuckets = kBlock;

__global__ __launch_bounds__(kBlock) void zero_words_kernel(uint32_t* __restrict__ p, uint32_t n) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i < n) p[i] = 0;
}

// tile_row[t] for t in [0, tiles]; with tile_bucket != nullptr also the bucket of every tile and the
// number of tiles per bucket (bucket_count must be zero on entry).
template <int IPT>
__global__ __launch_bounds__(kBlock) void merge_partition_kernel(idx_t m, idx_t nnz, idx_t base,
                                                                 const idx_t* __restrict__ row_ptr, uint32_t tiles,
                                                                 idx_t* __restrict__ tile_row,
                                                                 const idx_t* __restrict__ col, uint32_t key_shift,
                                                                 uint32_t* __restrict__ tile_bucket,
                                                                 uint32_t* __restrict__ bucket_count) {
    constexpr int kTile = kBlock * IPT;
    __shared__ uint32_t s_count[kOrderBuckets];
    const bool ordering = tile_bucket != nullptr;
    if (ordering) {
        s_count[threadIdx.x] = 0;
        __syncthreads();
    }
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    if (t <= tiles) {
        const uint64_t total = static_cast<uint64_t>(m) + nnz;
        uint64_t d = static_cast<uint64_t>(t) * kTile;
        if (d > total) d = total;
        const idx_t x = merge_search_global(d, m, nnz, base, row_ptr);
        tile_row[t] = x;
        if (ordering && t < tiles) {
            const uint64_t first = d - x;  // the tile's first nonzero, if it has one
            const uint32_t key = first < nnz ? col[first] - base : 0u;
            const uint32_t bucket = min(key >> key_shift, static_cast<uint32_t>(kOrderBuckets - 1));
            tile_bucket[t] = bucket;
            atomicAdd(&s_count[bucket], 1u);
        }
    }
    if (ordering) {
        __syncthreads();
        const uint32_t c = s_count[threadIdx.x];
        if (c != 0) atomicAdd(&bucket_count[threadIdx.x], c);
    }
}

// tile_order[position] = tile: bucket after bucket.  Every workgroup scans the bucket sizes for
// itself; bucket_cursor (zero on entry) hands out the slots inside a bucket, one stretch per
// workgroup and bucket: the tiles of a workgroup are first counted per bucket in LDS, so that the
// device-wide cursor of a bucket is moved once by each workgroup instead of once by each tile.
__global__ __launch_bounds__(kBlock) void merge_order_kernel(uint32_t tiles, const uint32_t* __restrict__ tile_bucket,
                                                             const uint32_t* __restrict__ bucket_count,
                                                             uint32_t* __restrict__ bucket_cursor,
                                                             uint32_t* __restrict__ tile_order) {
    __shared__ uint32_t s_start[kOrderBuckets];
    __shared__ uint32_t s_mine[kOrderBuckets];
    __shared__ uint32_t s_wave[kBlock / kWave];
    s_mine[threadIdx.x] = 0;
    const unsigned lane = threadIdx.x % kWave;
    const unsigned wave = threadIdx.x / kWave;
    const uint32_t size = bucket_count[threadIdx.x];
    uint32_t inc = size;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const uint32_t up = __shfl_up(inc, off, kWave);
        if (lane >= static_cast<unsigned>(off)) inc += up;
    }
    if (lane == kWave - 1) s_wave[wave] = inc;
    __syncthreads();
    uint32_t before = 0;
    for (unsigned w = 0; w < wave; ++w) before += s_wave[w];
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    const uint32_t bucket = t < tiles ? tile_bucket[t] : 0u;
    uint32_t slot = 0;
    if (t < tiles) slot = atomicAdd(&s_mine[bucket], 1u);
    __syncthreads();
    const uint32_t mine = s_mine[threadIdx.x];
    s_start[threadIdx.x] = before + inc - size + (mine != 0 ? atomicAdd(&bucket_cursor[threadIdx.x], mine) : 0u);
    __syncthreads();
    if (t < tiles) tile_order[s_start[bucket] + slot] = t;
}

// PRODUCTS: val holds value * x already (col and x are not read); the kernel only sums the rows.
template <typename T, bool BETA0, int IPT, bool PRODUCTS>
__global__ __launch_bounds__(kBlock) void spmv_merge_kernel(idx_t m, idx_t nnz, idx_t base,
                                                            const idx_t* __restrict__ row_ptr,
                                                            const idx_t* __restrict__ col, const T* __restrict__ val,
                                                            const T* __restrict__ x, T* __restrict__ y, T alpha,
                                                            T beta, const idx_t* __restrict__ tile_row,
                                                            idx_t* __restrict__ carry_row, T* __restrict__ carry_val,
                                                            const uint32_t* __restrict__ tile_order) {
    constexpr int kItemsPerThread = IPT;
    constexpr int kTile = kBlock * IPT;
    // s_row_end[i] = end offset of row x0+i; one extra slot closes the tile.
    __shared__ idx_t s_row_end[kTile + 1];
    // [0, tile_nnz) holds the products, [tile_nnz, tile_nnz + tile_rows) the finished row sums.
    __shared__ T s_data[kTile];
    __shared__ idx_t s_wave_key[kBlock / kWave];
    __shared__ T s_wave_val[kBlock / kWave];

    const uint32_t tile = tile_order != nullptr ? tile_order[blockIdx.x] : blockIdx.x;
    const uint32_t tid = threadIdx.x;
    const uint64_t total = static_cast<uint64_t>(m) + nnz;
    const uint64_t d0 = static_cast<uint64_t>(tile) * kTile;
    const uint64_t d1 = d0 + kTile < total ? d0 + kTile : total;
    const idx_t x0 = tile_row[tile];
    const idx_t x1 = tile_row[tile + 1];
    const idx_t y0 = static_cast<idx_t>(d0 - x0);
    const idx_t y1 = static_cast<idx_t>(d1 - x1);
    const idx_t tile_rows = x1 - x0;
    const idx_t tile_nnz = y1 - y0;
    const idx_t tile_items = tile_rows + tile_nnz;

    // A load that sits under a test of its own is waited for on the spot.  The loads of a thread's
    // items are therefore written without tests, from clamped indices, each kind back to back: the
    // row ends, the nonzeros, then the gathers from x; the tests come where the values are stored.
    idx_t ends[kItemsPerThread + 1];
#pragma unroll
    for (int i = 0; i <= kItemsPerThread; ++i) {
        // rows past the tile's last one are not needed: they all read that one's end again
        const idx_t r = min(x0 + tid + static_cast<idx_t>(i) * kBlock, min(x1, m - 1));  // m != 0 here
        ends[i] = row_ptr[r + 1];
    }
    const idx_t last_item = tile_nnz != 0 ? tile_nnz - 1 : 0;
    const idx_t* tile_col = tile_nnz != 0 && !PRODUCTS ? col + y0 : row_ptr;  // a tile of row ends only reads a valid word
    const T* tile_val = tile_nnz != 0 ? val + y0 : (PRODUCTS ? val : x);
#pragma unroll
    for (int i = 0; i <= kItemsPerThread; ++i) {
        const idx_t k = tid + static_cast<idx_t>(i) * kBlock;
        if (k <= tile_rows) s_row_end[k] = x0 + k < m ? ends[i] - base : 0xFFFFFFFFu;
    }
    constexpr int kGatherBatch = kItemsPerThread;  // items whose loads are in flight together
#pragma unroll
    for (int i0 = 0; i0 < kItemsPerThread; i0 += kGatherBatch) {
        idx_t c[kGatherBatch];
        T v[kGatherBatch], xv[kGatherBatch];
#pragma unroll
        for (int i = 0; i < kGatherBatch; ++i) {
            const idx_t k = min(tid + static_cast<idx_t>(i0 + i) * kBlock, last_item);
            if constexpr (!PRODUCTS) c[i] = load_stream(tile_col + k);
            v[i] = load_stream(tile_val + k);
        }
#pragma unroll
        for (int i = 0; i < kGatherBatch; ++i) {
            const idx_t k = tid + static_cast<idx_t>(i0 + i) * kBlock;
            if constexpr (PRODUCTS) xv[i] = T(1);
            else xv[i] = x[k < tile_nnz ? c[i] - base : 0];
        }
        // every gather of the batch is asked for before the first one is needed
#pragma unroll
        for (int i = 0; i < kGatherBatch; ++i) asm volatile("" : "+v"(xv[i]));
#pragma unroll
        for (int i = 0; i < kGatherBatch; ++i) {
            const idx_t k = tid + static_cast<idx_t>(i0 + i) * kBlock;
            if (k < tile_nnz) s_data[k] = PRODUCTS ? v[i] : v[i] * xv[i];
        }
    }
    __syncthreads();

    // this thread's start on the tile's path
    const idx_t dt = min(static_cast<idx_t>(tid * kItemsPerThread), tile_items);
    idx_t lo = dt > tile_nnz ? dt - tile_nnz : 0;
    idx_t hi = dt < tile_rows ? dt : tile_rows;
    while (lo < hi) {
        const idx_t mid = (lo + hi) >> 1;
        if (s_row_end[mid] <= y0 + (dt - mid - 1)) {
            lo = mid + 1;
        } else {
            hi = mid;
        }
    }
    idx_t row_l = lo;
    idx_t nz = y0 + (dt - lo);
    const idx_t first_row_l = row_l;
    bool emitted = false;
    T first_val = T(0);
    T running = T(0);
    T* s_out = s_data + tile_nnz;
#pragma unroll
    for (int i = 0; i < kItemsPerThread; ++i) {
        if (dt + i < tile_items) {
            if (nz < s_row_end[row_l]) {
                running += s_data[nz - y0];
                ++nz;
            } else {
                if (!emitted) {
                    first_val = running;  // completed below, once the carry-in is known
                    emitted = true;
                } else {
                    s_out[row_l] = running;
                }
                running = T(0);
                ++row_l;
            }
        }
    }

    // Exclusive reduce-by-row scan of (open row, partial sum) over the threads.  Keys never
    // decrease along the path, so "same key: add, else keep the later value" is associative.
    idx_t key = row_l;
    T value = running;
    const unsigned lane = tid % kWave;
    const unsigned wave = tid / kWave;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const idx_t k_up = __shfl_up(key, off, kWave);
        const T v_up = __shfl_up(value, off, kWave);
        if (lane >= static_cast<unsigned>(off) && k_up == key) value += v_up;
    }
    if (lane == kWave - 1) {
        s_wave_key[wave] = key;
        s_wave_val[wave] = value;
    }
    // exclusive within the wave
    idx_t ex_key = __shfl_up(key, 1, kWave);
    T ex_val = __shfl_up(value, 1, kWave);
    bool has_prefix = lane != 0;
    __syncthreads();
    {
        // fold the totals of the earlier waves
        bool w_has = false;
        idx_t w_key = 0;
        T w_val = T(0);
        for (unsigned w = 0; w < wave; ++w) {
            const idx_t k = s_wave_key[w];
            const T v = s_wave_val[w];
            w_val = (w_has && w_key == k) ? w_val + v : v;
            w_key = k;
            w_has = true;
        }
        if (w_has) {
            if (has_prefix) {
                if (w_key == ex_key) ex_val += w_val;
            } else {
                ex_key = w_key;
                ex_val = w_val;
                has_prefix = true;
            }
        }
    }
    const T carry_in = (has_prefix && ex_key == first_row_l) ? ex_val : T(0);
    if (emitted) s_out[first_row_l] = first_val + carry_in;

    if (tid == kBlock - 1) {
        // inclusive total of the whole tile = partial sum of the row left open at its end
        const T tile_total = (has_prefix && ex_key == key) ? ex_val + running : running;
        // `running` only covers this thread; if it emitted, earlier partials do not belong
        const T open_sum = emitted ? running : tile_total;
        carry_row[tile] = x1;
        carry_val[tile] = open_sum;
    }
    __syncthreads();

    for (idx_t i = tid; i < tile_rows; i += kBlock) {
        const idx_t r = x0 + i;
        if constexpr (BETA0) {
            y[r] = alpha * s_out[i];
        } else {
            y[r] = beta * y[r] + alpha * s_out[i];
        }
    }
}

// Adds the carries of rows that straddle tiles.  carry_row is non-decreasing; the first tile of
// each run of equal rows sums the run and updates y once.
template <typename T>
__global__ __launch_bounds__(kBlock) void spmv_merge_fixup_kernel(idx_t m, uint32_t tiles,
                                                                  const idx_t* __restrict__ carry_row,
                                                                  const T* __restrict__ carry_val, T* __restrict__ y,
                                                                  T alpha) {
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    if (t >= tiles) return;
    const idx_t r = carry_row[t];
    if (r >= m) return;
    if (t > 0 && carry_row[t - 1] == r) return;
    // A long row leaves a run of hundreds of carries to one thread.  Read one at a time, each costs a
    // trip to memory before the next is asked for; so they are read eight at a time from clamped
    // positions and added in the same order as before.
    constexpr uint32_t kAhead = 8;
    T sum = carry_val[t];
    bool open = true;
    for (uint32_t u = t + 1; open && u < tiles; u += kAhead) {
        idx_t rows[kAhead];
        T vals[kAhead];
#pragma unroll
        for (uint32_t i = 0; i < kAhead; ++i) {
            const uint32_t at = min(u + i, tiles - 1);
            rows[i] = carry_row[at];
            vals[i] = carry_val[at];
        }
#pragma unroll
        for (uint32_t i = 0; i < kAhead; ++i) {
            open = open && u + i < tiles && rows[i] == r;
            if (open) sum += vals[i];
        }
    }
    if (sum != T(0)) y[r] += alpha * sum;
}

inline uint32_t merge_tiles(idx_t m, idx_t nnz, int items_per_thread) {
    const uint64_t tile = static_cast<uint64_t>(kBlock) * items_per_thread;
    const uint64_t total = static_cast<uint64_t>(m) + nnz;
    return static_cast<uint32_t>((total + tile - 1) / tile);
}

}  // namespace

// Lanes per row for the vector family: the power of two nearest the mean row length from
// above, so that a typical row is read in one pass of its lane group.
int spmv_pick_lanes(idx_t m, idx_t nnz) {
    if (m == 0) return 1;
    const double mean = static_cast<double>(nnz) / static_cast<double>(m);
    int lanes = 1;
    while (lanes < 64 && static_cast<double>(lanes) < mean) lanes <<= 1;
    return lanes;
}

template <typename T>
void launch_spmv_vector(hipStream_t stream, const SpmvArgs& a, T alpha, T beta, int lanes) {
    if (a.m == 0) return;
    switch (lanes) {
        case 1: launch_vector_lu<T, 1, 2>(stream, a, alpha, beta); break;
        case 2: launch_vector_lu<T, 2, 4>(stream, a, alpha, beta); break;
        case 4: launch_vector_lu<T, 4, 4>(stream, a, alpha, beta); break;
        case 8: launch_vector_lu<T, 8, 4>(stream, a, alpha, beta); break;
        case 16: launch_vector_lu<T, 16, 4>(stream, a, alpha, beta); break;
        case 32: launch_vector_lu<T, 32, 4>(stream, a, alpha, beta); break;
        default: launch_vector_lu<T, 64, 4>(stream, a, alpha, beta); break;
    }
}

// Workspace layout: [tile_row: tiles+1 idx][carry_row: tiles idx][carry_val: tiles T]
// [tile_bucket: tiles][tile_order: tiles][bucket sizes, bucket cursors: 2 * kOrderBuckets], each
// sub-array aligned to 128 bytes.
size_t spmv_merge_workspace_bytes(idx_t m, idx_t nnz, size_t value_bytes) {
    const size_t tiles = merge_tiles(m, nnz, kItemsByColumn);  // the shorter tiles: room for either kind
    return align_up((tiles + 1) * sizeof(idx_t)) + align_up(tiles * sizeof(idx_t)) + align_up(tiles * value_bytes) +
           2 * align_up(tiles * sizeof(uint32_t)) + align_up(2 * kOrderBuckets * sizeof(uint32_t));
}

template <typename T, int IPT, bool PRODUCTS = false>
void launch_spmv_merge_tiles(hipStream_t stream, const SpmvArgs& a, T alpha, T beta, void* workspace, bool order_tiles) {
    const uint32_t tiles = merge_tiles(a.m, a.nnz, IPT);
    char* w = static_cast<char*>(workspace);
    idx_t* tile_row = reinterpret_cast<idx_t*>(w);
    w += align_up((static_cast<size_t>(tiles) + 1) * sizeof(idx_t));
    idx_t* carry_row = reinterpret_cast<idx_t*>(w);
    w += align_up(static_cast<size_t>(tiles) * sizeof(idx_t));
    T* carry_val = reinterpret_cast<T*>(w);
    w += align_up(static_cast<size_t>(tiles) * sizeof(T));
    uint32_t* tile_bucket = reinterpret_cast<uint32_t*>(w);
    w += align_up(static_cast<size_t>(tiles) * sizeof(uint32_t));
    uint32_t* tile_order = reinterpret_cast<uint32_t*>(w);
    w += align_up(static_cast<size_t>(tiles) * sizeof(uint32_t));
    uint32_t* bucket_count = reinterpret_cast<uint32_t*>(w);
    uint32_t* bucket_cursor = bucket_count + kOrderBuckets;

    const T* val = static_cast<const T*>(a.val);
    const T* x = static_cast<const T*>(a.x);
    T* y = static_cast<T*>(a.y);

    const dim3 per_tile((tiles + 1 + kBlock - 1) / kBlock);
    if (order_tiles) {
        // columns [0, n) fall into kOrderBuckets buckets of 2^key_shift columns
        uint32_t key_shift = 0;
        while ((static_cast<uint64_t>(kOrderBuckets) << key_shift) < a.n) ++key_shift;
        hipLaunchKernelGGL(zero_words_kernel, dim3(2), dim3(kBlock), 0, stream, bucket_count, 2u * kOrderBuckets);
        hipLaunchKernelGGL(merge_partition_kernel<IPT>, per_tile, dim3(kBlock), 0, stream, a.m, a.nnz, a.base, a.row_ptr, tiles,
                           tile_row, a.col, key_shift, tile_bucket, bucket_count);
        hipLaunchKernelGGL(merge_order_kernel, per_tile, dim3(kBlock), 0, stream, tiles,
                           static_cast<const uint32_t*>(tile_bucket), static_cast<const uint32_t*>(bucket_count),
                           bucket_cursor, tile_order);
    } else {
        hipLaunchKernelGGL(merge_partition_kernel<IPT>, per_tile, dim3(kBlock), 0, stream, a.m, a.nnz, a.base, a.row_ptr, tiles,
                           tile_row, a.col, 0u, static_cast<uint32_t*>(nullptr), static_cast<uint32_t*>(nullptr));
        tile_order = nullptr;
    }
    if (beta == T(0)) {
        hipLaunchKernelGGL((spmv_merge_kernel<T, true, IPT, PRODUCTS>), dim3(tiles), dim3(kBlock), 0, stream, a.m, a.nnz, a.base,
                           a.row_ptr, a.col, val, x, y, alpha, beta, tile_row, carry_row, carry_val,
                           static_cast<const uint32_t*>(tile_order));
    } else {
        hipLaunchKernelGGL((spmv_merge_kernel<T, false, IPT, PRODUCTS>), dim3(tiles), dim3(kBlock), 0, stream, a.m, a.nnz, a.base,
                           a.row_ptr, a.col, val, x, y, alpha, beta, tile_row, carry_row, carry_val,
                           static_cast<const uint32_t*>(tile_order));
    }
    hipLaunchKernelGGL((spmv_merge_fixup_kernel<T>), dim3((tiles + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, a.m,
                       tiles, carry_row, carry_val, y, alpha);
}

template <typename T>
void launch_spmv_merge(hipStream_t stream, const SpmvArgs& a, T alpha, T beta, void* workspace, bool order_tiles) {
    if (a.m == 0) return;
    if (order_tiles) launch_spmv_merge_tiles<T, kItemsByColumn>(stream, a, alpha, beta, workspace, true);
    else launch_spmv_merge_tiles<T, kItemsInOrder>(stream, a, alpha, beta, workspace, false);
}

template <typename T>
void launch_row_sums_merge(hipStream_t stream, const SpmvArgs& a, T alpha, T beta, void* workspace) {
    if (a.m == 0) return;
    launch_spmv_merge_tiles<T, kItemsInOrder, true>(stream, a, alpha, beta, workspace, false);
}

// ---- sums over the columns of bucketed products ----
// One workgroup per bucket of 2^shift neighbouring column keys: the sums of the bucket's columns live in
// LDS as doubles (fp32 products are widened: ds_add_f64 runs at four times the rate of ds_add_f32 on this
// chip), the bucket's (key, product) pairs stream past once, 2 * kBucketIpt of them in flight per thread, and
// every column of the bucket is written at the end, with or without products.
constexpr int kBucketBlock = 1024;
constexpr int kBucketIpt = 16;  // loads of two pairs each (8: 801 us on the power-law transpose, 16: 782 us)
constexpr uint32_t kBucketDigits = 256;  // rows of the sort's counter table: one per value of a digit

template <typename T>
struct PairOf { typedef float type __attribute__((ext_vector_type(2))); };
template <>
struct PairOf<double> { typedef double type __attribute__((ext_vector_type(2))); };

// Which part of which bucket a workgroup takes.  A bucket whose pairs number more than twice `share` (the mean of
// a bucket, rounded up) is dealt to several workgroups, ceil(count / share) of them, so that columns that crowd
// into a few buckets (a matrix sorted by degree) do not leave the work to a few CUs: workgroup b < 256 takes the
// first part of bucket b, the workgroups from 256 on the further parts, bucket by bucket.  The parts of a split
// bucket leave their sums as planes in `planes`, numbered in the same order, for bucket_merge_kernel.
struct BucketPart {
    uint32_t bucket;  // kBucketDigits: none
    uint32_t part, parts;
    uint32_t plane;   // of part 0 of this bucket, when parts > 1
};
__device__ __forceinline__ uint32_t bucket_count(const uint32_t* __restrict__ starts, uint32_t stride, idx_t nnz, uint32_t b,
                                                 idx_t* first) {
    idx_t e0 = starts[static_cast<uint64_t>(b) * stride];
    idx_t e1 = b + 1 < kBucketDigits ? starts[static_cast<uint64_t>(b + 1) * stride] : nnz;
    e0 = e0 < nnz ? e0 : nnz;
    e1 = e1 < nnz ? e1 : nnz;
    e1 = e1 > e0 ? e1 : e0;
    *first = e0;
    return e1 - e0;
}
// every thread of the workgroup must call this (it holds barriers); s_parts: kBucketDigits words of LDS
__device__ __forceinline__ BucketPart bucket_part(uint32_t group, bool merge, const uint32_t* __restrict__ starts,
                                                  uint32_t stride, idx_t nnz, uint32_t share, uint32_t* s_parts,
                                                  uint32_t* s_out) {
    for (uint32_t b = threadIdx.x; b < kBucketDigits; b += blockDim.x) {
        idx_t first;
        const uint32_t count = bucket_count(starts, stride, nnz, b, &first);
        s_parts[b] = count / 2 > share ? (count + share - 1) / share : 1u;  // more than twice the share: split
    }
    __syncthreads();
    if (threadIdx.x < kWave) {  // the first wavefront: four buckets per lane, prefix sums over the lanes
        static_assert(kBucketDigits == 4 * kWave, "four buckets per lane");
        const uint32_t lane = threadIdx.x;
        uint32_t parts[4], extra = 0, planes = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            parts[k] = s_parts[4 * lane + k];
            extra += parts[k] - 1;
            planes += parts[k] > 1 ? parts[k] : 0;
        }
        uint32_t extra_upto = extra, planes_upto = planes;  // inclusive over lanes
#pragma unroll
        for (int d = 1; d < kWave; d *= 2) {
            const uint32_t e = __shfl_up(extra_upto, d, kWave), q = __shfl_up(planes_upto, d, kWave);
            if (lane >= static_cast<uint32_t>(d)) {
                extra_upto += e;
                planes_upto += q;
            }
        }
        uint32_t bucket = kBucketDigits, part = 0;
        if (merge || group < kBucketDigits) {
            bucket = group;
        } else {
            // the further part number `further` lies with the lane whose buckets hold it
            const uint32_t further = group - kBucketDigits;
            const bool here = further >= extra_upto - extra && further < extra_upto;
            const uint64_t owner = __ballot(here);
            if (owner != 0) {
                const int src = __ffsll(static_cast<long long>(owner)) - 1;
                uint32_t left = further - __shfl(extra_upto - extra, src, kWave);
                uint32_t found = kBucketDigits, found_part = 0;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t e = __shfl(parts[k], src, kWave) - 1;
                    if (found == kBucketDigits) {
                        if (left < e) {
                            found = 4 * src + k;
                            found_part = left + 1;
                        } else {
                            left -= e;
                        }
                    }
                }
                bucket = found;
                part = found_part;
            }
        }
        // planes of the split buckets before `bucket`
        uint32_t plane = 0;
        if (bucket < kBucketDigits) {
            const int src = bucket / 4;
            plane = __shfl(planes_upto - planes, src, kWave);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t q = __shfl(parts[k], src, kWave);
                if (static_cast<uint32_t>(k) < bucket % 4) plane += q > 1 ? q : 0;
            }
        }
        if (lane == 0) {
            s_out[0] = bucket;
            s_out[1] = part;
            s_out[2] = plane;
        }
    }
    __syncthreads();
    BucketPart p;
    p.bucket = s_out[0];
    p.part = s_out[1];
    p.plane = s_out[2];
    p.parts = p.bucket < kBucketDigits ? s_parts[p.bucket] : 0;
    return p;
}

template <typename T>
__global__ __launch_bounds__(kBucketBlock) void bucket_sums_kernel(idx_t n, idx_t nnz, uint32_t shift,
                                                                  uint32_t stride, uint32_t buckets, uint32_t share,
                                                                  const uint32_t* __restrict__ starts,
                                                                  const uint16_t* __restrict__ keys,
                                                                  const T* __restrict__ products, T* __restrict__ y,
                                                                  double* __restrict__ planes, T alpha, T beta) {
    typedef typename PairOf<T>::type pair_t;
    extern __shared__ __align__(16) unsigned char s_raw[];
    __shared__ uint32_t s_parts[kBucketDigits];
    __shared__ uint32_t s_mine[3];
    double* s_acc = reinterpret_cast<double*>(s_raw);
    const uint32_t tid = threadIdx.x;
    // a workgroup whose own bucket is in one piece (the common case) need not look at the others
    BucketPart mine = {blockIdx.x, 0, 1, 0};
    bool look = blockIdx.x >= kBucketDigits;
    if (!look) {
        idx_t at;
        look = bucket_count(starts, stride, nnz, blockIdx.x, &at) / 2 > share;  // the same for the whole workgroup
    }
    if (look) mine = bucket_part(blockIdx.x, false, starts, stride, nnz, share, s_parts, s_mine);
    const uint32_t bucket = mine.bucket;
    if (bucket >= buckets) return;  // whole workgroup: no further part left for it, or no such bucket
    const uint32_t width = 1u << shift;
    for (uint32_t r = tid; r < width; r += kBucketBlock) s_acc[r] = 0.0;
    idx_t b0;
    const uint32_t count = bucket_count(starts, stride, nnz, bucket, &b0);
    const idx_t e0 = b0 + static_cast<idx_t>(static_cast<uint64_t>(count) * mine.part / mine.parts);
    const idx_t e1 = b0 + static_cast<idx_t>(static_cast<uint64_t>(count) * (mine.part + 1) / mine.parts);
    __syncthreads();
    // Two neighbouring pairs per load (the vector memory unit takes a load instruction of a wavefront in
    // the same time whatever its width): entries 2q and 2q + 1, of which the first of the part's first
    // load and the second of its last may belong to a neighbour.
    const uint32_t* keys2 = reinterpret_cast<const uint32_t*>(keys);
    const pair_t* products2 = reinterpret_cast<const pair_t*>(products);
    const idx_t q0 = e0 / 2;
    const idx_t q1 = e1 / 2 + (e1 & 1u);  // e1 <= nnz < 2^32: no overflow
    for (idx_t slab = q0; slab < q1; slab += kBucketBlock * kBucketIpt) {
        const uint32_t cnt = q1 - slab < static_cast<idx_t>(kBucketBlock * kBucketIpt) ? q1 - slab
                                                                                       : kBucketBlock * kBucketIpt;
        uint32_t key[kBucketIpt];
        pair_t p[kBucketIpt];
#pragma unroll
        for (int i = 0; i < kBucketIpt; ++i) {
            const uint32_t k = min(static_cast<uint32_t>(i) * kBucketBlock + tid, cnt - 1);
            key[i] = load_stream(keys2 + slab + k);
            p[i] = load_stream(products2 + slab + k);
        }
#pragma unroll
        for (int i = 0; i < kBucketIpt; ++i) {
            const uint32_t k = static_cast<uint32_t>(i) * kBucketBlock + tid;
            const uint64_t e = (static_cast<uint64_t>(slab) + k) * 2;
            // the low bits of a key are its place in the bucket, whatever the key holds
            if (k < cnt && e >= e0 && e < e1) unsafeAtomicAdd(&s_acc[key[i] & (width - 1)], static_cast<double>(p[i].x));
            if (k < cnt && e + 1 >= e0 && e + 1 < e1)
                unsafeAtomicAdd(&s_acc[(key[i] >> 16) & (width - 1)], static_cast<double>(p[i].y));
        }
    }
    __syncthreads();
    if (mine.parts > 1) {  // whole workgroup
        double* out = planes + (static_cast<uint64_t>(mine.plane) + mine.part) * width;
        for (uint32_t r = tid; r < width; r += kBucketBlock) out[r] = s_acc[r];
        return;
    }
    const uint64_t first = static_cast<uint64_t>(bucket) << shift;
    for (uint32_t r = tid; r < width; r += kBucketBlock) {
        const uint64_t c = first + r;
        if (c >= n) continue;  // the last bucket may reach past the last column
        const T s = alpha * static_cast<T>(s_acc[r]);
        y[c] = beta == T(0) ? s : s + beta * y[c];
    }
}

// The columns of the buckets that were dealt to several workgroups: their planes added up.  kBucketMergeParts
// workgroups per bucket, each with its share of the bucket's columns; those of a bucket in one piece have nothing
// to do.
constexpr uint32_t kBucketMergeParts = 16;
template <typename T>
__global__ __launch_bounds__(kBlock) void bucket_merge_kernel(idx_t n, idx_t nnz, uint32_t shift, uint32_t stride,
                                                              uint32_t buckets, uint32_t share,
                                                              const uint32_t* __restrict__ starts,
                                                              const double* __restrict__ planes, T* __restrict__ y,
                                                              T alpha, T beta) {
    __shared__ uint32_t s_parts[kBucketDigits];
    __shared__ uint32_t s_mine[3];
    {
        idx_t at;
        if (bucket_count(starts, stride, nnz, blockIdx.x / kBucketMergeParts, &at) / 2 <= share) return;  // whole workgroup
    }
    const BucketPart mine = bucket_part(blockIdx.x / kBucketMergeParts, true, starts, stride, nnz, share, s_parts, s_mine);
    if (mine.bucket >= buckets || mine.parts < 2) return;  // whole workgroup
    const uint32_t width = 1u << shift;
    const uint32_t slice = (width + kBucketMergeParts - 1) / kBucketMergeParts;
    const uint32_t r0 = (blockIdx.x % kBucketMergeParts) * slice;
    const uint32_t r1 = r0 + slice < width ? r0 + slice : width;
    const uint64_t first = static_cast<uint64_t>(mine.bucket) << shift;
    const double* in = planes + static_cast<uint64_t>(mine.plane) * width;
    for (uint32_t r = r0 + threadIdx.x; r < r1; r += kBlock) {
        const uint64_t c = first + r;
        if (c >= n) continue;
        double sum = 0.0;
        for (uint32_t part = 0; part < mine.parts; ++part) sum += in[static_cast<uint64_t>(part) * width + r];
        const T s = alpha * static_cast<T>(sum);
        y[c] = beta == T(0) ? s : s + beta * y[c];
    }
}

template <typename T>
bool launch_bucket_sums(hipStream_t stream, idx_t n, idx_t nnz, const BucketedProducts& b, const T* products, T* y,
                        T alpha, T beta) {
    if (b.buckets == 0 || b.buckets > kBucketDigits || b.shift > kBucketMaxShift) return false;
    const size_t lds = sizeof(double) << b.shift;
    // A bucket with more than twice `share` pairs is dealt to several workgroups, ceil(count / share) of them.  share
    // is the mean of a bucket, so that at most 256 further workgroups are needed, or more where the spare scratch is
    // short: the split buckets leave fewer than 2 * nnz / share planes (one per `share` pairs, and one more for each
    // of the fewer than nnz / share buckets that are split at all).
    const uint64_t max_planes = b.spare != nullptr ? b.spare_bytes / lds : 0;
    const bool split = max_planes >= 4;
    uint64_t share = (static_cast<uint64_t>(nnz) + kBucketDigits - 1) / kBucketDigits;
    if (split) {
        const uint64_t fits = (2 * static_cast<uint64_t>(nnz) + max_planes - 1) / max_planes + 1;
        share = share > fits ? share : fits;
    } else {
        share = nnz;  // no bucket holds more
    }
    double* planes = static_cast<double*>(b.spare);
    if (!allow_dynamic_lds(reinterpret_cast<const void*>(bucket_sums_kernel<T>), lds)) return false;
    hipLaunchKernelGGL((bucket_sums_kernel<T>), dim3(split ? 2 * kBucketDigits : b.buckets), dim3(kBucketBlock), lds, stream,
                       n, nnz, b.shift, b.stride, b.buckets, static_cast<uint32_t>(share), b.starts, b.keys, products, y,
                       planes, alpha, beta);
    if (split) {
        hipLaunchKernelGGL((bucket_merge_kernel<T>), dim3(kBucketDigits * kBucketMergeParts), dim3(kBlock), 0, stream, n,
                           nnz, b.shift, b.stride, b.buckets, static_cast<uint32_t>(share), b.starts,
                           static_cast<const double*>(planes), y, alpha, beta);
    }
    return launches_taken();
}

template bool launch_bucket_sums<float>(hipStream_t, idx_t, idx_t, const BucketedProducts&, const float*, float*, float,
                                        float);
template bool launch_bucket_sums<double>(hipStream_t, idx_t, idx_t, const BucketedProducts&, const double*, double*,
                                         double, double);
// ---- A^T x for a matrix with few columns ----
// With at most 2^14 columns all of y fits in the LDS of one workgroup, so nothing is sorted: each
// of kSkinnyGroups workgroups takes an equal share of the nonzeros as they lie, adds value * x[row] to
// its own copy of y in LDS (doubles), and writes the copy out as a plane of partial sums; a second
// kernel adds the planes up.  rows[] holds the row (+ base) of every nonzero: the COO row array, or
// what csr2coo makes of the offsets.
constexpr int kSkinnyGroups = 256;  // one per compute unit
constexpr int kSkinnyBlock = 1024;
constexpr int kSkinnyIpt = 8;

template <typename T>
__global__ __launch_bounds__(kSkinnyBlock) void skinny_products_kernel(idx_t m, idx_t n, idx_t nnz, idx_t base,
                                                                      const idx_t* __restrict__ rows,
                                                                      const idx_t* __restrict__ col,
                                                                      const T* __restrict__ val,
                                                                      const T* __restrict__ x,
                                                                      double* __restrict__ planes) {
    extern __shared__ __align__(16) unsigned char s_raw[];
    double* s_acc = reinterpret_cast<double*>(s_raw);
    const uint32_t tid = threadIdx.x;
    for (uint32_t c = tid; c < n; c += kSkinnyBlock) s_acc[c] = 0.0;
    __syncthreads();
    const idx_t e0 = static_cast<idx_t>(static_cast<uint64_t>(nnz) * blockIdx.x / kSkinnyGroups);
    const idx_t e1 = static_cast<idx_t>(static_cast<uint64_t>(nnz) * (blockIdx.x + 1) / kSkinnyGroups);
    for (idx_t slab = e0; slab < e1; slab += kSkinnyBlock * kSkinnyIpt) {
        const uint32_t cnt = e1 - slab < static_cast<idx_t>(kSkinnyBlock * kSkinnyIpt) ? e1 - slab
                                                                                       : kSkinnyBlock * kSkinnyIpt;
        idx_t c[kSkinnyIpt], r[kSkinnyIpt];
        T v[kSkinnyIpt], xr[kSkinnyIpt];
#pragma unroll
        for (int i = 0; i < kSkinnyIpt; ++i) {
            const uint32_t k = min(static_cast<uint32_t>(i) * kSkinnyBlock + tid, cnt - 1);
            c[i] = load_stream(col + slab + k);
            r[i] = load_stream(rows + slab + k);
            v[i] = load_stream(val + slab + k);
        }
#pragma unroll
        for (int i = 0; i < kSkinnyIpt; ++i) {
            const idx_t row = r[i] > base ? r[i] - base : 0;
            xr[i] = x[min(row, m - 1)];
        }
#pragma unroll
        for (int i = 0; i < kSkinnyIpt; ++i) {
            const uint32_t k = static_cast<uint32_t>(i) * kSkinnyBlock + tid;
            const idx_t column = c[i] > base ? c[i] - base : 0;
            if (k < cnt) unsafeAtomicAdd(&s_acc[min(column, n - 1)], static_cast<double>(v[i] * xr[i]));
        }
    }
    __syncthreads();
    double* out = planes + static_cast<uint64_t>(blockIdx.x) * n;
    for (uint32_t c = tid; c < n; c += kSkinnyBlock) out[c] = s_acc[c];
}

template <typename T>
__global__ __launch_bounds__(kBlock) void skinny_reduce_kernel(idx_t n, const double* __restrict__ planes,
                                                               T* __restrict__ y, T alpha, T beta) {
    const uint64_t c = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (c >= n) return;
    double sum = 0.0;
#pragma unroll 8
    for (int g = 0; g < kSkinnyGroups; ++g) sum += planes[static_cast<uint64_t>(g) * n + c];
    const T s = alpha * static_cast<T>(sum);
    y[c] = beta == T(0) ? s : s + beta * y[c];
}

bool skinny_transpose_shape(idx_t n, idx_t nnz) {
    // at most 2^14 columns: a copy of y fits in LDS as doubles; enough columns that the lanes of a wavefront
    // seldom meet on one sum; enough nonzeros that the planes are small beside them (and fit the scratch)
    return n <= (1u << kBucketMaxShift) && n >= 256 &&
           static_cast<uint64_t>(nnz) >= static_cast<uint64_t>(kSkinnyMinNonzerosPerColumn) * n;
}

size_t skinny_transpose_workspace_bytes(idx_t n) {
    return static_cast<size_t>(kSkinnyGroups) * n * sizeof(double);
}

template <typename T>
bool launch_skinny_transpose(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, idx_t base, const idx_t* rows,
                             const idx_t* col, const T* val, const T* x, T* y, T alpha, T beta, void* workspace) {
    if (m == 0 || n == 0 || nnz == 0) return true;
    double* planes = static_cast<double*>(workspace);
    const size_t lds = static_cast<size_t>(n) * sizeof(double);
    if (!allow_dynamic_lds(reinterpret_cast<const void*>(skinny_products_kernel<T>), lds)) return false;
    hipLaunchKernelGGL((skinny_products_kernel<T>), dim3(kSkinnyGroups), dim3(kSkinnyBlock), lds, stream, m, n, nnz, base,
                       rows, col, val, x, planes);
    hipLaunchKernelGGL((skinny_reduce_kernel<T>), dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, n,
                       static_cast<const double*>(planes), y, alpha, beta);
    return launches_taken();
}

template bool launch_skinny_transpose<float>(hipStream_t, idx_t, idx_t, idx_t, idx_t, const idx_t*, const idx_t*,
                                             const float*, const float*, float*, float, float, void*);
template bool launch_skinny_transpose<double>(hipStream_t, idx_t, idx_t, idx_t, idx_t, const idx_t*, const idx_t*,
                                              const double*, const double*, double*, double, double, void*);

template void launch_row_sums_merge<float>(hipStream_t, const SpmvArgs&, float, float, void*);
template void launch_row_sums_merge<double>(hipStream_t, const SpmvArgs&, double, double, void*);
template void launch_spmv_vector<float>(hipStream_t, const SpmvArgs&, float, float, int);
template void launch_spmv_vector<double>(hipStream_t, const SpmvArgs&, double, double, int);
template void launch_spmv_merge<float>(hipStream_t, const SpmvArgs&, float, float, void*, bool);
template void launch_spmv_merge<double>(hipStream_t, const SpmvArgs&, double, double, void*, bool);

}  // namespace mcsp
