// Column-banded CSR SpMV for gfx950: y = alpha*A*x + beta*y on a copy of A that is laid out so that
// the gathers from x hit in L2.
//
// A gather x[col] costs one 128-byte line fill from L2 when the line is there and a trip over the
// fabric when it is not; with x larger than an XCD's 4 MB L2 and columns spread over all of it, most
// gathers of the row kernels (spmv.hip) miss.  mcsparseSpMV_preprocess therefore re-lays the matrix
// out once: the columns are cut into bands narrow enough for a band of x to stay in L2, the rows
// into chunks, and the nonzeros are stored tile by tile (band-major, chunk-minor), inside a tile in
// CSR order.  An entry keeps (row inside the chunk, column inside the band) in one 32-bit word, so
// the stream is as long as CSR's.  The SpMV kernel hands every XCD a contiguous stretch of that
// tile list: an XCD works inside one band at a time and only that band of x lives in its L2.  A tile
// leaves one partial sum per row and band; a second kernel adds a row's partial sums in band order.
// No atomics: every sum is formed in a fixed order, so results are bit-reproducible run to run.
//
// A second form of the copy (BandedShape::by_column) trades that reproducibility for fewer requests to
// L2: tiles of up to 16384 rows whose entries are sorted by column, so that the lanes of a wavefront
// gather neighbouring elements of x (several per 128-byte line), and products added to the tile's row
// sums in LDS by ds_add_f64 in the order the wavefronts reach them.  Selected by
// MCSPARSE_SPMV_CSR_ALG1 in mcsparseSpMV_preprocess.
//
// Stands in, like spmv.hip, for the gather loop of the reference's row kernel
// (src/kernels/level2/spmv/csr_vector_device.hpp:40-57).
#include "device_util.h"
#include "internal.h"

namespace mcsp {

namespace {

constexpr int kBlock = 256;
// Entries per thread and slab.  Measured with 4, 8, 12 and 16 per thread: fp64 1M x 16 uniform 140, 118,
// 117, 114 us; the transposed power-law matrix (fp32, 28 per row) 557, 582, 498, 486 us.  512 threads with
// 8 or 16 entries each: 116 / 179 us and 518 / 614 us.
constexpr int kIpt = 16;
constexpr int kSlab = kBlock * kIpt;  // entries a workgroup stages at a time
constexpr int kRowsPerThread = kBandedMaxRowsPerTile / kBlock;
// The list of tiles (units) of a copy is cut into this many stretches, and workgroup i works on stretch i % 8: the
// eight XCDs of a whole MI355X, which take the workgroups of a launch in turn, so that one L2 holds one stretch's
// band of x.  It is part of the copy's layout, not read from the device: on a device with fewer XCDs (a partition)
// several stretches share an L2, which costs hit rate and nothing else.
constexpr uint32_t kXcds = 8;
constexpr uint32_t kColumnGroupsPerXcd = 32;  // workgroups per stretch of the kernel on tiles in column order (one per CU of an XCD)
static_assert(kBandedMaxRowsPerTile % kBlock == 0, "rows of a tile are dealt to the threads in rounds");
static_assert(kSlab <= 65536 && kBandedMaxRowsPerTile <= 65536, "16-bit positions in LDS");

// ------------------------------------------------------------------------------------------
// build
// ------------------------------------------------------------------------------------------
// Entry k of the band-sorted nonzeros becomes (row inside its chunk << band_shift) | (key inside the
// band); key = column index with the index base left in.  Tile of an entry = band * chunks + chunk;
// the entries are sorted by tile, and boundary k (between entries k-1 and k, 0 <= k <= nnz) writes
// the offsets of the tiles that begin there, so empty tiles are covered.
__global__ __launch_bounds__(kBlock) void banded_pack_kernel(idx_t nnz, idx_t base, uint32_t band_shift,
                                                             uint32_t rows_per_tile, uint32_t chunks, uint32_t tiles,
                                                             const idx_t* __restrict__ keys,
                                                             const idx_t* __restrict__ rows,
                                                             idx_t* __restrict__ entries,
                                                             idx_t* __restrict__ tile_ptr) {
    const uint64_t k = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (k > nnz) return;
    const idx_t band_mask = (1u << band_shift) - 1u;
    uint32_t tile = tiles;  // boundary nnz closes every remaining tile
    if (k < nnz) {
        const idx_t key = keys[k];
        const idx_t row = rows[k] - base;
        const uint32_t chunk = row / rows_per_tile;
        tile = (key >> band_shift) * chunks + chunk;
        entries[k] = ((row - chunk * rows_per_tile) << band_shift) | (key & band_mask);
    }
    uint32_t first = 0;  // first tile whose offset this boundary writes
    if (k != 0) {
        const uint32_t prev_chunk = (rows[k - 1] - base) / rows_per_tile;
        first = (keys[k - 1] >> band_shift) * chunks + prev_chunk + 1;
    }
    for (uint32_t t = first; t <= tile && t <= tiles; ++t) tile_ptr[t] = static_cast<idx_t>(k);
}

// xcd_start[i], i = 0..8: first tile of XCD i's stretch of the tile list, cut so that the stretches
// hold about the same number of nonzeros.
__global__ void banded_split_kernel(idx_t nnz, uint32_t tiles, const idx_t* __restrict__ tile_ptr,
                                    uint32_t* __restrict__ xcd_start) {
    const uint32_t i = threadIdx.x;
    if (i > kXcds) return;
    const uint64_t target = static_cast<uint64_t>(nnz) * i / kXcds;
    uint32_t lo = 0, hi = tiles;  // first tile whose offset is >= target
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (tile_ptr[mid] < target) lo = mid + 1; else hi = mid;
    }
    xcd_start[i] = i == 0 ? 0u : (i == kXcds ? tiles : lo);
}

// ------------------------------------------------------------------------------------------
// SpMV
// ------------------------------------------------------------------------------------------
// One tile per workgroup.  The tile's entries are staged a slab at a time: coalesced loads of the
// packed entries and values, the gathers from the band of x, products and row numbers to LDS; the
// ends of every row's run are found where neighbouring entries differ; then thread r adds up the run
// of row r (and r + 256, ...) in storage order into the row's accumulator in LDS.  A run longer than
// kLongRun entries (a long row of a power-law matrix puts thousands into one band) is left to a whole
// wavefront: lane l adds the entries l, l + 64, ... in order and the lane sums are added in a fixed
// tree, so the result does not depend on which wavefront picks the run up.
// Every index that comes out of the layout is clamped, so a layout the caller has overwritten gives
// wrong numbers but never an access outside the arrays.
constexpr uint32_t kLongRun = 48;
template <typename T>
__global__ __launch_bounds__(kBlock) void spmv_banded_kernel(idx_t m, idx_t n, idx_t nnz, idx_t base, uint32_t band_shift,
                                                             uint32_t rows_per_tile, uint32_t chunks, uint32_t tiles,
                                                             const uint32_t* __restrict__ xcd_start,
                                                             const idx_t* __restrict__ tile_ptr,
                                                             const idx_t* __restrict__ entries,
                                                             const T* __restrict__ vals, const T* __restrict__ x,
                                                             T* __restrict__ partials) {
    __shared__ T s_prod[kSlab];
    __shared__ T s_acc[kBandedMaxRowsPerTile];
    __shared__ uint16_t s_row[kSlab];
    __shared__ uint16_t s_beg[kBandedMaxRowsPerTile];
    __shared__ uint16_t s_end[kBandedMaxRowsPerTile];
    __shared__ uint16_t s_long[kSlab / kLongRun + 1];  // rows whose run in this slab is long
    __shared__ uint32_t s_long_count;

    const uint32_t tid = threadIdx.x;
    const uint32_t xcd = blockIdx.x % kXcds;
    const uint32_t tile = xcd_start[xcd] + blockIdx.x / kXcds;
    if (tile >= xcd_start[xcd + 1] || tile >= tiles) return;  // whole workgroup
    const uint32_t band = tile / chunks;
    const uint32_t chunk = tile - band * chunks;
    const uint64_t row0 = static_cast<uint64_t>(chunk) * rows_per_tile;
    if (row0 >= m) return;
    const uint32_t tile_rows = static_cast<uint32_t>(m - row0 < rows_per_tile ? m - row0 : rows_per_tile);
    idx_t e0 = tile_ptr[tile];
    idx_t e1 = tile_ptr[tile + 1];
    e0 = e0 < nnz ? e0 : nnz;
    e1 = e1 < nnz ? e1 : nnz;
    e1 = e1 > e0 ? e1 : e0;
    const idx_t band_mask = (1u << band_shift) - 1u;
    const idx_t band_key = band << band_shift;

#pragma unroll
    for (int q = 0; q < kRowsPerThread; ++q) {
        s_beg[q * kBlock + tid] = 0;
        s_end[q * kBlock + tid] = 0;
        s_acc[q * kBlock + tid] = T(0);
    }
    if (tid == 0) s_long_count = 0;

    for (idx_t slab = e0; slab < e1; slab += kSlab) {
        const uint32_t cnt = e1 - slab < static_cast<idx_t>(kSlab) ? e1 - slab : kSlab;
        // Loads without tests of their own (clamped positions), each kind back to back, so that all of
        // a thread's loads are on their way before the first is waited for.
        idx_t packed[kIpt];
        T v[kIpt], xv[kIpt];
#pragma unroll
        for (int i = 0; i < kIpt; ++i) {
            const uint32_t k = min(static_cast<uint32_t>(i) * kBlock + tid, cnt - 1);
            packed[i] = load_stream(entries + slab + k);
            v[i] = load_stream(vals + slab + k);
        }
#pragma unroll
        for (int i = 0; i < kIpt; ++i) {
            idx_t key = band_key | (packed[i] & band_mask);  // column + base
            key = key > base ? key : base;
            const idx_t c = min(key - base, n - 1);
            xv[i] = x[c];
        }
#pragma unroll
        for (int i = 0; i < kIpt; ++i) asm volatile("" : "+v"(xv[i]));
#pragma unroll
        for (int i = 0; i < kIpt; ++i) {
            const uint32_t k = static_cast<uint32_t>(i) * kBlock + tid;
            if (k < cnt) {
                s_prod[k] = v[i] * xv[i];
                s_row[k] = static_cast<uint16_t>(packed[i] >> band_shift);
            }
        }
        __syncthreads();
        // the run of row r is [s_beg[r], s_end[r]): entries of a tile are sorted by row
#pragma unroll
        for (int i = 0; i < kIpt; ++i) {
            const uint32_t k = static_cast<uint32_t>(i) * kBlock + tid;
            if (k < cnt) {
                const uint32_t r = s_row[k];
                if (r < tile_rows) {
                    if (k == 0 || s_row[k - 1] != r) s_beg[r] = static_cast<uint16_t>(k);
                    if (k + 1 == cnt || s_row[k + 1] != r) s_end[r] = static_cast<uint16_t>(k + 1);
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < kRowsPerThread; ++q) {
            const uint32_t r = q * kBlock + tid;
            if (r < tile_rows) {
                uint32_t end = s_end[r];
                uint32_t j = s_beg[r];
                end = end < cnt ? end : cnt;
                if (end > j + kLongRun) {
                    // at most cnt / kLongRun such runs fit a slab, so the list cannot overflow; its
                    // order does not matter, every run is summed on its own
                    s_long[atomicAdd(&s_long_count, 1u) % (kSlab / kLongRun + 1)] = static_cast<uint16_t>(r);
                } else {
                    T sum = T(0);
                    for (; j < end; ++j) sum += s_prod[j];
                    s_acc[r] += sum;
                    s_beg[r] = 0;
                    s_end[r] = 0;
                }
            }
        }
        __syncthreads();
        const uint32_t long_runs = min(s_long_count, static_cast<uint32_t>(kSlab / kLongRun + 1));
        if (long_runs != 0) {  // the same for the whole workgroup
            const uint32_t lane = tid % kWave;
            for (uint32_t w = tid / kWave; w < long_runs; w += kBlock / kWave) {
                const uint32_t r = min(static_cast<uint32_t>(s_long[w]), tile_rows - 1);
                uint32_t end = s_end[r];
                const uint32_t beg = min(static_cast<uint32_t>(s_beg[r]), cnt);
                end = end < cnt ? end : cnt;
                T sum = T(0);
                for (uint32_t j = beg + lane; j < end; j += kWave) sum += s_prod[j];
                sum = group_sum<kWave>(sum);
                if (lane == 0) {
                    s_acc[r] += sum;
                    s_beg[r] = 0;
                    s_end[r] = 0;
                }
            }
            __syncthreads();
            if (tid == 0) s_long_count = 0;
        }
        // the next slab's products may only be written once every run of this one has been read: the
        // barrier after the row sums (or the one after the long runs) stands between the two
    }
    __syncthreads();

    T* out = partials + static_cast<uint64_t>(band) * m + row0;
#pragma unroll
    for (int q = 0; q < kRowsPerThread; ++q) {
        const uint32_t r = q * kBlock + tid;
        if (r < tile_rows) out[r] = s_acc[r];
    }
}

// y[r] = beta*y[r] + alpha * (partials[0][r] + partials[1][r] + ...), the bands in order.
// next_unit (may be null): the work counters of spmv_column_order_kernel, put back to their start for the next call.
template <typename T, bool BETA0>
__global__ __launch_bounds__(kBlock) void banded_reduce_kernel(idx_t m, uint32_t bands, const T* __restrict__ partials,
                                                               T* __restrict__ y, T alpha, T beta,
                                                               uint32_t* __restrict__ next_unit) {
    if (next_unit != nullptr && blockIdx.x == 0 && threadIdx.x < kXcds) next_unit[threadIdx.x] = kColumnGroupsPerXcd;
    const uint64_t r = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (r >= m) return;
    constexpr uint32_t kAhead = 8;
    T sum = T(0);
    for (uint32_t b0 = 0; b0 < bands; b0 += kAhead) {
        T p[kAhead];
#pragma unroll
        for (uint32_t i = 0; i < kAhead; ++i) {
            const uint32_t b = min(b0 + i, bands - 1);
            p[i] = load_stream(partials + static_cast<uint64_t>(b) * m + r);
        }
#pragma unroll
        for (uint32_t i = 0; i < kAhead; ++i) {
            if (b0 + i < bands) sum = (b0 + i == 0) ? p[i] : sum + p[i];
        }
    }
    if constexpr (BETA0) {
        y[r] = alpha * sum;
    } else {
        y[r] = beta * y[r] + alpha * sum;
    }
}

// The same with 16 bytes per access: V = 16 / sizeof(T) neighbouring rows per thread.  m is a multiple of V and
// partials and y are 16-byte aligned (the launch checks).
template <typename T, bool BETA0>
__global__ __launch_bounds__(kBlock) void banded_reduce_wide_kernel(idx_t m, uint32_t bands, const T* __restrict__ partials,
                                                                    T* __restrict__ y, T alpha, T beta,
                                                                    uint32_t* __restrict__ next_unit) {
    constexpr int V = 16 / sizeof(T);
    typedef T vec_t __attribute__((ext_vector_type(V)));
    if (next_unit != nullptr && blockIdx.x == 0 && threadIdx.x < kXcds) next_unit[threadIdx.x] = kColumnGroupsPerXcd;
    const uint64_t r = (static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x) * V;
    if (r >= m) return;
    constexpr uint32_t kAhead = 8;
    vec_t sum = vec_t(0);
    for (uint32_t b0 = 0; b0 < bands; b0 += kAhead) {
        vec_t p[kAhead];
#pragma unroll
        for (uint32_t i = 0; i < kAhead; ++i) {
            const uint32_t b = min(b0 + i, bands - 1);
            p[i] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(partials + static_cast<uint64_t>(b) * m + r));
        }
#pragma unroll
        for (uint32_t i = 0; i < kAhead; ++i) {
            if (b0 + i < bands) sum = (b0 + i == 0) ? p[i] : sum + p[i];
        }
    }
    vec_t* out = reinterpret_cast<vec_t*>(y + r);
    if constexpr (BETA0) {
        *out = alpha * sum;
    } else {
        *out = beta * *out + alpha * sum;
    }
}

// ------------------------------------------------------------------------------------------
// tiles in column order
// ------------------------------------------------------------------------------------------
// A packed word has room for 32 - log2(rows per tile) column bits, which for tiles of 16384 rows is a
// band of 1 MiB of fp32: half of what an XCD's L2 holds comfortably.  `sub` consecutive bands therefore
// form a group that shares one plane of partial sums: the tiles of a row chunk in the bands of a group
// are neighbours in the tile list (tile = (group * chunks + chunk) * sub + band inside the group) and a
// workgroup takes them in one go, keeping the row sums in LDS across them.
//
// Nonzero k (row key r, column key c, both with the index base in) gets its tile number and the same
// packed word as above.  ids_out / packed_out may be the input arrays themselves (element k is read
// before it is written).
__global__ __launch_bounds__(kBlock) void column_order_pack_kernel(idx_t nnz, idx_t base, uint32_t band_shift,
                                                                   uint32_t rows_per_tile, uint32_t chunks, uint32_t sub,
                                                                   const idx_t* r_keys, const idx_t* c_keys,
                                                                   idx_t* ids_out, idx_t* packed_out) {
    const uint64_t k = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (k >= nnz) return;
    const idx_t band_mask = (1u << band_shift) - 1u;
    const idx_t key = c_keys[k];
    const idx_t row = r_keys[k] - base;
    const uint32_t chunk = row / rows_per_tile;
    const uint32_t band = key >> band_shift;
    const uint32_t group = band / sub;
    ids_out[k] = (group * chunks + chunk) * sub + (band - group * sub);
    packed_out[k] = ((row - chunk * rows_per_tile) << band_shift) | (key & band_mask);
}

// One workgroup per compute unit: workgroup i belongs to XCD i % 8 and takes every 32nd unit (the tiles
// of one row chunk in one band group) of that XCD's stretch.  The row sums of a unit live in LDS as
// doubles (fp32 products are widened: ds_add_f32 runs at a quarter of the rate of ds_add_f64 on this
// chip).  A thread keeps two sets of entries in registers, kColumnSet32 or kColumnSet64 each: what fits the 128
// registers a thread of a 1024-thread workgroup can have (fp64, one entry per load, 8 / 10 / 12 / 13: 75.0 / 73.7 /
// 72.5 / 70.3 us on 1 M rows x 16, 14 spills registers; fp32, four entries per load, 12 / 16: 340 / 346 us on the
// power-law matrix, 294 / 292 us on its transpose).
constexpr int kColumnBlock = 1024;
constexpr int kColumnSet32 = 12;
constexpr int kColumnSet64 = 13;
// fp32: the entries of a tile lie in blocks of kColumnQuad * 64, counted from the tile's first entry at a multiple
// of kColumnQuad (the up to three entries ahead of it are taken one by one).  A block of L entries in column order is
// stored so that lane l < L / 4 finds its entries l, L/4 + l, 2 L/4 + l, 3 L/4 + l of the block side by side at
// 4 l .. 4 l + 3 (the last L % 4 entries stay where they are): one 128-bit load per lane brings a wavefront four
// runs of neighbouring entries (the vector memory unit takes a load instruction in the same time whatever its
// width: power-law matrix 384 -> 343 us, its transpose 324 -> 295 us), an element is an entry of the block exactly
// when its place is below L, and a tile's last, partial block needs no code of its own.  With fp64 values the same
// layout with sets of 12 measured slower than one entry per load with sets of 13 (73.8 against 68.5 us on 1 M rows
// x 16; sets of 8: 75 us): that copy keeps its entries in column order, one per load.
constexpr int kColumnQuad = 4;
constexpr uint32_t kColumnQuadBlock = kColumnQuad * kWave;
static_assert(kColumnSet32 % kColumnQuad == 0, "whole blocks per set");
template <typename T>
constexpr bool column_order_quads() { return sizeof(T) == 4; }

// Puts the blocks of every tile into that order, in place.  kInterleaveParts workgroups per tile take turns at
// rounds of kInterleaveBlocks blocks, turned round in LDS so that reads and writes both run along the arrays.
constexpr uint32_t kInterleaveParts = 8;
constexpr int kInterleaveBlocks = 8;
template <typename T>
__global__ __launch_bounds__(kColumnQuadBlock) void column_order_interleave_kernel(idx_t nnz,
                                                                                  const idx_t* __restrict__ tile_ptr,
                                                                                  idx_t* entries, T* vals) {
    idx_t e0 = tile_ptr[blockIdx.x];
    idx_t e1 = tile_ptr[blockIdx.x + 1];
    e0 = e0 < nnz ? e0 : nnz;
    e1 = e1 < nnz ? e1 : nnz;
    e1 = e1 > e0 ? e1 : e0;
    const idx_t a0 = (e0 + kColumnQuad - 1) / kColumnQuad * kColumnQuad;
    if (a0 >= e1) return;  // whole workgroup
    const uint32_t len = e1 - a0;
    const uint32_t blocks = (len + kColumnQuadBlock - 1) / kColumnQuadBlock;
    __shared__ idx_t s_w[kInterleaveBlocks][kColumnQuadBlock];
    __shared__ T s_v[kInterleaveBlocks][kColumnQuadBlock];
    const uint32_t p = threadIdx.x;
    for (uint32_t b0 = blockIdx.y * kInterleaveBlocks; b0 < blocks; b0 += gridDim.y * kInterleaveBlocks) {  // whole workgroup
        idx_t w[kInterleaveBlocks];
        T v[kInterleaveBlocks];
#pragma unroll
        for (int i = 0; i < kInterleaveBlocks; ++i) {
            const uint32_t at = min((b0 + i) * kColumnQuadBlock + p, len - 1);
            w[i] = entries[a0 + at];
            v[i] = vals[a0 + at];
        }
#pragma unroll
        for (int i = 0; i < kInterleaveBlocks; ++i) {
            const uint32_t first = (b0 + i) * kColumnQuadBlock;
            if (first + p < len) {
                const uint32_t in_block = len - first < kColumnQuadBlock ? len - first : kColumnQuadBlock;
                const uint32_t q = in_block / kColumnQuad;
                const uint32_t to = p < q * kColumnQuad ? (p % q) * kColumnQuad + p / q : p;
                s_w[i][to] = w[i];
                s_v[i][to] = v[i];
            }
        }
        __syncthreads();  // every element of the round has been read and lies in its new place in LDS
#pragma unroll
        for (int i = 0; i < kInterleaveBlocks; ++i) {
            const uint32_t first = (b0 + i) * kColumnQuadBlock;
            if (first + p < len) {
                entries[a0 + first + p] = s_w[i][p];
                vals[a0 + first + p] = s_v[i][p];
            }
        }
        __syncthreads();
    }
}

// xcd_start for the kernel below, in units.  A stretch is dealt to the kColumnGroupsPerXcd workgroups of
// its XCD in turns, so what counts is the largest number of nonzeros any one workgroup ends up with.
// Two ways to cut the list of units are tried, equal nonzeros per XCD (good when units differ widely)
// and equal counts (good when they are alike: one unit too many on an XCD doubles a workgroup's
// share), and the better one is kept.
__global__ __launch_bounds__(kBlock) void column_order_split_kernel(idx_t nnz, uint32_t units, uint32_t sub,
                                                                    const idx_t* __restrict__ tile_ptr,
                                                                    uint32_t* __restrict__ xcd_start,
                                                                    uint32_t* __restrict__ next_unit) {
    static_assert(kBlock == kXcds * kColumnGroupsPerXcd, "one thread per workgroup of the SpMV kernel");
    __shared__ uint32_t s_start[2][kXcds + 1];
    __shared__ unsigned long long s_worst[2];
    const uint32_t tid = threadIdx.x;
    if (tid < kXcds) next_unit[tid] = kColumnGroupsPerXcd;  // the work counters of the SpMV kernel: see there
    if (tid == kXcds) next_unit[kXcds] = 0;                 // and its count of workgroups that are through
    if (tid <= kXcds) {
        const uint64_t target = static_cast<uint64_t>(nnz) * tid / kXcds;
        uint32_t lo = 0, hi = units;  // first unit whose offset is >= target
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (tile_ptr[static_cast<uint64_t>(mid) * sub] < target) lo = mid + 1; else hi = mid;
        }
        s_start[0][tid] = tid == 0 ? 0u : (tid == kXcds ? units : lo);
        s_start[1][tid] = static_cast<uint32_t>(static_cast<uint64_t>(units) * tid / kXcds);
    }
    if (tid < 2) s_worst[tid] = 0;
    __syncthreads();
    const uint32_t xcd = tid / kColumnGroupsPerXcd, slot = tid % kColumnGroupsPerXcd;
    for (int cut = 0; cut < 2; ++cut) {
        unsigned long long share = 0;
        for (uint32_t u = s_start[cut][xcd] + slot; u < s_start[cut][xcd + 1]; u += kColumnGroupsPerXcd)
            share += tile_ptr[static_cast<uint64_t>(u + 1) * sub] - tile_ptr[static_cast<uint64_t>(u) * sub];
        atomicMax(&s_worst[cut], share);
    }
    __syncthreads();
    if (tid <= kXcds) xcd_start[tid] = s_start[s_worst[1] <= s_worst[0] ? 1 : 0][tid];
}

// Adds product p to the sum of row r of the tile, for one entry per lane of a wavefront of which most lanes hold row
// `lead` (a row with an entry in nearly every column of the band: LDS would take the adds to its sum one after the
// other).  Those lanes are summed in registers and added once.  live: this lane's entry exists.
__device__ __forceinline__ void add_to_crowded_row(double* s_acc, uint32_t r, double p, bool live, uint32_t lead) {
    const bool with_lead = live && r == lead;
    const double sum = group_sum<kWave>(with_lead ? p : 0.0);
    if (lane_id() == 0) unsafeAtomicAdd(&s_acc[lead], sum);
    if (live && !with_lead) unsafeAtomicAdd(&s_acc[r], p);
}
constexpr int kCrowdedLanes = 40;  // lanes of a wavefront on one row from which they are summed in registers first

// Where the stretch of units of each XCD begins (and the last one ends), by value among the kernel's arguments.
struct XcdStarts {
    uint32_t first[kXcds + 1];
};

// CROWD: the matrix has a row that holds a large share of a tile (BandedShape::crowded_rows): where most lanes of a
// wavefront meet on one row in the first entries of a slab, the slab's products for that row are summed in registers
// (a matrix with dense rows: 0.78 -> 0.36 ms with one such row among 4 M, 0.99 -> 0.55 ms with four).  The test and
// the second copy of the loop cost the kernel 2 to 10 % on matrices without such rows, which is why it is a variant.
// DIRECT: one band group spans all of x, so a unit's sums are the rows of y themselves: the kernel writes
// y = alpha * sums + beta * y and no reduce kernel follows (11.7 us of 254 on the power-law matrix under op T).
// The work counters are then put back by the workgroup that is through last: next_unit[kXcds] counts them.
template <typename T, bool CROWD, bool DIRECT>
__global__ __launch_bounds__(kColumnBlock) void spmv_column_order_kernel(idx_t m, idx_t n, idx_t nnz, idx_t base,
                                                                        uint32_t band_shift, uint32_t rows_per_tile,
                                                                        uint32_t chunks, uint32_t units, uint32_t sub,
                                                                        const XcdStarts stretches,
                                                                        uint32_t* __restrict__ next_unit,
                                                                        const idx_t* __restrict__ tile_ptr,
                                                                        const idx_t* __restrict__ entries,
                                                                        const T* __restrict__ vals,
                                                                        const T* __restrict__ x,
                                                                        T* __restrict__ partials, T* __restrict__ y,
                                                                        T alpha, T beta) {
    const uint32_t* xcd_start = stretches.first;
    extern __shared__ __align__(16) unsigned char s_raw[];
    __shared__ uint32_t s_unit;
    double* s_acc = reinterpret_cast<double*>(s_raw);
    const uint32_t tid = threadIdx.x;
    const uint32_t xcd = blockIdx.x % kXcds;
    const uint32_t stretch_end = min(xcd_start[xcd + 1], units);
    const idx_t band_mask = (1u << band_shift) - 1u;
    for (uint32_t r = tid; r < rows_per_tile; r += kColumnBlock) s_acc[r] = 0.0;
    __syncthreads();
    // The units of an XCD's stretch differ in size (power-law rows): a workgroup starts with the unit of
    // its own number and takes the next off a counter whenever it gets free.  The counter starts at the
    // number of workgroups per XCD: the reduce kernel of the call before, or the build, has left it so.
    // Every workgroup ends when the counter has passed the stretch.
    bool first = true;
    while (true) {
        if (tid == 0)
            s_unit = xcd_start[xcd] + (first ? blockIdx.x / kXcds : atomicAdd(&next_unit[xcd], 1u));
        first = false;
        __syncthreads();
        const uint32_t unit = s_unit;
        __syncthreads();  // read by all before it is written again
        if (unit >= stretch_end) break;  // whole workgroup; also where an overwritten counter ends up
        const uint32_t group = unit / chunks;
        const uint32_t chunk = unit - group * chunks;
        const uint64_t row0 = static_cast<uint64_t>(chunk) * rows_per_tile;
        if (row0 >= m) continue;  // whole workgroup
        const uint32_t tile_rows = static_cast<uint32_t>(m - row0 < rows_per_tile ? m - row0 : rows_per_tile);
        for (uint32_t b = 0; b < sub; ++b) {
            const uint64_t tile = static_cast<uint64_t>(unit) * sub + b;
            idx_t e0 = tile_ptr[tile];
            idx_t e1 = tile_ptr[tile + 1];
            e0 = e0 < nnz ? e0 : nnz;
            e1 = e1 < nnz ? e1 : nnz;
            e1 = e1 > e0 ? e1 : e0;
            const idx_t band_key = (group * sub + b) << band_shift;
            // Two sets of kSet entries per thread take turns.  A set is gathered for and added while the loads of
            // the other are on their way: the gathers of a set are issued first, then the loads of the next set,
            // and only then are the gathers waited for (loads return in the order they were issued, so a wait for
            // gathers that had been issued after the next set's loads would wait for those as well; in that order
            // 1 M rows x 16 in fp64 took 78.3 us and the power-law matrix in fp32 395 us, in this one 70.3 and 384).
            constexpr int kSet = sizeof(T) == 4 ? kColumnSet32 : kColumnSet64;
            constexpr idx_t kPart = kColumnBlock * kSet;  // entries the workgroup takes per set
            idx_t packed[2][kSet];
            T v[2][kSet];
            // Element i of a thread's set lies at place(i) of the set.  In blocks: block i / 4 of the wavefront, at
            // 4 * lane + i % 4; else entry by entry across the workgroup.
            constexpr bool kQuads = column_order_quads<T>();
            const uint32_t lane_first = (tid / kWave) * kColumnQuadBlock + (tid % kWave) * kColumnQuad;
            auto place = [&](int i) {
                if constexpr (kQuads) {
                    return static_cast<uint32_t>(i / kColumnQuad) * (kColumnBlock * kColumnQuad) + lane_first +
                           static_cast<uint32_t>(i % kColumnQuad);
                } else {
                    return static_cast<uint32_t>(i) * kColumnBlock + tid;
                }
            };
            auto ask = [&](int h, idx_t start) {  // start < e1 (and a multiple of kColumnQuad where that matters)
                const uint32_t cnt = e1 - start < kPart ? e1 - start : kPart;
                if constexpr (kQuads) {
                    typedef idx_t quad_t __attribute__((ext_vector_type(4)));
                    const uint32_t last_quad = (cnt - 1) / kColumnQuad * kColumnQuad;
#pragma unroll
                    for (int j = 0; j < kSet / kColumnQuad; ++j) {
                        // (array + start) + place: a uniform base and a small offset per lane, one register
                        const uint32_t at = min(place(j * kColumnQuad), last_quad);
                        const quad_t q = __builtin_nontemporal_load(reinterpret_cast<const quad_t*>((entries + start) + at));
                        const quad_t f = __builtin_nontemporal_load(reinterpret_cast<const quad_t*>((vals + start) + at));
                        packed[h][j * 4 + 0] = q.x;
                        packed[h][j * 4 + 1] = q.y;
                        packed[h][j * 4 + 2] = q.z;
                        packed[h][j * 4 + 3] = q.w;
                        v[h][j * 4 + 0] = __uint_as_float(f.x);
                        v[h][j * 4 + 1] = __uint_as_float(f.y);
                        v[h][j * 4 + 2] = __uint_as_float(f.z);
                        v[h][j * 4 + 3] = __uint_as_float(f.w);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < kSet; ++i) {
                        const uint32_t k = min(place(i), cnt - 1);
                        packed[h][i] = load_stream(entries + start + k);
                        v[h][i] = load_stream(vals + start + k);
                    }
                }
            };
            auto gather = [&](int h, T (&xv)[kSet]) {
#pragma unroll
                for (int i = 0; i < kSet; ++i) {
                    idx_t key = band_key | (packed[h][i] & band_mask);  // column + base
                    key = key > base ? key : base;
                    xv[i] = x[min(key - base, n - 1)];
                }
            };
            auto add = [&](int h, idx_t start, const T (&xv)[kSet], bool whole_set) {
                const uint32_t cnt = e1 - start < kPart ? e1 - start : kPart;
                // a row past the end of the tile (an overwritten layout) still lies inside the sums
                if constexpr (CROWD) {
                    const uint32_t r_first = min(packed[h][0] >> band_shift, rows_per_tile - 1);
                    const uint32_t lead = __builtin_amdgcn_readfirstlane(r_first);
                    if (__popcll(__ballot(r_first == lead)) >= kCrowdedLanes) {  // whole wavefront
#pragma unroll
                        for (int i = 0; i < kSet; ++i) {
                            const uint32_t k = place(i);
                            const uint32_t r = min(packed[h][i] >> band_shift, rows_per_tile - 1);
                            add_to_crowded_row(s_acc, r, static_cast<double>(v[h][i] * xv[i]), whole_set || k < cnt, lead);
                        }
                        return;
                    }
                }
#pragma unroll
                for (int i = 0; i < kSet; ++i) {
                    const uint32_t k = place(i);
                    const uint32_t r = min(packed[h][i] >> band_shift, rows_per_tile - 1);
                    if (whole_set || k < cnt) unsafeAtomicAdd(&s_acc[r], static_cast<double>(v[h][i] * xv[i]));
                }
            };
            // A set with a successor: gathers, then the successor's loads, then the adds.  The loads are not
            // made conditional inside it: the compiler then counts the loads in flight for the path without them
            // and waits for all of them before the first add.  The last set of a tile runs without.
            auto step = [&](int h, idx_t start) {
                T xv[kSet];
                gather(h, xv);
                __builtin_amdgcn_sched_barrier(0);
                ask(h ^ 1, start + kPart);
                __builtin_amdgcn_sched_barrier(0);
                add(h, start, xv, true);
            };
            auto last = [&](int h, idx_t start) {
                T xv[kSet];
                gather(h, xv);
                add(h, start, xv, false);
            };
            if constexpr (kQuads) {  // the entries ahead of the first multiple of kColumnQuad, a lane each
                const idx_t a0 = (e0 + kColumnQuad - 1) / kColumnQuad * kColumnQuad;
                const idx_t head_end = a0 < e1 ? a0 : e1;
                if (tid < head_end - e0) {
                    const idx_t w = entries[e0 + tid];
                    idx_t key = band_key | (w & band_mask);
                    key = key > base ? key : base;
                    const uint32_t r = min(w >> band_shift, rows_per_tile - 1);
                    unsafeAtomicAdd(&s_acc[r], static_cast<double>(vals[e0 + tid] * x[min(key - base, n - 1)]));
                }
                e0 = head_end;
            }
            if (e0 < e1) {
                ask(0, e0);
                idx_t start = e0;
                int h = 0;  // the set that holds the entries from `start` (the same for the workgroup)
                while (e1 - start > kPart) {
                    step(0, start);
                    start += kPart;
                    h = 1;
                    if (e1 - start <= kPart) break;
                    step(1, start);
                    start += kPart;
                    h = 0;
                }
                if (h == 0) last(0, start);
                else last(1, start);
            }
        }
        __syncthreads();
        if constexpr (DIRECT) {
            T* out = y + row0;
            for (uint32_t r = tid; r < rows_per_tile; r += kColumnBlock) {
                if (r < tile_rows) {
                    const T sum = alpha * static_cast<T>(s_acc[r]);
                    out[r] = beta == T(0) ? sum : sum + beta * out[r];
                }
                s_acc[r] = 0.0;
            }
        } else {
            T* out = partials + static_cast<uint64_t>(group) * m + row0;
            for (uint32_t r = tid; r < rows_per_tile; r += kColumnBlock) {
                if (r < tile_rows) out[r] = static_cast<T>(s_acc[r]);
                s_acc[r] = 0.0;
            }
        }
        __syncthreads();
    }
    if constexpr (DIRECT) {
        // every workgroup comes here once, after its last look at a work counter
        if (tid == 0 && atomicAdd(&next_unit[kXcds], 1u) == gridDim.x - 1) {
            for (uint32_t i = 0; i < kXcds; ++i) atomicExch(&next_unit[i], static_cast<uint32_t>(kColumnGroupsPerXcd));
            atomicExch(&next_unit[kXcds], 0u);
        }
    }
}

}  // namespace

bool banded_shape(idx_t m, idx_t n, idx_t nnz, idx_t base, size_t value_bytes, size_t band_bytes, BandedShape* out) {
    if (m == 0 || n == 0 || nnz == 0 || (value_bytes != 4 && value_bytes != 8)) return false;
    uint32_t shift = 0;
    while ((static_cast<size_t>(value_bytes) << (shift + 1)) <= band_bytes) ++shift;  // keys per band = 2^shift
    const uint64_t max_key = static_cast<uint64_t>(n) - 1 + base;
    const uint64_t bands = (max_key >> shift) + 1;
    if (bands < 2 || bands > 256) return false;  // one band: x fits as it is; more than a sort pass orders
    // rows per tile: a typical tile fills three quarters of a slab
    const double per_row_and_band = static_cast<double>(nnz) / (static_cast<double>(m) * static_cast<double>(bands));
    double rows = 0.75 * kSlab / (per_row_and_band > 1e-9 ? per_row_and_band : 1e-9);
    if (rows > kBandedMaxRowsPerTile) rows = kBandedMaxRowsPerTile;
    if (rows < 32) rows = 32;
    uint32_t rows_per_tile = static_cast<uint32_t>(rows);
    if (rows_per_tile > m) rows_per_tile = m;
    if (bit_length(rows_per_tile - 1) + shift > 32) return false;
    const uint64_t chunks = (static_cast<uint64_t>(m) + rows_per_tile - 1) / rows_per_tile;
    if (bands * chunks >= (1ull << 31)) return false;
    out->band_shift = shift;
    out->band_bits = bit_length(static_cast<uint32_t>(bands - 1));
    out->bands = static_cast<uint32_t>(bands);
    out->rows_per_tile = rows_per_tile;
    out->chunks = static_cast<uint32_t>(chunks);
    out->tiles = static_cast<uint32_t>(bands * chunks);
    return true;
}

// ------------------------------------------------------------------------------------------
// how the gathers are spread over the lines of x
// ------------------------------------------------------------------------------------------
namespace {

__global__ __launch_bounds__(kBlock) void fill_u32_kernel(uint64_t n, uint32_t value, uint32_t* p) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < n) p[i] = value;
}

// counts[line] += gathers of that line.  Rows: the gathered element is the row itself (a transposing direction:
// element r is read once per nonzero of row r).  Indices: every stride-th index names the gathered element.
__global__ __launch_bounds__(kBlock) void line_gathers_of_rows_kernel(idx_t rows, const idx_t* __restrict__ ptr,
                                                                      uint32_t line_shift, uint32_t lines,
                                                                      uint32_t* counts) {
    const uint64_t r = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
    uint32_t len = r < rows ? ptr[r + 1] - ptr[r] : 0;
    // the rows of a line are neighbouring lanes (16 or 32 of them, aligned): summed first, one add per line
    for (uint32_t d = 1; d < (1u << line_shift); d <<= 1) len += __shfl_xor(len, static_cast<int>(d));
    if ((r & ((1u << line_shift) - 1u)) == 0 && r < rows && len != 0)
        atomicAdd(&counts[min(static_cast<uint32_t>(r >> line_shift), lines - 1)], len);
}
__global__ __launch_bounds__(kBlock) void line_gathers_of_indices_kernel(idx_t nnz, uint32_t stride, idx_t base,
                                                                         const idx_t* __restrict__ ind,
                                                                         uint32_t line_shift, uint32_t lines,
                                                                         uint32_t* counts) {
    const uint64_t k = (static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x) * stride;
    if (k >= nnz) return;
    const idx_t key = ind[k];
    const idx_t c = key > base ? key - base : 0;
    atomicAdd(&counts[min(static_cast<uint32_t>(c >> line_shift), lines - 1)], 1u);
}
// bins[2 b] = lines whose count has b as its highest bit, bins[2 b + 1] = their gathers
__global__ __launch_bounds__(kBlock) void line_gather_bins_kernel(uint32_t lines, const uint32_t* __restrict__ counts,
                                                                  unsigned long long* bins) {
    __shared__ unsigned long long s_bins[64];
    if (threadIdx.x < 64) s_bins[threadIdx.x] = 0;
    __syncthreads();
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const uint32_t c = i < lines ? counts[i] : 0;
    if (c != 0) {
        const uint32_t b = 31 - __clz(static_cast<int>(c));
        atomicAdd(&s_bins[2 * b], 1ull);
        atomicAdd(&s_bins[2 * b + 1], static_cast<unsigned long long>(c));
    }
    __syncthreads();
    if (threadIdx.x < 64 && s_bins[threadIdx.x] != 0) atomicAdd(&bins[threadIdx.x], s_bins[threadIdx.x]);
}

}  // namespace

size_t line_gathers_workspace_bytes(idx_t gathered, size_t value_bytes) {
    const uint32_t line_shift = value_bytes == 8 ? 4 : 5;
    const uint64_t lines = (static_cast<uint64_t>(gathered) >> line_shift) + 1;
    return 2 * kLineGatherBins * sizeof(unsigned long long) + lines * sizeof(uint32_t);
}

void launch_line_gathers(hipStream_t stream, bool of_rows, idx_t gathered, idx_t nnz, idx_t base, const idx_t* ptr,
                         const idx_t* ind, size_t value_bytes, void* workspace) {
    const uint32_t line_shift = value_bytes == 8 ? 4 : 5;
    const uint32_t lines = static_cast<uint32_t>((static_cast<uint64_t>(gathered) >> line_shift) + 1);
    unsigned long long* bins = static_cast<unsigned long long*>(workspace);
    uint32_t* counts = reinterpret_cast<uint32_t*>(bins + 2 * kLineGatherBins);
    const uint64_t words = 4ull * kLineGatherBins + lines;  // the pairs as 32-bit words, then the counts
    hipLaunchKernelGGL(fill_u32_kernel, dim3(static_cast<uint32_t>((words + kBlock - 1) / kBlock)), dim3(kBlock), 0, stream,
                       words, 0u, static_cast<uint32_t*>(workspace));
    if (of_rows) {
        hipLaunchKernelGGL(line_gathers_of_rows_kernel, dim3((gathered + kBlock - 1) / kBlock), dim3(kBlock), 0, stream,
                           gathered, ptr, line_shift, lines, counts);
    } else {
        const uint32_t stride = static_cast<uint32_t>((static_cast<uint64_t>(nnz) >> 20) + 1);  // about 1 M samples at most
        const uint64_t samples = (static_cast<uint64_t>(nnz) + stride - 1) / stride;
        hipLaunchKernelGGL(line_gathers_of_indices_kernel, dim3(static_cast<uint32_t>((samples + kBlock - 1) / kBlock)),
                           dim3(kBlock), 0, stream, nnz, stride, base, ind, line_shift, lines, counts);
    }
    hipLaunchKernelGGL(line_gather_bins_kernel, dim3((lines + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, lines, counts,
                       bins);
}

// bins: what line_gather_bins_kernel left (read back).  True when the kHotLines most gathered lines of x (half of what
// an XCD's L2 holds) take more than half of the gathers: the hot lines then stay in L2 whatever the width of a band
// group, and one group over all of x saves the planes of partial sums (power-law matrix, op T: 78 % of the gathers
// in the 16384 hottest lines, 294 -> 253 us; uniform columns: 12 %, 340 -> 425 us with groups of 8 MiB).
bool gathers_favour_wide_groups(const unsigned long long* bins) {
    unsigned long long all = 0;
    for (uint32_t b = 0; b < 32; ++b) all += bins[2 * b + 1];
    if (all == 0) return false;
    double lines = 0, gathers = 0;
    for (int b = 31; b >= 0 && lines < kHotLines; --b) {
        const double n = static_cast<double>(bins[2 * b]);
        if (n == 0) continue;
        const double take = n <= kHotLines - lines ? 1.0 : (kHotLines - lines) / n;
        lines += n * take;
        gathers += static_cast<double>(bins[2 * b + 1]) * take;
    }
    return 2.0 * gathers > static_cast<double>(all);
}

bool column_order_shape(idx_t m, idx_t n, idx_t nnz, idx_t base, size_t value_bytes, size_t band_bytes,
                        BandedShape* out) {
    if (m == 0 || n == 0 || nnz == 0 || (value_bytes != 4 && value_bytes != 8)) return false;
    uint32_t wanted = 0;  // log2 of the keys in band_bytes of x
    while ((static_cast<size_t>(value_bytes) << (wanted + 1)) <= band_bytes) ++wanted;
    const uint64_t max_key = static_cast<uint64_t>(n) - 1 + base;
    const uint64_t groups = (max_key >> wanted) + 1;  // planes of partial sums: every one costs a sum per row
    if (groups > 64) return false;
    // The taller a tile, the more of its entries share a line of x; but the kernel runs one workgroup per
    // compute unit, so there must be a unit of work for each: the tiles are halved until there is, and a
    // matrix too small for that is left to the other kernels.
    constexpr uint64_t kUnitsWanted = kXcds * kColumnGroupsPerXcd;
    uint32_t rows_per_tile = kColumnOrderRows;
    while (rows_per_tile > kColumnOrderMinRows &&
           groups * ((static_cast<uint64_t>(m) + rows_per_tile - 1) / rows_per_tile) < kUnitsWanted)
        rows_per_tile /= 2;
    const uint64_t chunks = (static_cast<uint64_t>(m) + rows_per_tile - 1) / rows_per_tile;
    if (groups * chunks < kUnitsWanted) return false;
    const uint32_t row_bits = bit_length(rows_per_tile - 1);
    const uint32_t shift = wanted > 32 - row_bits ? 32 - row_bits : wanted;
    const uint32_t sub = 1u << (wanted - shift);  // bands that share a plane of partial sums
    // the tile numbers are sorted in at most two passes of eight bits
    if (sub > 64 || groups * chunks * sub > 65536) return false;
    out->band_shift = shift;
    out->band_bits = bit_length(static_cast<uint32_t>(groups * sub - 1));
    out->bands = static_cast<uint32_t>(groups);
    out->rows_per_tile = rows_per_tile;
    out->chunks = static_cast<uint32_t>(chunks);
    out->tiles = static_cast<uint32_t>(groups * chunks * sub);
    out->sub = sub;
    out->by_column = true;
    return true;
}

BandedLayout banded_layout(const BandedShape& s, idx_t m, idx_t nnz, size_t value_bytes) {
    BandedLayout l;
    const size_t idx_bytes = align_up(static_cast<size_t>(nnz) * sizeof(idx_t));
    size_t off = 0;
    l.tile_ptr = off; off += align_up((static_cast<size_t>(s.tiles) + 1) * sizeof(idx_t));
    l.xcd_start = off; off += align_up((kXcds + 1) * sizeof(uint32_t));
    l.next_unit = off; off += align_up((kXcds + 1) * sizeof(uint32_t));  // the counters and the count of finished workgroups
    l.entries = off; off += idx_bytes;
    l.vals = off; off += align_up(static_cast<size_t>(nnz) * value_bytes);
    l.partials = off; off += align_up(static_cast<size_t>(s.bands) * m * value_bytes);
    l.keep = off;
    l.src_cols = l.src_rows = l.src_vals = l.tile_ids = 0;
    if (s.by_column) {
        l.tmp_keys = l.tmp_rows = 0;
        l.src_cols = off; off += idx_bytes;
        l.src_rows = off; off += idx_bytes;
        l.src_vals = off; off += align_up(static_cast<size_t>(nnz) * value_bytes);
        l.tile_ids = off; off += idx_bytes;
        l.sort_ws = off; off += align_up(csr2csc_workspace_bytes(m, 0, nnz, value_bytes));
        l.total = off;
        return l;
    }
    l.tmp_keys = off; off += idx_bytes;
    l.tmp_rows = off; off += idx_bytes;
    l.sort_ws = off; off += align_up(band_sort_workspace_bytes(nnz));
    l.total = off;
    return l;
}

void launch_column_order_build(hipStream_t stream, const BandedShape& s, idx_t m, idx_t nnz, idx_t base,
                               const idx_t* r_keys, const idx_t* c_keys, const void* vals, size_t value_bytes,
                               void* region) {
    const BandedLayout l = banded_layout(s, m, nnz, value_bytes);
    char* w = static_cast<char*>(region);
    // tile numbers and packed words take the place of the source arrays inside the region; a caller's
    // own arrays (the transposing directions hand them in) are copied from, never written
    idx_t* ids = reinterpret_cast<idx_t*>(w + l.src_cols);
    idx_t* packed = reinterpret_cast<idx_t*>(w + l.src_rows);
    hipLaunchKernelGGL(column_order_pack_kernel, dim3((nnz + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, nnz, base,
                       s.band_shift, s.rows_per_tile, s.chunks, s.sub, r_keys, c_keys, ids, packed);
    idx_t* sorted_ids = reinterpret_cast<idx_t*>(w + l.tile_ids);
    launch_sort_triples(stream, nnz, bit_length(s.tiles - 1), ids, packed, vals, sorted_ids,
                        reinterpret_cast<idx_t*>(w + l.entries), w + l.vals, value_bytes, w + l.sort_ws);
    launch_coo2csr(stream, nnz, s.tiles, sorted_ids, 0, reinterpret_cast<idx_t*>(w + l.tile_ptr));
    if (value_bytes == 4) {
        static_assert(column_order_quads<float>() && !column_order_quads<double>(), "the kernel's reading of the copy");
        hipLaunchKernelGGL(column_order_interleave_kernel<float>, dim3(s.tiles, kInterleaveParts), dim3(kColumnQuadBlock), 0, stream, nnz,
                           reinterpret_cast<const idx_t*>(w + l.tile_ptr), reinterpret_cast<idx_t*>(w + l.entries),
                           reinterpret_cast<float*>(w + l.vals));
    }
    hipLaunchKernelGGL(column_order_split_kernel, dim3(1), dim3(kBlock), 0, stream, nnz, s.tiles / s.sub, s.sub,
                       reinterpret_cast<const idx_t*>(w + l.tile_ptr), reinterpret_cast<uint32_t*>(w + l.xcd_start),
                       reinterpret_cast<uint32_t*>(w + l.next_unit));
}

void launch_banded_build(hipStream_t stream, const BandedShape& s, idx_t m, idx_t nnz, idx_t base, const idx_t* row_ptr,
                         const idx_t* col, const void* val, size_t value_bytes, void* region) {
    const BandedLayout l = banded_layout(s, m, nnz, value_bytes);
    char* w = static_cast<char*>(region);
    idx_t* tmp_keys = reinterpret_cast<idx_t*>(w + l.tmp_keys);
    idx_t* tmp_rows = reinterpret_cast<idx_t*>(w + l.tmp_rows);
    launch_sort_by_column_band(stream, m, nnz, base, row_ptr, col, val, value_bytes, s.band_shift, s.band_bits, tmp_keys,
                               tmp_rows, w + l.vals, w + l.sort_ws);
    const uint64_t boundaries = static_cast<uint64_t>(nnz) + 1;
    hipLaunchKernelGGL(banded_pack_kernel, dim3(static_cast<uint32_t>((boundaries + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       stream, nnz, base, s.band_shift, s.rows_per_tile, s.chunks, s.tiles,
                       static_cast<const idx_t*>(tmp_keys), static_cast<const idx_t*>(tmp_rows),
                       reinterpret_cast<idx_t*>(w + l.entries), reinterpret_cast<idx_t*>(w + l.tile_ptr));
    hipLaunchKernelGGL(banded_split_kernel, dim3(1), dim3(kWave), 0, stream, nnz, s.tiles,
                       reinterpret_cast<const idx_t*>(w + l.tile_ptr), reinterpret_cast<uint32_t*>(w + l.xcd_start));
}

uint32_t banded_grid(const uint32_t* xcd_start_host) {
    uint32_t longest = 0;
    for (uint32_t i = 0; i < kXcds; ++i) {
        const uint32_t len = xcd_start_host[i + 1] > xcd_start_host[i] ? xcd_start_host[i + 1] - xcd_start_host[i] : 0;
        longest = len > longest ? len : longest;
    }
    return longest * kXcds;
}

template <typename T>
bool launch_spmv_banded(hipStream_t stream, const BandedShape& s, uint32_t grid, const SpmvArgs& a, T alpha, T beta,
                        void* region) {
    if (a.m == 0) return true;
    const BandedLayout l = banded_layout(s, a.m, a.nnz, sizeof(T));
    char* w = static_cast<char*>(region);
    T* partials = reinterpret_cast<T*>(w + l.partials);
    if (s.by_column) {
        const int lds = static_cast<int>(s.rows_per_tile * sizeof(double));
        XcdStarts stretches;
        for (uint32_t i = 0; i <= kXcds; ++i) stretches.first[i] = s.xcd_start[i];
        // one band group: the kernel writes y itself, and no reduce follows
        const bool direct = s.bands == 1;
        auto* kernel = direct ? (s.crowded_rows ? spmv_column_order_kernel<T, true, true>
                                                : spmv_column_order_kernel<T, false, true>)
                              : (s.crowded_rows ? spmv_column_order_kernel<T, true, false>
                                                : spmv_column_order_kernel<T, false, false>);
        if (!allow_dynamic_lds(reinterpret_cast<const void*>(kernel), lds)) return false;
        hipLaunchKernelGGL(kernel, dim3(kColumnGroupsPerXcd * kXcds), dim3(kColumnBlock), lds, stream, a.m, a.n, a.nnz,
                           a.base, s.band_shift, s.rows_per_tile, s.chunks, s.tiles / s.sub, s.sub,
                           stretches, reinterpret_cast<uint32_t*>(w + l.next_unit),
                           reinterpret_cast<const idx_t*>(w + l.tile_ptr), reinterpret_cast<const idx_t*>(w + l.entries),
                           reinterpret_cast<const T*>(w + l.vals), static_cast<const T*>(a.x), partials,
                           static_cast<T*>(a.y), alpha, beta);
        if (direct) return launches_taken();
    } else if (grid != 0) {
        hipLaunchKernelGGL((spmv_banded_kernel<T>), dim3(grid), dim3(kBlock), 0, stream, a.m, a.n, a.nnz, a.base,
                           s.band_shift, s.rows_per_tile, s.chunks, s.tiles,
                           reinterpret_cast<const uint32_t*>(w + l.xcd_start),
                           reinterpret_cast<const idx_t*>(w + l.tile_ptr), reinterpret_cast<const idx_t*>(w + l.entries),
                           reinterpret_cast<const T*>(w + l.vals), static_cast<const T*>(a.x), partials);
    }
    uint32_t* next_unit = s.by_column ? reinterpret_cast<uint32_t*>(w + l.next_unit) : nullptr;
    constexpr idx_t kWide = 16 / sizeof(T);
    // 16 bytes per access: 1 M rows, four planes of fp64 10.9 -> 8.8 us; eight planes of fp32 (four rows per thread) 1 us slower
    if (sizeof(T) == 8 && a.m % kWide == 0 &&
        ((reinterpret_cast<uintptr_t>(partials) | reinterpret_cast<uintptr_t>(a.y)) & 15u) == 0) {
        const dim3 wide_grid((a.m / kWide + kBlock - 1) / kBlock);
        if (beta == T(0)) {
            hipLaunchKernelGGL((banded_reduce_wide_kernel<T, true>), wide_grid, dim3(kBlock), 0, stream, a.m, s.bands,
                               static_cast<const T*>(partials), static_cast<T*>(a.y), alpha, beta, next_unit);
        } else {
            hipLaunchKernelGGL((banded_reduce_wide_kernel<T, false>), wide_grid, dim3(kBlock), 0, stream, a.m, s.bands,
                               static_cast<const T*>(partials), static_cast<T*>(a.y), alpha, beta, next_unit);
        }
        return launches_taken();
    }
    const dim3 rows_grid((a.m + kBlock - 1) / kBlock);
    if (beta == T(0)) {
        hipLaunchKernelGGL((banded_reduce_kernel<T, true>), rows_grid, dim3(kBlock), 0, stream, a.m, s.bands,
                           static_cast<const T*>(partials), static_cast<T*>(a.y), alpha, beta, next_unit);
    } else {
        hipLaunchKernelGGL((banded_reduce_kernel<T, false>), rows_grid, dim3(kBlock), 0, stream, a.m, s.bands,
                           static_cast<const T*>(partials), static_cast<T*>(a.y), alpha, beta, next_unit);
    }
    return launches_taken();
}

template bool launch_spmv_banded<float>(hipStream_t, const BandedShape&, uint32_t, const SpmvArgs&, float, float, void*);
template bool launch_spmv_banded<double>(hipStream_t, const BandedShape&, uint32_t, const SpmvArgs&, double, double, void*);

}  // namespace mcsp
