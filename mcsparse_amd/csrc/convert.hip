// Index conversions for gfx950: csr2coo, coo2csr and csr2csc.
//
// csr2csc must reproduce the reference's order exactly: a stable sort of the nonzeros by
// column (src/kernels/conversion/mcsp_csr2csc.cpp:97-98, LSD radix sort with 2-bit digits,
// src/mcprim/device_radix_sort.hpp:283-306), so entries of one column keep their CSR order.
// A stable sort has exactly one result, which leaves the digit width free: here the (column,
// row, value) triples are carried through ceil(bits/8) LSD passes of up to 8 bits instead of
// sorting a permutation in bits/2 passes and gathering through it afterwards, which on HBM
// trades ~24 sweeps plus two random gathers for 3 sweeps.
#include "device_util.h"
#include "internal.h"

namespace mcsp {

namespace {

constexpr int kBlock = 256;

// ------------------------------------------------------------------------------------------
// row lookups in row_ptr, shared by csr2coo and the sorts that read a CSR matrix in place
// ------------------------------------------------------------------------------------------
// Number of rows r in [0, m] whose first nonzero index row_ptr[r] - base is <= g, found with
// 64 probes per round, which shrink the interval 64-fold (4M rows: 4 dependent loads instead of 22);
// with g a nonzero index the answer minus one is the row that holds g.
// Every lane of the wave must call this; all lanes return the same value.
__device__ __forceinline__ idx_t wave_count_row_starts(const idx_t* __restrict__ row_ptr, idx_t m, idx_t base, idx_t g) {
    uint64_t lo = 0;
    uint64_t hi = static_cast<uint64_t>(m) + 1;
    const unsigned lane = lane_id();
    while (lo < hi) {
        const uint64_t span = hi - lo;
        const uint64_t step = (span + kWave - 1) / kWave;
        const uint64_t probe = lo + lane * step;
        const bool pred = probe < hi && row_ptr[probe] - base <= g;
        const unsigned count = __popcll(__ballot(pred));
        if (count == 0) {
            hi = lo;
        } else {
            const uint64_t new_hi = lo + static_cast<uint64_t>(count) * step;
            lo = lo + static_cast<uint64_t>(count - 1) * step + 1;
            hi = new_hi < hi ? new_hi : hi;
        }
    }
    return static_cast<idx_t>(lo);
}

// Inclusive sum over the 64 lanes of a wavefront: four shifted adds inside each row of 16 lanes,
// then the last lane of rows 0 and 2 is added to rows 1 and 3, then lane 31 to rows 2 and 3.
__device__ __forceinline__ uint32_t wave_inclusive_sum(uint32_t v) {
    constexpr int kRowShr = 0x110, kRowBcast15 = 0x142, kRowBcast31 = 0x143;
    int x = static_cast<int>(v);
    x += __builtin_amdgcn_update_dpp(0, x, kRowShr + 1, 0xF, 0xF, false);
    x += __builtin_amdgcn_update_dpp(0, x, kRowShr + 2, 0xF, 0xF, false);
    x += __builtin_amdgcn_update_dpp(0, x, kRowShr + 4, 0xF, 0xF, false);
    x += __builtin_amdgcn_update_dpp(0, x, kRowShr + 8, 0xF, 0xF, false);
    x += __builtin_amdgcn_update_dpp(0, x, kRowBcast15, 0xA, 0xF, false);
    x += __builtin_amdgcn_update_dpp(0, x, kRowBcast31, 0xC, 0xF, false);
    return static_cast<uint32_t>(x);
}

// coo_rows[j] = row of nonzero j (+ base) = the number of rows that begin at or before j, minus one.
// A tile is 4096 nonzeros.  The rows that begin inside it are read from row_ptr (the first of them is
// known from the tile before; only where a workgroup's first tile begins is searched for, a chain of
// dependent loads) and set bits in a 4096-bit map in LDS; a thread then writes four neighbouring rows at a
// time, each a count of bits, as one 16-byte store.  A tile in which two rows begin at the same nonzero
// (an empty row) cannot be told from the map: its threads search the staged row starts instead, or
// row_ptr itself when more rows begin in the tile than LDS holds.  A workgroup takes kExpandTiles tiles in
// a row.  Reference semantics: src/kernels/conversion/coo2csr_device.hpp:26-41.
constexpr int kExpandTiles = 8;
constexpr int kCooBlock = 256;
constexpr int kCooTile = kCooBlock * 16;  // four stores of four rows per thread
constexpr int kCooWords = kCooTile / kWave;
constexpr int kCooLoads = 4;  // row starts per thread and round
__global__ __launch_bounds__(kCooBlock) void csr2coo_kernel(idx_t m, idx_t nnz, idx_t base,
                                                         const idx_t* __restrict__ row_ptr,
                                                         idx_t* __restrict__ coo_rows) {
    typedef idx_t idx4 __attribute__((ext_vector_type(4)));
    static_assert((kCooWords % kWave == 0 || kCooWords < kWave) && kCooWords <= kCooBlock && kCooBlock % kWave == 0,
                  "the words of the map are counted a wavefront at a time");
    constexpr int kScanLanes = (kCooWords + kWave - 1) / kWave * kWave;
    __shared__ idx_t s_start[kCooTile];
    __shared__ unsigned long long s_begins[kCooWords];
    __shared__ uint32_t s_begins_before[kCooWords];
    __shared__ uint32_t s_wave_begins[(kCooWords + kWave - 1) / kWave];
    __shared__ idx_t s_first;
    __shared__ uint32_t s_empty_rows;
    __shared__ uint32_t s_inside;

    const uint32_t tid = threadIdx.x;
    const unsigned lane = tid % kWave;
    const uint64_t group_first = static_cast<uint64_t>(blockIdx.x) * kExpandTiles * kCooTile;
    if (group_first >= nnz) return;  // whole workgroup
    if (tid / kWave == 0) {
        const idx_t c = wave_count_row_starts(row_ptr, m, base, static_cast<idx_t>(group_first));
        if (tid == 0) s_first = c;
    }
    __syncthreads();
    uint64_t before = s_first;  // rows (of the m + 1 offsets) that begin at or before the tile's first nonzero
    const bool wide = (reinterpret_cast<uintptr_t>(coo_rows) & 15u) == 0;
    for (int t = 0; t < kExpandTiles; ++t) {
        const uint64_t j0 = group_first + static_cast<uint64_t>(t) * kCooTile;
        if (j0 >= nnz) break;  // whole workgroup
        const uint32_t count = static_cast<uint32_t>(nnz - j0 < kCooTile ? nnz - j0 : kCooTile);
        if (tid < kCooWords) s_begins[tid] = 0;
        if (tid == 0) {
            s_empty_rows = 0;
            s_inside = 0;
        }
        __syncthreads();
        // the offsets from `before` on, until one lies past the tile: those up to j0 + 4096 begin a row of this
        // tile (or, at j0 + 4096 itself, are counted for the next one)
        uint32_t inside = 0;
        for (uint32_t loaded = 0;; loaded += kCooBlock * kCooLoads) {
            uint64_t at[kCooLoads];
#pragma unroll
            for (int k = 0; k < kCooLoads; ++k) {
                const uint64_t r = before + loaded + static_cast<uint32_t>(k) * kCooBlock + tid;
                const uint64_t r_read = r <= m ? r : m;
                const idx_t v = row_ptr[r_read];
                at[k] = r <= m ? static_cast<uint64_t>(v - base) - j0 : ~0ull;  // > 0: row `before` begins after j0
            }
            uint32_t mine = 0;  // one past the last offset of this thread that lies inside
#pragma unroll
            for (int k = 0; k < kCooLoads; ++k) {
                if (at[k] > static_cast<uint64_t>(kCooTile)) continue;
                const uint32_t i = loaded + static_cast<uint32_t>(k) * kCooBlock + tid;
                mine = i + 1;
                if (i < static_cast<uint32_t>(kCooTile)) s_start[i] = static_cast<idx_t>(at[k]);
                if (at[k] < static_cast<uint64_t>(kCooTile)) {
                    const unsigned long long bit = 1ull << (at[k] % kWave);
                    if ((atomicOr(&s_begins[at[k] / kWave], bit) & bit) != 0) s_empty_rows = 1;
                }
            }
            // the offsets ascend, so those inside come first: their number is where the last one stands
            if (mine != 0) atomicMax(&s_inside, mine);
            __syncthreads();
            inside = s_inside;
            if (inside < loaded + kCooBlock * kCooLoads) break;  // whole workgroup: the round held one past the tile
        }
        const bool by_bits = s_empty_rows == 0;  // the same for the whole workgroup
        if (by_bits) {
            if (tid < kScanLanes) {  // whole wavefronts
                const uint32_t c = tid < kCooWords ? __popcll(s_begins[tid]) : 0;
                const uint32_t upto = wave_inclusive_sum(c);
                if (tid < kCooWords) s_begins_before[tid] = upto - c;
                if (lane == kWave - 1) s_wave_begins[tid / kWave] = upto;
            }
            __syncthreads();
        }
        const bool staged = inside <= static_cast<uint32_t>(kCooTile);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t p = (static_cast<uint32_t>(k) * kCooBlock + tid) * 4;  // four neighbouring nonzeros of the tile
            if (p >= count) continue;
            idx_t rows[4];
            if (by_bits) {
                const uint32_t word = p / kWave, bit = p % kWave;
                const unsigned long long w = s_begins[word];
                // rows that begin before nonzero p, then one more for every bit of the four at p .. p + 3
                uint64_t upto = before + s_begins_before[word];
                for (uint32_t v = 0; v < word / kWave; ++v) upto += s_wave_begins[v];  // wavefronts of words before this one
                idx_t row = static_cast<idx_t>(upto + __popcll(w & ((1ull << bit) - 1ull)) - 1 + base);
                const uint32_t four = static_cast<uint32_t>(w >> bit) & 0xFu;  // bit <= 60
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    row += (four >> e) & 1u;
                    rows[e] = row;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    uint32_t lo = 0, hi = inside;  // row starts of the tile at or before nonzero p + e
                    while (lo < hi) {
                        const uint32_t mid = (lo + hi) >> 1;
                        const uint64_t begins = staged ? s_start[mid] : static_cast<uint64_t>(row_ptr[before + mid] - base) - j0;
                        if (begins <= p + e) lo = mid + 1; else hi = mid;
                    }
                    rows[e] = static_cast<idx_t>(before + lo - 1 + base);
                }
            }
            idx_t* out = coo_rows + j0 + p;
            if (wide && p + 4 <= count) {
                idx4 v = {rows[0], rows[1], rows[2], rows[3]};
                __builtin_nontemporal_store(v, reinterpret_cast<idx4*>(out));
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (p + e < count) out[e] = rows[e];
            }
        }
        before += inside;
        __syncthreads();  // the next tile clears the map
    }
}

// Offsets from sorted row indices: boundary t (between entry t-1 and entry t, 0 <= t <= nnz) fills
// the offsets of the rows that lie in between, so empty rows are covered.  A thread takes kCooVectors
// times four consecutive entries (one 128-bit load each when the array allows it, all asked for before the
// first is used; 1, 2, 4, 8 vectors: 127, 121, 120, 158 us on 117 M entries) and the boundaries in front of
// them; the entry before a thread's four comes from the neighbouring lane.
// Reference semantics: src/kernels/conversion/coo2csr_device.hpp:8-24.
constexpr int kCooPerThread = 4;
constexpr int kCooVectors = 2;
constexpr uint32_t kCooFillRows = 4096;        // offsets a workgroup of the fill kernel looks after
constexpr uint64_t kCooDeferredFill = 8192;    // stretches of more offsets than this are its work (>= kCooFillRows)
template <bool VEC>
__global__ __launch_bounds__(kBlock) void coo2csr_kernel(idx_t nnz, idx_t m, idx_t base,
                                                         const idx_t* __restrict__ coo_rows,
                                                         idx_t* __restrict__ row_ptr) {
    typedef idx_t idx4 __attribute__((ext_vector_type(4)));
    const unsigned lane = threadIdx.x % kWave;
    // entries t0 .. t0+3 of every vector; past the end they read as row m, which makes boundary nnz close
    // the offsets up to m and the boundaries after it empty
    uint64_t first[kCooVectors];
    idx_t r[kCooVectors][kCooPerThread];
    idx_t lead[kCooVectors];  // entry t0-1 for the first lane of a wavefront
#pragma unroll
    for (int j = 0; j < kCooVectors; ++j) {
        const uint64_t t0 = ((static_cast<uint64_t>(blockIdx.x) * kCooVectors + j) * kBlock + threadIdx.x) * kCooPerThread;
        first[j] = t0;
        if (VEC && t0 + kCooPerThread <= nnz) {
            const idx4 v = __builtin_nontemporal_load(reinterpret_cast<const idx4*>(coo_rows + t0));
#pragma unroll
            for (int e = 0; e < kCooPerThread; ++e) r[j][e] = v[e] - base;
        } else {
#pragma unroll
            for (int e = 0; e < kCooPerThread; ++e) r[j][e] = t0 + e < nnz ? load_stream(coo_rows + t0 + e) - base : m;
        }
        lead[j] = lane == 0 && t0 != 0 && t0 <= nnz ? coo_rows[t0 - 1] - base : 0;
    }
#pragma unroll
    for (int j = 0; j < kCooVectors; ++j) {
        const uint64_t t0 = first[j];
        // entry t0-1: the last entry of the lane below, a load of its own for the first lane of a wavefront
        idx_t before = __shfl_up(r[j][kCooPerThread - 1], 1, kWave);
        if (lane == 0) before = lead[j];
        // rows [prev, cur) get offset t: prev = row of entry t-1 plus one (0 in front of the first entry).
        // A thread fills short stretches itself; a longer stretch of empty rows is left to the whole
        // wavefront below, lane by lane 64 offsets at a time; one of more than kCooDeferredFill offsets (up to
        // all m of them after the last entry) to the kernel after this one.
        constexpr uint64_t kSerialFill = 16;
        uint64_t prev = t0 == 0 ? 0 : static_cast<uint64_t>(before) + 1;
        uint64_t long_from = 0, long_to = 0;  // at most one long stretch is kept per thread; more are filled serially
        idx_t long_value = 0;
        if (t0 <= nnz) {
#pragma unroll
            for (int e = 0; e < kCooPerThread; ++e) {
                const uint64_t t = t0 + e;
                if (t > nnz) break;
                const uint64_t cur = static_cast<uint64_t>(r[j][e]) + 1;  // t == nnz: m + 1
                if (cur > prev + kCooDeferredFill) {
                    // left to coo2csr_fill_kernel: the rows of a matrix with few entries, or all those after the
                    // last entry, would keep one wavefront busy for as long as the rest of the launch takes
                } else if (cur > prev + kSerialFill && long_to == long_from) {
                    long_from = prev;
                    long_to = cur;
                    long_value = static_cast<idx_t>(t) + base;
                } else {
                    for (uint64_t i = prev; i < cur; ++i) row_ptr[i] = static_cast<idx_t>(t) + base;
                }
                prev = cur;
            }
        }
        // every lane of the wavefront gets here: the stretches are handed round and filled cooperatively
        uint64_t pending = __ballot(long_to > long_from);
        while (pending != 0) {
            const int src = __ffsll(static_cast<long long>(pending)) - 1;
            pending &= pending - 1;
            const uint64_t from = __shfl(long_from, src, kWave);
            const uint64_t to = __shfl(long_to, src, kWave);
            const idx_t value = __shfl(long_value, src, kWave);
            for (uint64_t i = from + lane; i < to; i += kWave) row_ptr[i] = value;
        }
    }
}

// Number of entries whose row (index base taken off) is below p, in sorted rows, found with 64 probes per
// round.  Every lane of the wave must call this; all lanes return the same value.
__device__ __forceinline__ idx_t wave_count_rows_below(const idx_t* __restrict__ coo_rows, idx_t nnz, idx_t base, uint64_t p) {
    uint64_t lo = 0;
    uint64_t hi = nnz;
    const unsigned lane = lane_id();
    while (lo < hi) {
        const uint64_t span = hi - lo;
        const uint64_t step = (span + kWave - 1) / kWave;
        const uint64_t probe = lo + lane * step;
        const bool pred = probe < hi && static_cast<uint64_t>(coo_rows[probe] - base) < p;
        const unsigned count = __popcll(__ballot(pred));
        if (count == 0) {
            hi = lo;
        } else {
            const uint64_t new_hi = lo + static_cast<uint64_t>(count) * step;
            lo = lo + static_cast<uint64_t>(count - 1) * step + 1;
            hi = new_hi < hi ? new_hi : hi;
        }
    }
    return static_cast<idx_t>(lo);
}

// The stretches of more than kCooDeferredFill equal offsets that coo2csr_kernel leaves out: a workgroup looks
// after kCooFillRows offsets.  Such a stretch is longer than that, so if it touches the workgroup's offsets it holds
// the first or the last of them: for both, the number t of entries in rows below says which stretch they lie in
// (from the row of entry t-1, exclusive, to the row of entry t, inclusive) and what it holds (t + base).
__global__ __launch_bounds__(kBlock) void coo2csr_fill_kernel(idx_t nnz, idx_t m, idx_t base,
                                                              const idx_t* __restrict__ coo_rows,
                                                              idx_t* __restrict__ row_ptr) {
    __shared__ uint64_t s_from[2], s_to[2];
    __shared__ idx_t s_value[2];
    const uint32_t tid = threadIdx.x;
    const uint64_t i0 = static_cast<uint64_t>(blockIdx.x) * kCooFillRows;
    const uint64_t total = static_cast<uint64_t>(m) + 1;  // offsets 0 .. m
    if (i0 >= total) return;  // whole workgroup
    const uint64_t i1 = i0 + kCooFillRows < total ? i0 + kCooFillRows : total;
    const uint32_t which = tid / kWave;
    if (which < 2) {  // whole wavefronts
        const uint64_t p = which == 0 ? i0 : i1 - 1;
        const idx_t t = wave_count_rows_below(coo_rows, nnz, base, p);
        // offsets (row of entry t-1, row of entry t] hold t + base; before the first entry from 0, after the last to m
        const uint64_t from = t == 0 ? 0 : static_cast<uint64_t>(coo_rows[t - 1] - base) + 1;
        const uint64_t to = t == nnz ? total : static_cast<uint64_t>(coo_rows[t] - base) + 1;
        if (tid % kWave == 0) {
            const bool deferred = to > from + kCooDeferredFill;
            s_from[which] = deferred ? (from > i0 ? from : i0) : 0;
            s_to[which] = deferred ? (to < i1 ? to : i1) : 0;
            s_value[which] = t + base;
        }
    }
    __syncthreads();
    const int stretches = s_from[1] == s_from[0] && s_to[1] == s_to[0] ? 1 : 2;  // one stretch may hold both ends
    for (int k = 0; k < stretches; ++k) {
        const idx_t value = s_value[k];
        for (uint64_t i = s_from[k] + tid; i < s_to[k]; i += kBlock) row_ptr[i] = value;
    }
}

// ------------------------------------------------------------------------------------------
// device-wide exclusive scan of uint32 (in place), chunks of 4096
// ------------------------------------------------------------------------------------------
constexpr int kScanIpt = 16;
constexpr int kScanChunk = kBlock * kScanIpt;

__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* s_wave, uint32_t* total) {
    const unsigned lane = threadIdx.x % kWave;
    const unsigned wave = threadIdx.x / kWave;
    uint32_t inc = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const uint32_t up = __shfl_up(inc, off, kWave);
        if (lane >= static_cast<unsigned>(off)) inc += up;
    }
    if (lane == kWave - 1) s_wave[wave] = inc;
    __syncthreads();
    uint32_t wave_off = 0, all = 0;
#pragma unroll
    for (unsigned w = 0; w < kBlock / kWave; ++w) {
        const uint32_t s = s_wave[w];
        if (w < wave) wave_off += s;
        all += s;
    }
    __syncthreads();  // s_wave may be reused by the caller
    *total = all;
    return wave_off + inc - v;
}

__global__ __launch_bounds__(kBlock) void scan_reduce_kernel(const uint32_t* __restrict__ data, uint64_t n,
                                                             uint32_t* __restrict__ chunk_sums) {
    __shared__ uint32_t s_wave[kBlock / kWave];
    const uint64_t start = static_cast<uint64_t>(blockIdx.x) * kScanChunk;
    // loads without a test of their own (clamped index), so that they are all on their way at once
    uint32_t got[kScanIpt];
#pragma unroll
    for (int i = 0; i < kScanIpt; ++i) {
        const uint64_t p = start + static_cast<uint64_t>(i) * kBlock + threadIdx.x;
        got[i] = data[p < n ? p : n - 1];  // n != 0: the grid has no workgroup otherwise
    }
    uint32_t v = 0;
#pragma unroll
    for (int i = 0; i < kScanIpt; ++i) {
        const uint64_t p = start + static_cast<uint64_t>(i) * kBlock + threadIdx.x;
        v += p < n ? got[i] : 0u;
    }
    uint32_t total;
    block_exclusive_scan(v, s_wave, &total);
    if (threadIdx.x == 0) chunk_sums[blockIdx.x] = total;
}

// chunk_offsets == nullptr: single chunk starting at 0.
__global__ __launch_bounds__(kBlock) void scan_chunks_kernel(uint32_t* __restrict__ data, uint64_t n,
                                                             const uint32_t* __restrict__ chunk_offsets) {
    __shared__ uint32_t s_wave[kBlock / kWave];
    // thread owns kScanIpt consecutive elements so that its local prefix is sequential
    const uint64_t start = static_cast<uint64_t>(blockIdx.x) * kScanChunk + static_cast<uint64_t>(threadIdx.x) * kScanIpt;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    // whole runs of an aligned array move as 128-bit loads and stores
    const bool whole = (reinterpret_cast<uintptr_t>(data) & 15u) == 0 && start + kScanIpt <= n;
    uint32_t v[kScanIpt];
    uint32_t sum = 0;
    if (whole) {
#pragma unroll
        for (int q = 0; q < kScanIpt / 4; ++q) {
            const u32x4 four = *reinterpret_cast<const u32x4*>(data + start + 4 * q);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[4 * q + e] = four[e];
        }
    } else {
#pragma unroll
        for (int i = 0; i < kScanIpt; ++i) v[i] = start + i < n ? data[start + i] : 0;
    }
#pragma unroll
    for (int i = 0; i < kScanIpt; ++i) sum += v[i];
    uint32_t total;
    uint32_t off = block_exclusive_scan(sum, s_wave, &total);
    if (chunk_offsets != nullptr) off += chunk_offsets[blockIdx.x];
    if (whole) {
#pragma unroll
        for (int q = 0; q < kScanIpt / 4; ++q) {
            u32x4 four;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                four[e] = off;
                off += v[4 * q + e];
            }
            *reinterpret_cast<u32x4*>(data + start + 4 * q) = four;
        }
    } else {
#pragma unroll
        for (int i = 0; i < kScanIpt; ++i) {
            if (start + i < n) data[start + i] = off;
            off += v[i];
        }
    }
}

size_t scan_workspace_elems(uint64_t n) {
    size_t elems = 0;
    while (n > kScanChunk) {
        n = (n + kScanChunk - 1) / kScanChunk;
        elems += align_up(n * sizeof(uint32_t)) / sizeof(uint32_t);
    }
    return elems;
}

void launch_exclusive_scan(hipStream_t stream, uint32_t* data, uint64_t n, uint32_t* workspace) {
    if (n == 0) return;
    if (n <= kScanChunk) {
        hipLaunchKernelGGL(scan_chunks_kernel, dim3(1), dim3(kBlock), 0, stream, data, n,
                           static_cast<const uint32_t*>(nullptr));
        return;
    }
    const uint64_t chunks = (n + kScanChunk - 1) / kScanChunk;
    uint32_t* sums = workspace;
    uint32_t* next_ws = workspace + align_up(chunks * sizeof(uint32_t)) / sizeof(uint32_t);
    hipLaunchKernelGGL(scan_reduce_kernel, dim3(static_cast<uint32_t>(chunks)), dim3(kBlock), 0, stream, data, n, sums);
    launch_exclusive_scan(stream, sums, chunks, next_ws);
    hipLaunchKernelGGL(scan_chunks_kernel, dim3(static_cast<uint32_t>(chunks)), dim3(kBlock), 0, stream, data, n,
                       static_cast<const uint32_t*>(sums));
}

// ------------------------------------------------------------------------------------------
// one stable LSD radix pass over (key, row, value) triples
// ------------------------------------------------------------------------------------------
constexpr int kSortBlock = 1024;                       // threads per tile: many waves hide the barriers
constexpr int kSortIpt = 4;
constexpr int kSortTile = kSortBlock * kSortIpt;       // 4096 triples per workgroup
constexpr int kSortWaves = kSortBlock / kWave;         // 16
constexpr int kSortWaveItems = kWave * kSortIpt;       // each wave owns 256 consecutive triples
constexpr int kMaxRadix = 256;
static_assert(kSortBlock >= kMaxRadix, "one thread per digit");

// counters[digit * tiles + tile] = how many keys of `tile` carry `digit` (the digit of key - bias).  256 threads, 16 keys
// each, read as four 128-bit loads (tiles start at multiples of 4096 keys, so they are aligned).
constexpr int kHistBlock = 256;
__global__ __launch_bounds__(kHistBlock) void radix_hist_kernel(const idx_t* __restrict__ keys, idx_t count,
                                                                uint32_t shift, uint32_t bits, uint32_t tiles,
                                                                uint32_t* __restrict__ counters, idx_t bias,
                                                                uint32_t xcds) {
    typedef idx_t idx4 __attribute__((ext_vector_type(4)));
    __shared__ uint32_t s_cnt[kMaxRadix];
    const uint32_t radix = 1u << bits;
    const uint32_t mask = radix - 1;
    // The same tile order as the scatter kernel below: an XCD counts a contiguous range of tiles,
    // so the sixteen neighbouring tiles whose counters share a cache line write it in one L2.
    const uint32_t tiles_per_xcd = (tiles + xcds - 1) / xcds;
    const uint32_t tile = (blockIdx.x % xcds) * tiles_per_xcd + blockIdx.x / xcds;
    if (tile >= tiles) return;  // whole workgroup
    s_cnt[threadIdx.x] = 0;
    __syncthreads();
    const uint64_t start = static_cast<uint64_t>(tile) * kSortTile;
    // tiles start at multiples of 4096 keys, so a 16-byte aligned array allows 128-bit loads; the keys
    // of the first pass are the caller's own array, which may start anywhere
    const bool wide = (reinterpret_cast<uintptr_t>(keys) & 15u) == 0;
    const uint32_t lane = lane_id();
#pragma unroll
    for (int i = 0; i < kSortTile / (kHistBlock * 4); ++i) {
        const uint64_t p = start + (static_cast<uint64_t>(i) * kHistBlock + threadIdx.x) * 4;
        const bool full = wide && p + 4 <= count;
        idx4 k = {0, 0, 0, 0};
        if (full) k = __builtin_nontemporal_load(reinterpret_cast<const idx4*>(keys + p));
        uint32_t d[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) d[e] = ((k[e] - bias) >> shift) & mask;
        // Keys that are sorted inside long rows carry the same high digit many times in a row, and LDS
        // takes the adds of a wavefront to one counter one after the other.  A lane whose four keys
        // share a digit joins the lanes before it that hold the same one: the first lane of such a run
        // adds for all of them.
        const bool uni = full && d[0] == d[1] && d[1] == d[2] && d[2] == d[3];
        const uint32_t before = __shfl_up(uni ? d[0] : ~0u, 1, kWave);  // ~0u is no digit
        const bool head = lane == 0 || !uni || before != d[0];
        const uint64_t heads = __ballot(head);
        if (head) {
            if (uni) {
                const uint64_t later = lane == kWave - 1 ? 0 : heads >> (lane + 1);
                const uint32_t run = later != 0 ? static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(later)))
                                                : kWave - lane;
                atomicAdd(&s_cnt[d[0]], 4u * run);
            } else if (full) {
#pragma unroll
                for (int e = 0; e < 4; ++e) atomicAdd(&s_cnt[d[e]], 1u);
            } else {
                const uint64_t stop = p + 4 < count ? p + 4 : count;
                for (uint64_t q = p; q < stop; ++q) atomicAdd(&s_cnt[((keys[q] - bias) >> shift) & mask], 1u);
            }
        }
    }
    __syncthreads();
    if (threadIdx.x < radix) counters[static_cast<uint64_t>(threadIdx.x) * tiles + tile] = s_cnt[threadIdx.x];
}

// Exclusive scan of one value per digit, held by the first kMaxRadix threads of the scatter
// kernel; the other wavefronts only take part in the barrier.
__device__ __forceinline__ uint32_t digit_exclusive_scan(uint32_t v, uint32_t* s_wave) {
    constexpr unsigned kDigitWaves = kMaxRadix / kWave;
    const unsigned lane = threadIdx.x % kWave;
    const unsigned wave = threadIdx.x / kWave;
    uint32_t inc = 0;
    if (wave < kDigitWaves) {
        inc = wave_inclusive_sum(v);
        if (lane == kWave - 1) s_wave[wave] = inc;
    }
    __syncthreads();
    uint32_t wave_off = 0;
#pragma unroll
    for (unsigned w = 0; w + 1 < kDigitWaves; ++w) {
        if (w < wave) wave_off += s_wave[w];
    }
    return wave_off + inc - v;
}

// VB = bytes per value (0 = no values).  counters hold, after the exclusive scan, the output
// position of the first key of each (digit, tile).  FROM_CSR: the triples are the nonzeros of a
// CSR matrix in place -- rows_in is its row_ptr array (m + 1 offsets, index base `base`) and the
// row of every nonzero (+ base) is worked out here instead of being read.
template <int VB>
struct ValueOf { typedef uint32_t type; };
template <>
struct ValueOf<8> { typedef uint64_t type; };

// AUX = false: (key, value) pairs, rows_out is not written.  TIMES_X (with FROM_CSR, without AUX): the
// value that travels is value * x[row of the nonzero], in the floating-point type of VB bytes.
// short_keys (TIMES_X only, shift <= 16): keys_out is an array of uint16_t that receives the bits of key - bias below
// `shift`.  bias is subtracted from a key wherever a digit is taken from it (the index base, where that saves a bit).
template <int VB>
struct RealOf { typedef float type; };
template <>
struct RealOf<8> { typedef double type; };

template <int VB, bool FROM_CSR, bool AUX, bool TIMES_X>
__global__ __launch_bounds__(kSortBlock) void radix_scatter_kernel(
    const idx_t* __restrict__ keys_in, const idx_t* __restrict__ rows_in, const void* __restrict__ vals_in_v,
    idx_t* __restrict__ keys_out, idx_t* __restrict__ rows_out, void* __restrict__ vals_out_v, idx_t count,
    uint32_t shift, uint32_t bits, uint32_t tiles, const uint32_t* __restrict__ counters,
    const idx_t* __restrict__ tile_rows, idx_t base, const void* __restrict__ x_v, bool short_keys, idx_t bias,
    uint32_t xcds) {
    static_assert(AUX || VB != 0, "pairs carry a value");
    static_assert(!TIMES_X || (FROM_CSR && !AUX), "products are formed where the rows are worked out");
    typedef typename ValueOf<VB>::type val_t;
    const val_t* vals_in = static_cast<const val_t*>(vals_in_v);
    val_t* vals_out = static_cast<val_t*>(vals_out_v);

    __shared__ uint32_t s_cnt[kSortWaves][kMaxRadix];  // per-wave digit counts, then wave offsets
    __shared__ uint32_t s_start[kMaxRadix];            // first sorted slot of each digit in the tile
    __shared__ uint32_t s_dest[kMaxRadix];             // global position of that slot
    __shared__ uint32_t s_wave[kSortWaves];
    __shared__ idx_t s_keys[kSortTile];
    __shared__ idx_t s_rows[(AUX || FROM_CSR) ? kSortTile : 1];
    __shared__ val_t s_vals[VB ? kSortTile : 1];
    // FROM_CSR: one bit per nonzero of the tile that begins a row, how many rows begin before each 64 of
    // them, and whether two rows begin at the same nonzero (an empty row)
    __shared__ unsigned long long s_begins[FROM_CSR ? kSortTile / kWave : 1];
    __shared__ uint32_t s_begins_before[FROM_CSR ? kSortTile / kWave : 1];
    __shared__ uint32_t s_empty_rows;

    const uint32_t tid = threadIdx.x;
    const unsigned lane = tid % kWave;
    const unsigned wave = tid / kWave;
    const uint32_t radix = 1u << bits;
    const uint32_t mask = radix - 1;
    // Workgroups are handed to the device's XCDs in turn.  Tile t+1 appends to the digit runs tile t
    // started, so each XCD walks a contiguous range of tiles: the partial cache lines at the run
    // ends then meet in one L2 and leave as full lines.
    const uint32_t tiles_per_xcd = (tiles + xcds - 1) / xcds;
    const uint32_t tile = (blockIdx.x % xcds) * tiles_per_xcd + blockIdx.x / xcds;
    if (tile >= tiles) return;  // whole workgroup
    const uint64_t tile_start = static_cast<uint64_t>(tile) * kSortTile;
    const uint32_t tile_count =
        static_cast<uint32_t>(count - tile_start < kSortTile ? count - tile_start : kSortTile);

    for (uint32_t i = tid; i < kSortWaves * kMaxRadix; i += kSortBlock) (&s_cnt[0][0])[i] = 0;
    if constexpr (FROM_CSR) {
        if (tid < kSortTile / kWave) s_begins[tid] = 0;
        if (tid == 0) s_empty_rows = 0;
    }
    __syncthreads();

    // FROM_CSR: the row starts that fall inside the tile, relative to it, go to LDS (s_rows is
    // free until the tile is sorted); the row of a nonzero is the row of the tile's first nonzero
    // plus the number of starts at or before it.  They are asked for here and parked in LDS after
    // the ranking below, which covers their latency.
    idx_t first_row = 0, inside = 0, tile_first = 0;
    const idx_t* starts_in = nullptr;
    bool staged = false;
    idx_t start_of[kSortIpt];
    if constexpr (FROM_CSR) {
        const idx_t before = tile_rows[tile];  // row starts at or before the tile's first nonzero
        first_row = before - 1;
        inside = tile_rows[tile + 1] - before;
        starts_in = rows_in + before;
        tile_first = static_cast<idx_t>(tile_start) + base;
        staged = inside <= static_cast<idx_t>(kSortTile);
    }

    // Position inside the tile of this thread's i-th triple: waves own consecutive slabs, lanes
    // are interleaved inside a slab, so (wave, i, lane) order is input order.
    idx_t key[kSortIpt], row[kSortIpt];
    val_t val[kSortIpt];
    uint32_t rank[kSortIpt];
    const uint64_t lanemask_lt = (1ull << lane) - 1ull;
#pragma unroll
    for (int i = 0; i < kSortIpt; ++i) {
        const uint32_t p = wave * kSortWaveItems + i * kWave + lane;
        const bool live = p < tile_count;
        key[i] = live ? load_stream(keys_in + tile_start + p) : 0;
        if constexpr (!FROM_CSR && AUX) row[i] = live ? load_stream(rows_in + tile_start + p) : 0;
        if constexpr (VB != 0) val[i] = live ? load_stream(vals_in + tile_start + p) : val_t(0);
    }
    if constexpr (FROM_CSR) {
#pragma unroll
        for (int i = 0; i < kSortIpt; ++i) {
            const idx_t j = i * kSortBlock + tid;
            start_of[i] = staged && j < inside ? starts_in[j] : 0;
        }
    }
#pragma unroll
    for (int i = 0; i < kSortIpt; ++i) {
        const uint32_t p = wave * kSortWaveItems + i * kWave + lane;
        const bool live = p < tile_count;
        const uint32_t d = ((key[i] - bias) >> shift) & mask;
        // lanes of this wave holding the same digit in this round: per bit of the digit, keep the
        // lanes that voted as this lane did (vote xor own bit, spread over the word, is 0 there)
        uint64_t peers = __ballot(live);
#pragma unroll
        for (uint32_t b = 0; b < 8; ++b) {
            if (b < bits) {
                const uint32_t own = static_cast<uint32_t>(static_cast<int32_t>(d << (31 - b)) >> 31);  // bit b, spread
                const uint64_t vote = __ballot(own != 0);
                peers &= ~(vote ^ ((static_cast<uint64_t>(own) << 32) | own));
            }
        }
        rank[i] = 0;
        if (live) {
            // The counter is shared by the lanes of this wave across rounds: every peer reads it,
            // then the lowest peer alone adds the round's count.  LDS operations of one wave
            // complete in program order; the relaxed atomics keep the compiler from reordering or
            // merging them and keep them LDS instructions.
            uint32_t* counter = &s_cnt[wave][d];
            const uint32_t before = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
            rank[i] = before + __popcll(peers & lanemask_lt);
            if ((peers & lanemask_lt) == 0) {
                __hip_atomic_store(counter, before + __popcll(peers), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
            }
        }
    }
    if constexpr (FROM_CSR) {
#pragma unroll
        for (int i = 0; i < kSortIpt; ++i) {
            const idx_t j = i * kSortBlock + tid;
            if (staged && j < inside) {
                const idx_t at = start_of[i] - tile_first;
                s_rows[j] = at;
                if (at < static_cast<idx_t>(kSortTile)) {  // the tile's last row may end where the next tile begins
                    const unsigned long long bit = 1ull << (at % kWave);
                    if ((atomicOr(&s_begins[at / kWave], bit) & bit) != 0) s_empty_rows = 1;
                }
            }
        }
    }
    __syncthreads();

    if constexpr (FROM_CSR) {
        // The row of a nonzero is the first row of the tile plus the rows that begin at or before it.  Without
        // empty rows that is a count of bits: the lanes of a wavefront hold 64 neighbouring nonzeros, one word
        // of s_begins, in every round.  Otherwise, a search per nonzero.
        const bool by_bits = staged && s_empty_rows == 0;  // the same for the whole workgroup
        if (by_bits) {
            static_assert(kSortWaveItems / kWave == kSortIpt && kSortTile / kWave == kWave, "a word per wavefront and round");
            if (wave == 0) {
                const uint32_t c = __popcll(s_begins[lane]);
                s_begins_before[lane] = wave_inclusive_sum(c) - c;
            }
            __syncthreads();
            const unsigned long long up_to_lane = (2ull << lane) - 1ull;  // lane 63: all ones
#pragma unroll
            for (int i = 0; i < kSortIpt; ++i) {
                const uint32_t word = wave * kSortIpt + i;
                row[i] = first_row + s_begins_before[word] + __popcll(s_begins[word] & up_to_lane) + base;
            }
        }
#pragma unroll
        for (int i = 0; i < kSortIpt; ++i) {
            if (by_bits) break;
            const uint32_t p = wave * kSortWaveItems + i * kWave + lane;
            idx_t lo = 0;
            idx_t hi = inside;
            if (staged) {
                while (lo < hi) {
                    const idx_t mid = (lo + hi) >> 1;
                    if (s_rows[mid] <= p) lo = mid + 1; else hi = mid;
                }
            } else {  // more than a tile's worth of (mostly empty) rows: search the offsets in place
                while (lo < hi) {
                    const idx_t mid = (lo + hi) >> 1;
                    if (starts_in[mid] - tile_first <= p) lo = mid + 1; else hi = mid;
                }
            }
            row[i] = first_row + lo + base;
        }
        if constexpr (TIMES_X) {
            typedef typename RealOf<VB>::type real_t;
            const real_t* x = static_cast<const real_t*>(x_v);
            real_t xr[kSortIpt];
#pragma unroll
            for (int i = 0; i < kSortIpt; ++i) {
                const uint32_t p = wave * kSortWaveItems + i * kWave + lane;
                xr[i] = x[p < tile_count ? row[i] - base : first_row];  // first_row: a row of the matrix
            }
#pragma unroll
            for (int i = 0; i < kSortIpt; ++i) {
                val[i] = __builtin_bit_cast(val_t, __builtin_bit_cast(real_t, val[i]) * xr[i]);
            }
        }
    }

    // per digit: turn the wave counts into wave offsets, then lay the digits out in order
    uint32_t digit_total = 0;
    if (tid < radix) {
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) {
            const uint32_t c = s_cnt[w][tid];
            s_cnt[w][tid] = digit_total;
            digit_total += c;
        }
    }
    const uint32_t digit_start = digit_exclusive_scan(digit_total, s_wave);
    if (tid < radix) {
        s_start[tid] = digit_start;
        s_dest[tid] = counters[static_cast<uint64_t>(tid) * tiles + tile];
    }
    __syncthreads();

#pragma unroll
    for (int i = 0; i < kSortIpt; ++i) {
        const uint32_t p = wave * kSortWaveItems + i * kWave + lane;
        if (p < tile_count) {
            const uint32_t d = ((key[i] - bias) >> shift) & mask;
            const uint32_t slot = s_start[d] + s_cnt[wave][d] + rank[i];
            s_keys[slot] = key[i];
            if constexpr (AUX) s_rows[slot] = row[i];
            if constexpr (VB != 0) s_vals[slot] = val[i];
        }
    }
    __syncthreads();

    // sorted tile -> global: neighbouring threads write neighbouring addresses inside a digit run
#pragma unroll
    for (int i = 0; i < kSortIpt; ++i) {
        const uint32_t slot = i * kSortBlock + tid;
        if (slot < tile_count) {
            const idx_t k = s_keys[slot];
            const uint32_t d = ((k - bias) >> shift) & mask;
            const uint64_t out = static_cast<uint64_t>(s_dest[d]) + (slot - s_start[d]);
            if constexpr (TIMES_X) {
                // short_keys: the last pass of a sort on the top bits keeps only what lies below them, in 16 bits
                if (short_keys) reinterpret_cast<uint16_t*>(keys_out)[out] = static_cast<uint16_t>((k - bias) & ((1u << shift) - 1u));
                else keys_out[out] = k;
            } else {
                keys_out[out] = k;
            }
            if constexpr (AUX) rows_out[out] = s_rows[slot];
            if constexpr (VB != 0) vals_out[out] = s_vals[slot];
        }
    }
}

// tile_rows[t] = number of rows that start at or before the first nonzero of sort tile t
// (t = tiles: all m + 1 offsets).  One wavefront per entry.
__global__ __launch_bounds__(kBlock) void tile_row_starts_kernel(const idx_t* __restrict__ row_ptr, idx_t m, idx_t base,
                                                                 idx_t nnz, uint32_t tiles, idx_t* __restrict__ tile_rows) {
    const uint32_t t = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (t > tiles) return;  // whole wavefront
    const uint64_t first = static_cast<uint64_t>(t) * kSortTile;
    const idx_t starts = wave_count_row_starts(row_ptr, m, base, first < nnz ? static_cast<idx_t>(first) : nnz);
    if (threadIdx.x % kWave == 0) tile_rows[t] = starts;
}

uint32_t sort_tiles(idx_t nnz) { return static_cast<uint32_t>((static_cast<uint64_t>(nnz) + kSortTile - 1) / kSortTile); }

size_t sort_counter_elems(idx_t count) { return static_cast<size_t>(kMaxRadix) * sort_tiles(count); }

// Temporaries of one sort: two sets of (keys, aux, values) that the passes alternate between,
// the per-(digit, tile) counters and the scratch of their scan.
struct SortScratch {
    idx_t* keys[2];
    idx_t* aux[2];
    void* vals[2];
    uint32_t* counters;
    uint32_t* scan_ws;
    idx_t* tile_rows = nullptr;  // sort_tiles(count) + 1 entries, only for sorts that read a CSR matrix in place
};

template <int VB>
void launch_scatter(hipStream_t stream, bool from_csr, uint32_t grid, const idx_t* keys_in, const idx_t* aux_in,
                    const void* vals_in, idx_t* keys_out, idx_t* aux_out, void* vals_out, idx_t count, uint32_t shift,
                    uint32_t bits, uint32_t tiles, const uint32_t* counters, const idx_t* tile_rows, idx_t base,
                    bool pairs, const void* x, bool short_keys, idx_t bias, uint32_t xcds) {
    const void* none = nullptr;
    if constexpr (VB != 0) {
        if (pairs && from_csr) {
            hipLaunchKernelGGL((radix_scatter_kernel<VB, true, false, true>), dim3(grid), dim3(kSortBlock), 0, stream, keys_in,
                               aux_in, vals_in, keys_out, aux_out, vals_out, count, shift, bits, tiles, counters, tile_rows,
                               base, x, short_keys, bias, xcds);
            return;
        }
        if (pairs) {
            hipLaunchKernelGGL((radix_scatter_kernel<VB, false, false, false>), dim3(grid), dim3(kSortBlock), 0, stream, keys_in,
                               aux_in, vals_in, keys_out, aux_out, vals_out, count, shift, bits, tiles, counters, tile_rows,
                               base, none, false, bias, xcds);
            return;
        }
    }
    if (from_csr) {
        hipLaunchKernelGGL((radix_scatter_kernel<VB, true, true, false>), dim3(grid), dim3(kSortBlock), 0, stream, keys_in,
                           aux_in, vals_in, keys_out, aux_out, vals_out, count, shift, bits, tiles, counters, tile_rows, base,
                           none, false, bias, xcds);
    } else {
        hipLaunchKernelGGL((radix_scatter_kernel<VB, false, true, false>), dim3(grid), dim3(kSortBlock), 0, stream, keys_in,
                           aux_in, vals_in, keys_out, aux_out, vals_out, count, shift, bits, tiles, counters, tile_rows, base,
                           none, false, bias, xcds);
    }
}

// A sort whose triples are the nonzeros of a CSR matrix where they lie.
struct CsrSource {
    idx_t rows = 0;  // > 0: aux_in is the row_ptr of a CSR matrix with this many rows, and the first
                     // pass derives the aux of every triple, its row + base, from it
    idx_t base = 0;  // index base of row_ptr
    // != nullptr: no aux travels; the value of every triple is multiplied by x[its row] in the first
    // pass (x in the floating-point type of the values), and (key, product) pairs are sorted
    const void* times_x = nullptr;
    // lowest key bit the sort looks at: the keys are ordered by bits [first_bit, first_bit + key_bits)
    uint32_t first_bit = 0;
    // with times_x, in a sort of one pass: keys_out is an array of uint16_t that receives the key bits below
    // first_bit (<= 16 of them), which is all that tells the keys of one digit apart
    bool short_keys = false;
    // subtracted from every key before its digits are taken (the keys themselves travel unchanged)
    idx_t bias = 0;
};

// Stable LSD radix sort of (key, aux, value) triples on the low key_bits of the keys, in
// ceil(key_bits / 8) passes of equal width.  The last pass writes keys_out / aux_out / vals_out,
// which must not overlap the inputs.  value_bytes is 0 (no values), 4 or 8.
void radix_sort_triples(hipStream_t stream, idx_t count, uint32_t key_bits, const idx_t* keys_in, const idx_t* aux_in,
                        const void* vals_in, idx_t* keys_out, idx_t* aux_out, void* vals_out, size_t value_bytes,
                        const SortScratch& t, const CsrSource& csr = CsrSource()) {
    const uint32_t passes = key_bits == 0 ? 1 : (key_bits + 7) / 8;
    const uint32_t bits = key_bits == 0 ? 1 : (key_bits + passes - 1) / passes;
    const uint32_t radix = 1u << bits;
    const uint32_t tiles = sort_tiles(count);
    const uint32_t xcds = device_topology().xcds;
    const uint32_t scatter_grid = (tiles + xcds - 1) / xcds * xcds;
    uint32_t shift = csr.first_bit;
    if (csr.rows > 0) {
        const uint32_t waves_per_block = kBlock / kWave;
        hipLaunchKernelGGL(tile_row_starts_kernel, dim3((tiles + 1 + waves_per_block - 1) / waves_per_block), dim3(kBlock),
                           0, stream, aux_in, csr.rows, csr.base, count, tiles, t.tile_rows);
    }
    for (uint32_t p = 0; p < passes; ++p) {
        const bool last = p + 1 == passes;
        const bool from_csr = p == 0 && csr.rows > 0;
        idx_t* k_out = last ? keys_out : t.keys[p & 1];
        idx_t* a_out = last ? aux_out : t.aux[p & 1];
        void* v_out = last ? vals_out : t.vals[p & 1];
        hipLaunchKernelGGL(radix_hist_kernel, dim3(scatter_grid), dim3(kHistBlock), 0, stream, keys_in, count, shift, bits,
                           tiles, t.counters, csr.bias, xcds);
        launch_exclusive_scan(stream, t.counters, static_cast<uint64_t>(radix) * tiles, t.scan_ws);
        auto* launch = value_bytes == 0 ? launch_scatter<0> : value_bytes == 4 ? launch_scatter<4> : launch_scatter<8>;
        launch(stream, from_csr, scatter_grid, keys_in, aux_in, vals_in, k_out, a_out, v_out, count, shift, bits, tiles,
               t.counters, t.tile_rows, csr.base, csr.times_x != nullptr, csr.times_x,
               csr.short_keys && last && from_csr, csr.bias, xcds);
        keys_in = k_out;
        aux_in = a_out;
        vals_in = v_out;
        shift += bits;
    }
}

struct Csr2CscLayout {
    size_t sorted_keys, keys_a, rows_a, vals_a, keys_b, rows_b, vals_b, counters, scan_ws, tile_rows, total;
};

// pairs: no row arrays (the sort of a transposing SpMV, which carries no rows)
Csr2CscLayout csr2csc_layout(idx_t nnz, size_t value_bytes, bool pairs = false) {
    Csr2CscLayout l;
    const size_t idx_bytes = align_up(static_cast<size_t>(nnz) * sizeof(idx_t));
    const size_t row_bytes = pairs ? 0 : idx_bytes;
    const size_t val_bytes = align_up(static_cast<size_t>(nnz) * value_bytes);
    const size_t counter_elems = sort_counter_elems(nnz);
    size_t off = 0;
    l.sorted_keys = off; off += idx_bytes;
    l.keys_a = off; off += idx_bytes;
    l.rows_a = off; off += row_bytes;
    l.vals_a = off; off += val_bytes;
    l.keys_b = off; off += idx_bytes;
    l.rows_b = off; off += row_bytes;
    l.vals_b = off; off += val_bytes;
    l.counters = off; off += align_up(counter_elems * sizeof(uint32_t));
    l.scan_ws = off; off += align_up(scan_workspace_elems(counter_elems) * sizeof(uint32_t)) + kAlign;
    l.tile_rows = off; off += align_up((static_cast<size_t>(sort_tiles(nnz)) + 1) * sizeof(idx_t));
    l.total = off;
    return l;
}

// Scratch of the index sorts: three sets of (keys, aux, permutation) -- the two the passes
// alternate between and the result of the minor-key sort -- plus one spare index array.
struct IndexSortLayout {
    size_t set[3][3];
    size_t spare, counters, scan_ws, total;
};

IndexSortLayout index_sort_layout(idx_t nnz) {
    IndexSortLayout l;
    const size_t idx_bytes = align_up(static_cast<size_t>(nnz) * sizeof(idx_t));
    const size_t counter_elems = sort_counter_elems(nnz);
    size_t off = 0;
    for (int s = 0; s < 3; ++s) {
        for (int a = 0; a < 3; ++a) {
            l.set[s][a] = off;
            off += idx_bytes;
        }
    }
    l.spare = off; off += idx_bytes;
    l.counters = off; off += align_up(counter_elems * sizeof(uint32_t));
    l.scan_ws = off; off += align_up(scan_workspace_elems(counter_elems) * sizeof(uint32_t)) + kAlign;
    l.total = off;
    return l;
}

// Sorts (major, minor, perm) triples by (major, minor): a stable sort on the minor key followed
// by a stable sort on the major key.  Outputs may be the input arrays themselves: both sorts
// write to arrays their own inputs do not overlap.  perm_in == nullptr sorts without a payload.
void sort_by_two_keys(hipStream_t stream, idx_t nnz, uint32_t major_bits, uint32_t minor_bits, const idx_t* major_in,
                      const idx_t* minor_in, const idx_t* perm_in, idx_t* major_out, idx_t* minor_out, idx_t* perm_out,
                      char* w, const IndexSortLayout& l) {
    SortScratch t;
    for (int s = 0; s < 2; ++s) {
        t.keys[s] = reinterpret_cast<idx_t*>(w + l.set[s][0]);
        t.aux[s] = reinterpret_cast<idx_t*>(w + l.set[s][1]);
        t.vals[s] = w + l.set[s][2];
    }
    t.counters = reinterpret_cast<uint32_t*>(w + l.counters);
    t.scan_ws = reinterpret_cast<uint32_t*>(w + l.scan_ws);
    idx_t* mid_minor = reinterpret_cast<idx_t*>(w + l.set[2][0]);
    idx_t* mid_major = reinterpret_cast<idx_t*>(w + l.set[2][1]);
    idx_t* mid_perm = reinterpret_cast<idx_t*>(w + l.set[2][2]);
    const size_t vb = perm_in != nullptr ? sizeof(idx_t) : 0;
    radix_sort_triples(stream, nnz, minor_bits, minor_in, major_in, perm_in, mid_minor, mid_major, mid_perm, vb, t);
    radix_sort_triples(stream, nnz, major_bits, mid_major, mid_minor, mid_perm, major_out, minor_out, perm_out, vb, t);
}

__global__ __launch_bounds__(kBlock) void identity_kernel(idx_t n, idx_t* __restrict__ p) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < static_cast<uint64_t>(n)) p[i] = static_cast<idx_t>(i);
}

// Eight elements per thread, the indices first, then the eight gathers, then the stores: a thread has
// eight gathers in flight, as the SpMV kernels have, so what this kernel takes is what the gathers cost.
constexpr int kGatherPerThread = 8;
template <typename T>
__global__ __launch_bounds__(kBlock) void gather_kernel(idx_t nnz, const T* __restrict__ y, T* __restrict__ x_val,
                                                        const idx_t* __restrict__ x_ind, idx_t base) {
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * (kBlock * kGatherPerThread) + threadIdx.x;
    const uint64_t last = static_cast<uint64_t>(nnz) - 1;  // nnz != 0: the grid has no workgroup otherwise
    idx_t ind[kGatherPerThread];
    T got[kGatherPerThread];
#pragma unroll
    for (int k = 0; k < kGatherPerThread; ++k) {
        const uint64_t i = first + static_cast<uint64_t>(k) * kBlock;
        ind[k] = load_stream(x_ind + (i < last ? i : last));
    }
#pragma unroll
    for (int k = 0; k < kGatherPerThread; ++k) got[k] = y[ind[k] - base];
#pragma unroll
    for (int k = 0; k < kGatherPerThread; ++k) {
        const uint64_t i = first + static_cast<uint64_t>(k) * kBlock;
        if (i <= last) x_val[i] = got[k];
    }
}

}  // namespace

void launch_csr2coo(hipStream_t stream, idx_t m, idx_t nnz, const idx_t* row_ptr, idx_t base, idx_t* coo_rows) {
    if (nnz == 0) return;
    const uint64_t per_group = static_cast<uint64_t>(kExpandTiles) * kCooTile;
    const uint32_t groups = static_cast<uint32_t>((static_cast<uint64_t>(nnz) + per_group - 1) / per_group);
    hipLaunchKernelGGL(csr2coo_kernel, dim3(groups), dim3(kCooBlock), 0, stream, m, nnz, base, row_ptr, coo_rows);
}

void launch_coo2csr(hipStream_t stream, idx_t nnz, idx_t m, const idx_t* coo_rows, idx_t base, idx_t* row_ptr) {
    const uint64_t threads = (static_cast<uint64_t>(nnz) + kCooPerThread) / kCooPerThread;  // boundaries 0 .. nnz
    const uint64_t per_block = static_cast<uint64_t>(kBlock) * kCooVectors;
    const dim3 grid(static_cast<uint32_t>((threads + per_block - 1) / per_block));
    if (reinterpret_cast<uintptr_t>(coo_rows) % 16 == 0) {
        hipLaunchKernelGGL(coo2csr_kernel<true>, grid, dim3(kBlock), 0, stream, nnz, m, base, coo_rows, row_ptr);
    } else {
        hipLaunchKernelGGL(coo2csr_kernel<false>, grid, dim3(kBlock), 0, stream, nnz, m, base, coo_rows, row_ptr);
    }
    if (static_cast<uint64_t>(m) + 1 > kCooDeferredFill) {  // else no stretch is long enough to have been left out
        const uint64_t blocks = (static_cast<uint64_t>(m) + 1 + kCooFillRows - 1) / kCooFillRows;
        hipLaunchKernelGGL(coo2csr_fill_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0, stream, nnz, m, base,
                           coo_rows, row_ptr);
    }
}

size_t csr2csc_workspace_bytes(idx_t /*m*/, idx_t /*n*/, idx_t nnz, size_t value_bytes) {
    return csr2csc_layout(nnz, value_bytes).total;
}

size_t transposed_products_workspace_bytes(idx_t nnz, size_t value_bytes) {
    return csr2csc_layout(nnz, value_bytes, true).total;
}

// The nonzeros are sorted by column where they lie: the first pass reads col / val in place and
// works the row indices out of row_ptr; the sorted columns then give the offsets.
void launch_csr2csc(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, const void* csr_val, const idx_t* row_ptr,
                    const idx_t* col, void* csc_val, idx_t* row_ind, idx_t* col_ptr, size_t value_bytes, idx_t base,
                    void* workspace) {
    if (m == 0 || n == 0 || nnz == 0) return;
    const Csr2CscLayout l = csr2csc_layout(nnz, value_bytes);
    char* w = static_cast<char*>(workspace);
    idx_t* sorted_keys = reinterpret_cast<idx_t*>(w + l.sorted_keys);
    SortScratch t;
    t.keys[0] = reinterpret_cast<idx_t*>(w + l.keys_a);
    t.keys[1] = reinterpret_cast<idx_t*>(w + l.keys_b);
    t.aux[0] = reinterpret_cast<idx_t*>(w + l.rows_a);
    t.aux[1] = reinterpret_cast<idx_t*>(w + l.rows_b);
    t.vals[0] = w + l.vals_a;
    t.vals[1] = w + l.vals_b;
    t.counters = reinterpret_cast<uint32_t*>(w + l.counters);
    t.scan_ws = reinterpret_cast<uint32_t*>(w + l.scan_ws);
    t.tile_rows = reinterpret_cast<idx_t*>(w + l.tile_rows);
    CsrSource csr;
    csr.rows = m;
    csr.base = base;
    // keys are the raw column indices (index base included); the digits are taken from key - base, so that a
    // one-based matrix with 2^16 or 2^24 columns does not pay a pass for the one key that needs another bit
    csr.bias = base;
    radix_sort_triples(stream, nnz, bit_length(n - 1), col, row_ptr, csr_val, sorted_keys, row_ind, csc_val, value_bytes,
                       t, csr);
    launch_coo2csr(stream, nnz, n, sorted_keys, base, col_ptr);
}

// What a transposing SpMV needs of A^T: the products value * x[row] of all nonzeros in the order of a
// stable sort by column, and the column offsets.  (column, product) pairs are sorted instead of
// (column, row, value) triples, so the later passes move 8 or 12 bytes per nonzero instead of 12 or
// 16, and the sums over the columns then need no gather from x.
// workspace: transposed_products_workspace_bytes.
void launch_transposed_products(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, const void* csr_val, const idx_t* row_ptr,
                                const idx_t* col, const void* x, void* products, idx_t* col_ptr, size_t value_bytes,
                                idx_t base, void* workspace) {
    if (m == 0 || n == 0 || nnz == 0) return;
    const Csr2CscLayout l = csr2csc_layout(nnz, value_bytes, true);
    char* w = static_cast<char*>(workspace);
    idx_t* sorted_keys = reinterpret_cast<idx_t*>(w + l.sorted_keys);
    SortScratch t;
    t.keys[0] = reinterpret_cast<idx_t*>(w + l.keys_a);
    t.keys[1] = reinterpret_cast<idx_t*>(w + l.keys_b);
    t.aux[0] = t.aux[1] = nullptr;
    t.vals[0] = w + l.vals_a;
    t.vals[1] = w + l.vals_b;
    t.counters = reinterpret_cast<uint32_t*>(w + l.counters);
    t.scan_ws = reinterpret_cast<uint32_t*>(w + l.scan_ws);
    t.tile_rows = reinterpret_cast<idx_t*>(w + l.tile_rows);
    CsrSource csr;
    csr.rows = m;
    csr.base = base;
    csr.times_x = x;
    csr.bias = base;  // as in launch_csr2csc
    radix_sort_triples(stream, nnz, bit_length(n - 1), col, row_ptr, csr_val, sorted_keys, nullptr, products, value_bytes,
                       t, csr);
    launch_coo2csr(stream, nnz, n, sorted_keys, base, col_ptr);
}

bool bucketed_products_shape(idx_t n, uint32_t* shift) {
    const uint32_t bits = bit_length(n - 1);  // of the columns without their index base
    // fewer keys than that: the full sort is two short passes; more: a bucket's sums no longer fit in LDS
    if (bits < kBucketMinKeyBits || bits > 8 + kBucketMaxShift) return false;
    *shift = bits - 8;
    return true;
}

// One pass of the same sort, for a transposing SpMV that may add the products of a column in any order:
// (column, value * x[row]) pairs ordered by the top eight bits of the columns (index base taken off) only, that is
// in up to 256 buckets of 2^shift neighbouring columns, inside a bucket in CSR order.  The sums over a bucket's
// columns then fit in LDS.  Of a key only its place in the bucket is written, as 16 bits: a quarter fewer
// bytes for this pass to write and the sums to read.  workspace as for launch_transposed_products.
void launch_bucketed_products(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, const void* csr_val, const idx_t* row_ptr,
                              const idx_t* col, const void* x, void* products, size_t value_bytes, idx_t base,
                              void* workspace, BucketedProducts* out) {
    uint32_t shift = 0;
    if (m == 0 || nnz == 0 || !bucketed_products_shape(n, &shift)) return;
    const Csr2CscLayout l = csr2csc_layout(nnz, value_bytes, true);
    char* w = static_cast<char*>(workspace);
    idx_t* keys = reinterpret_cast<idx_t*>(w + l.sorted_keys);  // room for 32-bit keys, used for 16-bit ones
    SortScratch t;  // one pass writes the outputs directly: no alternating sets
    t.keys[0] = t.keys[1] = nullptr;
    t.aux[0] = t.aux[1] = nullptr;
    t.vals[0] = t.vals[1] = nullptr;
    t.counters = reinterpret_cast<uint32_t*>(w + l.counters);
    t.scan_ws = reinterpret_cast<uint32_t*>(w + l.scan_ws);
    t.tile_rows = reinterpret_cast<idx_t*>(w + l.tile_rows);
    CsrSource csr;
    csr.rows = m;
    csr.base = base;
    csr.times_x = x;
    csr.first_bit = shift;
    csr.short_keys = true;
    csr.bias = base;
    radix_sort_triples(stream, nnz, 8, col, row_ptr, csr_val, keys, nullptr, products, value_bytes, t, csr);
    out->keys = reinterpret_cast<const uint16_t*>(keys);
    out->starts = t.counters;  // after the scan, counters[digit * tiles] is where the digit's keys begin
    out->stride = sort_tiles(nnz);
    out->shift = shift;
    out->buckets = static_cast<uint32_t>((n - 1) >> shift) + 1;
    out->spare = w + l.keys_a;  // the sets the passes of a full sort alternate between
    out->spare_bytes = l.counters - l.keys_a;
}

// Scratch of launch_sort_by_column_band: the counters of one pass, their scan, the row starts per tile.
namespace {
struct BandSortLayout {
    size_t counters, scan_ws, tile_rows, total;
};
BandSortLayout band_sort_layout(idx_t nnz) {
    BandSortLayout l;
    const size_t counter_elems = sort_counter_elems(nnz);
    size_t off = 0;
    l.counters = off; off += align_up(counter_elems * sizeof(uint32_t));
    l.scan_ws = off; off += align_up(scan_workspace_elems(counter_elems) * sizeof(uint32_t)) + kAlign;
    l.tile_rows = off; off += align_up((static_cast<size_t>(sort_tiles(nnz)) + 1) * sizeof(idx_t));
    l.total = off;
    return l;
}
}  // namespace

size_t band_sort_workspace_bytes(idx_t nnz) { return band_sort_layout(nnz).total; }

void launch_sort_by_column_band(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, const idx_t* row_ptr, const idx_t* col,
                                const void* val, size_t value_bytes, uint32_t band_shift, uint32_t band_bits,
                                idx_t* cols_out, idx_t* rows_out, void* vals_out, void* workspace) {
    if (m == 0 || nnz == 0) return;
    const BandSortLayout l = band_sort_layout(nnz);
    char* w = static_cast<char*>(workspace);
    SortScratch t;  // one pass writes the outputs directly: no alternating sets
    t.keys[0] = t.keys[1] = nullptr;
    t.aux[0] = t.aux[1] = nullptr;
    t.vals[0] = t.vals[1] = nullptr;
    t.counters = reinterpret_cast<uint32_t*>(w + l.counters);
    t.scan_ws = reinterpret_cast<uint32_t*>(w + l.scan_ws);
    t.tile_rows = reinterpret_cast<idx_t*>(w + l.tile_rows);
    CsrSource csr;
    csr.rows = m;
    csr.base = base;
    csr.first_bit = band_shift;
    radix_sort_triples(stream, nnz, band_bits > 8 ? 8 : band_bits, col, row_ptr, val, cols_out, rows_out, vals_out,
                       value_bytes, t, csr);
}

namespace {
// The two sets of arrays the passes of a sort alternate between, the counters and their scan, carved
// out of a workspace of csr2csc_workspace_bytes.
SortScratch sort_scratch_in(char* w, const Csr2CscLayout& l) {
    SortScratch t;
    t.keys[0] = reinterpret_cast<idx_t*>(w + l.keys_a);
    t.keys[1] = reinterpret_cast<idx_t*>(w + l.keys_b);
    t.aux[0] = reinterpret_cast<idx_t*>(w + l.rows_a);
    t.aux[1] = reinterpret_cast<idx_t*>(w + l.rows_b);
    t.vals[0] = w + l.vals_a;
    t.vals[1] = w + l.vals_b;
    t.counters = reinterpret_cast<uint32_t*>(w + l.counters);
    t.scan_ws = reinterpret_cast<uint32_t*>(w + l.scan_ws);
    t.tile_rows = reinterpret_cast<idx_t*>(w + l.tile_rows);
    return t;
}
}  // namespace

// The nonzeros of a CSR matrix in the order of a stable sort by column, as (column, row, value)
// arrays with the index base left in: csr2csc without the offsets.  low_bits > 0 leaves that many low
// bits of the column keys out of the sort: columns that differ only there stay in CSR order.
// workspace: csr2csc_workspace_bytes.
void launch_sort_by_column(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, idx_t base, const idx_t* row_ptr,
                           const idx_t* col, const void* val, size_t value_bytes, uint32_t low_bits, idx_t* cols_out,
                           idx_t* rows_out, void* vals_out, void* workspace) {
    if (m == 0 || n == 0 || nnz == 0) return;
    const SortScratch t = sort_scratch_in(static_cast<char*>(workspace), csr2csc_layout(nnz, value_bytes));
    CsrSource csr;
    csr.rows = m;
    csr.base = base;
    csr.first_bit = low_bits;
    const uint32_t bits = bit_length(n - 1 + base);
    radix_sort_triples(stream, nnz, bits > low_bits ? bits - low_bits : 0, col, row_ptr, val, cols_out, rows_out,
                       vals_out, value_bytes, t, csr);
}

// Stable sort of (key, aux, value) triples on the low key_bits (at most 16) of the keys.  The outputs
// must not overlap the inputs or the workspace (csr2csc_workspace_bytes).
void launch_sort_triples(hipStream_t stream, idx_t nnz, uint32_t key_bits, const idx_t* keys_in, const idx_t* aux_in,
                         const void* vals_in, idx_t* keys_out, idx_t* aux_out, void* vals_out, size_t value_bytes,
                         void* workspace) {
    if (nnz == 0) return;
    const SortScratch t = sort_scratch_in(static_cast<char*>(workspace), csr2csc_layout(nnz, value_bytes));
    radix_sort_triples(stream, nnz, key_bits, keys_in, aux_in, vals_in, keys_out, aux_out, vals_out, value_bytes, t);
}

size_t index_sort_workspace_bytes(idx_t nnz) { return index_sort_layout(nnz).total; }

void launch_coosort(hipStream_t stream, idx_t major_extent, idx_t minor_extent, idx_t nnz, idx_t* major, idx_t* minor,
                    idx_t* perm, void* workspace) {
    if (nnz == 0) return;
    // indices may be zero- or one-based: keys reach the extent itself in the second case
    sort_by_two_keys(stream, nnz, bit_length(major_extent), bit_length(minor_extent), major, minor, perm, major, minor,
                     perm, static_cast<char*>(workspace), index_sort_layout(nnz));
}

void launch_csrsort(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, idx_t base, const idx_t* row_ptr, idx_t* col,
                    idx_t* perm, void* workspace) {
    if (m == 0 || n == 0 || nnz == 0) return;
    const IndexSortLayout l = index_sort_layout(nnz);
    char* w = static_cast<char*>(workspace);
    idx_t* rows = reinterpret_cast<idx_t*>(w + l.spare);  // row of every entry, then the sorted rows
    launch_csr2coo(stream, m, nnz, row_ptr, base, rows);
    sort_by_two_keys(stream, nnz, bit_length(m - 1 + base), bit_length(n - 1 + base), rows, col, perm, rows, col, perm,
                     w, l);
}

void launch_identity(hipStream_t stream, idx_t n, idx_t* p) {
    if (n == 0) return;
    hipLaunchKernelGGL(identity_kernel, dim3((static_cast<uint32_t>(n) + kBlock - 1) / kBlock), dim3(kBlock), 0, stream,
                       n, p);
}

template <typename T>
void launch_gather(hipStream_t stream, idx_t nnz, const T* y, T* x_val, const idx_t* x_ind, idx_t base) {
    if (nnz == 0) return;
    constexpr uint32_t per_block = kBlock * kGatherPerThread;
    hipLaunchKernelGGL((gather_kernel<T>), dim3((static_cast<uint32_t>(nnz) + per_block - 1) / per_block), dim3(kBlock),
                       0, stream, nnz, y, x_val, x_ind, base);
}

namespace {
__global__ __launch_bounds__(kBlock) void narrow_indices_kernel(const int64_t* __restrict__ src, idx_t* __restrict__ dst,
                                                                uint64_t n) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < n) dst[i] = static_cast<idx_t>(load_stream(src + i));
}
}  // namespace

void launch_narrow_indices(hipStream_t stream, const int64_t* src, idx_t* dst, uint64_t n) {
    if (n == 0) return;
    hipLaunchKernelGGL(narrow_indices_kernel, dim3(static_cast<uint32_t>((n + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       stream, src, dst, n);
}

size_t exclusive_scan_workspace_bytes(uint64_t n) {
    return align_up(scan_workspace_elems(n) * sizeof(uint32_t)) + kAlign;
}

void launch_exclusive_scan_u32(hipStream_t stream, uint32_t* data, uint64_t n, void* workspace) {
    launch_exclusive_scan(stream, data, n, static_cast<uint32_t*>(workspace));
}

template void launch_gather<float>(hipStream_t, idx_t, const float*, float*, const idx_t*, idx_t);
template void launch_gather<double>(hipStream_t, idx_t, const double*, double*, const idx_t*, idx_t);

}  // namespace mcsp
