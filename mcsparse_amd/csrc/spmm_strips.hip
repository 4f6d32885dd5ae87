// CSR SpMM from a schedule of diagonal blocks over groups of row strips, for matrices in which rows a fixed
// distance apart hold the same diagonals shifted by that distance (structured grids: the rows of neighbouring
// grid lines).
//
// The reference's kernel (src/kernels/level3/spmm/csr_spmm_device.hpp:121-137) walks a row's nonzeros once per
// output column.  The block schedule of spmm_blocks.hip shares a loaded row of op(B) between the neighbouring rows
// of one group of eight; here a group is kSpmmStrips strips of kSpmmStripRows consecutive rows, strip q beginning
// `stride` rows behind strip q - 1 (a grid line further on).  Row i of any strip that holds column c + i + p lies on
// diagonal p of block c, so the strips that reach the same rows of op(B) through different diagonals of the matrix
// (line l through its offset +stride, line l + 1 through offset 0, line l + 2 through -stride) share one block: its
// kSpmmStripRows + n - 1 rows of op(B) are loaded once for all of them.  On a 27-point stencil a row of A costs 6.75
// loaded rows of op(B) instead of 11.25 with groups of eight consecutive rows and 27 without sharing.
//
// A block is sixteen bytes: {int32 c, uint32 n | j_first << 4 | j_last << 8, uint32 held_lo, uint32 held_hi}; bit
// 3 * r + p of the 48 bits held_hi:held_lo says that row r of the group (strip r / kSpmmStripRows, row r %
// kSpmmStripRows of it) holds diagonal p, i.e. column c + r % kSpmmStripRows + p; j_first .. j_last are the rows of
// op(B), counted from c, that the held diagonals need.  The blocks of a group consume every row's nonzeros in
// storage order, and the values are read from the CSR array on every call.
#include "spmm_device.h"

namespace mcsp {

namespace {

using namespace spmm_detail;

constexpr int H = kSpmmStripRows;
constexpr int Q = kSpmmStrips;
constexpr int R = H * Q;  // rows of a group
constexpr int D = kSpmmBlockMaxDiagonals;
constexpr int kRowsOfB = H + D - 1;
constexpr int kLanes = 16;  // lanes per group: one per row where the values are fetched
constexpr int kNoKey = 0x7fffffff;
static_assert(R == kLanes && H == 4 && D == 3, "a lane per row; quads of lanes are strips; three bits per row");

struct StripCounters {
    unsigned long long span_sum;  // sum over the groups of (last column - first column)
    unsigned long long loads;     // rows of op(B) all blocks load together
    unsigned int longest_strip;   // most nonzeros in one strip of a group that has blocks
    unsigned int reserved;        // keeps `stride` at byte 24, where readers of the buffer look for it
    unsigned int stride;          // rows between the strips of a group
};

struct StripPartial {
    unsigned long long span, loads;
    unsigned int longest, padding;
};

__global__ void zero_strip_counters_kernel(StripCounters* c, uint32_t stride) {
    c->span_sum = 0;
    c->loads = 0;
    c->longest_strip = 0;
    c->reserved = 0;
    c->stride = stride;
}

__device__ __forceinline__ uint64_t first_row_of_group(uint64_t group, uint32_t stride) {
    const uint64_t per_tile = stride / H;  // groups in a stretch of Q * stride rows
    return group / per_tile * (static_cast<uint64_t>(Q) * stride) + group % per_tile * H;
}

// v of another lane of the same row of 16 lanes, chosen by a DPP control (quad permutes and mirrors, as in group_sum).
template <int CTRL>
__device__ __forceinline__ int dpp_int(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}
// min / max / or over the sixteen lanes of a group; every lane ends with the result
template <typename F>
__device__ __forceinline__ int group16_reduce(int v, F f) {
    v = f(v, dpp_int<kDppQuadXor1>(v));
    v = f(v, dpp_int<kDppQuadXor2>(v));
    v = f(v, dpp_int<kDppRowHalfMirror>(v));
    v = f(v, dpp_int<kDppRowMirror>(v));
    return v;
}

// Sixteen lanes cover the nonzeros of one group with blocks, lane r walking row r of the group.  The rows are merged
// by the key column - (row inside its strip): rows of one strip on one diagonal of the matrix share a key, and so do
// rows of different strips that name the same rows of op(B).  A step takes the lowest key among the rows' next
// nonzeros; a block grows while that key follows the last one, up to D keys; which rows hold a key is recorded bit
// by bit, so any set of rows may.  Every row's nonzeros are consumed in storage order, whatever that order is: the
// values of a row inside a block are always the next ones it has not used yet.
constexpr int kCoverGroupsPerBlock = kBlock / kLanes;
constexpr int kColRoom = 136;  // entries of a strip's copy: 128 and the neighbours its first and last piece bring along
template <bool FILL>
__global__ __launch_bounds__(kBlock) void strip_cover_kernel(idx_t m, idx_t nnz, idx_t base, uint32_t stride,
                                                             const idx_t* __restrict__ row_ptr,
                                                             const idx_t* __restrict__ col,
                                                             uint32_t* __restrict__ block_ptr, uint4* __restrict__ blocks,
                                                             StripCounters* __restrict__ counters,
                                                             StripPartial* __restrict__ partials) {
    __shared__ __attribute__((aligned(16))) idx_t s_col[kCoverGroupsPerBlock * Q][kColRoom];
    const uint64_t groups = spmm_strip_groups(m, stride);
    const uint64_t group = static_cast<uint64_t>(blockIdx.x) * kCoverGroupsPerBlock + threadIdx.x / kLanes;
    const uint32_t lane = threadIdx.x % kLanes;
    // (lane groups behind the last group leave a zero for the scan, or nothing, and add nothing to the counters)
    const bool slot_exists = group <= groups;
    auto imin = [](int a, int b) { return a < b ? a : b; };
    auto imax = [](int a, int b) { return a > b ? a : b; };
    auto ior = [](int a, int b) { return a | b; };
    uint32_t count = 0;
    uint32_t loads = 0;
    int first_col = 0x7fffffff, last_col = -1;
    int longest_strip = 0;
    if (group < groups) {
        const uint64_t row = first_row_of_group(group, stride) + static_cast<uint64_t>(lane / H) * stride + lane % H;
        const bool exists = row < static_cast<uint64_t>(m);
        idx_t i = exists ? row_ptr[row] - base : 0;
        const idx_t e = exists ? row_ptr[row + 1] - base : 0;
        const int row_nnz = static_cast<int>(e - i);
        int strip_nnz = row_nnz + dpp_int<kDppQuadXor1>(row_nnz);
        strip_nnz += dpp_int<kDppQuadXor2>(strip_nnz);
        const int group_nnz = strip_nnz + dpp_int<kDppRowHalfMirror>(strip_nnz) +
                              dpp_int<kDppRowMirror>(strip_nnz + dpp_int<kDppRowHalfMirror>(strip_nnz));
        if (static_cast<idx_t>(group_nnz) <= kSpmmMaxMergedGroup) {
            longest_strip = group16_reduce(strip_nnz, imax);
            const uint32_t out = FILL ? block_ptr[group] : 0;
            // A strip's column indices are one contiguous stretch: its four lanes copy it into LDS in 16-byte pieces
            // first (read entry by entry while the merge goes on, the lines would be fetched again and again: the
            // many groups in flight push each other's out of L2).  Longer strips, or an unaligned array, are read in
            // place.
            const idx_t strip_begin = static_cast<idx_t>(dpp_int<0x00>(static_cast<int>(i)));   // the quad's first lane
            const idx_t strip_end = static_cast<idx_t>(dpp_int<0xFF>(static_cast<int>(e)));     // the quad's last lane
            const idx_t stage_first = strip_begin & ~idx_t(3);
            const bool staged = strip_end >= strip_begin && strip_end - stage_first <= static_cast<idx_t>(kColRoom) &&
                                reinterpret_cast<uintptr_t>(col) % 16 == 0;
            idx_t* mine_staged = s_col[(threadIdx.x / kLanes) * Q + lane / H];
            if (staged) {
                typedef idx_t Piece __attribute__((ext_vector_type(4)));
                const idx_t pieces = (strip_end - stage_first + 3) / 4;  // at most kColRoom / 4
                const idx_t whole_pieces = nnz / 4;                      // pieces that lie inside the array altogether
                for (idx_t piece = lane % H; piece < pieces; piece += H) {
                    const idx_t at = stage_first / 4 + piece;
                    if (at < whole_pieces) {
                        reinterpret_cast<Piece*>(mine_staged)[piece] = reinterpret_cast<const Piece*>(col)[at];
                    } else {  // the array's last entries, when they do not fill a piece
                        for (idx_t t = at * 4; t < nnz; ++t) mine_staged[t - stage_first] = col[t];
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            int start = 0;
            uint32_t width = 0;
            uint32_t mine = 0;  // bit p: this lane's row holds diagonal p of the block being grown
            auto flush = [&]() {
                if (width == 0) return;
                // the rows of op(B) the held diagonals need, and the 48 bits
                int j_lo = 0xff, j_hi = 0;
#pragma unroll
                for (int p = 0; p < D; ++p) {
                    if ((mine >> p) & 1u) {
                        j_lo = imin(j_lo, static_cast<int>(lane % H) + p);
                        j_hi = imax(j_hi, static_cast<int>(lane % H) + p);
                    }
                }
                const uint32_t j_first = static_cast<uint32_t>(group16_reduce(j_lo, imin));
                const uint32_t j_last = static_cast<uint32_t>(group16_reduce(j_hi, imax));
                const unsigned long long my_bits = static_cast<unsigned long long>(mine) << (3 * lane);
                const uint32_t held_lo = static_cast<uint32_t>(group16_reduce(static_cast<int>(static_cast<uint32_t>(my_bits)), ior));
                const uint32_t held_hi = static_cast<uint32_t>(group16_reduce(static_cast<int>(static_cast<uint32_t>(my_bits >> 32)), ior));
                if (FILL && lane == 0)
                    blocks[out + count] = make_uint4(static_cast<uint32_t>(start), width | (j_first << 4) | (j_last << 8), held_lo, held_hi);
                ++count;
                loads += j_last - j_first + 1;
                width = 0;
                mine = 0;
            };
            while (true) {
                int key = kNoKey;
                if (i < e) {
                    const int c = static_cast<int>((staged ? mine_staged[i - stage_first] : col[i]) - base);
                    key = c - static_cast<int>(lane % H);
                }
                const int low = group16_reduce(key, imin);
                if (low == kNoKey) break;  // the whole lane group
                if (!(width != 0 && width < static_cast<uint32_t>(D) && low == start + static_cast<int>(width))) {
                    flush();
                    start = low;
                }
                const uint32_t p = width++;
                if (key == low) {
                    mine |= 1u << p;
                    const int c = key + static_cast<int>(lane % H);
                    first_col = imin(first_col, c);
                    last_col = imax(last_col, c);
                    ++i;
                }
            }
            flush();
            first_col = group16_reduce(first_col, imin);
            last_col = group16_reduce(last_col, imax);
        }
    }
    if (!FILL) {
        if (lane == 0 && slot_exists) block_ptr[group] = count;  // slot `groups` receives the total after the scan
        // the four groups of a wavefront add to the counters together (every lane of a group holds the group's figures)
        unsigned long long span = count != 0 ? static_cast<unsigned long long>(last_col - first_col) : 0ull;
        unsigned long long all_loads = loads;
        int longest = count != 0 ? longest_strip : 0;
#pragma unroll
        for (int off = kLanes; off < kWave; off <<= 1) {
            span += __shfl_xor(span, off, kWave);
            all_loads += __shfl_xor(all_loads, off, kWave);
            longest = imax(longest, __shfl_xor(longest, off, kWave));
        }
        // and the wavefronts of the workgroup: adds of all workgroups to the three counters would queue on one line
        // (a millisecond for 2 M rows), so every workgroup leaves its figures in a slot of its own where there is room
        __shared__ StripPartial s_part[kBlock / kWave];
        if (lane_id() == 0) s_part[threadIdx.x / kWave] = {span, all_loads, static_cast<unsigned int>(longest), 0u};
        __syncthreads();
        if (threadIdx.x == 0) {
            StripPartial sum = s_part[0];
#pragma unroll
            for (int w = 1; w < kBlock / kWave; ++w) {
                sum.span += s_part[w].span;
                sum.loads += s_part[w].loads;
                sum.longest = sum.longest > s_part[w].longest ? sum.longest : s_part[w].longest;
            }
            if (partials != nullptr) {
                partials[blockIdx.x] = sum;
            } else {
                if (sum.span != 0) atomicAdd(&counters->span_sum, sum.span);
                if (sum.loads != 0) atomicAdd(&counters->loads, sum.loads);
                if (sum.longest != 0) atomicMax(&counters->longest_strip, sum.longest);
            }
        }
    }
}

// The figures the workgroups of the count pass left, added up into the counters (one workgroup, no atomics).
__global__ __launch_bounds__(kBlock) void strip_counters_sum_kernel(const StripPartial* __restrict__ partials, uint32_t count,
                                                                    StripCounters* __restrict__ counters) {
    __shared__ StripPartial s_part[kBlock / kWave];
    StripPartial sum = {0ull, 0ull, 0u, 0u};
    for (uint32_t i = threadIdx.x; i < count; i += kBlock) {
        const StripPartial p = partials[i];
        sum.span += p.span;
        sum.loads += p.loads;
        sum.longest = sum.longest > p.longest ? sum.longest : p.longest;
    }
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        sum.span += __shfl_xor(sum.span, off, kWave);
        sum.loads += __shfl_xor(sum.loads, off, kWave);
        const unsigned int other = static_cast<unsigned int>(__shfl_xor(static_cast<int>(sum.longest), off, kWave));
        sum.longest = sum.longest > other ? sum.longest : other;
    }
    if (lane_id() == 0) s_part[threadIdx.x / kWave] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kBlock / kWave; ++w) {
            sum.span += s_part[w].span;
            sum.loads += s_part[w].loads;
            sum.longest = sum.longest > s_part[w].longest ? sum.longest : s_part[w].longest;
        }
        counters->span_sum = sum.span;
        counters->loads = sum.loads;
        counters->longest_strip = sum.longest;
    }
}

// The four lane groups of a wavefront walk their block lists in lockstep, so the groups are handed out in an order
// in which neighbours hold equal lists: inside every stretch of kOrderChunk consecutive groups, sorted (stably) by a
// hash of their blocks' shapes.  Any permutation gives the right product.
constexpr uint32_t kOrderChunk = 1024;
__global__ __launch_bounds__(kOrderChunk) void strip_order_kernel(uint64_t groups, const uint32_t* __restrict__ block_ptr,
                                                                  const uint4* __restrict__ blocks,
                                                                  uint32_t* __restrict__ order) {
    __shared__ uint32_t keys[kOrderChunk];
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * kOrderChunk;
    const uint64_t group = first + threadIdx.x;
    uint32_t hash = 0x3fffffu;  // groups past the end sort last
    if (group < groups) {
        hash = 2166136261u;
        for (uint32_t s = block_ptr[group]; s < block_ptr[group + 1]; ++s) {
            const uint4 d = blocks[s];
            hash = (hash ^ d.y) * 16777619u;
            hash = (hash ^ d.z) * 16777619u;
            hash = (hash ^ d.w) * 16777619u;
        }
        hash = (hash ^ (hash >> 15)) & 0x3ffffeu;
    }
    keys[threadIdx.x] = (hash << 10) | threadIdx.x;
    __syncthreads();
    for (uint32_t size = 2; size <= kOrderChunk; size <<= 1) {
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            const uint32_t partner = threadIdx.x ^ stride;
            if (partner > threadIdx.x) {
                const uint32_t a = keys[threadIdx.x], b = keys[partner];
                const bool ascending = (threadIdx.x & size) == 0;
                if ((a > b) == ascending) {
                    keys[threadIdx.x] = b;
                    keys[partner] = a;
                }
            }
            __syncthreads();
        }
    }
    if (group < groups) order[group] = static_cast<uint32_t>(first) + (keys[threadIdx.x] & (kOrderChunk - 1));
}

// Values a strip may hold for its copy in LDS to be used, and the room of a copy (the 16-byte pieces a copy is made
// of bring along up to a piece's worth of neighbours at either end).
template <typename T>
constexpr int strip_capacity() { return static_cast<int>(kSpmmStripStagedValues); }  // 512 bytes of fp32, 1024 of fp64 (a 27-point stencil's strip: 108 values)
template <typename T>
constexpr int strip_room() { return strip_capacity<T>() + 2 * (16 / static_cast<int>(sizeof(T))); }

// 16 lanes per group, V = 16 B / sizeof(T) adjacent columns of C per lane; blockIdx.y walks panels of 16 * V columns.
// Lane l of a group looks after row l of the group where values are concerned: it knows where the row's next unused
// value lies and fetches the (at most D) values the row has in a block; they reach the multiply-adds as DPP row
// broadcasts.  STAGED: no strip holds more than strip_capacity<T>() nonzeros and the value array is 16-byte aligned;
// the four lanes of a strip then copy its values into LDS once, in whole 16-byte pieces, and the blocks read them
// there.
// A workgroup is one wavefront (four groups): a wavefront that is through makes room for the next at once instead of
// waiting for the others of its workgroup (256 threads: 360 us at N = 64 on the 128^3 stencil, 128 or 64: 349 us).
constexpr int kStripBlock = kWave;
template <typename T, bool WIDE, bool STAGED>
__global__ __launch_bounds__(kStripBlock, 3) void spmm_strips_kernel(idx_t m, idx_t n, idx_t base, uint32_t stride,
                                                             const idx_t* __restrict__ row_ptr,
                                                             const idx_t* __restrict__ col, const T* __restrict__ val,
                                                             const uint32_t* __restrict__ block_ptr,
                                                             const uint4* __restrict__ blocks,
                                                             const uint32_t* __restrict__ order, const T* __restrict__ B,
                                                             int64_t ldb, T* __restrict__ C, int64_t ldc,
                                                             bool c_row_major, T alpha, T beta, uint32_t xcd_chunk,
                                                             uint32_t xcds, idx_t k, idx_t nnz, uint32_t total_blocks) {
    typedef typename ByteOffset<WIDE>::type off_t;
    constexpr int V = 16 / sizeof(T);
    constexpr int kGroupsPerBlock = kStripBlock / kLanes;
    const idx_t lane = threadIdx.x % kLanes;
    const uint64_t turn = xcd_position(blockIdx.x, xcd_chunk, xcds) * kGroupsPerBlock + threadIdx.x / kLanes;
    const uint64_t groups = spmm_strip_groups(m, stride);
    if (turn >= groups) return;  // whole lane groups
    // which group takes this turn (held to the groups that exist, whatever the buffer holds)
    const uint64_t group = min(static_cast<uint64_t>(order[turn]), groups - 1);
    const uint64_t g0 = first_row_of_group(group, stride);
    const uint64_t c_own = (static_cast<uint64_t>(blockIdx.y) * kLanes + lane) * V;
    const bool stores = c_own < static_cast<uint64_t>(n);  // lanes past the last column only help fetching
    const uint64_t c0 = stores ? c_own : 0;

    T acc[R][V];
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int c = 0; c < V; ++c) acc[r][c] = T(0);
    }
    const char* B_bytes = reinterpret_cast<const char*>(B);
    const off_t lane_off = static_cast<off_t>(c0 * sizeof(T));
    const off_t ldb_bytes = static_cast<off_t>(ldb * sizeof(T));

    // this lane's row of the group: where its nonzeros begin and end (a row past the matrix's end holds none)
    const uint64_t my_row = g0 + static_cast<uint64_t>(lane / H) * stride + lane % H;
    const uint64_t row_at = my_row < static_cast<uint64_t>(m) ? my_row : static_cast<uint64_t>(m);
    const idx_t row_begin = row_ptr[row_at] - base;
    const idx_t row_end = (my_row < static_cast<uint64_t>(m) ? row_ptr[row_at + 1] : row_ptr[row_at]) - base;
    // its strip's nonzeros: from the first row's begin to the last row's end (DPP inside the quad of lanes)
    const idx_t strip_begin = static_cast<idx_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(row_begin), 0x00, 0xF, 0xF, true));
    const idx_t strip_end = static_cast<idx_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(row_end), 0xFF, 0xF, 0xF, true));
    const idx_t strip_nnz = strip_end >= strip_begin ? strip_end - strip_begin : 0;
    const idx_t group_nnz = group_bcast<kLanes, 0>(strip_nnz) + group_bcast<kLanes, H>(strip_nnz) +
                            group_bcast<kLanes, 2 * H>(strip_nnz) + group_bcast<kLanes, 3 * H>(strip_nnz);

    if (group_nnz <= kSpmmMaxMergedGroup) {
        // The schedule lives in the caller's buffer.  Whatever it holds, nothing is read outside the arrays: list
        // bounds are held to the list, a block whose rows of op(B) do not all exist counts as a block that holds
        // nothing, value positions are held to the copy in LDS or to the nonzeros.
        const uint32_t s_end = min(block_ptr[group + 1], total_blocks);
        const uint32_t s_begin = min(block_ptr[group], s_end);
        const idx_t last_value = nnz - 1;  // nnz != 0: total_blocks != 0
        const uint32_t last_block = total_blocks - 1;
        idx_t pos = row_begin;  // where the next unused value of this lane's row lies

        constexpr int kRoom = strip_room<T>();
        constexpr int E = 16 / sizeof(T);  // values per 16-byte piece
        __shared__ __attribute__((aligned(16))) T s_val[STAGED ? kGroupsPerBlock * Q : 1][STAGED ? kRoom : 1];
        T* staged = s_val[STAGED ? (threadIdx.x / kLanes) * Q + lane / H : 0];
        const idx_t stage_first = strip_begin & ~static_cast<idx_t>(E - 1);  // the piece the strip's first value lies in
        if constexpr (STAGED) {
            typedef T Piece __attribute__((ext_vector_type(E)));
            constexpr int kPieces = kRoom / E;              // pieces a copy has room for
            constexpr int kRounds = (kPieces + H - 1) / H;  // pieces a lane copies
            // the strip's pieces (at most kPieces: the launcher has checked the longest strip)
            const idx_t pieces = min(static_cast<idx_t>((strip_end - stage_first + E - 1) / E), static_cast<idx_t>(kPieces));
            const idx_t whole_pieces = nnz / E;  // pieces that lie inside the array altogether
            const idx_t first_piece = stage_first / E;
            auto copy_rounds = [&](int from, int to) {
                // all loads of a call on their way together, each held to a piece that exists; pieces past the strip's
                // end are copies of its last one and land on it
                Piece got[kRounds];
#pragma unroll
                for (int c = from; c < to; ++c) {
                    const idx_t piece = min(static_cast<idx_t>(c * H + lane % H), pieces != 0 ? pieces - 1 : 0);
                    const idx_t at = min(first_piece + piece, whole_pieces != 0 ? whole_pieces - 1 : 0);
                    got[c] = reinterpret_cast<const Piece*>(val)[at];
                }
#pragma unroll
                for (int c = from; c < to; ++c) {
                    const idx_t piece = min(static_cast<idx_t>(c * H + lane % H), pieces != 0 ? pieces - 1 : 0);
                    reinterpret_cast<Piece*>(staged)[piece] = got[c];
                }
            };
            copy_rounds(0, kRounds / 2);
            if (pieces > static_cast<idx_t>(kRounds / 2 * H)) copy_rounds(kRounds / 2, kRounds);
            // the array's last values, when they do not fill a piece, one by one (nothing is read past the end)
            if (strip_end > whole_pieces * E) {
                const idx_t at = max(whole_pieces * E, strip_begin) + lane % H;
                if (at < strip_end && at - stage_first < static_cast<idx_t>(kRoom)) staged[at - stage_first] = val[at];
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }

        // Everything a block needs is asked for while the block before it is being worked on: its descriptor two
        // blocks ahead, its values and its rows of op(B) one block ahead, into a second set of registers.  None of
        // these loads sits under a test: a block past the end of the list, or one that is not sound, turns into a
        // block that holds nothing and whose loads go to places that exist.
        struct Shape {
            int cbase;
            uint32_t held_lo, held_hi;  // bit 3 * r + p: row r of the group holds diagonal p
            uint32_t j_first, j_last;   // rows of op(B) the block needs, counted from cbase
            uint32_t mine;              // the three bits of this lane's row
        };
        auto decode = [&](uint4 d, bool exists) {
            Shape sh;
            sh.cbase = static_cast<int>(d.x);
            const uint32_t width = d.y & 15u;
            sh.j_first = (d.y >> 4) & 15u;
            sh.j_last = (d.y >> 8) & 15u;
            // diagonals past the block's width are held by nobody: 001, 011 or 111 for every row
            const uint32_t keep_lo = width >= 3 ? 0xffffffffu : width == 2 ? 0xdb6db6dbu : 0x49249249u;
            const uint32_t keep_hi = width >= 3 ? 0x0000ffffu : width == 2 ? 0x00006db6u : 0x00002492u;
            sh.held_lo = d.z & keep_lo;
            sh.held_hi = d.w & keep_hi;
            // (every extent is below 2^31 here, so the sums cannot wrap)
            const bool sound = exists && width - 1u < static_cast<uint32_t>(D) && sh.j_first <= sh.j_last &&
                               sh.j_last < static_cast<uint32_t>(kRowsOfB) && sh.cbase + static_cast<int>(sh.j_first) >= 0 &&
                               sh.cbase + static_cast<int>(sh.j_last) <= static_cast<int>(k) - 1;
            if (!sound) {
                sh.cbase = 0;
                sh.held_lo = sh.held_hi = 0;
                sh.j_first = sh.j_last = 0;
            }
            const unsigned long long held = (static_cast<unsigned long long>(sh.held_hi) << 32) | sh.held_lo;
            sh.mine = static_cast<uint32_t>(held >> (3 * lane)) & 7u;
            return sh;
        };
        struct Operands {
            T v[D];  // this lane's row: its value of diagonal p (anything where it holds none)
            Vec<T, V> b[kRowsOfB];
        };
        auto fetch = [&](const Shape& sh, idx_t at_value, Operands& o) {
            // the row's next three values; the one of diagonal p is its (held diagonals below p)-th
            T next[D];
            if constexpr (STAGED) {
                const idx_t at = at_value - stage_first;  // a place past the copy (an overwritten schedule) is held inside it
#pragma unroll
                for (int t = 0; t < D; ++t) next[t] = staged[min(at + t, static_cast<idx_t>(kRoom - 1))];
            } else {
#pragma unroll
                for (int t = 0; t < D; ++t) next[t] = val[min(at_value + t, last_value)];
            }
            o.v[0] = next[0];
            o.v[1] = (sh.mine & 1u) ? next[1] : next[0];
            const uint32_t below = __popc(sh.mine & 3u);
            o.v[2] = below == 2 ? next[2] : below == 1 ? next[1] : next[0];
            // rows j_first .. j_last of the block are needed; the others are asked for at the nearest needed one
            const off_t roff = static_cast<off_t>(static_cast<int64_t>(sh.cbase)) * ldb_bytes + lane_off;
            static_for<kRowsOfB>([&](auto jc) {
                constexpr uint32_t j = decltype(jc)::value;
                const uint32_t jj = min(max(j, sh.j_first), sh.j_last);
                o.b[j] = load_vec<T, V>(reinterpret_cast<const T*>(B_bytes + (roff + static_cast<off_t>(jj) * ldb_bytes)));
            });
        };
        auto consume = [&](const Shape& sh, const Operands& o) {
            static_for<Q>([&](auto qc) {
                constexpr int q = decltype(qc)::value;
                // the twelve bits of strip q (the same for the lanes of the group)
                const uint32_t bits = q == 0 ? sh.held_lo & 0xfffu
                                             : q == 1 ? (sh.held_lo >> 12) & 0xfffu
                                                      : q == 2 ? ((sh.held_lo >> 24) | (sh.held_hi << 8)) & 0xfffu
                                                               : (sh.held_hi >> 4) & 0xfffu;
                if (bits == 0xfffu) {
                    // every row of the strip holds every diagonal: the multiply-adds follow in the order the rows of
                    // op(B) arrive
                    static_for<kRowsOfB>([&](auto jc) {
                        constexpr int j = decltype(jc)::value;
                        static_for<D>([&](auto pc) {
                            constexpr int p = decltype(pc)::value;
                            constexpr int i = j - p;
                            if constexpr (i >= 0 && i < H) {
                                const T a = group_bcast<kLanes, q * H + i>(o.v[p]);
#pragma unroll
                                for (int c = 0; c < V; ++c) acc[q * H + i][c] += a * o.b[j].v[c];
                            }
                        });
                    });
                } else if (bits != 0) {
                    // the tests sit around the multiply-adds, so that a row only ever sees the rows of op(B) it names
                    static_for<kRowsOfB>([&](auto jc) {
                        constexpr int j = decltype(jc)::value;
                        static_for<D>([&](auto pc) {
                            constexpr int p = decltype(pc)::value;
                            constexpr int i = j - p;
                            if constexpr (i >= 0 && i < H) {
                                if ((bits >> (3 * i + p)) & 1u) {
                                    const T a = group_bcast<kLanes, q * H + i>(o.v[p]);
#pragma unroll
                                    for (int c = 0; c < V; ++c) acc[q * H + i][c] += a * o.b[j].v[c];
                                }
                            }
                        });
                    });
                }
            });
        };
        auto advance = [&](const Shape& sh) -> idx_t { return static_cast<idx_t>(__popc(sh.mine)); };
        auto descriptor = [&](uint32_t s) { return blocks[min(s, last_block)]; };

        Operands even, odd;
        uint4 d_next = descriptor(s_begin + 1);
        Shape now = decode(descriptor(s_begin), s_begin < s_end);
        fetch(now, pos, even);
        uint32_t s = s_begin;
        for (; s + 2 < s_end; s += 2) {
            // block s is in `even`; s + 1 goes to `odd` while s is worked on, s + 2 to `even` while s + 1 is
            const uint4 d_after = descriptor(s + 2);
            const Shape next = decode(d_next, true);
            pos += advance(now);
            fetch(next, pos, odd);
            consume(now, even);
            const uint4 d_after2 = descriptor(s + 3);
            const Shape after = decode(d_after, true);
            pos += advance(next);
            fetch(after, pos, even);
            consume(next, odd);
            now = after;
            d_next = d_after2;
        }
        // the last block, or the last two
        if (s + 1 < s_end) {
            const Shape next = decode(d_next, true);
            pos += advance(now);
            fetch(next, pos, odd);
            consume(now, even);
            consume(next, odd);
        } else {
            consume(now, even);  // holds nothing when the list is empty
        }
    } else {
        // a group too long to be worth covering: one row after the other
        static_for<R>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            const idx_t b = group_bcast<kLanes, r>(row_begin);
            const idx_t e = group_bcast<kLanes, r>(row_end);
            row_times_b<T, kLanes, V, WIDE>(b, e, lane, base, col, val, B_bytes, lane_off, ldb_bytes, acc[r]);
        });
    }

    if (!stores) return;
    // A column-major C holds the rows of a strip next to each other in every column: 16 or 32 bytes.
    const bool whole_columns = !c_row_major && ((reinterpret_cast<uintptr_t>(C) | static_cast<uintptr_t>(ldc * sizeof(T))) & 15u) == 0;
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const uint64_t strip_row = g0 + static_cast<uint64_t>(q) * stride;  // a multiple of H
        if (whole_columns && strip_row + H <= static_cast<uint64_t>(m)) {
#pragma unroll
            for (int c = 0; c < V; ++c)
                store_c_four_rows<T>(C + static_cast<int64_t>(c0 + c) * ldc + strip_row, acc[q * H][c], acc[q * H + 1][c],
                                     acc[q * H + 2][c], acc[q * H + 3][c], alpha, beta);
        } else {
#pragma unroll
            for (int h = 0; h < H; ++h) {
                if (strip_row + h < static_cast<uint64_t>(m))
                    store_c<T, V>(C, ldc, c_row_major, strip_row + h, c0, acc[q * H + h], alpha, beta);
            }
        }
    }
}

// The strip schedule inside the region spmm_schedule_layout describes: the offsets where the merged lists keep
// theirs, the blocks from the start of the entries' place, the order of the groups at its end.
struct Carved {
    uint32_t* block_ptr;
    StripCounters* counters;
    uint4* blocks;
    uint32_t* order;
    char* scan_ws;
};
Carved carve(idx_t m, idx_t nnz, uint32_t stride, void* schedule) {
    const SpmmScheduleLayout l = spmm_schedule_layout(m, nnz);
    char* w = static_cast<char*>(schedule);
    const size_t order_bytes = spmm_strip_groups(m, stride) * sizeof(uint32_t);
    const size_t entries_bytes = static_cast<size_t>(nnz) * sizeof(uint32_t);
    const size_t order_at = entries_bytes >= order_bytes ? (entries_bytes - order_bytes) / 16 * 16 : 0;
    return {reinterpret_cast<uint32_t*>(w + l.group_ptr), reinterpret_cast<StripCounters*>(w + l.span_sum),
            reinterpret_cast<uint4*>(w + l.entries), reinterpret_cast<uint32_t*>(w + l.entries + order_at), w + l.scan_ws};
}

}  // namespace

bool spmm_strip_stride_usable(idx_t m, uint32_t stride) {
    // whole strips per stretch, more than one group per stretch, and no more offsets than the region has slots for
    return stride >= 2 * H && stride % H == 0 && static_cast<uint64_t>(stride) * 8 <= static_cast<uint64_t>(m) &&
           spmm_strip_groups(m, stride) + 1 <= spmm_groups(m) + 1;
}

void launch_spmm_strip_count(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, uint32_t stride, const idx_t* row_ptr,
                             const idx_t* col, void* schedule) {
    const Carved c = carve(m, nnz, stride, schedule);
    const uint64_t slots = spmm_strip_groups(m, stride) + 1;
    const dim3 grid(static_cast<uint32_t>((slots + kCoverGroupsPerBlock - 1) / kCoverGroupsPerBlock));
    hipLaunchKernelGGL(zero_strip_counters_kernel, dim3(1), dim3(1), 0, stream, c.counters, stride);
    // the place of the blocks, not yet written, takes the workgroups' figures when it has room for them
    StripPartial* partials = static_cast<uint64_t>(grid.x) * sizeof(StripPartial) <= static_cast<uint64_t>(nnz) * sizeof(uint32_t)
                                 ? reinterpret_cast<StripPartial*>(c.blocks) : nullptr;
    hipLaunchKernelGGL((strip_cover_kernel<false>), grid, dim3(kBlock), 0, stream, m, nnz, base, stride, row_ptr, col, c.block_ptr,
                       c.blocks, c.counters, partials);
    if (partials != nullptr)
        hipLaunchKernelGGL(strip_counters_sum_kernel, dim3(1), dim3(kBlock), 0, stream, partials, grid.x, c.counters);
    launch_exclusive_scan_u32(stream, c.block_ptr, slots, c.scan_ws);
}

void launch_spmm_strip_fill(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, uint32_t stride, const idx_t* row_ptr,
                            const idx_t* col, void* schedule) {
    const Carved c = carve(m, nnz, stride, schedule);
    const uint64_t groups = spmm_strip_groups(m, stride);
    const dim3 grid(static_cast<uint32_t>((groups + kCoverGroupsPerBlock - 1) / kCoverGroupsPerBlock));
    hipLaunchKernelGGL((strip_cover_kernel<true>), grid, dim3(kBlock), 0, stream, m, nnz, base, stride, row_ptr, col, c.block_ptr,
                       c.blocks, c.counters, static_cast<StripPartial*>(nullptr));
    hipLaunchKernelGGL(strip_order_kernel, dim3(static_cast<uint32_t>((groups + kOrderChunk - 1) / kOrderChunk)),
                       dim3(kOrderChunk), 0, stream, groups, c.block_ptr, c.blocks, c.order);
}

bool spmm_strip_schedule_fits(idx_t m, idx_t nnz, uint32_t stride, uint32_t blocks) {
    return static_cast<uint64_t>(blocks) * sizeof(uint4) + spmm_strip_groups(m, stride) * sizeof(uint32_t) + 16 <=
           static_cast<uint64_t>(nnz) * sizeof(uint32_t);
}

template <typename T>
void launch_spmm_strips(hipStream_t stream, const SpmmArgs& a, const void* schedule, uint32_t stride, uint32_t total_blocks,
                        uint32_t longest_strip, uint64_t mean_span, T alpha, T beta) {
    if (a.m == 0 || a.n == 0) return;
    constexpr int V = 16 / sizeof(T);
    constexpr int kGroupsPerBlock = kStripBlock / kLanes;
    const Carved c = carve(a.m, a.nnz, stride, const_cast<void*>(schedule));
    const uint64_t groups = spmm_strip_groups(a.m, stride);
    const uint64_t group_blocks = (groups + kGroupsPerBlock - 1) / kGroupsPerBlock;
    const uint64_t panels = (static_cast<uint64_t>(a.n) + kLanes * V - 1) / (kLanes * V);
    // An XCD works through a stretch of consecutive workgroups at a time, so that the rows of op(B) neighbouring
    // workgroups share stay in its own L2, as long as such a stretch of op(B) is small against the 4 MB of an L2.
    constexpr uint64_t kRowsPerBlock = static_cast<uint64_t>(kGroupsPerBlock) * R;
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
    const bool staged = longest_strip <= static_cast<uint32_t>(strip_capacity<T>()) && reinterpret_cast<uintptr_t>(val) % 16 == 0;
    auto launch = [&](auto wide_c, auto staged_c) {
        hipLaunchKernelGGL((spmm_strips_kernel<T, decltype(wide_c)::value, decltype(staged_c)::value>), grid, dim3(kStripBlock), 0,
                           stream, a.m, a.n, a.base, stride, a.row_ptr, a.col, val, c.block_ptr, c.blocks, c.order, B, a.ldb, C,
                           a.ldc, a.c_row_major, alpha, beta, xcd_chunk, xcds, a.k, a.nnz, total_blocks);
    };
    if (narrow_offsets(a, sizeof(T))) {
        if (staged) launch(std::false_type{}, std::true_type{});
        else launch(std::false_type{}, std::false_type{});
    } else {
        launch(std::true_type{}, std::false_type{});
    }
}

template void launch_spmm_strips<float>(hipStream_t, const SpmmArgs&, const void*, uint32_t, uint32_t, uint32_t, uint64_t,
                                        float, float);
template void launch_spmm_strips<double>(hipStream_t, const SpmmArgs&, const void*, uint32_t, uint32_t, uint32_t, uint64_t,
                                         double, double);

}  // namespace mcsp
