// CSR SpMM from a schedule of diagonal blocks, for matrices whose neighbouring rows hold the same
// diagonals (stencils, banded and structured-grid matrices).
//
// The reference's kernel (src/kernels/level3/spmm/csr_spmm_device.hpp:121-137) walks a row's nonzeros
// once per output column.  Here a lane group owns kSpmmBlockRows consecutive rows of A and a few adjacent
// columns of C.  mcsparseSpMM_preprocess has covered the nonzeros of those rows with blocks of up to
// kSpmmBlockMaxDiagonals consecutive diagonals, each with its own range of rows: block
// (c, n, lo_0, hi_0, .., lo_{n-1}, hi_{n-1}) says that row r of the group holds column c + r + p for every
// p < n with lo_p <= r < hi_p.  The block needs at most kSpmmBlockRows + n - 1 consecutive rows of op(B),
// each loaded once into registers and used by up to n rows of A, and which loaded row feeds which
// accumulator is fixed in the code: no per-nonzero flags, ballots or masks.  The values are read from the
// CSR array on every call (a row's values inside a block are the next ones in storage order), so the
// caller may change them freely between calls.
//
// A block is eight bytes: {int32 c, uint32 shape}; shape bits 0-2 hold n, bits 8+8p..11+8p hold lo_p and
// bits 12+8p..15+8p hold hi_p.
#include "spmm_device.h"

namespace mcsp {

namespace {

using namespace spmm_detail;

constexpr int K = kSpmmBlockRows;
constexpr int D = kSpmmBlockMaxDiagonals;
constexpr int kNoKey = 0x7fffffff;

struct BlockCounters {
    unsigned long long span_sum;  // sum over the groups of (last column - first column)
    unsigned long long loads;     // rows of op(B) all blocks load together
    unsigned int longest_group;   // most nonzeros in one group that has blocks
};

__global__ void zero_block_counters_kernel(BlockCounters* c) {
    c->span_sum = 0;
    c->loads = 0;
    c->longest_group = 0;
}

// One thread covers the nonzeros of one group of K rows with blocks.  It merges the rows by the key
// column - row (the diagonal a nonzero lies on, counted from the group's first row): nonzeros of
// neighbouring rows on one diagonal share a key, consecutive diagonals have consecutive keys.  A block
// grows while the next key follows the last one and the same rows hold it; a set of rows with gaps is cut
// into its contiguous stretches.  Every row's nonzeros are consumed in storage order, whatever that order
// is, so the p-th value of a row inside a block is always the next one the row has not used yet.
//
// The 64 groups of a wavefront read one contiguous stretch of the column indices; read thread by thread
// they would cost a cache line per element, so the wavefront first copies the stretch into LDS when it
// fits.
constexpr uint32_t kStage = 16384;
template <bool FILL>
__global__ __launch_bounds__(kWave) void block_cover_kernel(idx_t m, idx_t base, const idx_t* __restrict__ row_ptr,
                                                            const idx_t* __restrict__ col,
                                                            uint32_t* __restrict__ block_ptr, uint2* __restrict__ blocks,
                                                            BlockCounters* __restrict__ counters) {
    __shared__ idx_t s_col[kStage];
    const uint64_t groups = spmm_block_groups(m);
    const uint64_t first_group = static_cast<uint64_t>(blockIdx.x) * kWave;
    const uint64_t group = first_group + threadIdx.x;
    const uint64_t first_row = first_group * K < m ? first_group * K : m;
    const uint64_t end_row = (first_group + kWave) * K < m ? (first_group + kWave) * K : m;
    const idx_t stretch_begin = row_ptr[first_row] - base;
    const idx_t stretch_end = row_ptr[end_row] - base;
    const bool staged = stretch_end - stretch_begin <= kStage;
    if (staged) {
        constexpr int kAhead = 16;  // loads on their way before the first is parked
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
    __syncthreads();

    uint32_t count = 0;
    unsigned long long loads = 0;
    uint32_t first_col = 0xffffffffu, last_col = 0;
    uint32_t group_nnz = 0;
    if (group < groups) {
        idx_t i[K], e[K];
        const uint64_t r0 = group * K;
        idx_t next = row_ptr[r0] - base;
#pragma unroll
        for (int r = 0; r < K; ++r) {
            i[r] = next;
            if (r0 + r < static_cast<uint64_t>(m)) next = row_ptr[r0 + r + 1] - base;
            e[r] = next;
        }
        if (e[K - 1] - i[0] <= kSpmmMaxMergedGroup) {
            group_nnz = e[K - 1] - i[0];
            uint32_t out = FILL ? block_ptr[group] : 0;
            auto cover = [&](auto staged_c) {
                constexpr bool kStaged = decltype(staged_c)::value;
                auto key_of = [&](int r) -> int {
                    if (i[r] >= e[r]) return kNoKey;
                    const uint32_t c = static_cast<uint32_t>((kStaged ? s_col[i[r] - stretch_begin] : col[i[r]]) - base);
                    first_col = c < first_col ? c : first_col;
                    last_col = c > last_col ? c : last_col;
                    return static_cast<int>(c) - r;
                };
                int key[K];
#pragma unroll
                for (int r = 0; r < K; ++r) key[r] = key_of(r);
                // the block being grown: keys start .. start + width - 1, key start + p held by rows lo[p] .. hi[p] - 1
                int start = 0;
                uint32_t width = 0;
                uint32_t lo[D], hi[D];
                auto emit = [&](int c, uint32_t w, const uint32_t (&l)[D], const uint32_t (&h)[D]) {
                    uint32_t shape = w;
                    uint32_t j_min = 0xffffffffu, j_max = 0;
#pragma unroll
                    for (int q = 0; q < D; ++q) {
                        if (static_cast<uint32_t>(q) < w) {
                            shape |= (l[q] | (h[q] << 4)) << (8 + 8 * q);
                            j_min = min(j_min, l[q] + q);
                            j_max = max(j_max, h[q] - 1 + q);
                        }
                    }
                    if (FILL) blocks[out + count] = make_uint2(static_cast<uint32_t>(c), shape);
                    ++count;
                    loads += j_max - j_min + 1;
                };
                auto flush = [&]() {
                    if (width != 0) emit(start, width, lo, hi);
                    width = 0;
                };
                while (true) {
                    int low = kNoKey;
#pragma unroll
                    for (int r = 0; r < K; ++r) low = key[r] < low ? key[r] : low;
                    if (low == kNoKey) break;
                    uint32_t holders = 0;
#pragma unroll
                    for (int r = 0; r < K; ++r) {
                        if (key[r] == low) {
                            holders |= 1u << r;
                            ++i[r];
                            key[r] = key_of(r);
                        }
                    }
                    // the rows that hold this key, one contiguous stretch at a time
                    while (holders != 0) {
                        const uint32_t first = __ffs(holders) - 1;
                        const uint32_t run = __ffs(~(holders >> first)) - 1;  // set bits from `first` on
                        holders &= ~(((1u << run) - 1u) << first);
                        // The last stretch may carry on the block being grown (the next diagonal of the same rows,
                        // or of rows shifted by a grid line's end); the others are blocks of their own.
                        if (holders == 0 && width != 0 && width < static_cast<uint32_t>(D) && low == start + static_cast<int>(width)) {
                            lo[width] = first;
                            hi[width] = first + run;
                            ++width;
                        } else if (holders == 0) {
                            flush();
                            start = low;
                            lo[0] = first;
                            hi[0] = first + run;
                            width = 1;
                        } else {
                            flush();
                            const uint32_t l1[D] = {first, 0, 0}, h1[D] = {first + run, 0, 0};
                            emit(low, 1, l1, h1);
                        }
                    }
                }
                flush();
            };
            if (staged) cover(std::true_type{});
            else cover(std::false_type{});
        }
    }
    if (!FILL) {
        if (group <= groups) block_ptr[group] = count;  // slot `groups` receives the total after the scan
        unsigned long long span = count != 0 ? last_col - first_col : 0;
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            span += __shfl_xor(span, off, kWave);
            loads += __shfl_xor(loads, off, kWave);
            group_nnz = max(group_nnz, static_cast<uint32_t>(__shfl_xor(static_cast<int>(group_nnz), off, kWave)));
        }
        if (lane_id() == 0) {
            if (span != 0) atomicAdd(&counters->span_sum, span);
            if (loads != 0) atomicAdd(&counters->loads, loads);
            if (group_nnz != 0) atomicMax(&counters->longest_group, group_nnz);
        }
    }
}

// The lane groups of a wavefront walk their block lists in lockstep: a wavefront whose groups hold different
// lists runs every list's code one after the other (on a stencil the groups at the ends of a grid line, an
// eighth of all, made half of the wavefronts take twice as long).  So the groups are handed out in an order in
// which neighbours hold equal lists: inside every stretch of kOrderChunk consecutive groups, sorted (stably) by
// a hash of the shapes of their blocks.  Any permutation gives the right product; this one also keeps a
// stretch's rows of op(B) together.
constexpr uint32_t kOrderChunk = 1024;
__global__ __launch_bounds__(kOrderChunk) void block_order_kernel(uint64_t groups, const uint32_t* __restrict__ block_ptr,
                                                                  const uint2* __restrict__ blocks,
                                                                  uint32_t* __restrict__ order) {
    __shared__ uint32_t keys[kOrderChunk];
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * kOrderChunk;
    const uint64_t group = first + threadIdx.x;
    uint32_t hash = 0x3fffffu;  // groups past the end sort last
    if (group < groups) {
        hash = 2166136261u;
        for (uint32_t s = block_ptr[group]; s < block_ptr[group + 1]; ++s) hash = (hash ^ blocks[s].y) * 16777619u;
        hash = (hash ^ (hash >> 15)) & 0x3ffffeu;
    }
    keys[threadIdx.x] = (hash << 10) | threadIdx.x;
    __syncthreads();
    // bitonic sort of the chunk's 1024 keys; the thread number in the low bits makes equal hashes keep their order
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

// LR lanes (8..64) per group of K rows, V = 16 B / sizeof(T) adjacent columns per lane; blockIdx.y walks
// panels of LR * V columns.  Every lane of a group reads the block descriptors itself (one address for the
// whole group: one access); a block's values are read by the lanes together (lane l reads for row
// l / (LR / K)) and reach the multiply-adds as DPP row broadcasts.
// STAGED: no group holds more nonzeros than stage_capacity<T, LR>() and the value array is 16-byte aligned.  A
// group's values are then copied into LDS once, in whole 16-byte pieces, and every block reads its values from
// there.  (Read from memory block by block, the sixteen lanes of a group ask for two values in each of eight
// rows: eight cache lines touched for 128 bytes, nine times over per row, which cost the vector memory path
// twice what a block's rows of op(B) cost.)
template <typename T, int LR>
constexpr int stage_capacity() { return (LR >= 16 ? 2048 : 1024) / static_cast<int>(sizeof(T)); }

template <typename T, int LR, bool WIDE, bool STAGED>
__global__ __launch_bounds__(kBlock) void spmm_blocks_kernel(idx_t m, idx_t n, idx_t base,
                                                             const idx_t* __restrict__ row_ptr,
                                                             const idx_t* __restrict__ col, const T* __restrict__ val,
                                                             const uint32_t* __restrict__ block_ptr,
                                                             const uint2* __restrict__ blocks,
                                                             const uint32_t* __restrict__ order, const T* __restrict__ B,
                                                             int64_t ldb, T* __restrict__ C, int64_t ldc,
                                                             bool c_row_major, T alpha, T beta, uint32_t xcd_chunk, uint32_t xcds,
                                                             idx_t k, idx_t nnz, uint32_t total_blocks) {
    typedef typename ByteOffset<WIDE>::type off_t;
    constexpr int V = 16 / sizeof(T);
    constexpr int kGroupsPerBlock = kBlock / LR;
    constexpr int kLanesPerRow = LR / K;                                 // lanes that fetch the values of one row
    constexpr int kValuesPerLane = (D + kLanesPerRow - 1) / kLanesPerRow;
    static_assert(LR >= K && LR % K == 0, "a lane group fetches the values of its K rows in one go");
    const idx_t lane = threadIdx.x % LR;
    const uint64_t turn = xcd_position(blockIdx.x, xcd_chunk, xcds) * kGroupsPerBlock + threadIdx.x / LR;
    const uint64_t groups = spmm_block_groups(m);
    if (turn >= groups) return;  // whole lane groups
    // which group takes this turn (held to the groups that exist, whatever the buffer holds)
    const uint64_t group = min(static_cast<uint64_t>(order[turn]), groups - 1);
    const uint64_t r0 = group * K;
    const uint64_t c_own = (static_cast<uint64_t>(blockIdx.y) * LR + lane) * V;
    const bool stores = c_own < static_cast<uint64_t>(n);  // lanes past the last column only help fetching
    const uint64_t c0 = stores ? c_own : 0;

    T acc[K][V];
#pragma unroll
    for (int r = 0; r < K; ++r) {
#pragma unroll
        for (int c = 0; c < V; ++c) acc[r][c] = T(0);
    }
    const char* B_bytes = reinterpret_cast<const char*>(B);
    const off_t lane_off = static_cast<off_t>(c0 * sizeof(T));
    const off_t ldb_bytes = static_cast<off_t>(ldb * sizeof(T));
    const uint64_t last_row = static_cast<uint64_t>(m) - 1;
    const uint64_t group_end_row = r0 + K < static_cast<uint64_t>(m) ? r0 + K : static_cast<uint64_t>(m);
    const idx_t group_begin = row_ptr[r0] - base;
    const idx_t group_end = row_ptr[group_end_row] - base;

    if (group_end - group_begin <= kSpmmMaxMergedGroup) {
        // The schedule lives in the caller's buffer.  Whatever it holds, nothing is read outside the arrays:
        // list bounds are held to the list, a block whose rows of op(B) do not all exist counts as a block of
        // no width, value positions are held to the nonzeros.  (An overwritten schedule gives wrong numbers,
        // never a fault.)
        const uint32_t s_end = min(block_ptr[group + 1], total_blocks);
        const uint32_t s_begin = min(block_ptr[group], s_end);
        const idx_t last_value = nnz - 1;  // nnz != 0: total_blocks != 0
        const uint32_t last_block = total_blocks - 1;
        const uint32_t my_row = lane / kLanesPerRow;
        // where the next unused value of this lane's row lies
        const uint64_t my_abs_row = r0 + my_row < last_row ? r0 + my_row : last_row;
        const uint32_t my_place = (lane % kLanesPerRow) * kValuesPerLane;  // the first diagonal this lane fetches for
        idx_t pos = row_ptr[my_abs_row] - base;

        constexpr int kCap = stage_capacity<T, LR>();
        constexpr int E = 16 / sizeof(T);  // values per 16-byte piece
        __shared__ __attribute__((aligned(16))) T s_val[STAGED ? kGroupsPerBlock : 1][STAGED ? kCap : 1];
        T* staged = s_val[STAGED ? threadIdx.x / LR : 0];
        const idx_t stage_first = group_begin & ~static_cast<idx_t>(E - 1);  // the piece the group's first value lies in
        if constexpr (STAGED) {
            typedef T Piece __attribute__((ext_vector_type(E)));
            constexpr int kPerLane = kCap / E / LR;  // pieces a lane copies
            static_assert(kPerLane >= 2 && kPerLane % 2 == 0, "two rounds of copies");
            const idx_t pieces = (group_end - stage_first + E - 1) / E;  // at most kCap / E: the launcher has checked
            const idx_t whole_pieces = nnz / E;  // pieces that lie inside the array altogether
            const idx_t first_piece = stage_first / E;
            auto copy_round = [&](int from) {
                // all loads of a round on their way together, each held to a piece that exists; pieces past the
                // group's end land in places nothing reads
                Piece got[kPerLane / 2];
#pragma unroll
                for (int c = 0; c < kPerLane / 2; ++c) {
                    const idx_t piece = static_cast<idx_t>(from + c) * LR + lane;
                    const idx_t at = min(first_piece + min(piece, pieces - 1), whole_pieces != 0 ? whole_pieces - 1 : 0);
                    got[c] = reinterpret_cast<const Piece*>(val)[at];
                }
#pragma unroll
                for (int c = 0; c < kPerLane / 2; ++c) {
                    const idx_t piece = static_cast<idx_t>(from + c) * LR + lane;
                    reinterpret_cast<Piece*>(staged)[piece] = got[c];
                }
            };
            copy_round(0);
            if (pieces > static_cast<idx_t>(kPerLane / 2 * LR)) copy_round(kPerLane / 2);
            // the array's last values, when they do not fill a piece, one by one (nothing is read past the end)
            if (group_end > whole_pieces * E) {
                const idx_t at = whole_pieces * E + lane;
                if (at < group_end) staged[at - stage_first] = val[at];
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }

        // What a wavefront waits for is the latency of its loads, not their number: with a block's loads
        // asked for when the block's turn comes, a group's blocks cost one trip to memory each, one after the
        // other.  So everything a block needs is asked for while the block before it is being worked on: its
        // descriptor two blocks ahead (every lane of the group reads it itself), its values and its rows of
        // op(B) one block ahead, into a second set of registers.  None of these loads sits under a test (a load
        // under a test makes the compiler wait for every load in flight at the join): a block past the end of
        // the list, or one that is not sound, turns into a block of no width whose loads go to places that exist.
        // A block as the kernel sees it.  `mine` says which of the block's diagonals this lane's row holds (bit p:
        // diagonal p): the row's values of the block are its next popcount(mine) ones, in the order of the bits.
        struct Shape {
            int cbase;
            uint32_t w;
            uint32_t lo[D], len[D];  // diagonal p is held by rows lo[p] .. lo[p] + len[p] - 1
            uint32_t j_first, j_last;  // rows of op(B) the block needs, counted from cbase
            uint32_t mine;
            bool whole;  // every row of the group holds every diagonal of the block
        };
        auto decode = [&](uint2 d, bool exists) {
            Shape sh;
            sh.cbase = static_cast<int>(d.x);
            sh.w = d.y & 7u;
            bool sound = exists && sh.w - 1u < static_cast<uint32_t>(D);
            sh.whole = true;
            sh.mine = 0;
            sh.j_first = 0xffffu;
            sh.j_last = 0;
#pragma unroll
            for (int q = 0; q < D; ++q) {
                const uint32_t lo = (d.y >> (8 + 8 * q)) & 15u;
                const uint32_t hi = (d.y >> (12 + 8 * q)) & 15u;
                const bool used = static_cast<uint32_t>(q) < sh.w;
                sound = sound && (!used || (lo < hi && hi <= static_cast<uint32_t>(K)));
                sh.lo[q] = lo;
                sh.len[q] = used ? hi - lo : 0u;
                sh.whole = sh.whole && (!used || (lo == 0 && hi == static_cast<uint32_t>(K)));
                if (used) {
                    sh.j_first = min(sh.j_first, lo + q);
                    sh.j_last = max(sh.j_last, hi - 1 + q);
                    if (my_row - lo < hi - lo) sh.mine |= 1u << q;
                }
            }
            // (every extent is below 2^31 here, so the sums cannot wrap)
            sound = sound && sh.cbase + static_cast<int>(sh.j_first) >= 0 &&
                    sh.cbase + static_cast<int>(sh.j_last) <= static_cast<int>(k) - 1;
            if (!sound) {
                sh.cbase = 0;
                sh.w = 0;
                sh.j_first = sh.j_last = 0;
                sh.mine = 0;
                sh.whole = false;
#pragma unroll
                for (int q = 0; q < D; ++q) sh.len[q] = 0;
            }
            return sh;
        };
        struct Operands {
            T v[kValuesPerLane];
            Vec<T, V> b[K + D - 1];
        };
        // at_value: where the first unused value of this lane's row lies
        auto fetch = [&](const Shape& sh, idx_t at_value, Operands& o) {
            // this lane fetches for the diagonals my_place .. my_place + kValuesPerLane - 1 of its row: the value of
            // diagonal p is the row's (number of held diagonals below p)-th unused one
            idx_t at[kValuesPerLane];
#pragma unroll
            for (int q = 0; q < kValuesPerLane; ++q)
                at[q] = at_value + static_cast<idx_t>(__popc(sh.mine & ((1u << (my_place + q)) - 1u)));
            if constexpr (STAGED) {
                // from the group's copy in LDS; a place past the copy (an overwritten schedule) is held inside it
#pragma unroll
                for (int q = 0; q < kValuesPerLane; ++q)
                    o.v[q] = staged[min(at[q] - stage_first, static_cast<idx_t>(kCap - 1))];
            } else {
#pragma unroll
                for (int q = 0; q < kValuesPerLane; ++q) o.v[q] = val[min(at[q], last_value)];
            }
            // rows j_first .. j_last of the block are needed; the others are asked for at the nearest needed one
            const off_t roff = static_cast<off_t>(static_cast<int64_t>(sh.cbase)) * ldb_bytes + lane_off;
            static_for<K + D - 1>([&](auto jc) {
                constexpr uint32_t j = decltype(jc)::value;
                const uint32_t jj = min(max(j, sh.j_first), sh.j_last);
                o.b[j] = load_vec<T, V>(reinterpret_cast<const T*>(B_bytes + (roff + static_cast<off_t>(jj) * ldb_bytes)));
            });
        };
        auto consume = [&](const Shape& sh, const Operands& o) {
            // Every row of the group takes part (all but the groups at the edge of a grid line): the
            // multiply-adds follow in the order the rows of op(B) arrive.
            auto whole = [&](auto wc) {
                constexpr int W = decltype(wc)::value;
                static_for<K + W - 1>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    static_for<W>([&](auto pc) {
                        constexpr int p = decltype(pc)::value;
                        constexpr int r = j - p;
                        if constexpr (r >= 0 && r < K) {
                            const T a = group_bcast<LR, r * kLanesPerRow + p / kValuesPerLane>(o.v[p % kValuesPerLane]);
#pragma unroll
                            for (int c = 0; c < V; ++c) acc[r][c] += a * o.b[j].v[c];
                        }
                    });
                });
            };
            // Some rows lack some diagonals (a grid line begins or ends inside the group): the tests sit around
            // the multiply-adds, so that a row only ever sees the rows of op(B) it names.
            auto partial = [&]() {
                static_for<K + D - 1>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    static_for<D>([&](auto pc) {
                        constexpr int p = decltype(pc)::value;
                        constexpr int r = j - p;
                        if constexpr (r >= 0 && r < K) {
                            if (static_cast<uint32_t>(r) - sh.lo[p] < sh.len[p]) {
                                const T a = group_bcast<LR, r * kLanesPerRow + p / kValuesPerLane>(o.v[p % kValuesPerLane]);
#pragma unroll
                                for (int c = 0; c < V; ++c) acc[r][c] += a * o.b[j].v[c];
                            }
                        }
                    });
                });
            };
            if (sh.whole) {
                static_assert(D == 3, "one case per width");
                switch (sh.w) {
                    case 1: whole(std::integral_constant<int, 1>{}); break;
                    case 2: whole(std::integral_constant<int, 2>{}); break;
                    case 3: whole(std::integral_constant<int, 3>{}); break;
                    default: break;
                }
            } else if (sh.w != 0) {
                partial();
            }
        };
        auto advance = [&](const Shape& sh) -> idx_t { return static_cast<idx_t>(__popc(sh.mine)); };
        auto descriptor = [&](uint32_t s) { return blocks[min(s, last_block)]; };

        Operands even, odd;
        uint2 d_next = descriptor(s_begin + 1);
        Shape now = decode(descriptor(s_begin), s_begin < s_end);
        fetch(now, pos, even);
        uint32_t s = s_begin;
        for (; s + 2 < s_end; s += 2) {
            // block s is in `even`; s + 1 goes to `odd` while s is worked on, s + 2 to `even` while s + 1 is
            const uint2 d_after = descriptor(s + 2);
            const Shape next = decode(d_next, true);
            pos += advance(now);
            fetch(next, pos, odd);
            consume(now, even);
            const uint2 d_after2 = descriptor(s + 3);
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
            consume(now, even);  // no width when the list is empty
        }
    } else {
        // a group too long to be worth covering: one row after the other
        idx_t i[K], e[K];
        idx_t next = group_begin;
#pragma unroll
        for (int r = 0; r < K; ++r) {
            i[r] = next;
            if (r0 + r < static_cast<uint64_t>(m)) next = row_ptr[r0 + r + 1] - base;
            e[r] = next;
        }
#pragma unroll
        for (int r = 0; r < K; ++r)
            row_times_b<T, LR, V, WIDE>(i[r], e[r], lane, base, col, val, B_bytes, lane_off, ldb_bytes, acc[r]);
    }

    // A column-major C holds the rows of the group next to each other in every column: 32 or 64 bytes per
    // column and lane, which the lane groups of a workgroup complete to whole lines.
    static_assert(K % 4 == 0, "rows of a group are written four at a time into a column-major C");
    const bool whole_columns = !c_row_major && r0 + K <= static_cast<uint64_t>(m) &&
                               ((reinterpret_cast<uintptr_t>(C) | static_cast<uintptr_t>(ldc * sizeof(T))) & 15u) == 0;
    if constexpr (sizeof(T) == 4 && K == 8) {
        // Written lane by lane, a wavefront's store touches 64 pieces of 16 bytes, each in a line of its own.  Two
        // neighbouring lanes swap halves instead: of every column of the two, the even lane then writes rows 0-3 and
        // the odd lane rows 4-7, 32 adjacent bytes per store and pair.  (Both lanes of a pair belong to one group;
        // every lane takes part in the swap, also those that store nothing.)
        const bool odd = (lane & 1u) != 0;
        const uint64_t partner_c_own = odd ? c_own - V : c_own + V;
        const bool paired = whole_columns && stores && partner_c_own < static_cast<uint64_t>(n);
        if (__builtin_amdgcn_ballot_w64(paired) != 0) {  // same for the whole wavefront
            T got[4][V];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int c = 0; c < V; ++c) got[i][c] = dpp_mov<kDppQuadXor1>(odd ? acc[i][c] : acc[4 + i][c]);
            }
            if (paired) {
                const uint64_t pair_c0 = odd ? c0 - V : c0;
                T* first = C + r0 + (odd ? 4 : 0);
#pragma unroll
                for (int c = 0; c < V; ++c) {
                    // a column of the even lane: its own rows 0-3, and the rows 4-7 it gave to the odd lane
                    T* at = first + static_cast<int64_t>(pair_c0 + c) * ldc;
                    if (odd) store_c_four_rows<T>(at, got[0][c], got[1][c], got[2][c], got[3][c], alpha, beta);
                    else store_c_four_rows<T>(at, acc[0][c], acc[1][c], acc[2][c], acc[3][c], alpha, beta);
                }
#pragma unroll
                for (int c = 0; c < V; ++c) {
                    // a column of the odd lane: the rows 0-3 it gave to the even lane, and its own rows 4-7
                    T* at = first + static_cast<int64_t>(pair_c0 + V + c) * ldc;
                    if (odd) store_c_four_rows<T>(at, acc[4][c], acc[5][c], acc[6][c], acc[7][c], alpha, beta);
                    else store_c_four_rows<T>(at, got[0][c], got[1][c], got[2][c], got[3][c], alpha, beta);
                }
                return;
            }
        }
    }
    if (!stores) return;
    if (whole_columns) {
#pragma unroll
        for (int c = 0; c < V; ++c) {
#pragma unroll
            for (int q = 0; q < K / 4; ++q)
                store_c_four_rows<T>(C + static_cast<int64_t>(c0 + c) * ldc + r0 + 4 * q, acc[4 * q][c], acc[4 * q + 1][c],
                                     acc[4 * q + 2][c], acc[4 * q + 3][c], alpha, beta);
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < K; ++r) {
        if (r0 + r < static_cast<uint64_t>(m)) store_c<T, V>(C, ldc, c_row_major, r0 + r, c0, acc[r], alpha, beta);
    }
}

template <typename T, int LR>
void launch_blocks(hipStream_t stream, const SpmmArgs& a, const uint32_t* block_ptr, const uint2* blocks,
                   const uint32_t* order, uint32_t total_blocks, uint32_t longest_group, T alpha, T beta,
                   uint64_t mean_span) {
    constexpr int V = 16 / sizeof(T);
    const uint64_t groups = spmm_block_groups(a.m);
    const uint64_t group_blocks = (groups + (kBlock / LR) - 1) / (kBlock / LR);
    const uint64_t panels = (static_cast<uint64_t>(a.n) + LR * V - 1) / (LR * V);
    // An XCD works through mean_span / 16 consecutive rows at a time, so that the rows of op(B) which
    // neighbouring stretches share (the neighbouring grid lines of a stencil) stay in its own L2, as long as
    // such a stretch of op(B) is small against the 4 MB of an L2.
    constexpr uint64_t kRowsPerBlock = static_cast<uint64_t>(kBlock / LR) * K;
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
    // a group's values fit its share of LDS, with the pieces before and behind that the 16-byte copies bring along
    const bool staged = static_cast<uint64_t>(longest_group) + 2 * (16 / sizeof(T)) <= static_cast<uint64_t>(stage_capacity<T, LR>()) &&
                        reinterpret_cast<uintptr_t>(val) % 16 == 0;
    auto launch = [&](auto wide_c, auto staged_c) {
        hipLaunchKernelGGL((spmm_blocks_kernel<T, LR, decltype(wide_c)::value, decltype(staged_c)::value>), grid, dim3(kBlock),
                           0, stream, a.m, a.n, a.base, a.row_ptr, a.col, val, block_ptr, blocks, order, B, a.ldb, C, a.ldc,
                           a.c_row_major, alpha, beta, xcd_chunk, xcds, a.k, a.nnz, total_blocks);
    };
    if (narrow_offsets(a, sizeof(T))) {
        if (staged) launch(std::false_type{}, std::true_type{});
        else launch(std::false_type{}, std::false_type{});
    } else {
        launch(std::true_type{}, std::false_type{});
    }
}

// The block schedule inside the region spmm_schedule_layout describes: the offsets where the merged lists
// keep theirs, the blocks from the start of the entries' place, the order of the groups at its end.
struct Carved {
    uint32_t* block_ptr;
    BlockCounters* counters;
    uint2* blocks;
    uint32_t* order;
    char* scan_ws;
};
Carved carve(idx_t m, idx_t nnz, void* schedule) {
    const SpmmScheduleLayout l = spmm_schedule_layout(m, nnz);
    char* w = static_cast<char*>(schedule);
    const size_t order_bytes = spmm_block_groups(m) * sizeof(uint32_t);
    const size_t entries_bytes = static_cast<size_t>(nnz) * sizeof(uint32_t);
    const size_t order_at = entries_bytes >= order_bytes ? (entries_bytes - order_bytes) / 8 * 8 : 0;
    return {reinterpret_cast<uint32_t*>(w + l.group_ptr), reinterpret_cast<BlockCounters*>(w + l.span_sum),
            reinterpret_cast<uint2*>(w + l.entries), reinterpret_cast<uint32_t*>(w + l.entries + order_at), w + l.scan_ws};
}

}  // namespace

void launch_spmm_block_count(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, const idx_t* row_ptr, const idx_t* col,
                             void* schedule) {
    const Carved c = carve(m, nnz, schedule);
    const uint64_t slots = spmm_block_groups(m) + 1;
    const dim3 grid(static_cast<uint32_t>((slots + kWave - 1) / kWave));
    hipLaunchKernelGGL(zero_block_counters_kernel, dim3(1), dim3(1), 0, stream, c.counters);
    hipLaunchKernelGGL((block_cover_kernel<false>), grid, dim3(kWave), 0, stream, m, base, row_ptr, col, c.block_ptr,
                       c.blocks, c.counters);
    launch_exclusive_scan_u32(stream, c.block_ptr, slots, c.scan_ws);
}

void launch_spmm_block_fill(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, const idx_t* row_ptr, const idx_t* col,
                            void* schedule) {
    const Carved c = carve(m, nnz, schedule);
    const uint64_t slots = spmm_block_groups(m) + 1;
    const dim3 grid(static_cast<uint32_t>((slots + kWave - 1) / kWave));
    hipLaunchKernelGGL((block_cover_kernel<true>), grid, dim3(kWave), 0, stream, m, base, row_ptr, col, c.block_ptr,
                       c.blocks, c.counters);
    const uint64_t groups = spmm_block_groups(m);
    hipLaunchKernelGGL(block_order_kernel, dim3(static_cast<uint32_t>((groups + kOrderChunk - 1) / kOrderChunk)),
                       dim3(kOrderChunk), 0, stream, groups, c.block_ptr, c.blocks, c.order);
}

bool spmm_block_schedule_fits(idx_t m, idx_t nnz, uint32_t blocks) {
    return static_cast<uint64_t>(blocks) * sizeof(uint2) + spmm_block_groups(m) * sizeof(uint32_t) + 8 <=
           static_cast<uint64_t>(nnz) * sizeof(uint32_t);
}

bool spmm_blocks_usable(const SpmmArgs& a, size_t value_bytes) {
    const int64_t wide = static_cast<int64_t>(16 / value_bytes);
    // at least five 128-bit vectors per row: lane groups of eight and more
    return a.b_row_major && a.n >= 4 * wide + 1 && a.k <= kSpmmMaxScheduledColumns && a.m < (idx_t(1) << 31) &&
           reinterpret_cast<uintptr_t>(a.B) % 16 == 0 && a.ldb % wide == 0 && a.n % wide == 0 &&
           (!a.c_row_major || (reinterpret_cast<uintptr_t>(a.C) % 16 == 0 && a.ldc % wide == 0));
}

template <typename T>
void launch_spmm_blocks(hipStream_t stream, const SpmmArgs& a, const void* schedule, uint32_t total_blocks,
                        uint32_t longest_group, uint64_t mean_span, T alpha, T beta) {
    if (a.m == 0 || a.n == 0) return;
    constexpr int V = 16 / sizeof(T);
    const Carved c = carve(a.m, a.nnz, const_cast<void*>(schedule));
    const uint64_t lanes_needed = (static_cast<uint64_t>(a.n) + V - 1) / V;
    // Beyond 32 lanes a lane group would be a whole wavefront with eight rows to itself, too little work to hide
    // the chain of loads a group begins with: wider operands are cut into panels of 64 bytes x 16 lanes.
    if (lanes_needed <= 8) launch_blocks<T, 8>(stream, a, c.block_ptr, c.blocks, c.order, total_blocks, longest_group, alpha, beta, mean_span);
    else if (lanes_needed <= 16 || lanes_needed > 32) launch_blocks<T, 16>(stream, a, c.block_ptr, c.blocks, c.order, total_blocks, longest_group, alpha, beta, mean_span);
    else launch_blocks<T, 32>(stream, a, c.block_ptr, c.blocks, c.order, total_blocks, longest_group, alpha, beta, mean_span);
}

template void launch_spmm_blocks<float>(hipStream_t, const SpmmArgs&, const void*, uint32_t, uint32_t, uint64_t, float, float);
template void launch_spmm_blocks<double>(hipStream_t, const SpmmArgs&, const void*, uint32_t, uint32_t, uint64_t, double,
                                         double);

}  // namespace mcsp
