// Host-side objects behind the opaque handles of mcsparse.h, and the launch entry points
// the host layer calls.  Not installed; the ABI is include/mcsparse.h only.
#ifndef MCSPARSE_AMD_INTERNAL_H_
#define MCSPARSE_AMD_INTERNAL_H_

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

#include "mcsparse.h"

// Sub-buffer alignment and the smallest size any *_bufferSize reports
// (reference: src/include/mcsp_config.h:13-15).
constexpr size_t kAlign = 128;
constexpr size_t kMinBuffer = 128;

static constexpr inline size_t align_up(size_t n, size_t a = kAlign) { return (n + a - 1) / a * a; }

// reference: src/include/mcsp_handle.h:11-27 (device pool dropped, see mcsparse.h)
struct mcsparseContext {
    hipStream_t stream = nullptr;
    mcsparsePointerMode_t ptr_mode = MCSPARSE_POINTER_MODE_HOST;
    // mcsparseSetSpMVDeterministic: every SpMV call of this handle is treated as MCSPARSE_SPMV_CSR_ALG2
    bool spmv_deterministic = false;
    // mcsparseSetSpMVPreprocessTrial: mcsparseSpMV_preprocess times its copy against the row kernels and keeps
    // it only where it is faster
    bool spmv_preprocess_trial = true;
};

// reference: src/include/mcsp_internal_types.h:86-94
struct mcsparseMatDescr {
    mcsparseMatrixType_t type = MCSPARSE_MATRIX_TYPE_GENERAL;
    mcsparseFillMode_t fill_mode = MCSPARSE_FILL_MODE_FULL;
    mcsparseDiagType_t diag_type = MCSPARSE_DIAG_TYPE_NON_UNIT;
    mcsparseStorageMode_t storage_mode = MCSPARSE_STORAGE_MODE_SORTED;
    mcsparseIndexBase_t base = MCSPARSE_INDEX_BASE_ZERO;
};

// reference: src/include/mcsp_internal_types.h:127-133
struct mcsparseDnVecDescr {
    macaDataType valueType = MACA_R_32F;
    int64_t size = 0;
    void* values = nullptr;
};

// reference: src/include/mcsp_internal_types.h:135-147
struct mcsparseDnMatDescr {
    macaDataType valueType = MACA_R_32F;
    mcsparseOrder_t order = MCSPARSE_ORDER_COL;
    int64_t row_num = 0;
    int64_t col_num = 0;
    int64_t ld = 0;
    void* values = nullptr;
    int64_t batchCount = 1;
    int64_t batchStride = 0;
};

// Kernel family of an SpMV call.
enum SpmvFamily : int { kFamilyAuto = 0, kFamilyVector = 1, kFamilyMerge = 2 };
// Path items (row ends + nonzeros) per workgroup of the merge family when its tiles run in column
// order, and the size of x from which the analysis asks for that order.
constexpr uint32_t kMergeTileItems = 1024;
constexpr int64_t kMergeOrderMinVectorBytes = 2 << 20;

// Result of the row-length analysis of one CSR structure.  It only steers which kernel
// runs; both kernel families are correct for any structure, so a stale plan costs time,
// never correctness.
struct SpmvPlan {
    bool valid = false;
    // signature of the structure the plan was computed for
    const void* rows = nullptr;
    int64_t m = 0, nnz = 0;
    int base = 0;
    // outcome
    int family = kFamilyAuto;
    int lanes = 0;
    uint32_t max_row_len = 0;
    uint32_t hist[MCSPARSE_ROW_BIN_COUNT] = {0};
    // user override (mcsparseSpMatSetSpMVPlan); kFamilyAuto = none
    int forced_family = kFamilyAuto;
    int forced_lanes = 0;
};

// Row-group schedule built by mcsparseSpMM_preprocess inside the caller's buffer.  Unlike the
// SpMV plan it is part of the computation: SpMM uses it only while the buffer and the CSR
// arrays it was built from are the ones of the call, and the caller must not change the
// structure or the buffer's contents in between (the contract of a preprocess step).
struct SpmmSchedule {
    bool valid = false;
    bool useful = false;   // the merged lists are short enough to pay off
    const void* buffer = nullptr;
    const void* rows = nullptr;
    const void* cols = nullptr;
    int64_t m = 0, nnz = 0;
    int base = 0;
    uint32_t entries = 0;  // length of all merged lists together, or the number of diagonal blocks
    uint64_t mean_span = 0;  // mean distance between the first and the last column of a group
    bool blocks = false;   // the schedule holds diagonal blocks (spmm_blocks.hip) instead of merged lists
    uint32_t longest_group = 0;  // blocks: the most nonzeros in one group of rows (strips: in one strip)
    uint32_t stride = 0;   // blocks: != 0 says the groups are strips this many rows apart (spmm_strips.hip)
};

// Column-banded copy of a CSR matrix built by mcsparseSpMV_preprocess inside the caller's buffer
// (spmv_banded.hip).  Like the SpMM schedule it is part of the computation, and it holds a copy of the
// values: SpMV uses it only while the buffer, the three CSR arrays and the extents of the call are the
// ones it was built from.
struct BandedShape {
    uint32_t band_shift;     // a band holds 2^band_shift keys (column index + index base)
    uint32_t band_bits;      // bits needed to number the bands
    uint32_t bands;
    uint32_t rows_per_tile;
    uint32_t chunks;         // row chunks = tiles per band
    uint32_t tiles;
    // false: entries of a tile in CSR order, row sums formed in a fixed order (bit-reproducible);
    // true: entries of a tile in column order, products added to the row sums in LDS as they come
    bool by_column = false;
    uint32_t sub = 1;        // by_column: bands per group; `bands` then counts the groups (planes of partial sums)
    // by_column: some row holds more than half of what a row chunk holds on average, so that the wavefronts of its
    // tile would queue on its sum in LDS; the kernel variant that sums such a row's products in registers is used
    bool crowded_rows = false;
    // by_column: where each XCD's stretch of units begins (what the build left at BandedLayout::xcd_start, read back
    // once): handed to the kernel with its arguments, which saves its workgroups a dependent load from memory
    uint32_t xcd_start[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
};
struct SpmvBanded {
    bool valid = false;
    bool useful = false;     // false: preprocess built the copy, timed it against the row kernels and found it
                             // no faster; calls run the row kernels
    const void* buffer = nullptr;
    const void* rows = nullptr;
    const void* cols = nullptr;
    const void* vals = nullptr;
    int64_t m = 0, n = 0, nnz = 0;
    int base = 0;
    macaDataType type = MACA_R_32F;
    mcsparseFormat_t format = MCSPARSE_FORMAT_CSR;
    bool transposed = false; // the copy is of the transpose of the arrays (CSR with op T, CSC with op N)
    size_t region = 0;       // offset of the banded copy inside the buffer
    BandedShape shape = {};
    uint32_t grid = 0;       // workgroups of the SpMV kernel
    size_t band_bytes = 0;   // user override of the band width (mcsparseSpMatSetSpMVBandBytes); 0 = default
};

// reference: src/include/mcsp_internal_types.h:184-225.  rows/cols follow the reference's
// convention: for CSR rows = row offsets, cols = column indices; for CSC rows = row indices,
// cols = column offsets (src/common/mcsp_helper.cpp:447-452).
struct mcsparseSpMatDescr {
    mcsparseFormat_t format = MCSPARSE_FORMAT_CSR;
    mcsparseIndexType_t rowIdxType = MCSPARSE_INDEX_32I;
    mcsparseIndexType_t colIdxType = MCSPARSE_INDEX_32I;
    mcsparseIndexBase_t idxBase = MCSPARSE_INDEX_BASE_ZERO;
    macaDataType valueType = MACA_R_32F;
    int64_t row_num = 0;
    int64_t col_num = 0;
    int64_t nnz = 0;
    void* rows = nullptr;
    void* cols = nullptr;
    void* vals = nullptr;
    // strided batches (:194-196): batchStride moves the index and value arrays, offsetsBatchStride
    // the offsets array of CSR / CSC
    int64_t batchCount = 1;
    int64_t batchStride = 0;
    int64_t offsetsBatchStride = 0;
    // sizes of the transpose scratch layout, filled by *_bufferSize
    // (reference: src/common/mcsp_internal_transpose_sparse.hpp:517-549)
    int is_buffersize_called = 0;
    size_t assist_index_buffer_size = 0;
    size_t fixed_length_buffer_size = 0;
    SpmvPlan plan;
    SpmmSchedule schedule;
    SpmvBanded banded;
};

// How many compute units the current device shows and how many XCDs (L2 domains that take the workgroups of a
// launch in turn) they make up: topology.cpp.
namespace mcsp {
constexpr uint32_t kMaxXcds = 8;
struct Topology {
    uint32_t cus = 256;
    uint32_t xcds = 8;
};
Topology topology_of_cu_count(int cus);
Topology device_topology();
}  // namespace mcsp

// The kernels that ask for more dynamic LDS than the default limit: raises the limit for `kernel`; false when the
// device refuses (another LDS size), in which case the launcher launches nothing and its caller reports
// MCSP_STATUS_INTERNAL_ERROR instead of returning success with the output unwritten.
inline bool allow_dynamic_lds(const void* kernel, size_t bytes) {
    return hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)) == hipSuccess;
}
// After the launches of a path that raised an LDS limit: whether the runtime took them.
inline bool launches_taken() { return hipGetLastError() == hipSuccess; }

// Internal status, mapped to the public one exactly as the reference's wrapper does
// (src/include/mcsp_internal_types.h:13-30, src/wrapper/mcsp_interface_wrapper.cpp:5-42).
enum mcspStatus_t {
    MCSP_STATUS_SUCCESS = 0,
    MCSP_STATUS_INVALID_HANDLE = 1,
    MCSP_STATUS_NOT_IMPLEMENTED = 2,
    MCSP_STATUS_INVALID_POINTER = 3,
    MCSP_STATUS_INVALID_SIZE = 4,
    MCSP_STATUS_MEMORY_ERROR = 5,
    MCSP_STATUS_INTERNAL_ERROR = 6,
    MCSP_STATUS_INVALID_VALUE = 7,
    MCSP_STATUS_ARCH_MISMATCH = 8,
    MCSP_STATUS_ZERO_PIVOT = 9,
    MCSP_STATUS_NOT_INITIALIZED = 10,
    MCSP_STATUS_TYPE_MISMATCH = 11,
    MCSP_STATUS_MAPPING_ERROR = 12,
    MCSP_STATUS_EXECUTION_FAILED = 13,
    MCSP_STATUS_MATRIX_TYPE_NOT_SUPPORTED = 14,
    MCSP_STATUS_INSUFFICIENT_RESOURCES = 15
};
mcsparseStatus_t to_public_status(mcspStatus_t s);

static inline size_t value_size(macaDataType t) {
    switch (t) {
        case MACA_R_32F: return 4;
        case MACA_R_64F: return 8;
        case MACA_C_32F: return 8;
        case MACA_C_64F: return 16;
        case MACA_R_16F: case MACA_R_16BF: return 2;
        case MACA_C_16F: case MACA_C_16BF: return 4;
        case MACA_R_8I: return 1;
        case MACA_R_32I: return 4;
        default: return 0;
    }
}

// Bits needed to write n: 0 -> 0, 1 -> 1, 2..3 -> 2 ...
// (reference: src/include/mcsp_internal_host_utils.hpp:25-32)
static inline uint32_t bit_length(uint32_t n) {
    uint32_t b = 0;
    while (n) { ++b; n >>= 1; }
    return b;
}

// ---------------------------------------------------------------------------------------
// Device work.  Every function enqueues on `stream` and returns without synchronising
// unless stated.  Index arrays are unsigned 32-bit.  "base" is 0 or 1.
// ---------------------------------------------------------------------------------------
namespace mcsp {

typedef uint32_t idx_t;

// ---- host layer shared between entry points (api_compute.cpp) ----
// spmv_check: the argument checks of mcsparseSpMV.  buffer_bytes != 0 states how large `buffer` is:
// a call that needs more is refused with INSUFFICIENT_RESOURCES.  may_read_back = false asks for a
// call free of device-to-host copies: no row-length analysis (a structure without a plan runs the
// merge family) and host scalars only.  spmv_call: the checks, then the launches.
mcspStatus_t spmv_check(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha, mcsparseSpMatDescr_t matA,
                        mcsparseDnVecDescr_t vecX, const void* beta, mcsparseDnVecDescr_t vecY,
                        macaDataType computeType, const void* buffer, size_t buffer_bytes, bool may_read_back);
mcspStatus_t spmv_call(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha, mcsparseSpMatDescr_t matA,
                       mcsparseDnVecDescr_t vecX, const void* beta, mcsparseDnVecDescr_t vecY,
                       macaDataType computeType, void* buffer, size_t buffer_bytes, bool may_read_back,
                       mcsparseSpMVAlg_t alg = MCSPARSE_SPMV_ALG_DEFAULT);

// Kernel family (and lanes per row / tile order) for a structure with these row-length bins: the
// 33 counters and the longest row that launch_row_bins leaves, read back to the host.  A pure
// function, so the choice can be pinned on a table of histograms without a GPU.
void spmv_plan_from_bins(const uint32_t* bins, int64_t m, int64_t nnz, int64_t x_bytes, int* family, int* lanes);

// ---- row-length analysis (analysis.hip) ----
// hist_out: MCSPARSE_ROW_BIN_COUNT counters followed by the longest row length (34 x u32),
// zeroed by this call.  row_bins may be null.
void launch_row_bins(hipStream_t stream, idx_t m, const idx_t* row_ptr, idx_t base, uint8_t* row_bins,
                     uint32_t* hist_out);

// ---- SpMV (spmv.hip) ----
struct SpmvArgs {
    idx_t m, n, nnz, base;
    const idx_t* row_ptr;
    const idx_t* col;
    const void* val;
    const void* x;
    void* y;
};
// y = alpha*A*x + beta*y; beta == 0 never reads y.
template <typename T>
void launch_spmv_vector(hipStream_t stream, const SpmvArgs& a, T alpha, T beta, int lanes);
// workspace: spmv_merge_workspace_bytes(m, nnz, sizeof(T)) bytes of device scratch.
size_t spmv_merge_workspace_bytes(idx_t m, idx_t nnz, size_t value_bytes);
// order_tiles: the tiles run in the order of their first column.
template <typename T>
void launch_spmv_merge(hipStream_t stream, const SpmvArgs& a, T alpha, T beta, void* workspace, bool order_tiles);
// The same sums over rows when a.val already holds the products value * x (a.col and a.x unused).
template <typename T>
void launch_row_sums_merge(hipStream_t stream, const SpmvArgs& a, T alpha, T beta, void* workspace);
int spmv_pick_lanes(idx_t m, idx_t nnz);

// ---- column-banded SpMV (spmv_banded.hip) ----
// Rows of a tile (one workgroup's share of a band) and the width of a band of x in bytes.
constexpr int kBandedMaxRowsPerTile = 1024;
constexpr size_t kBandedBandBytes = size_t(2) << 20;
struct BandedLayout {
    // kept between preprocess and SpMV: [0, keep); scratch of the build: [keep, total)
    size_t tile_ptr, xcd_start, entries, vals, partials, keep, tmp_keys, tmp_rows, sort_ws, total;
    // by_column only: the nonzeros sorted by column (the source of the build) and the sorted tile numbers
    size_t src_cols, src_rows, src_vals, tile_ids;
    size_t next_unit;  // by_column: one work counter per XCD
};
// The same decision for the copy whose tiles are in column order (BandedShape::by_column): tiles of
// kColumnOrderMinRows .. kColumnOrderRows rows, at most 64 planes of partial sums and 65536 tiles, and at
// least one unit of work per compute unit.
constexpr uint32_t kColumnOrderRows = 16384;
constexpr uint32_t kColumnOrderMinRows = 2048;
bool column_order_shape(idx_t m, idx_t n, idx_t nnz, idx_t base, size_t value_bytes, size_t band_bytes,
                        BandedShape* out);
// How the gathers of an SpMV are spread over the 128-byte lines of x: launch_line_gathers fills, at the head of
// `workspace` (line_gathers_workspace_bytes), kLineGatherBins pairs (lines, gathers) binned by the highest bit of a
// line's count: of_rows from the row lengths (the gathered element is the row: a transposing direction), else from
// a sample of the indices.  gathers_favour_wide_groups reads the pairs once they are on the host.
constexpr uint32_t kLineGatherBins = 32;
constexpr double kHotLines = 16384;
size_t line_gathers_workspace_bytes(idx_t gathered, size_t value_bytes);
void launch_line_gathers(hipStream_t stream, bool of_rows, idx_t gathered, idx_t nnz, idx_t base, const idx_t* ptr,
                         const idx_t* ind, size_t value_bytes, void* workspace);
bool gathers_favour_wide_groups(const unsigned long long* bins);
// r_keys / c_keys: row + base and column + base of every nonzero of the matrix to copy, in an order
// sorted by the 128-byte line of x the column lies in (any order inside a line); vals in the same
// order.  Neither is written.
void launch_column_order_build(hipStream_t stream, const BandedShape& s, idx_t m, idx_t nnz, idx_t base,
                               const idx_t* r_keys, const idx_t* c_keys, const void* vals, size_t value_bytes,
                               void* region);
// False when the banded copy cannot help or cannot be built: x fits one band, more than 256 bands.
bool banded_shape(idx_t m, idx_t n, idx_t nnz, idx_t base, size_t value_bytes, size_t band_bytes, BandedShape* out);
BandedLayout banded_layout(const BandedShape& s, idx_t m, idx_t nnz, size_t value_bytes);
// Builds the banded copy in `region` (banded_layout(...).total bytes); xcd_start (9 x u32 at
// region + layout.xcd_start) is then read back by the caller and turned into the grid by banded_grid.
void launch_banded_build(hipStream_t stream, const BandedShape& s, idx_t m, idx_t nnz, idx_t base, const idx_t* row_ptr,
                         const idx_t* col, const void* val, size_t value_bytes, void* region);
uint32_t banded_grid(const uint32_t* xcd_start_host);
template <typename T>
bool launch_spmv_banded(hipStream_t stream, const BandedShape& s, uint32_t grid, const SpmvArgs& a, T alpha, T beta,
                        void* region);

// Streaming kernels that measure what the memory takes by itself (analysis.hip): mode 0 reads src, 1 writes dst,
// 2 copies; bytes a multiple of 16 and below 2^44, arrays 16-byte aligned, sink = at least one uint32 for mode 0.
void launch_stream_probe(hipStream_t stream, int mode, const void* src, void* dst, uint64_t bytes, uint32_t* sink,
                         uint32_t sink_words);

// ---- SpMM (spmm.hip) ----
struct SpmmArgs {
    idx_t m, n, k, nnz, base;   // C is m x n, A is m x k
    const idx_t* row_ptr;
    const idx_t* col;
    const void* val;
    const void* B;
    int64_t ldb;
    bool b_row_major;           // element (kk, j) of op(B) at kk*ldb + j, else at j*ldb + kk
    void* C;
    int64_t ldc;
    bool c_row_major;
    // Rows of more than long_row nonzeros (0: none are treated apart) are left out by the row kernels and taken in
    // pieces by the kernels of spmm_long.hip, which need spmm_long_rows_bytes(nnz, long_n, value size) bytes at
    // long_ws; long_n is the width the area was sized for (at least n).
    idx_t long_row = 0;
    void* long_ws = nullptr;
    int64_t long_n = 0;
};
template <typename T>
void launch_spmm(hipStream_t stream, const SpmmArgs& a, T alpha, T beta);

// Long rows (spmm_long.hip): a lane group of the row kernels walks a row by itself, so a row of tens of thousands
// of nonzeros outlasts the rest of the launch.  Rows above kSpmmLongRow nonzeros are cut into pieces of
// kSpmmLongChunk, a workgroup each.  The first 2 * kAlign bytes of the area are not used by these kernels (the
// row-length analysis of the call writes its counters there).
constexpr idx_t kSpmmLongRow = 1024;
constexpr idx_t kSpmmLongChunk = 4096;
size_t spmm_long_rows_bytes(idx_t nnz, int64_t n, size_t value_bytes);
void launch_spmm_long_find(hipStream_t stream, const SpmmArgs& a, size_t value_bytes);
template <typename T>
void launch_spmm_long_rows(hipStream_t stream, const SpmmArgs& a, T alpha, T beta);

// Row-group schedule of a CSR structure (spmm.hip): for every group of kSpmmGroupRows
// consecutive rows the merged list of their column indices, each entry =
// (zero-based column << kSpmmGroupRows) | one bit per row of the group that has the column.
// group_ptr has groups+1 offsets into entries; span_sum (one u64) is the sum over the groups of
// the distance between their first and last column.  Groups holding more than kSpmmMaxMergedGroup
// nonzeros get no entries and are processed row by row.
constexpr int kSpmmGroupRows = 4;
constexpr idx_t kSpmmMaxMergedGroup = 2048;
constexpr int64_t kSpmmMaxScheduledColumns = int64_t(1) << (32 - kSpmmGroupRows);
constexpr uint64_t spmm_groups(idx_t m) { return (static_cast<uint64_t>(m) + kSpmmGroupRows - 1) / kSpmmGroupRows; }
struct SpmmScheduleLayout {
    size_t group_ptr, span_sum, entries, scan_ws, total;
};
SpmmScheduleLayout spmm_schedule_layout(idx_t m, idx_t nnz);
// Fills group_ptr and entries inside `schedule` (laid out as spmm_schedule_layout says).
void launch_spmm_schedule(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, const idx_t* row_ptr, const idx_t* col,
                          void* schedule);
// Same result as launch_spmm for a row-major op(B) whose rows allow 128-bit accesses
// (spmm_schedule_usable says so), reading every B row once per row group.
bool spmm_schedule_usable(const SpmmArgs& a, size_t value_bytes);
template <typename T>
void launch_spmm_scheduled(hipStream_t stream, const SpmmArgs& a, const void* schedule, uint32_t total_entries,
                           uint64_t mean_span, T alpha, T beta);

// Diagonal-block schedule of a CSR structure (spmm_blocks.hip), the second kind mcsparseSpMM_preprocess can leave in
// the region spmm_schedule_layout describes: for every group of kSpmmBlockRows consecutive rows a list of blocks
// {int32 c, uint32 shape}.  A block holds n <= kSpmmBlockMaxDiagonals consecutive diagonals (shape bits 0-2: n); its
// p-th diagonal is held by the rows lo_p .. hi_p - 1 of the group (shape bits 8+8p..11+8p: lo_p, 12+8p..15+8p: hi_p),
// and row r holds it in column c + r + p (zero-based).  The blocks of a group consume every row's nonzeros in
// storage order.  group_ptr's place holds the groups+1 offsets into the blocks, entries' place the blocks (8 bytes
// each) and, at its end, the order in which the kernel takes the groups (the schedule is only kept when they fit),
// span_sum's place three counters: the sum of the groups' column spans and the number of rows of op(B) all blocks
// load (u64), the most nonzeros in one group (u32).
constexpr int kSpmmBlockRows = 8;
constexpr int kSpmmBlockMaxDiagonals = 3;
constexpr uint64_t spmm_block_groups(idx_t m) { return (static_cast<uint64_t>(m) + kSpmmBlockRows - 1) / kSpmmBlockRows; }
// Counts the blocks of every group and scans the counts (the total lands in slot `groups` of the offsets).
void launch_spmm_block_count(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, const idx_t* row_ptr, const idx_t* col,
                             void* schedule);
// Strip schedule of a CSR structure (spmm_strips.hip), the third kind: a group is kSpmmStrips strips of
// kSpmmStripRows consecutive rows, strip q beginning `stride` rows behind strip q - 1; the rows are cut into stretches
// of kSpmmStrips * stride rows, each holding stride / kSpmmStripRows groups.  Blocks are 16 bytes (see the file), the
// region is used like the one of the block schedule, and the counters' place also holds the stride.
constexpr int kSpmmStripRows = 4;
constexpr int kSpmmStrips = 4;
// values of a strip the kernel copies into LDS; a structure with longer strips is left to the groups of eight rows
constexpr uint32_t kSpmmStripStagedValues = 128;
constexpr uint64_t spmm_strip_groups(idx_t m, uint32_t stride) {
    return (static_cast<uint64_t>(m) + static_cast<uint64_t>(kSpmmStrips) * stride - 1) /
           (static_cast<uint64_t>(kSpmmStrips) * stride) * (stride / kSpmmStripRows);
}
// stride is one the schedule can be built with for a matrix of m rows
bool spmm_strip_stride_usable(idx_t m, uint32_t stride);
void launch_spmm_strip_count(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, uint32_t stride, const idx_t* row_ptr,
                             const idx_t* col, void* schedule);
void launch_spmm_strip_fill(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, uint32_t stride, const idx_t* row_ptr,
                            const idx_t* col, void* schedule);
bool spmm_strip_schedule_fits(idx_t m, idx_t nnz, uint32_t stride, uint32_t blocks);
// Same conditions on the operands as the block schedule (spmm_blocks_usable).
template <typename T>
void launch_spmm_strips(hipStream_t stream, const SpmmArgs& a, const void* schedule, uint32_t stride, uint32_t total_blocks,
                        uint32_t longest_strip, uint64_t mean_span, T alpha, T beta);

// Whether `blocks` blocks of 8 bytes and the order of the groups (4 bytes each) fit the entries' place.
bool spmm_block_schedule_fits(idx_t m, idx_t nnz, uint32_t blocks);
// Writes the blocks and the order in which the kernel takes the groups; only after the count, and only when
// spmm_block_schedule_fits says so.
void launch_spmm_block_fill(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, const idx_t* row_ptr, const idx_t* col,
                            void* schedule);
bool spmm_blocks_usable(const SpmmArgs& a, size_t value_bytes);
// longest_group: the most nonzeros any group with blocks holds (the third counter the count leaves).
template <typename T>
void launch_spmm_blocks(hipStream_t stream, const SpmmArgs& a, const void* schedule, uint32_t total_blocks,
                        uint32_t longest_group, uint64_t mean_span, T alpha, T beta);

// Dense transposes for column-major SpMM operands (spmm.hip).  src is rows x cols, row-major with
// leading dimension lds.  launch_transpose: dst (cols x rows_padded, ldd) = transpose(src), the columns
// [rows, rows_padded) of dst zero.  launch_transpose_accumulate: dst = beta * dst + transpose(src);
// beta == 0 does not read dst.
template <typename T>
void launch_transpose(hipStream_t stream, idx_t rows, idx_t cols, idx_t rows_padded, const T* src, int64_t lds, T* dst,
                      int64_t ldd);
template <typename T>
void launch_transpose_accumulate(hipStream_t stream, idx_t rows, idx_t cols, const T* src, int64_t lds, T* dst,
                                 int64_t ldd, T beta);

// ---- conversions (convert.hip) ----
void launch_csr2coo(hipStream_t stream, idx_t m, idx_t nnz, const idx_t* row_ptr, idx_t base, idx_t* coo_rows);
void launch_coo2csr(hipStream_t stream, idx_t nnz, idx_t m, const idx_t* coo_rows, idx_t base, idx_t* row_ptr);
size_t csr2csc_workspace_bytes(idx_t m, idx_t n, idx_t nnz, size_t value_bytes);
// value_bytes 0 = structure only.  Writes col_ptr[n+1], row_ind[nnz] (both + base) and csc_val.
void launch_csr2csc(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, const void* csr_val, const idx_t* row_ptr,
                    const idx_t* col, void* csc_val, idx_t* row_ind, idx_t* col_ptr, size_t value_bytes,
                    idx_t base, void* workspace);
// products[nnz] = value * x[row] of every nonzero in the order of a stable sort by column, and
// col_ptr[n+1] (+ base): what op(A) = A^T needs of the transpose.  value_bytes is 4 (fp32 values and
// x) or 8 (fp64); workspace of transposed_products_workspace_bytes(nnz, value_bytes) bytes.
size_t transposed_products_workspace_bytes(idx_t nnz, size_t value_bytes);
void launch_transposed_products(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, const void* csr_val, const idx_t* row_ptr,
                                const idx_t* col, const void* x, void* products, idx_t* col_ptr, size_t value_bytes,
                                idx_t base, void* workspace);

// The same products in up to 256 buckets of 2^shift neighbouring columns (index base taken off: bucket b
// holds columns [b << shift, (b + 1) << shift)), bucket b starting at starts[b * stride] and ending where
// the next begins (the last at nnz); inside a bucket the pairs are in CSR order, not sorted, and keys[]
// holds a column's low `shift` bits, its place in the bucket.  Both arrays may be read up to the next even index past nnz.  One pass over the nonzeros instead of the three of a
// full sort: for callers that then add the products of a column in any order.  The shape function says
// whether the shape allows it (more than 2^14 and at most 2^22 columns: a bucket's sums must fit in LDS as
// doubles).
constexpr uint32_t kBucketMinKeyBits = 15;
constexpr uint32_t kBucketMaxShift = 14;
struct BucketedProducts {
    const uint16_t* keys = nullptr;
    const uint32_t* starts = nullptr;
    uint32_t stride = 0, shift = 0, buckets = 0;
    void* spare = nullptr;  // part of the workspace the pass did not use, for the sums of buckets that are split
    size_t spare_bytes = 0;
};
bool bucketed_products_shape(idx_t n, uint32_t* shift);
void launch_bucketed_products(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, const void* csr_val, const idx_t* row_ptr,
                              const idx_t* col, const void* x, void* products, size_t value_bytes, idx_t base,
                              void* workspace, BucketedProducts* out);
// y[c] = alpha * (sum of the products of column c) + beta * y[c] for all n columns, from such buckets;
// the sums are formed in LDS in the order the wavefronts reach the products.
template <typename T>
bool launch_bucket_sums(hipStream_t stream, idx_t n, idx_t nnz, const BucketedProducts& b, const T* products, T* y,
                        T alpha, T beta);

// y = alpha * A^T x + beta * y for an m x n matrix with at most 2^14 columns and many nonzeros per
// column, without sorting anything: shares of the nonzeros are summed into copies of y in LDS, the copies
// into y.  rows[nnz] = row + base of every nonzero (COO rows, or csr2coo of the offsets); workspace of
// skinny_transpose_workspace_bytes(n) bytes, which the shape function keeps below 16 bytes per nonzero.
constexpr uint32_t kSkinnyMinNonzerosPerColumn = 128;
bool skinny_transpose_shape(idx_t n, idx_t nnz);
size_t skinny_transpose_workspace_bytes(idx_t n);
template <typename T>
bool launch_skinny_transpose(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, idx_t base, const idx_t* rows,
                             const idx_t* col, const T* val, const T* x, T* y, T alpha, T beta, void* workspace);

// One stable radix pass over the nonzeros of a CSR matrix where they lie, on band_bits (<= 8) bits
// of the keys from bit band_shift on (key = column index, index base included): cols_out / rows_out
// (row + base) / vals_out hold the nonzeros band by band, inside a band in CSR order.
size_t band_sort_workspace_bytes(idx_t nnz);
void launch_sort_by_column_band(hipStream_t stream, idx_t m, idx_t nnz, idx_t base, const idx_t* row_ptr, const idx_t* col,
                                const void* val, size_t value_bytes, uint32_t band_shift, uint32_t band_bits,
                                idx_t* cols_out, idx_t* rows_out, void* vals_out, void* workspace);

// (column, row + base, value) arrays of the nonzeros in the order of a stable sort by column: csr2csc
// without the offsets; the low_bits lowest bits of the column keys are left out of the sort.
// workspace: csr2csc_workspace_bytes.
void launch_sort_by_column(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, idx_t base, const idx_t* row_ptr,
                           const idx_t* col, const void* val, size_t value_bytes, uint32_t low_bits, idx_t* cols_out,
                           idx_t* rows_out, void* vals_out, void* workspace);
// Stable sort of (key, aux, value) triples on the low key_bits (<= 16) of the keys; outputs apart from
// the inputs and from the workspace (csr2csc_workspace_bytes).
void launch_sort_triples(hipStream_t stream, idx_t nnz, uint32_t key_bits, const idx_t* keys_in, const idx_t* aux_in,
                         const void* vals_in, idx_t* keys_out, idx_t* aux_out, void* vals_out, size_t value_bytes,
                         void* workspace);

// ---- index sorts (convert.hip) --------------------------------------------------------------
size_t index_sort_workspace_bytes(idx_t nnz);
// In-place stable sort of COO entries by (major, minor); perm (may be null) moves with them.
// The extents bound the index values (inclusive, so one-based indices are covered).
void launch_coosort(hipStream_t stream, idx_t major_extent, idx_t minor_extent, idx_t nnz, idx_t* major, idx_t* minor,
                    idx_t* perm, void* workspace);
// Sorts the column indices inside every row of a CSR structure; perm (may be null) moves along.
void launch_csrsort(hipStream_t stream, idx_t m, idx_t n, idx_t nnz, idx_t base, const idx_t* row_ptr, idx_t* col,
                    idx_t* perm, void* workspace);
void launch_identity(hipStream_t stream, idx_t n, idx_t* p);
// In-place exclusive prefix sum of n 32-bit counters.
size_t exclusive_scan_workspace_bytes(uint64_t n);
void launch_exclusive_scan_u32(hipStream_t stream, uint32_t* data, uint64_t n, void* workspace);
// x_val[i] = y[x_ind[i] - base]
template <typename T>
void launch_gather(hipStream_t stream, idx_t nnz, const T* y, T* x_val, const idx_t* x_ind, idx_t base);
// dst[i] = low 32 bits of src[i]
void launch_narrow_indices(hipStream_t stream, const int64_t* src, idx_t* dst, uint64_t n);

}  // namespace mcsp

#endif  // MCSPARSE_AMD_INTERNAL_H_
