// mcsparseSpMV / mcsparseSpMM / conversion entry points: argument validation in the order of the
// reference's host drivers, scratch-buffer carving, kernel-family choice and launches.
#include <cmath>
#include <cstring>

#include "internal.h"

#include <algorithm>

using mcsp::idx_t;

namespace {

// Leading part of every SpMV scratch buffer: the 34 counters of the row-length analysis.
constexpr size_t kAnalysisBytes = align_up((MCSPARSE_ROW_BIN_COUNT + 1) * sizeof(uint32_t));

bool fits_32(int64_t v) { return (v >> 32) == 0; }

// A stream that is being captured into a HIP graph cannot be synchronised: trying to would fail and
// invalidate the caller's capture.
bool stream_is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing(stream, &status) == hipSuccess && status != hipStreamCaptureStatusNone;
}

// Reads a scalar of the compute type.  Device pointer mode costs one blocking copy, like the
// reference (src/include/mcsp_internal_host_utils.hpp:34-63).
template <typename T>
bool scalar_to_host(mcsparseHandle_t h, const void* p, T* out) {
    if (h->ptr_mode == MCSPARSE_POINTER_MODE_HOST) {
        std::memcpy(out, p, sizeof(T));
        return true;
    }
    if (stream_is_capturing(h->stream)) return false;  // a blocking read cannot be captured
    if (hipMemcpyAsync(out, p, sizeof(T), hipMemcpyDeviceToHost, h->stream) != hipSuccess) return false;
    return hipStreamSynchronize(h->stream) == hipSuccess;
}

// The CSR-shaped view a call works on.  CSC inputs are re-read as the CSR of the transpose
// (src/kernels/level2/spmv/mcsp_spmv_gpu.cpp:734-739); row-sorted COO inputs get their row
// offsets built in the scratch buffer by coo2csr (:817-825), so `ptr` is null until then.
struct CsrView {
    int64_t m, n;        // shape of the matrix whose CSR arrays these are
    const idx_t* ptr;    // m+1 offsets (null for COO: built into the scratch buffer)
    const idx_t* ind;    // nnz indices
    const void* val;
    const idx_t* coo_rows;  // COO only: the nnz row indices the offsets are built from
    bool transpose;      // the call needs view^T
};

CsrView make_view(const mcsparseSpMatDescr* A, mcsparseOperation_t op, const idx_t* rows32 = nullptr,
                  const idx_t* cols32 = nullptr) {
    const idx_t* a_rows = rows32 != nullptr ? rows32 : static_cast<const idx_t*>(A->rows);
    const idx_t* a_cols = cols32 != nullptr ? cols32 : static_cast<const idx_t*>(A->cols);
    CsrView v;
    const bool op_t = op != MCSPARSE_OPERATION_NON_TRANSPOSE;
    v.coo_rows = nullptr;
    if (A->format == MCSPARSE_FORMAT_CSC) {
        v.m = A->col_num;
        v.n = A->row_num;
        v.ptr = a_cols;  // column offsets
        v.ind = a_rows;  // row indices
        v.transpose = !op_t;
    } else {
        v.m = A->row_num;
        v.n = A->col_num;
        v.ptr = a_rows;
        v.ind = a_cols;
        v.transpose = op_t;
        if (A->format == MCSPARSE_FORMAT_COO) {
            v.coo_rows = v.ptr;
            v.ptr = nullptr;
        }
    }
    v.val = A->vals;
    return v;
}

bool format_is_built(mcsparseFormat_t f) {
    return f == MCSPARSE_FORMAT_CSR || f == MCSPARSE_FORMAT_CSC || f == MCSPARSE_FORMAT_COO;
}

// Scratch layout of an SpMV call, all parts aligned to 128 bytes:
//   [analysis][merge workspace][COO only: row offsets m+1]
//   transposing calls add [col_ptr n+1][products nnz][workspace of the sort by column]
//   64-bit index arrays add their narrowed copies at the end
// (the reference keeps the whole transpose there, mcsp_spmv_gpu.cpp:308 and :813-831).
struct SpmvLayout {
    size_t merge_ws, coo_ptr, col_ptr, vals, csr2csc_ws, narrow, total;
};

SpmvLayout spmv_layout(const CsrView& v, int64_t nnz, size_t value_bytes, size_t narrow) {
    SpmvLayout l = {};
    const int64_t out_rows = v.transpose ? v.n : v.m;  // rows of the matrix the SpMV kernel sees
    size_t off = kAnalysisBytes;
    l.merge_ws = off;
    off += align_up(mcsp::spmv_merge_workspace_bytes(static_cast<idx_t>(out_rows), static_cast<idx_t>(nnz),
                                                     value_bytes));
    l.coo_ptr = off;
    if (v.coo_rows != nullptr) off += align_up(static_cast<size_t>(v.m + 1) * sizeof(idx_t));
    if (v.transpose) {
        l.col_ptr = off;
        off += align_up(static_cast<size_t>(v.n + 1) * sizeof(idx_t));
        l.vals = off;
        off += align_up(static_cast<size_t>(nnz) * value_bytes);
        l.csr2csc_ws = off;
        off += align_up(mcsp::transposed_products_workspace_bytes(static_cast<idx_t>(nnz), value_bytes));
    }
    l.narrow = off;
    off += narrow;
    l.total = off < kMinBuffer ? kMinBuffer : off;
    return l;
}

// Checks shared by SpMV and SpMV_bufferSize, in the reference's order
// (mcsp_spmv_gpu.cpp:686-714 and :309-334).  `need_buffer` is the SpMV-only externalBuffer check,
// which sits between the size-range and the format checks; `other_pointers_ok` carries the
// bufferSize pointer of SpMV_bufferSize, which the reference tests with the other pointers.
mcspStatus_t check_spmv_args(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha,
                             const mcsparseSpMatDescr* A, const mcsparseDnVecDescr* x, const void* beta,
                             const mcsparseDnVecDescr* y, bool other_pointers_ok, bool need_buffer,
                             const void* buffer) {
    if (handle == nullptr) return MCSP_STATUS_INVALID_HANDLE;
    if (alpha == nullptr || beta == nullptr || A == nullptr || x == nullptr || y == nullptr || !other_pointers_ok)
        return MCSP_STATUS_INVALID_POINTER;
    if (!fits_32(A->row_num) || !fits_32(A->col_num) || !fits_32(A->nnz) || !fits_32(x->size) || !fits_32(y->size))
        return MCSP_STATUS_NOT_IMPLEMENTED;
    if (need_buffer && buffer == nullptr) return MCSP_STATUS_INVALID_POINTER;
    if (!(A->format == MCSPARSE_FORMAT_CSR || A->format == MCSPARSE_FORMAT_COO ||
          A->format == MCSPARSE_FORMAT_COO_AOS || A->format == MCSPARSE_FORMAT_CSC))
        return MCSP_STATUS_NOT_IMPLEMENTED;
    const bool op_n = opA == MCSPARSE_OPERATION_NON_TRANSPOSE;
    if (!((op_n && x->size == A->col_num && y->size == A->row_num) ||
          (!op_n && x->size == A->row_num && y->size == A->col_num)))
        return MCSP_STATUS_INVALID_SIZE;
    return MCSP_STATUS_SUCCESS;
}

// Row and column index types must agree; 32I and 64I are the two the reference dispatches on
// (mcsp_spmv_gpu.cpp:1123-1133).
mcspStatus_t check_index_types(const mcsparseSpMatDescr* A) {
    if (A->rowIdxType == MCSPARSE_INDEX_32I && A->colIdxType == MCSPARSE_INDEX_32I) return MCSP_STATUS_SUCCESS;
    if (A->rowIdxType == MCSPARSE_INDEX_64I && A->colIdxType == MCSPARSE_INDEX_64I) return MCSP_STATUS_SUCCESS;
    return MCSP_STATUS_NOT_IMPLEMENTED;
}

// The kernels work on 32-bit indices.  Every extent of a matrix is checked to be below 2^32
// (as in the reference, mcsp_spmv_gpu.cpp:698-701), so the entries of 64-bit index arrays fit
// 32 bits: a call on such a matrix first copies its two index arrays, narrowed, into the
// scratch buffer and runs on the copies.  The reference instantiates its kernels for int64
// instead (mcsp_spmv_gpu.cpp:1128-1129); the results are the same.
bool wide_indices(const mcsparseSpMatDescr* A) { return A->rowIdxType == MCSPARSE_INDEX_64I; }

// Lengths of the descriptor's `rows` and `cols` arrays.
void index_array_lengths(const mcsparseSpMatDescr* A, size_t* rows_len, size_t* cols_len) {
    const size_t nnz = static_cast<size_t>(A->nnz);
    switch (A->format) {
        case MCSPARSE_FORMAT_CSR: *rows_len = static_cast<size_t>(A->row_num) + 1; *cols_len = nnz; break;
        case MCSPARSE_FORMAT_CSC: *rows_len = nnz; *cols_len = static_cast<size_t>(A->col_num) + 1; break;
        default: *rows_len = nnz; *cols_len = nnz; break;  // COO
    }
}

size_t narrow_bytes(const mcsparseSpMatDescr* A) {
    if (!wide_indices(A)) return 0;
    size_t rl, cl;
    index_array_lengths(A, &rl, &cl);
    return align_up(rl * sizeof(idx_t)) + align_up(cl * sizeof(idx_t));
}

// 32-bit `rows` and `cols` arrays of the descriptor: the caller's own, or narrowed copies
// written to `region` (narrow_bytes(A) bytes).
struct IndexArrays {
    const idx_t* rows;
    const idx_t* cols;
};
IndexArrays index_arrays(mcsparseHandle_t h, const mcsparseSpMatDescr* A, char* region) {
    IndexArrays out = {static_cast<const idx_t*>(A->rows), static_cast<const idx_t*>(A->cols)};
    if (!wide_indices(A)) return out;
    size_t rl, cl;
    index_array_lengths(A, &rl, &cl);
    idx_t* r32 = reinterpret_cast<idx_t*>(region);
    idx_t* c32 = reinterpret_cast<idx_t*>(region + align_up(rl * sizeof(idx_t)));
    if (A->rows != nullptr) mcsp::launch_narrow_indices(h->stream, static_cast<const int64_t*>(A->rows), r32, rl);
    if (A->cols != nullptr) mcsp::launch_narrow_indices(h->stream, static_cast<const int64_t*>(A->cols), c32, cl);
    out.rows = A->rows != nullptr ? r32 : nullptr;
    out.cols = A->cols != nullptr ? c32 : nullptr;
    return out;
}

// Chooses the kernel family for a structure; runs the row-length analysis (one kernel, one
// blocking 136-byte read-back) the first time a structure is seen.  `ptr` are the offsets to
// analyse, `signature` the caller's array that identifies the structure.
mcspStatus_t ensure_plan(mcsparseHandle_t h, mcsparseSpMatDescr* A, const idx_t* ptr, const void* signature,
                         int64_t m, int64_t nnz, int64_t x_bytes, void* buffer, bool may_read_back) {
    SpmvPlan& p = A->plan;
    if (p.valid && p.rows == signature && p.m == m && p.nnz == nnz && p.base == static_cast<int>(A->idxBase))
        return MCSP_STATUS_SUCCESS;
    // The analysis ends in a blocking read-back, which a stream under graph capture cannot do: the
    // plan only steers speed, so such a call goes without one.
    if (may_read_back && p.forced_family == kFamilyAuto && stream_is_capturing(h->stream)) may_read_back = false;
    if (!may_read_back && p.forced_family == kFamilyAuto) {
        // No analysis without its read-back: the merge family in storage order is correct and balanced
        // for every structure.  The plan stays invalid, so a later call that may read back analyses.
        p.valid = false;
        p.family = kFamilyMerge;
        p.lanes = 0;
        return MCSP_STATUS_SUCCESS;
    }
    p.rows = signature;
    p.m = m;
    p.nnz = nnz;
    p.base = static_cast<int>(A->idxBase);
    const int mean_lanes = mcsp::spmv_pick_lanes(static_cast<idx_t>(m), static_cast<idx_t>(nnz));
    if (p.forced_family != kFamilyAuto) {
        p.family = p.forced_family;
        // merge family: lanes != 0 asks for the tiles to run in the order of their first column
        p.lanes = p.family == kFamilyVector ? (p.forced_lanes ? p.forced_lanes : mean_lanes) : (p.forced_lanes ? 1 : 0);
        p.max_row_len = 0;
        p.valid = true;
        return MCSP_STATUS_SUCCESS;
    }
    uint32_t* dev_hist = static_cast<uint32_t*>(buffer);
    mcsp::launch_row_bins(h->stream, static_cast<idx_t>(m), ptr, static_cast<idx_t>(A->idxBase), nullptr, dev_hist);
    uint32_t host_hist[MCSPARSE_ROW_BIN_COUNT + 1];
    if (hipMemcpyAsync(host_hist, dev_hist, sizeof(host_hist), hipMemcpyDeviceToHost, h->stream) != hipSuccess ||
        hipStreamSynchronize(h->stream) != hipSuccess)
        return MCSP_STATUS_INTERNAL_ERROR;
    std::memcpy(p.hist, host_hist, sizeof(p.hist));
    p.max_row_len = host_hist[MCSPARSE_ROW_BIN_COUNT];
    mcsp::spmv_plan_from_bins(host_hist, m, nnz, x_bytes, &p.family, &p.lanes);
    if (p.family == kFamilyVector && p.forced_lanes) p.lanes = p.forced_lanes;
    p.valid = true;
    return MCSP_STATUS_SUCCESS;
}

// Where the banded copy of mcsparseSpMV_preprocess sits in its buffer: behind the scratch of a plain
// SpMV call, which mcsparseSpMV may still write (row-length analysis) when handed the same buffer.
size_t banded_region_offset(const mcsparseSpMatDescr* A, mcsparseOperation_t op, size_t value_bytes) {
    const CsrView v = make_view(A, op);
    return align_up(spmv_layout(v, A->nnz, value_bytes, narrow_bytes(A)).total);
}

// What mcsparseSpMV_preprocess builds a copy for: CSR, CSC and COO, 32- or 64-bit indices, fp32 / fp64.
// The copy is of the matrix the row kernels would run on: the arrays as they lie (CSR with op N, CSC
// with op T) or, for the transposing directions (CSR with op T, CSC with op N), their transpose, which
// the preprocess call builds once with csr2csc.  `shape` is that matrix's; *rows its number of rows.
bool banded_candidate(const mcsparseSpMatDescr* A, mcsparseOperation_t op, mcsparseSpMVAlg_t alg, BandedShape* shape) {
    if (!format_is_built(A->format)) return false;
    if (A->valueType != MACA_R_32F && A->valueType != MACA_R_64F) return false;
    const CsrView v = make_view(A, op);
    const int64_t rows = v.transpose ? v.n : v.m;
    const int64_t cols = v.transpose ? v.m : v.n;
    const size_t band_bytes = A->banded.band_bytes != 0 ? A->banded.band_bytes : mcsp::kBandedBandBytes;
    shape->by_column = false;
    // Only MCSPARSE_SPMV_CSR_ALG2 promises the same bits on every run (the meaning APIs of this family
    // give the values; the reference ignores alg).  Every other algorithm gets the faster copy, tiles in
    // column order with sums formed in LDS as the products arrive, where the shape allows it.
    if (alg != MCSPARSE_SPMV_CSR_ALG2 &&
        mcsp::column_order_shape(static_cast<idx_t>(rows), static_cast<idx_t>(cols), static_cast<idx_t>(A->nnz),
                                 static_cast<idx_t>(A->idxBase), value_size(A->valueType), band_bytes, shape))
        return true;
    return mcsp::banded_shape(static_cast<idx_t>(rows), static_cast<idx_t>(cols), static_cast<idx_t>(A->nnz),
                              static_cast<idx_t>(A->idxBase), value_size(A->valueType), band_bytes, shape);
}

// Scratch of the preprocess call behind the banded copy of a transposing direction: the transpose in
// CSR form and the workspace of the csr2csc that produces it.
struct TransposeScratch {
    size_t ptr, ind, vals, ws, total;
};
TransposeScratch transpose_scratch(const CsrView& v, int64_t nnz, size_t value_bytes) {
    TransposeScratch t;
    size_t off = 0;
    t.ptr = off; off += align_up(static_cast<size_t>(v.n + 1) * sizeof(idx_t));
    t.ind = off; off += align_up(static_cast<size_t>(nnz) * sizeof(idx_t));
    t.vals = off; off += align_up(static_cast<size_t>(nnz) * value_bytes);
    t.ws = off;
    off += align_up(mcsp::csr2csc_workspace_bytes(static_cast<idx_t>(v.m), static_cast<idx_t>(v.n),
                                                  static_cast<idx_t>(nnz), value_bytes));
    t.total = off;
    return t;
}

// The banded copy on the descriptor belongs to this call: same buffer, same arrays, same extents, same
// direction.
bool banded_matches(const mcsparseSpMatDescr* A, const void* buffer, size_t value_bytes, bool transposing,
                    mcsparseSpMVAlg_t alg) {
    const SpmvBanded& b = A->banded;
    // MCSPARSE_SPMV_CSR_ALG2 asks for the same bits on every run, which the copy in column order does not give
    if (b.shape.by_column && alg == MCSPARSE_SPMV_CSR_ALG2) return false;
    return b.valid && b.useful && b.buffer == buffer && b.rows == A->rows && b.cols == A->cols && b.vals == A->vals &&
           b.m == A->row_num && b.n == A->col_num && b.nnz == A->nnz && b.base == static_cast<int>(A->idxBase) &&
           b.type == A->valueType && value_size(b.type) == value_bytes && b.format == A->format &&
           b.transposed == transposing;
}

template <typename T>
mcspStatus_t spmv_typed(mcsparseHandle_t h, mcsparseSpMatDescr* A, mcsparseOperation_t op, const void* alpha,
                        const void* beta, const mcsparseDnVecDescr* x, mcsparseDnVecDescr* y, void* buffer,
                        bool may_read_back, mcsparseSpMVAlg_t alg) {
    T h_alpha, h_beta;
    if (!scalar_to_host(h, beta, &h_beta) || !scalar_to_host(h, alpha, &h_alpha))
        return stream_is_capturing(h->stream) ? MCSP_STATUS_NOT_IMPLEMENTED : MCSP_STATUS_INTERNAL_ERROR;
    // reference: mcsp_spmv_gpu.cpp:235-237 -- y is left untouched in both cases
    if (A->nnz == 0 || (h_alpha == T(0) && h_beta == T(0))) return MCSP_STATUS_SUCCESS;

    const idx_t nnz = static_cast<idx_t>(A->nnz);
    const idx_t base = static_cast<idx_t>(A->idxBase);
    char* buf = static_cast<char*>(buffer);
    CsrView v = make_view(A, op);
    const SpmvLayout l = spmv_layout(v, A->nnz, sizeof(T), narrow_bytes(A));
    // what identifies the structure to the plan cache: the caller's own array
    const void* signature = v.coo_rows != nullptr ? static_cast<const void*>(v.coo_rows) : v.ptr;
    if ((v.transpose || A->plan.forced_family == kFamilyAuto) && banded_matches(A, buffer, sizeof(T), v.transpose, alg)) {
        // mcsparseSpMV_preprocess has copied the matrix of this direction (for a transposing one, its
        // transpose) into the buffer: the caller's arrays are not read at all
        mcsp::SpmvArgs a;
        a.nnz = nnz;
        a.base = base;
        a.x = x->values;
        a.y = y->values;
        a.m = static_cast<idx_t>(v.transpose ? v.n : v.m);
        a.n = static_cast<idx_t>(v.transpose ? v.m : v.n);
        a.row_ptr = nullptr;
        a.col = nullptr;
        a.val = nullptr;
        // (a device that refuses the kernel's LDS size launches nothing: an error, not a y left unwritten)
        return mcsp::launch_spmv_banded<T>(h->stream, A->banded.shape, A->banded.grid, a, h_alpha, h_beta,
                                           buf + A->banded.region)
                   ? MCSP_STATUS_SUCCESS
                   : MCSP_STATUS_INTERNAL_ERROR;
    }
    // A call that does not run from the copy but is handed the copy's buffer may write over it: the copy
    // sits behind the scratch of its own direction only, and the scratch of this call (the other
    // direction, another value size) can reach further.  Such a call ends the copy; the next matching
    // call runs the direct kernels until preprocess is called again.
    if (A->banded.valid && A->banded.buffer == buffer && l.total > A->banded.region) A->banded.valid = false;
    if (wide_indices(A)) {
        const IndexArrays ia = index_arrays(h, A, buf + l.narrow);
        v = make_view(A, op, ia.rows, ia.cols);
    }
    if (v.coo_rows != nullptr) {
        idx_t* built = reinterpret_cast<idx_t*>(buf + l.coo_ptr);
        mcsp::launch_coo2csr(h->stream, nnz, static_cast<idx_t>(v.m), v.coo_rows, base, built);
        v.ptr = built;
    }
    mcsp::SpmvArgs a;
    a.nnz = nnz;
    a.base = base;
    a.x = x->values;
    a.y = y->values;

    if (!v.transpose) {
        a.m = static_cast<idx_t>(v.m);
        a.n = static_cast<idx_t>(v.n);
        a.row_ptr = v.ptr;
        a.col = v.ind;
        a.val = v.val;
        const mcspStatus_t st =
            ensure_plan(h, A, v.ptr, signature, v.m, A->nnz, v.n * static_cast<int64_t>(sizeof(T)), buffer,
                        may_read_back);
        if (st != MCSP_STATUS_SUCCESS) return st;
        if (A->plan.family == kFamilyMerge) {
            mcsp::launch_spmv_merge<T>(h->stream, a, h_alpha, h_beta, buf + l.merge_ws, A->plan.lanes != 0);
        } else {
            mcsp::launch_spmv_vector<T>(h->stream, a, h_alpha, h_beta, A->plan.lanes);
        }
        return MCSP_STATUS_SUCCESS;
    }

    // Transposing call.  The reference materialises the transpose in the scratch buffer on every call
    // (mcsp_spmv_gpu.cpp:797-845) -- the caller may have changed the values -- and then runs its row
    // kernel on it.  Here every call sorts (column, value * x[row]) pairs by column with the machinery
    // of csr2csc, which is a stable sort of one array less, and then sums the products of each column:
    // the sum of a column adds the same products in the same order (row order) as a row kernel on the
    // transpose would, without the gathers from x.
    idx_t* t_ptr = reinterpret_cast<idx_t*>(buf + l.col_ptr);
    void* t_val = buf + l.vals;
    // Unless the caller asked for the algorithm whose bits repeat (MCSPARSE_SPMV_CSR_ALG2): one pass of
    // that sort, into buckets of neighbouring columns, and the sums of a bucket's columns formed in LDS
    // in whatever order the products arrive.
    if (alg != MCSPARSE_SPMV_CSR_ALG2 && mcsp::skinny_transpose_shape(static_cast<idx_t>(v.n), nnz)) {
        // few columns, many nonzeros in each: nothing is ordered at all.  The scratch of the sort holds the
        // rows of the nonzeros (for CSR offsets) and the partial sums.
        char* ws = buf + l.csr2csc_ws;
        const idx_t* rows = v.coo_rows;
        if (rows == nullptr) {
            idx_t* expanded = reinterpret_cast<idx_t*>(ws);
            mcsp::launch_csr2coo(h->stream, static_cast<idx_t>(v.m), nnz, v.ptr, base, expanded);
            rows = expanded;
        }
        return mcsp::launch_skinny_transpose<T>(h->stream, static_cast<idx_t>(v.m), static_cast<idx_t>(v.n), nnz, base, rows,
                                                v.ind, static_cast<const T*>(v.val), static_cast<const T*>(x->values),
                                                static_cast<T*>(y->values), h_alpha, h_beta,
                                                ws + align_up(static_cast<size_t>(nnz) * sizeof(idx_t)))
                   ? MCSP_STATUS_SUCCESS
                   : MCSP_STATUS_INTERNAL_ERROR;
    }
    uint32_t bucket_shift = 0;
    if (alg != MCSPARSE_SPMV_CSR_ALG2 &&
        mcsp::bucketed_products_shape(static_cast<idx_t>(v.n), &bucket_shift)) {
        mcsp::BucketedProducts b;
        mcsp::launch_bucketed_products(h->stream, static_cast<idx_t>(v.m), static_cast<idx_t>(v.n), nnz, v.val, v.ptr,
                                       v.ind, x->values, t_val, sizeof(T), base, buf + l.csr2csc_ws, &b);
        return mcsp::launch_bucket_sums<T>(h->stream, static_cast<idx_t>(v.n), nnz, b, static_cast<const T*>(t_val),
                                           static_cast<T*>(y->values), h_alpha, h_beta)
                   ? MCSP_STATUS_SUCCESS
                   : MCSP_STATUS_INTERNAL_ERROR;
    }
    mcsp::launch_transposed_products(h->stream, static_cast<idx_t>(v.m), static_cast<idx_t>(v.n), nnz, v.val, v.ptr, v.ind,
                                     x->values, t_val, t_ptr, sizeof(T), base, buf + l.csr2csc_ws);
    a.m = static_cast<idx_t>(v.n);
    a.n = static_cast<idx_t>(v.m);
    a.row_ptr = t_ptr;
    a.col = nullptr;
    a.val = t_val;
    a.x = nullptr;
    mcsp::launch_row_sums_merge<T>(h->stream, a, h_alpha, h_beta, buf + l.merge_ws);
    return MCSP_STATUS_SUCCESS;
}

// Scratch layout of an SpMM call: CSR gets room for the row-group schedule that
// mcsparseSpMM_preprocess builds (SpMM itself writes nothing there); COO gets [row offsets m+1];
// CSC gets the transposed copy [row_ptr m+1 | col_ind nnz][values][csr2csc workspace]
// (mcsp_spmm_gpu.cpp:818-849); 64-bit index arrays add their narrowed copies at the end.
struct SpmmLayout {
    size_t ptr, ind, vals, csr2csc_ws, bt, ct, long_ws, narrow, total;
    int64_t n_padded;  // leading dimension of the row-major copies of op(B) and C
    bool copy_b, copy_c;
};

// op(B)(kk, j) sits at kk*ldb + j for (N, row-major) and (T, column-major), else at j*ldb + kk.
bool b_image_is_row_major(mcsparseOperation_t opB, const mcsparseDnMatDescr* B) {
    const bool op_n = opB == MCSPARSE_OPERATION_NON_TRANSPOSE;
    return (op_n && B->order == MCSPARSE_ORDER_ROW) || (!op_n && B->order == MCSPARSE_ORDER_COL);
}

bool schedulable(const mcsparseSpMatDescr* A) {
    return A->format == MCSPARSE_FORMAT_CSR && A->row_num > 0 && A->nnz > 0 &&
           A->col_num <= mcsp::kSpmmMaxScheduledColumns;
}

// The schedule of the descriptor belongs to this call: same buffer, same arrays, same extents.
bool schedule_matches(const mcsparseSpMatDescr* A, const void* buffer) {
    const SpmmSchedule& s = A->schedule;
    return s.valid && s.useful && s.buffer == buffer && s.rows == A->rows && s.cols == A->cols && s.m == A->row_num &&
           s.nnz == A->nnz && s.base == static_cast<int>(A->idxBase);
}

// A column-major op(B) would be gathered element by element and a column-major C written element by
// element; with room in the scratch buffer they are transposed instead (the reference copies the other
// way round, into memory it allocates: mcsp_spmm_gpu.cpp:119-133): op(B) into a row-major copy before
// the product, the product from a row-major C out into the caller's.
SpmmLayout spmm_layout(const mcsparseSpMatDescr* A, const mcsparseDnMatDescr* B, const mcsparseDnMatDescr* C,
                       mcsparseOperation_t opB, size_t value_bytes) {
    SpmmLayout l = {};
    size_t off = 0;
    if (A->format == MCSPARSE_FORMAT_CSR) {
        if (schedulable(A)) off += mcsp::spmm_schedule_layout(static_cast<idx_t>(A->row_num), static_cast<idx_t>(A->nnz)).total;
    } else if (A->format == MCSPARSE_FORMAT_COO) {
        off += align_up(static_cast<size_t>(A->row_num + 1) * sizeof(idx_t));
    } else if (A->format == MCSPARSE_FORMAT_CSC) {
        l.ind = static_cast<size_t>(A->row_num + 1) * sizeof(idx_t);
        off += align_up(static_cast<size_t>(A->row_num + 1 + A->nnz) * sizeof(idx_t));
        l.vals = off;
        off += align_up(static_cast<size_t>(A->nnz) * value_bytes);
        l.csr2csc_ws = off;
        off += align_up(mcsp::csr2csc_workspace_bytes(static_cast<idx_t>(A->col_num), static_cast<idx_t>(A->row_num),
                                                      static_cast<idx_t>(A->nnz), value_bytes));
    }
    const int64_t n = C->col_num;
    l.n_padded = (n + 3) / 4 * 4;
    l.copy_b = !b_image_is_row_major(opB, B) && A->col_num > 0 && n > 0;
    l.copy_c = C->order != MCSPARSE_ORDER_ROW && A->row_num > 0 && n > 0;
    l.bt = off;
    if (l.copy_b) off += align_up(static_cast<size_t>(A->col_num) * l.n_padded * value_bytes);
    l.ct = off;
    if (l.copy_c) off += align_up(static_cast<size_t>(A->row_num) * l.n_padded * value_bytes);
    // the pieces long rows are cut into, their partial sums, and the counters of the row-length analysis
    l.long_ws = off;
    if (A->nnz > 0 && A->row_num > 0 && n > 0)
        off += align_up(mcsp::spmm_long_rows_bytes(static_cast<idx_t>(A->nnz), l.n_padded, value_bytes));
    l.narrow = off;
    off += narrow_bytes(A);
    l.total = off < kMinBuffer ? kMinBuffer : off;
    return l;
}

template <typename T>
mcspStatus_t spmm_typed(mcsparseHandle_t h, mcsparseSpMatDescr* A, mcsparseOperation_t opB, const void* alpha,
                        const void* beta, const mcsparseDnMatDescr* B, mcsparseDnMatDescr* C, void* buffer) {
    T h_alpha, h_beta;
    if (!scalar_to_host(h, beta, &h_beta) || !scalar_to_host(h, alpha, &h_alpha))
        return stream_is_capturing(h->stream) ? MCSP_STATUS_NOT_IMPLEMENTED : MCSP_STATUS_INTERNAL_ERROR;
    // reference: mcsp_spmm_gpu.cpp:110-114
    if (A->nnz == 0 && h_beta == T(1)) return MCSP_STATUS_SUCCESS;

    char* buf = static_cast<char*>(buffer);
    const SpmmLayout l = spmm_layout(A, B, C, opB, sizeof(T));
    // Strided batches (csr_spmm_device.hpp:102-108): batch b works on the arrays moved on by b
    // strides; the reference runs them as blockIdx.z of one launch, here they are launches in a
    // row on the stream, sharing the scratch buffer.
    const int64_t batches = C->batchCount;
    const bool shared_structure = A->offsetsBatchStride == 0 && A->batchStride == 0;
    const size_t idx_bytes = wide_indices(A) ? sizeof(int64_t) : sizeof(idx_t);
    for (int64_t b = 0; b < batches; ++b) {
        mcsparseSpMatDescr Ab = *A;  // this batch's view of A
        const int64_t rows_stride = A->format == MCSPARSE_FORMAT_CSR ? A->offsetsBatchStride : A->batchStride;
        const int64_t cols_stride = A->format == MCSPARSE_FORMAT_CSC ? A->offsetsBatchStride : A->batchStride;
        if (A->rows != nullptr) Ab.rows = static_cast<char*>(A->rows) + b * rows_stride * static_cast<int64_t>(idx_bytes);
        if (A->cols != nullptr) Ab.cols = static_cast<char*>(A->cols) + b * cols_stride * static_cast<int64_t>(idx_bytes);
        if (A->vals != nullptr) Ab.vals = static_cast<char*>(A->vals) + b * A->batchStride * static_cast<int64_t>(sizeof(T));
        const IndexArrays ia = index_arrays(h, &Ab, buf + l.narrow);

        mcsp::SpmmArgs a;
        a.m = static_cast<idx_t>(A->row_num);
        a.n = static_cast<idx_t>(C->col_num);
        a.k = static_cast<idx_t>(A->col_num);
        a.nnz = static_cast<idx_t>(A->nnz);
        a.base = static_cast<idx_t>(A->idxBase);
        a.row_ptr = ia.rows;
        a.col = ia.cols;
        a.val = Ab.vals;
        if (A->format == MCSPARSE_FORMAT_COO && A->nnz != 0) {
            idx_t* built = reinterpret_cast<idx_t*>(buf + l.ptr);
            mcsp::launch_coo2csr(h->stream, a.nnz, a.m, ia.rows, a.base, built);
            a.row_ptr = built;
        } else if (A->format == MCSPARSE_FORMAT_CSC && A->nnz != 0) {
            // the CSC arrays are the CSR of A^T (col_num x row_num); transposing them gives the CSR of A
            idx_t* t_ptr = reinterpret_cast<idx_t*>(buf + l.ptr);
            idx_t* t_ind = reinterpret_cast<idx_t*>(buf + l.ind);
            void* t_val = buf + l.vals;
            mcsp::launch_csr2csc(h->stream, static_cast<idx_t>(A->col_num), static_cast<idx_t>(A->row_num), a.nnz,
                                 Ab.vals, ia.cols, ia.rows, t_val, t_ind, t_ptr, sizeof(T), a.base,
                                 buf + l.csr2csc_ws);
            a.row_ptr = t_ptr;
            a.col = t_ind;
            a.val = t_val;
        } else if (A->format != MCSPARSE_FORMAT_CSR) {
            // no nonzeros: C = beta*C over m empty rows; coo2csr with nnz = 0 writes the m+1 offsets
            idx_t* built = reinterpret_cast<idx_t*>(buf + l.ptr);
            mcsp::launch_coo2csr(h->stream, 0, a.m, built, a.base, built);
            a.row_ptr = built;
        }
        const T* b_user = reinterpret_cast<const T*>(static_cast<const char*>(B->values) +
                                                     b * B->batchStride * static_cast<int64_t>(sizeof(T)));
        T* c_user = reinterpret_cast<T*>(static_cast<char*>(C->values) +
                                         b * C->batchStride * static_cast<int64_t>(sizeof(T)));
        a.B = b_user;
        a.ldb = B->ld;
        a.b_row_major = b_image_is_row_major(opB, B);
        a.C = c_user;
        a.ldc = C->ld;
        a.c_row_major = C->order == MCSPARSE_ORDER_ROW;
        // Rows far longer than the rest are cut into pieces (spmm_long.hip), which costs four small launches: only
        // where the matrix has such rows.  Whether it has is part of the row-length analysis that SpMV keeps on the
        // descriptor (one kernel and a 136-byte read-back the first time a structure is seen); a call that cannot
        // use it (a stream under capture, batches with offsets of their own, COO and CSC inputs, whose offsets are
        // built in the buffer) takes the launches.
        if (A->nnz != 0 && a.m != 0 && a.n != 0) {
            bool may_have_long_rows = true;
            if (A->format == MCSPARSE_FORMAT_CSR && (batches == 1 || shared_structure)) {
                const mcspStatus_t ps = ensure_plan(h, A, ia.rows, A->rows, A->row_num, A->nnz,
                                                    A->col_num * static_cast<int64_t>(sizeof(T)), buf + l.long_ws, true);
                if (ps != MCSP_STATUS_SUCCESS) return ps;
                if (A->plan.valid && A->plan.forced_family == kFamilyAuto)
                    may_have_long_rows = A->plan.max_row_len > mcsp::kSpmmLongRow;
            }
            if (may_have_long_rows) {
                a.long_row = mcsp::kSpmmLongRow;
                a.long_ws = buf + l.long_ws;
                a.long_n = l.n_padded;
            }
        }
        T beta_inner = h_beta;
        if (l.copy_b && A->nnz != 0) {  // without nonzeros op(B) is never read (and may be NULL)
            // the column-major image is a row-major n x k matrix: its transpose is op(B), row-major
            T* bt = reinterpret_cast<T*>(buf + l.bt);
            mcsp::launch_transpose<T>(h->stream, a.n, a.k, static_cast<idx_t>(l.n_padded), b_user, B->ld, bt, l.n_padded);
            a.B = bt;
            a.ldb = l.n_padded;
            a.b_row_major = true;
        }
        // The kernel that works from the schedule owns four consecutive rows per lane group and writes them
        // into a column-major C as they lie there, 16 bytes per column: no row-major copy of C then.
        const bool scheduled_here = (b == 0 || shared_structure) && schedule_matches(A, buffer);
        const bool by_blocks = A->schedule.blocks;
        auto schedule_usable = [&]() {
            return by_blocks ? mcsp::spmm_blocks_usable(a, sizeof(T)) : mcsp::spmm_schedule_usable(a, sizeof(T));
        };
        const bool direct_c = l.copy_c && scheduled_here && schedule_usable() &&
                              reinterpret_cast<uintptr_t>(c_user) % 16 == 0 &&
                              (static_cast<uint64_t>(C->ld) * sizeof(T)) % 16 == 0;
        const bool copy_c = l.copy_c && !direct_c;
        if (copy_c) {
            a.C = buf + l.ct;
            a.ldc = l.n_padded;
            a.c_row_major = true;
            beta_inner = T(0);  // beta * C is added when the product is transposed out
            // with both copies at hand the padded columns of op(B) are zeros: whole 128-bit vectors
            if (l.copy_b && A->nnz != 0) a.n = static_cast<idx_t>(l.n_padded);
        }
        // the schedule was built from batch 0's structure
        if (scheduled_here && schedule_usable()) {
            if (by_blocks && A->schedule.stride != 0)
                mcsp::launch_spmm_strips<T>(h->stream, a, buffer, A->schedule.stride, A->schedule.entries,
                                            A->schedule.longest_group, A->schedule.mean_span, h_alpha, beta_inner);
            else if (by_blocks)
                mcsp::launch_spmm_blocks<T>(h->stream, a, buffer, A->schedule.entries, A->schedule.longest_group,
                                            A->schedule.mean_span, h_alpha,
                                            beta_inner);
            else
                mcsp::launch_spmm_scheduled<T>(h->stream, a, buffer, A->schedule.entries, A->schedule.mean_span, h_alpha,
                                               beta_inner);
        } else {
            mcsp::launch_spmm<T>(h->stream, a, h_alpha, beta_inner);
        }
        if (copy_c) {
            mcsp::launch_transpose_accumulate<T>(h->stream, a.m, static_cast<idx_t>(C->col_num),
                                                 reinterpret_cast<const T*>(buf + l.ct), l.n_padded, c_user, C->ld,
                                                 h_beta);
        }
    }
    // a launch the runtime refused (a kernel image that does not fit the device) must not pass for a product
    return launches_taken() ? MCSP_STATUS_SUCCESS : MCSP_STATUS_INTERNAL_ERROR;
}

mcspStatus_t check_spmm_args(mcsparseHandle_t handle, const void* alpha, const mcsparseSpMatDescr* A,
                             const mcsparseDnMatDescr* B, const void* beta, const mcsparseDnMatDescr* C) {
    // reference: mcsp_spmm_gpu.cpp:313-332 / :789-807
    if (handle == nullptr) return MCSP_STATUS_INVALID_HANDLE;
    if (A == nullptr || B == nullptr || C == nullptr || alpha == nullptr || beta == nullptr)
        return MCSP_STATUS_INVALID_POINTER;
    if (!fits_32(A->row_num) || !fits_32(A->col_num) || !fits_32(A->nnz) || !fits_32(B->row_num) ||
        !fits_32(B->col_num) || !fits_32(B->ld) || !fits_32(C->row_num) || !fits_32(C->col_num) || !fits_32(C->ld))
        return MCSP_STATUS_NOT_IMPLEMENTED;
    if (A->format != MCSPARSE_FORMAT_CSR && A->format != MCSPARSE_FORMAT_COO &&
        A->format != MCSPARSE_FORMAT_BLOCKED_ELL && A->format != MCSPARSE_FORMAT_CSC)
        return MCSP_STATUS_NOT_IMPLEMENTED;
    return MCSP_STATUS_SUCCESS;
}

}  // namespace

namespace mcsp {

// Kernel family for a CSR structure from its row-length bins (bins[b], b >= 1: rows of length in
// [2^(b-1), 2^b); bins[0]: empty rows; bins[MCSPARSE_ROW_BIN_COUNT]: the longest row).
//
// The vector family gives L lanes to a row (L = the power of two at or above the mean length) and a
// wavefront keeps k = 64/L * 4 rows in flight; it loops until the longest of them is done, so the
// share of its lane slots that hold a nonzero is mean / (L * E[max over k rows of ceil(len / L)]).
// The expectation comes from the bins, with the lengths inside a bin placed so that the overall
// mean is the true one (rows of exactly 16 fall into [16, 32) and count as 16, not 24).  The merge
// family spends about one slot per nonzero and row whatever the lengths are, at ~5 % more work per
// item.  Measured: rows of exactly 16 (share 1.0) run 10 % faster in the vector family; rows of
// 28 +- 5 (share 0.48) 13 % faster in the merge family; Poisson rows of mean 20 (share 0.6) faster in
// the vector family.  The families change places at a share of about one half.  A row far longer
// than the rest serialises one wavefront, so such matrices take the merge family whatever the share.
void spmv_plan_from_bins(const uint32_t* bins, int64_t m, int64_t nnz, int64_t x_bytes, int* family, int* lanes) {
    const int mean_lanes = spmv_pick_lanes(static_cast<idx_t>(m), static_cast<idx_t>(nnz));
    const uint32_t max_row_len = bins[MCSPARSE_ROW_BIN_COUNT];
    const uint32_t limit = static_cast<uint32_t>(32 * mean_lanes > 512 ? 32 * mean_lanes : 512);
    bool merge = max_row_len > limit;
    if (!merge && m > 0 && nnz > 0) {
        // lengths inside a bin: lower edge times a common factor in [1, 2) that makes the mean right
        double edge_sum = 0;
        for (int b = 1; b < MCSPARSE_ROW_BIN_COUNT; ++b) edge_sum += static_cast<double>(bins[b]) * std::ldexp(1.0, b - 1);
        double factor = edge_sum > 0 ? static_cast<double>(nnz) / edge_sum : 1.0;
        factor = factor < 1.0 ? 1.0 : (factor > 2.0 ? 2.0 : factor);
        const double k = 64.0 / mean_lanes * 4.0;
        double below = static_cast<double>(bins[0]) / static_cast<double>(m);  // share of rows in lower bins
        double below_pow = std::pow(below, k);
        double expected_max = 0;
        for (int b = 1; b < MCSPARSE_ROW_BIN_COUNT; ++b) {
            if (bins[b] == 0) continue;
            double len = std::ldexp(1.0, b - 1) * factor;
            if (len > max_row_len) len = max_row_len;  // no row is longer than the longest
            const double passes = std::ceil(len / mean_lanes - 1e-9);
            const double upto = below + static_cast<double>(bins[b]) / static_cast<double>(m);
            const double upto_pow = std::pow(upto < 1.0 ? upto : 1.0, k);
            expected_max += passes * (upto_pow - below_pow);
            below = upto;
            below_pow = upto_pow;
        }
        const double mean = static_cast<double>(nnz) / static_cast<double>(m);
        const double share = expected_max > 0 ? mean / (mean_lanes * expected_max) : 1.0;
        merge = share < 0.5;
    }
    if (merge) {
        *family = kFamilyMerge;
        // Rows longer than a tile of the merge path put whole tiles inside one row; when x is too
        // large to stay in an XCD's L2 next to the streamed matrix, those tiles run in the order of
        // their first column (lanes = 1), which costs two small kernels per call.
        // That order pays where such rows hold most of the nonzeros (the power-law matrix: two thirds); where a few
        // long rows sit among many short ones it costs more than it brings (1 M rows of 16 plus 64 rows of 100000:
        // 155 us against 140 us in storage order).
        double in_long_rows = 0;
        for (int b = 1; b < MCSPARSE_ROW_BIN_COUNT; ++b) {
            const double lower_edge = std::ldexp(1.0, b - 1);
            if (lower_edge >= kMergeTileItems) in_long_rows += static_cast<double>(bins[b]) * lower_edge;
        }
        const bool mostly_long = nnz > 0 && in_long_rows * 2 >= static_cast<double>(nnz);  // lower edges: an underestimate
        *lanes = max_row_len >= kMergeTileItems && x_bytes > kMergeOrderMinVectorBytes && mostly_long ? 1 : 0;
    } else {
        *family = kFamilyVector;
        *lanes = mean_lanes;
    }
}

// The argument checks of mcsparseSpMV in the reference's order, then the ones this build adds.
mcspStatus_t spmv_check(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha, mcsparseSpMatDescr_t matA,
                        mcsparseDnVecDescr_t vecX, const void* beta, mcsparseDnVecDescr_t vecY,
                        macaDataType computeType, const void* buffer, size_t buffer_bytes, bool may_read_back) {
    if (matA != nullptr) {
        const mcspStatus_t it = check_index_types(matA);
        if (it != MCSP_STATUS_SUCCESS) return it;
    }
    const mcspStatus_t st = check_spmv_args(handle, opA, alpha, matA, vecX, beta, vecY, true, true, buffer);
    if (st != MCSP_STATUS_SUCCESS) return st;
    const bool real_type = computeType == MACA_R_32F || computeType == MACA_R_64F || computeType == MACA_R_16F ||
                           computeType == MACA_R_16BF;
    if (real_type && opA == MCSPARSE_OPERATION_CONJUGATE_TRANSPOSE) return MCSP_STATUS_INVALID_VALUE;
    if (!format_is_built(matA->format)) return MCSP_STATUS_NOT_IMPLEMENTED;  // COO_AOS
    // Same-type real fp32/fp64 only; the reference's mixed-precision and complex routes
    // (:848-860) are outside this path.  x is checked too, which the reference omits.
    if (!(computeType == matA->valueType && computeType == vecY->valueType && computeType == vecX->valueType))
        return MCSP_STATUS_NOT_IMPLEMENTED;
    if (computeType != MACA_R_32F && computeType != MACA_R_64F) return MCSP_STATUS_NOT_IMPLEMENTED;
    if (!may_read_back && handle->ptr_mode != MCSPARSE_POINTER_MODE_HOST) return MCSP_STATUS_NOT_IMPLEMENTED;
    if (buffer_bytes != 0) {
        const CsrView v = make_view(matA, opA);
        if (spmv_layout(v, matA->nnz, value_size(computeType), narrow_bytes(matA)).total > buffer_bytes)
            return MCSP_STATUS_INSUFFICIENT_RESOURCES;
    }
    // The reference hands NULL arrays back as INVALID_POINTER (mcsp_spmv_gpu.cpp:217-220); a kernel
    // would fault on them.  A call without nonzeros reads none of them.
    if (matA->nnz != 0 && (matA->rows == nullptr || matA->cols == nullptr || matA->vals == nullptr ||
                           vecX->values == nullptr || vecY->values == nullptr))
        return MCSP_STATUS_INVALID_POINTER;
    return MCSP_STATUS_SUCCESS;
}

mcspStatus_t spmv_call(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha, mcsparseSpMatDescr_t matA,
                       mcsparseDnVecDescr_t vecX, const void* beta, mcsparseDnVecDescr_t vecY,
                       macaDataType computeType, void* buffer, size_t buffer_bytes, bool may_read_back,
                       mcsparseSpMVAlg_t alg) {
    const mcspStatus_t st =
        spmv_check(handle, opA, alpha, matA, vecX, beta, vecY, computeType, buffer, buffer_bytes, may_read_back);
    if (st != MCSP_STATUS_SUCCESS) return st;
    if (handle->spmv_deterministic) alg = MCSPARSE_SPMV_CSR_ALG2;
    if (computeType == MACA_R_32F)
        return spmv_typed<float>(handle, matA, opA, alpha, beta, vecX, vecY, buffer, may_read_back, alg);
    return spmv_typed<double>(handle, matA, opA, alpha, beta, vecX, vecY, buffer, may_read_back, alg);
}

// mcsparseSpMV_preprocess has just built a copy for a direction that does not transpose.  Whether calls run
// faster from it than from the caller's arrays depends on what the row kernels already get from the caches (a
// banded matrix reads x line by line as it is; an x that fits an L2 next to rows long enough to fill the lanes
// leaves the copy's extra partial sums as pure cost), so both are run here, on the handle's stream, with the
// caller's x and a y inside the buffer, and timed with events: once each, which settles it where one takes more
// than twice the other's time (or, for long runs, a quarter more), else twice more.  *copy_wins says whether the copy was faster by more than a
// twentieth.
mcspStatus_t spmv_trial(mcsparseHandle_t handle, mcsparseOperation_t opA, mcsparseSpMatDescr_t matA,
                        mcsparseDnVecDescr_t vecX, void* trial_y, macaDataType computeType, void* buffer,
                        mcsparseSpMVAlg_t alg, bool* copy_wins) {
    mcsparseDnVecDescr y = {};
    const CsrView v = make_view(matA, opA);
    y.valueType = computeType;
    y.size = v.transpose ? v.n : v.m;
    y.values = trial_y;
    const double one64 = 1.0, zero64 = 0.0;
    const float one32 = 1.0f, zero32 = 0.0f;
    const void* one = computeType == MACA_R_32F ? static_cast<const void*>(&one32) : &one64;
    const void* zero = computeType == MACA_R_32F ? static_cast<const void*>(&zero32) : &zero64;
    const mcsparsePointerMode_t callers_mode = handle->ptr_mode;
    handle->ptr_mode = MCSPARSE_POINTER_MODE_HOST;
    hipEvent_t marks[3] = {nullptr, nullptr, nullptr};  // before the row kernels, between the two, after the copy
    mcspStatus_t st = MCSP_STATUS_SUCCESS;
    for (hipEvent_t& e : marks)
        if (st == MCSP_STATUS_SUCCESS && hipEventCreate(&e) != hipSuccess) st = MCSP_STATUS_INTERNAL_ERROR;
    float rows_ms = 0.0f, copy_ms = 0.0f;
    for (int runs = 1; runs <= 2 && st == MCSP_STATUS_SUCCESS; ++runs) {
        for (int leg = 0; leg < 2 && st == MCSP_STATUS_SUCCESS; ++leg) {
            matA->banded.useful = leg == 1;  // leg 0 runs the row kernels, leg 1 the copy
            if (hipEventRecord(marks[leg], handle->stream) != hipSuccess) st = MCSP_STATUS_INTERNAL_ERROR;
            for (int run = 0; run < runs && st == MCSP_STATUS_SUCCESS; ++run)
                st = computeType == MACA_R_32F
                         ? spmv_typed<float>(handle, matA, opA, one, zero, vecX, &y, buffer, true, alg)
                         : spmv_typed<double>(handle, matA, opA, one, zero, vecX, &y, buffer, true, alg);
        }
        if (st == MCSP_STATUS_SUCCESS &&
            (hipEventRecord(marks[2], handle->stream) != hipSuccess || hipEventSynchronize(marks[2]) != hipSuccess ||
             hipEventElapsedTime(&rows_ms, marks[0], marks[1]) != hipSuccess ||
             hipEventElapsedTime(&copy_ms, marks[1], marks[2]) != hipSuccess))
            st = MCSP_STATUS_INTERNAL_ERROR;
        // the first runs of the two are their slowest (cold caches, by some tens of microseconds): enough to tell two
        // from one, or five from four where a run takes a third of a millisecond and more, not 20 from 19
        const float slower = rows_ms > copy_ms ? rows_ms : copy_ms, faster = rows_ms > copy_ms ? copy_ms : rows_ms;
        if (slower > 2.0f * faster || (faster > 0.3f && slower > 1.25f * faster)) break;
    }
    for (hipEvent_t e : marks)
        if (e != nullptr) (void)hipEventDestroy(e);
    handle->ptr_mode = callers_mode;
    matA->banded.useful = true;
    *copy_wins = copy_ms * 20.0f < rows_ms * 19.0f;
    return st;
}

}  // namespace mcsp

extern "C" {

// reference: src/kernels/level2/spmv/mcsp_spmv_gpu.cpp:309-352, :1108-1121
mcsparseStatus_t mcsparseSpMV_bufferSize(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha,
                                         mcsparseSpMatDescr_t matA, mcsparseDnVecDescr_t vecX, const void* beta,
                                         mcsparseDnVecDescr_t vecY, macaDataType /*computeType*/,
                                         mcsparseSpMVAlg_t /*alg*/, size_t* bufferSize) {
    if (matA != nullptr) {
        const mcspStatus_t it = check_index_types(matA);
        if (it != MCSP_STATUS_SUCCESS) return to_public_status(it);
    }
    const mcspStatus_t st =
        check_spmv_args(handle, opA, alpha, matA, vecX, beta, vecY, bufferSize != nullptr, false, nullptr);
    if (st != MCSP_STATUS_SUCCESS) return to_public_status(st);
    if (!format_is_built(matA->format)) return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);  // COO_AOS

    const size_t vb = value_size(matA->valueType);
    const CsrView v = make_view(matA, opA);
    const SpmvLayout l = spmv_layout(v, matA->nnz, vb, narrow_bytes(matA));
    if (v.transpose) {
        matA->assist_index_buffer_size = l.vals - l.col_ptr;
        matA->fixed_length_buffer_size = l.csr2csc_ws;
        matA->is_buffersize_called = 1;
    }
    *bufferSize = l.total;
    return MCSPARSE_STATUS_SUCCESS;
}

// reference: src/kernels/level2/spmv/mcsp_spmv_gpu.cpp:686-903, :1123-1147
mcsparseStatus_t mcsparseSpMV(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha,
                              mcsparseSpMatDescr_t matA, mcsparseDnVecDescr_t vecX, const void* beta,
                              mcsparseDnVecDescr_t vecY, macaDataType computeType, mcsparseSpMVAlg_t alg,
                              void* externalBuffer) {
    return to_public_status(
        mcsp::spmv_call(handle, opA, alpha, matA, vecX, beta, vecY, computeType, externalBuffer, 0, true, alg));
}

// EXTENSION
mcsparseStatus_t mcsparseSpMV_preprocess_bufferSize(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha,
                                                    mcsparseSpMatDescr_t matA, mcsparseDnVecDescr_t vecX,
                                                    const void* beta, mcsparseDnVecDescr_t vecY,
                                                    macaDataType computeType, mcsparseSpMVAlg_t alg,
                                                    size_t* bufferSize) {
    const mcsparseStatus_t st =
        mcsparseSpMV_bufferSize(handle, opA, alpha, matA, vecX, beta, vecY, computeType, alg, bufferSize);
    if (st != MCSPARSE_STATUS_SUCCESS) return st;
    if (handle->spmv_deterministic) alg = MCSPARSE_SPMV_CSR_ALG2;
    BandedShape shape;
    if (banded_candidate(matA, opA, alg, &shape)) {
        const size_t vb = value_size(matA->valueType);
        const CsrView v = make_view(matA, opA);
        const idx_t rows = static_cast<idx_t>(v.transpose ? v.n : v.m);
        // the copy in column order carries its own scratch; the other builds a transpose behind itself
        // and, for a direction that does not transpose, a y for the runs that time the copy against the row kernels
        *bufferSize = banded_region_offset(matA, opA, vb) +
                      align_up(mcsp::banded_layout(shape, rows, static_cast<idx_t>(matA->nnz), vb).total) +
                      (v.transpose ? (shape.by_column ? 0 : transpose_scratch(v, matA->nnz, vb).total)
                                   : align_up(static_cast<size_t>(rows) * vb));
    }
    return MCSPARSE_STATUS_SUCCESS;
}

// EXTENSION
mcsparseStatus_t mcsparseSpMV_preprocess(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha,
                                         mcsparseSpMatDescr_t matA, mcsparseDnVecDescr_t vecX, const void* beta,
                                         mcsparseDnVecDescr_t vecY, macaDataType computeType,
                                         mcsparseSpMVAlg_t alg, void* externalBuffer) {
    const mcspStatus_t st =
        mcsp::spmv_check(handle, opA, alpha, matA, vecX, beta, vecY, computeType, externalBuffer, 0, true);
    if (st != MCSP_STATUS_SUCCESS) return to_public_status(st);
    matA->banded.valid = false;
    if (stream_is_capturing(handle->stream)) return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);  // it blocks
    if (handle->spmv_deterministic) alg = MCSPARSE_SPMV_CSR_ALG2;
    BandedShape shape;
    if (matA->nnz == 0 || !banded_candidate(matA, opA, alg, &shape)) return MCSPARSE_STATUS_SUCCESS;  // nothing to prepare

    CsrView v = make_view(matA, opA);
    const idx_t m = static_cast<idx_t>(v.transpose ? v.n : v.m);  // rows of the matrix that is banded
    const idx_t nnz = static_cast<idx_t>(matA->nnz);
    const idx_t base = static_cast<idx_t>(matA->idxBase);
    const size_t vb = value_size(matA->valueType);
    // 64-bit indices are narrowed and COO rows turned into offsets in the part of the buffer a plain call
    // uses for the same purpose; the copy does not refer to them afterwards
    const void* signature = v.coo_rows != nullptr ? static_cast<const void*>(v.coo_rows) : v.ptr;
    {
        char* buf = static_cast<char*>(externalBuffer);
        const SpmvLayout sl = spmv_layout(v, matA->nnz, vb, narrow_bytes(matA));
        if (wide_indices(matA)) {
            const IndexArrays ia = index_arrays(handle, matA, buf + sl.narrow);
            v = make_view(matA, opA, ia.rows, ia.cols);
        }
        if (v.coo_rows != nullptr) {
            idx_t* built = reinterpret_cast<idx_t*>(buf + sl.coo_ptr);
            mcsp::launch_coo2csr(handle->stream, nnz, static_cast<idx_t>(v.m), v.coo_rows, base, built);
            v.ptr = built;
        }
    }
    if (!v.transpose) {
        // the plan of the row kernels is worked out here as well, so that no later call has to block for it
        const mcspStatus_t ps = ensure_plan(handle, matA, v.ptr, signature, v.m, matA->nnz,
                                            v.n * static_cast<int64_t>(vb), externalBuffer, true);
        if (ps != MCSP_STATUS_SUCCESS) return to_public_status(ps);
    }
    // Where a few lines of x take most of the gathers (long rows under a transposing direction, popular columns),
    // one band group over all of x does better than groups that fit an XCD's L2: the hot lines stay in L2 anyway
    // and the planes of partial sums go.  Measured on the matrix, unless the caller has set the width.
    if (shape.by_column && matA->banded.band_bytes == 0 && shape.bands > 1) {
        const idx_t gathered = static_cast<idx_t>(v.transpose ? v.m : v.n);
        const size_t region_at = banded_region_offset(matA, opA, vb);
        const size_t room = align_up(mcsp::banded_layout(shape, m, nnz, vb).total);
        if (mcsp::line_gathers_workspace_bytes(gathered, vb) <= room) {
            char* ws = static_cast<char*>(externalBuffer) + region_at;
            mcsp::launch_line_gathers(handle->stream, v.transpose, gathered, nnz, base, v.ptr, v.ind, vb, ws);
            unsigned long long bins[2 * mcsp::kLineGatherBins];
            if (hipMemcpyAsync(bins, ws, sizeof(bins), hipMemcpyDeviceToHost, handle->stream) != hipSuccess ||
                hipStreamSynchronize(handle->stream) != hipSuccess)
                return to_public_status(MCSP_STATUS_INTERNAL_ERROR);
            if (mcsp::gathers_favour_wide_groups(bins)) {
                size_t all_of_x = mcsp::kBandedBandBytes;
                while (all_of_x < (static_cast<size_t>(gathered) + base) * vb) all_of_x *= 2;
                BandedShape wide;
                if (mcsp::column_order_shape(m, gathered, nnz, base, vb, all_of_x, &wide) &&
                    wide.rows_per_tile == shape.rows_per_tile &&
                    align_up(mcsp::banded_layout(wide, m, nnz, vb).total) <= room)
                    shape = wide;
            }
        }
    }
    SpmvBanded& b = matA->banded;
    b.buffer = externalBuffer;
    b.rows = matA->rows;
    b.cols = matA->cols;
    b.vals = matA->vals;
    b.m = matA->row_num;
    b.n = matA->col_num;
    b.nnz = matA->nnz;
    b.base = static_cast<int>(matA->idxBase);
    b.type = matA->valueType;
    b.format = matA->format;
    b.transposed = v.transpose;
    b.shape = shape;
    // the longest row is known from the analysis above; for a transposing direction (rows = the view's columns) it
    // is not, and the plain kernel is used
    b.shape.crowded_rows = shape.by_column && !v.transpose && matA->plan.valid && shape.chunks != 0 &&
                           2 * static_cast<uint64_t>(matA->plan.max_row_len) > static_cast<uint64_t>(nnz) / shape.chunks;
    b.region = banded_region_offset(matA, opA, vb);
    b.grid = 0;
    char* region = static_cast<char*>(externalBuffer) + b.region;
    if (shape.by_column) {
        const mcsp::BandedLayout cl = mcsp::banded_layout(shape, m, nnz, vb);
        idx_t* src_cols = reinterpret_cast<idx_t*>(region + cl.src_cols);
        idx_t* src_rows = reinterpret_cast<idx_t*>(region + cl.src_rows);
        if (v.transpose) {
            // the nonzeros of the transpose sorted by its columns are the arrays as they lie: its
            // columns are the rows of the view, its rows the column indices
            mcsp::launch_csr2coo(handle->stream, static_cast<idx_t>(v.m), nnz, v.ptr, base, src_rows);
            mcsp::launch_column_order_build(handle->stream, shape, m, nnz, base, v.ind, src_rows, matA->vals, vb, region);
        } else {
            // what the kernel gains from is lanes that share a 128-byte line of x: the order of the columns
            // inside a line does not matter, so the sort leaves the bits that tell them apart alone
            const uint32_t line_bits = vb == 8 ? 4 : 5;
            mcsp::launch_sort_by_column(handle->stream, static_cast<idx_t>(v.m), static_cast<idx_t>(v.n), nnz, base, v.ptr,
                                        v.ind, matA->vals, vb, line_bits, src_cols, src_rows, region + cl.src_vals,
                                        region + cl.sort_ws);
            mcsp::launch_column_order_build(handle->stream, shape, m, nnz, base, src_rows, src_cols, region + cl.src_vals,
                                            vb, region);
        }
    } else if (v.transpose) {
        // the transpose in CSR form, behind the banded copy it is only the source of
        char* scratch = region + align_up(mcsp::banded_layout(shape, m, nnz, vb).total);
        const TransposeScratch t = transpose_scratch(v, matA->nnz, vb);
        idx_t* t_ptr = reinterpret_cast<idx_t*>(scratch + t.ptr);
        idx_t* t_ind = reinterpret_cast<idx_t*>(scratch + t.ind);
        mcsp::launch_csr2csc(handle->stream, static_cast<idx_t>(v.m), static_cast<idx_t>(v.n), nnz, matA->vals, v.ptr,
                             v.ind, scratch + t.vals, t_ind, t_ptr, vb, base, scratch + t.ws);
        mcsp::launch_banded_build(handle->stream, shape, m, nnz, base, t_ptr, t_ind, scratch + t.vals, vb, region);
    } else {
        mcsp::launch_banded_build(handle->stream, shape, m, nnz, base, v.ptr, v.ind, matA->vals, vb, region);
    }
    uint32_t xcd_start[9];
    const mcsp::BandedLayout l = mcsp::banded_layout(shape, m, nnz, vb);
    if (hipMemcpyAsync(xcd_start, region + l.xcd_start, sizeof(xcd_start), hipMemcpyDeviceToHost, handle->stream) !=
            hipSuccess ||
        hipStreamSynchronize(handle->stream) != hipSuccess)
        return to_public_status(MCSP_STATUS_INTERNAL_ERROR);
    b.grid = mcsp::banded_grid(xcd_start);
    for (int i = 0; i < 9; ++i) b.shape.xcd_start[i] = xcd_start[i];
    b.useful = true;
    b.valid = true;
    // A caller who has set the band width or the kernel family is measuring one of the two by itself.  The
    // transposing directions need no trial: without a copy each call sorts the products by column.
    if (handle->spmv_preprocess_trial && !v.transpose && matA->banded.band_bytes == 0 &&
        matA->plan.forced_family == kFamilyAuto) {
        bool copy_wins = true;
        const mcspStatus_t ts = mcsp::spmv_trial(handle, opA, matA, vecX, region + align_up(l.total), computeType,
                                                 externalBuffer, alg, &copy_wins);
        if (ts != MCSP_STATUS_SUCCESS) {
            b.valid = false;
            return to_public_status(ts);
        }
        b.useful = copy_wins;
    }
    return MCSPARSE_STATUS_SUCCESS;
}

// reference: src/kernels/level3/spmm/mcsp_spmm_gpu.cpp:309-342, :950-963
mcsparseStatus_t mcsparseSpMM_bufferSize(mcsparseHandle_t handle, mcsparseOperation_t /*opA*/,
                                         mcsparseOperation_t opB, const void* alpha, mcsparseSpMatDescr_t matA,
                                         mcsparseDnMatDescr_t matB, const void* beta, mcsparseDnMatDescr_t matC,
                                         macaDataType /*computeType*/, mcsparseSpMMAlg_t /*alg*/,
                                         size_t* bufferSize) {
    if (matA != nullptr) {
        const mcspStatus_t it = check_index_types(matA);
        if (it != MCSP_STATUS_SUCCESS) return to_public_status(it);
    }
    const mcspStatus_t st = check_spmm_args(handle, alpha, matA, matB, beta, matC);
    if (st != MCSP_STATUS_SUCCESS) return to_public_status(st);
    if (bufferSize == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (!format_is_built(matA->format)) return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);  // Blocked-ELL
    *bufferSize = spmm_layout(matA, matB, matC, opB, value_size(matA->valueType)).total;
    if (matA->format == MCSPARSE_FORMAT_CSC) matA->is_buffersize_called = 1;
    return MCSPARSE_STATUS_SUCCESS;
}

// reference: src/kernels/level3/spmm/mcsp_spmm_gpu.cpp:965-970 -- a no-op there.  Here a CSR
// matrix gets its row-group schedule built into externalBuffer (sized by mcsparseSpMM_bufferSize);
// mcsparseSpMM uses it when it is handed the same buffer and the same CSR arrays, and falls back
// to the schedule-free kernel otherwise.  Until then the caller must leave the buffer and the
// structure of A alone; the values of A may change freely.
namespace {

// The distance, in rows, at which the strips of a strip schedule would lie for this matrix, or 0: the smallest
// distance between the beginnings of two runs of consecutive diagonals in the middle row that is a whole number of
// strips and leaves the matrix at least eight such stretches (a 27-point stencil on a grid of lines of 128 points
// has runs of three diagonals 128 apart).  Reads the row back: blocks.
uint32_t strip_stride_of_middle_row(hipStream_t stream, idx_t m, idx_t base, const idx_t* row_ptr, const idx_t* col) {
    constexpr idx_t kMostLooked = 256;
    const idx_t row = m / 2;
    idx_t ends[2] = {0, 0};
    if (hipMemcpyAsync(ends, row_ptr + row, sizeof(ends), hipMemcpyDeviceToHost, stream) != hipSuccess ||
        hipStreamSynchronize(stream) != hipSuccess)
        return 0;
    if (ends[1] < ends[0] || ends[0] < base) return 0;
    const idx_t count = ends[1] - ends[0];
    if (count < 2 || count > kMostLooked) return 0;
    idx_t cols[kMostLooked];
    if (hipMemcpyAsync(cols, col + (ends[0] - base), count * sizeof(idx_t), hipMemcpyDeviceToHost, stream) != hipSuccess ||
        hipStreamSynchronize(stream) != hipSuccess)
        return 0;
    std::sort(cols, cols + count);
    uint32_t best = 0;
    idx_t run_start = cols[0];
    for (idx_t i = 1; i < count; ++i) {
        if (cols[i] <= cols[i - 1] + 1) continue;  // the run goes on (or a duplicate)
        const uint64_t gap = static_cast<uint64_t>(cols[i]) - run_start;
        run_start = cols[i];
        if (gap > 0xffffffffull) continue;
        const uint32_t stride = static_cast<uint32_t>(gap);
        if (mcsp::spmm_strip_stride_usable(m, stride) && (best == 0 || stride < best)) best = stride;
    }
    return best;
}

}  // namespace

mcsparseStatus_t mcsparseSpMM_preprocess(mcsparseHandle_t handle, mcsparseOperation_t opA, mcsparseOperation_t opB,
                                         const void* alpha, mcsparseSpMatDescr_t matA, mcsparseDnMatDescr_t matB,
                                         const void* beta, mcsparseDnMatDescr_t matC, macaDataType /*computeType*/,
                                         mcsparseSpMMAlg_t /*alg*/, void* externalBuffer) {
    if (matA != nullptr) {
        const mcspStatus_t it = check_index_types(matA);
        if (it != MCSP_STATUS_SUCCESS) return to_public_status(it);
    }
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (externalBuffer == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    const mcspStatus_t st = check_spmm_args(handle, alpha, matA, matB, beta, matC);
    if (st != MCSP_STATUS_SUCCESS) return to_public_status(st);
    matA->schedule.valid = false;
    // the schedule's size is read back: not possible on a stream under graph capture
    if (stream_is_capturing(handle->stream)) return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);
    if (opA != MCSPARSE_OPERATION_NON_TRANSPOSE || !schedulable(matA) || matA->rows == nullptr || matA->cols == nullptr ||
        matC->col_num <= 0)
        return MCSPARSE_STATUS_SUCCESS;  // nothing to prepare for this call

    const idx_t m = static_cast<idx_t>(matA->row_num);
    const idx_t nnz = static_cast<idx_t>(matA->nnz);
    const IndexArrays ia = index_arrays(handle, matA, static_cast<char*>(externalBuffer) +
                                                          spmm_layout(matA, matB, matC, opB, value_size(matA->valueType)).narrow);
    const mcsp::SpmmScheduleLayout l = mcsp::spmm_schedule_layout(m, nnz);
    SpmmSchedule& s = matA->schedule;
    s.buffer = externalBuffer;
    s.rows = matA->rows;
    s.cols = matA->cols;
    s.m = matA->row_num;
    s.nnz = matA->nnz;
    s.base = static_cast<int>(matA->idxBase);
    s.blocks = false;
    s.stride = 0;
    {
        // The kernels that work from a schedule walk every row in one piece; a matrix with rows of thousands of
        // nonzeros is left to the row kernels, which hand such rows to the kernels of spmm_long.hip.
        const size_t vb0 = value_size(matA->valueType);
        const mcspStatus_t ps =
            ensure_plan(handle, matA, ia.rows, matA->rows, matA->row_num, matA->nnz, matA->col_num * static_cast<int64_t>(vb0),
                        static_cast<char*>(externalBuffer) + spmm_layout(matA, matB, matC, opB, vb0).long_ws, true);
        if (ps != MCSP_STATUS_SUCCESS) return to_public_status(ps);
        if (matA->plan.valid && matA->plan.forced_family == kFamilyAuto && matA->plan.max_row_len > mcsp::kSpmmLongRow) {
            s.entries = 0;
            s.useful = false;
            s.valid = true;
            return MCSPARSE_STATUS_SUCCESS;
        }
    }
    const char* span_slot = static_cast<const char*>(externalBuffer) + l.span_sum;

    // First choice, for operands of 65 (fp64: 129) to 1024 bytes per row (the widths its kernel was measured faster at: by 35 %,
    // 16 %, 29 % and 4 % at 32, 64, 128 and 256 fp32 columns of a 27-point stencil): diagonal blocks over groups of
    // eight rows.  Kept when the blocks are large (a stencil's are 24 nonzeros each) and each loaded row of op(B)
    // serves about two nonzeros or more; matrices without such structure get the merged column lists.
    const size_t vb = value_size(matA->valueType);
    const int64_t row_bytes = matC->col_num * static_cast<int64_t>(vb);
    // (in fp64 from 129 bytes: at 12 and 16 columns of a 27-point stencil the kernel without a schedule is 2 and 5 %
    // faster)
    const bool wide_enough = row_bytes > (vb == 8 ? 128 : 64) && row_bytes <= 1024 && matA->row_num < (int64_t(1) << 31);
    if (wide_enough) {
        mcsp::launch_spmm_block_count(handle->stream, m, nnz, static_cast<idx_t>(matA->idxBase), ia.rows, ia.cols,
                                      externalBuffer);
        const uint64_t block_groups = mcsp::spmm_block_groups(m);
        uint32_t blocks = 0;
        unsigned long long counters[3] = {0, 0, 0};  // span sum, rows of op(B) loaded, longest group (low 32 bits)
        const char* total_slot = static_cast<const char*>(externalBuffer) + l.group_ptr + block_groups * sizeof(uint32_t);
        if (hipMemcpyAsync(&blocks, total_slot, sizeof(blocks), hipMemcpyDeviceToHost, handle->stream) != hipSuccess ||
            hipMemcpyAsync(counters, span_slot, sizeof(counters), hipMemcpyDeviceToHost, handle->stream) != hipSuccess ||
            hipStreamSynchronize(handle->stream) != hipSuccess)
            return to_public_status(MCSP_STATUS_INTERNAL_ERROR);
        const uint64_t nz = static_cast<uint64_t>(matA->nnz);
        if (blocks != 0 && static_cast<uint64_t>(blocks) * 8 <= nz && counters[1] * 9 <= nz * 5 &&
            mcsp::spmm_block_schedule_fits(m, nnz, blocks)) {
            // The matrix has diagonals.  Where rows a fixed distance apart hold the same ones (the neighbouring lines
            // of a structured grid), groups of strips that far apart share more of the loaded rows of op(B): the
            // distance is read off a row in the middle, the gain is measured by covering the matrix that way, and the
            // strips are kept when they load a fifth fewer rows.
            // (Their kernel gives sixteen lanes of 16 bytes to a group and writes a column-major C in pieces of four
            // rows: for operands of up to 128 bytes per row, and for a column-major C, the groups of eight rows stay.)
            const bool strips_suit = row_bytes > 128 && matC->order == MCSPARSE_ORDER_ROW;
            const uint32_t stride = !strips_suit ? 0u
                                                 : strip_stride_of_middle_row(handle->stream, m, static_cast<idx_t>(matA->idxBase),
                                                                              ia.rows, ia.cols);
            if (stride != 0) {
                mcsp::launch_spmm_strip_count(handle->stream, m, nnz, static_cast<idx_t>(matA->idxBase), stride, ia.rows,
                                              ia.cols, externalBuffer);
                const uint64_t strip_groups = mcsp::spmm_strip_groups(m, stride);
                uint32_t strip_blocks = 0;
                unsigned long long strip_counters[3] = {0, 0, 0};  // span sum, rows of op(B) loaded, longest strip
                const char* strip_total = static_cast<const char*>(externalBuffer) + l.group_ptr + strip_groups * sizeof(uint32_t);
                if (hipMemcpyAsync(&strip_blocks, strip_total, sizeof(strip_blocks), hipMemcpyDeviceToHost, handle->stream) != hipSuccess ||
                    hipMemcpyAsync(strip_counters, span_slot, sizeof(strip_counters), hipMemcpyDeviceToHost, handle->stream) != hipSuccess ||
                    hipStreamSynchronize(handle->stream) != hipSuccess)
                    return to_public_status(MCSP_STATUS_INTERNAL_ERROR);
                // (and its strips' values fit the copies in LDS: read where they lie, 16 rows' values cost more than they save)
                if (strip_blocks != 0 && strip_counters[1] * 5 <= counters[1] * 4 &&
                    (strip_counters[2] & 0xffffffffull) <= mcsp::kSpmmStripStagedValues &&
                    mcsp::spmm_strip_schedule_fits(m, nnz, stride, strip_blocks)) {
                    mcsp::launch_spmm_strip_fill(handle->stream, m, nnz, static_cast<idx_t>(matA->idxBase), stride, ia.rows,
                                                 ia.cols, externalBuffer);
                    s.entries = strip_blocks;
                    s.mean_span = strip_groups != 0 ? strip_counters[0] / strip_groups : 0;
                    s.blocks = true;
                    s.stride = stride;
                    s.longest_group = static_cast<uint32_t>(strip_counters[2] & 0xffffffffull);
                    s.useful = true;
                    s.valid = true;
                    return MCSPARSE_STATUS_SUCCESS;
                }
                // not worth it: the offsets of the groups of eight rows are counted again (the region is shared)
                mcsp::launch_spmm_block_count(handle->stream, m, nnz, static_cast<idx_t>(matA->idxBase), ia.rows, ia.cols,
                                              externalBuffer);
            }
            mcsp::launch_spmm_block_fill(handle->stream, m, nnz, static_cast<idx_t>(matA->idxBase), ia.rows, ia.cols,
                                         externalBuffer);
            s.entries = blocks;
            s.mean_span = block_groups != 0 ? counters[0] / block_groups : 0;
            s.blocks = true;
            s.longest_group = static_cast<uint32_t>(counters[2] & 0xffffffffull);
            s.useful = true;
            s.valid = true;
            return MCSPARSE_STATUS_SUCCESS;
        }
    }

    mcsp::launch_spmm_schedule(handle->stream, m, nnz, static_cast<idx_t>(matA->idxBase), ia.rows, ia.cols,
                               externalBuffer);
    const uint64_t groups = mcsp::spmm_groups(m);
    uint32_t entries = 0;
    const char* total_slot = static_cast<const char*>(externalBuffer) + l.group_ptr + groups * sizeof(uint32_t);
    unsigned long long span_sum = 0;
    if (hipMemcpyAsync(&entries, total_slot, sizeof(entries), hipMemcpyDeviceToHost, handle->stream) != hipSuccess ||
        hipMemcpyAsync(&span_sum, span_slot, sizeof(span_sum), hipMemcpyDeviceToHost, handle->stream) != hipSuccess ||
        hipStreamSynchronize(handle->stream) != hipSuccess)
        return to_public_status(MCSP_STATUS_INTERNAL_ERROR);
    s.entries = entries;
    s.mean_span = groups != 0 ? span_sum / groups : 0;
    // Worth it when the merged lists are clearly shorter than the rows they replace; groups too
    // long to merge contribute no entries and are not evidence either way.
    s.useful = entries != 0 && static_cast<uint64_t>(entries) * 100 <= static_cast<uint64_t>(matA->nnz) * 85;
    s.valid = true;
    return MCSPARSE_STATUS_SUCCESS;
}

// reference: src/kernels/level3/spmm/mcsp_spmm_gpu.cpp:785-867, :972-982, :82-162
mcsparseStatus_t mcsparseSpMM(mcsparseHandle_t handle, mcsparseOperation_t opA, mcsparseOperation_t opB,
                              const void* alpha, mcsparseSpMatDescr_t matA, mcsparseDnMatDescr_t matB,
                              const void* beta, mcsparseDnMatDescr_t matC, macaDataType computeType,
                              mcsparseSpMMAlg_t /*alg*/, void* externalBuffer) {
    if (matA != nullptr) {
        const mcspStatus_t it = check_index_types(matA);
        if (it != MCSP_STATUS_SUCCESS) return to_public_status(it);
    }
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (externalBuffer == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    mcspStatus_t st = check_spmm_args(handle, alpha, matA, matB, beta, matC);
    if (st != MCSP_STATUS_SUCCESS) return to_public_status(st);
    if (!format_is_built(matA->format)) return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);  // Blocked-ELL
    if (!(computeType == matA->valueType && computeType == matC->valueType && computeType == matB->valueType))
        return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);
    // op(A) != N is not implemented by the reference for CSR, COO or transposed CSC (:105-108)
    if (opA != MCSPARSE_OPERATION_NON_TRANSPOSE) return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);
    // Shapes the reference never checks and then reads out of bounds on: C is m x n, op(B) is k x n.
    const bool op_n = opB == MCSPARSE_OPERATION_NON_TRANSPOSE;
    const int64_t b_rows = op_n ? matB->row_num : matB->col_num;
    const int64_t b_cols = op_n ? matB->col_num : matB->row_num;
    if (matC->row_num != matA->row_num || b_rows != matA->col_num || b_cols != matC->col_num)
        return to_public_status(MCSP_STATUS_INVALID_SIZE);
    const int64_t b_lead = matB->order == MCSPARSE_ORDER_ROW ? matB->col_num : matB->row_num;
    const int64_t c_lead = matC->order == MCSPARSE_ORDER_ROW ? matC->col_num : matC->row_num;
    if (matB->ld < b_lead || matC->ld < c_lead) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    // reference: mcsp_spmm_gpu.cpp:96-98
    if (!(matC->batchCount == matA->batchCount && matC->batchCount == matB->batchCount))
        return to_public_status(MCSP_STATUS_INVALID_SIZE);
    // the reference hands NULL arrays back as INVALID_POINTER (mcsp_spmm_gpu.cpp:100-103); a kernel
    // would fault on them.  Arrays that a call without nonzeros never reads may be NULL.
    if (matC->values == nullptr || (matA->format == MCSPARSE_FORMAT_CSR && matA->rows == nullptr) ||
        (matA->nnz != 0 && (matA->rows == nullptr || matA->cols == nullptr || matA->vals == nullptr ||
                            matB->values == nullptr)))
        return to_public_status(MCSP_STATUS_INVALID_POINTER);

    switch (computeType) {
        case MACA_R_32F: st = spmm_typed<float>(handle, matA, opB, alpha, beta, matB, matC, externalBuffer); break;
        case MACA_R_64F: st = spmm_typed<double>(handle, matA, opB, alpha, beta, matB, matC, externalBuffer); break;
        default: st = MCSP_STATUS_NOT_IMPLEMENTED;
    }
    return to_public_status(st);
}

// reference: src/kernels/conversion/mcsp_coo2csr.cpp:7-32, :85-88
mcsparseStatus_t mcsparseXcoo2csr(mcsparseHandle_t handle, const int* coo_rows, int nnz, int m, int* csr_rows,
                                  mcsparseIndexBase_t idx_base) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (nnz == 0) return MCSPARSE_STATUS_SUCCESS;  // csr_rows is left untouched, as in the reference
    // negative sizes arrive as huge unsigned values in the reference (uint32 casts); refuse them
    if (m < 0 || nnz < 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    if (coo_rows == nullptr || csr_rows == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    mcsp::launch_coo2csr(handle->stream, static_cast<idx_t>(nnz), static_cast<idx_t>(m),
                         reinterpret_cast<const idx_t*>(coo_rows), static_cast<idx_t>(idx_base),
                         reinterpret_cast<idx_t*>(csr_rows));
    return MCSPARSE_STATUS_SUCCESS;
}

// reference: src/kernels/conversion/mcsp_coo2csr.cpp:34-59, :90-93
mcsparseStatus_t mcsparseXcsr2coo(mcsparseHandle_t handle, const int* csr_rows, int nnz, int m, int* coo_rows,
                                  mcsparseIndexBase_t idx_base) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (nnz == 0) return MCSPARSE_STATUS_SUCCESS;
    if (m < 0 || nnz < 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    if (coo_rows == nullptr || csr_rows == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    mcsp::launch_csr2coo(handle->stream, static_cast<idx_t>(m), static_cast<idx_t>(nnz),
                         reinterpret_cast<const idx_t*>(csr_rows), static_cast<idx_t>(idx_base),
                         reinterpret_cast<idx_t*>(coo_rows));
    return MCSPARSE_STATUS_SUCCESS;
}

// reference: src/kernels/conversion/mcsp_csr2csc.cpp:9-41, :312-320
mcsparseStatus_t mcsparseCsr2cscEx2_bufferSize(mcsparseHandle_t handle, int m, int n, int nnz, const void* /*csr_val*/,
                                               const int* /*csr_rows*/, const int* /*csr_cols*/, void* /*csc_val*/,
                                               int* /*csc_cols*/, int* /*csc_rows*/, macaDataType val_type,
                                               mcsparseAction_t csc_action, mcsparseIndexBase_t /*idx_base*/,
                                               mcsparseCsr2CscAlg_t /*alg*/, size_t* buffer_size) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (n < 0 || m < 0 || nnz < 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    if (buffer_size == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (n == 0 || m == 0 || nnz == 0) {
        *buffer_size = kMinBuffer;
        return MCSPARSE_STATUS_SUCCESS;
    }
    // The reference sizes for the numeric case whatever the action; so does this.
    size_t vb = value_size(val_type);
    if (vb != 4 && vb != 8) vb = 8;
    (void)csc_action;
    *buffer_size = mcsp::csr2csc_workspace_bytes(static_cast<idx_t>(m), static_cast<idx_t>(n),
                                                 static_cast<idx_t>(nnz), vb);
    if (*buffer_size < kMinBuffer) *buffer_size = kMinBuffer;
    return MCSPARSE_STATUS_SUCCESS;
}

// reference: src/kernels/conversion/mcsp_csr2csc.cpp:43-132, :293-310
mcsparseStatus_t mcsparseCsr2cscEx2(mcsparseHandle_t handle, int m, int n, int nnz, const void* csr_val,
                                    const int* csr_rows, const int* csr_cols, void* csc_val, int* csc_cols,
                                    int* csc_rows, macaDataType val_type, mcsparseAction_t csc_action,
                                    mcsparseIndexBase_t idx_base, mcsparseCsr2CscAlg_t /*alg*/, void* temp_buffer) {
    // value types the reference's switch accepts (:297-309); complex ones are not built here
    size_t vb;
    switch (val_type) {
        case MACA_R_32F: vb = 4; break;
        case MACA_R_64F: vb = 8; break;
        case MACA_C_32F: case MACA_C_64F: return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);
        default: return to_public_status(MCSP_STATUS_TYPE_MISMATCH);
    }
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (n < 0 || m < 0 || nnz < 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    if (n == 0 || m == 0 || nnz == 0) return MCSPARSE_STATUS_SUCCESS;  // outputs untouched (:56-58)
    // value pointers are required even for SYMBOLIC (:60-63)
    if (csr_val == nullptr || csr_rows == nullptr || csr_cols == nullptr || csc_val == nullptr ||
        csc_rows == nullptr || csc_cols == nullptr || temp_buffer == nullptr)
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (csc_action == MCSPARSE_ACTION_SYMBOLIC) vb = 0;
    mcsp::launch_csr2csc(handle->stream, static_cast<idx_t>(m), static_cast<idx_t>(n), static_cast<idx_t>(nnz), csr_val,
                         reinterpret_cast<const idx_t*>(csr_rows), reinterpret_cast<const idx_t*>(csr_cols), csc_val,
                         reinterpret_cast<idx_t*>(csc_rows), reinterpret_cast<idx_t*>(csc_cols), vb,
                         static_cast<idx_t>(idx_base), temp_buffer);
    return MCSPARSE_STATUS_SUCCESS;
}

// EXTENSION
mcsparseStatus_t mcsparseXcsrRowBinsPlan(const uint32_t* bin_hist, int64_t m, int64_t nnz, int64_t x_bytes, int* family,
                                         int* lanes_per_row) {
    if (bin_hist == nullptr || family == nullptr || lanes_per_row == nullptr)
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (m < 0 || nnz < 0 || !fits_32(m) || !fits_32(nnz)) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    mcsp::spmv_plan_from_bins(bin_hist, m, nnz, x_bytes, family, lanes_per_row);
    return MCSPARSE_STATUS_SUCCESS;
}

// EXTENSION
mcsparseStatus_t mcsparseXcsrRowBins(mcsparseHandle_t handle, int m, const int* csr_rows, mcsparseIndexBase_t idx_base,
                                     uint8_t* row_bins, uint32_t* bin_hist) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (m < 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    if (csr_rows == nullptr || bin_hist == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    mcsp::launch_row_bins(handle->stream, static_cast<idx_t>(m), reinterpret_cast<const idx_t*>(csr_rows),
                          static_cast<idx_t>(idx_base), row_bins, bin_hist);
    return MCSPARSE_STATUS_SUCCESS;
}

// EXTENSION: a measuring stick, not part of the path (see include/mcsparse.h)
mcsparseStatus_t mcsparseXstreamProbe(mcsparseHandle_t handle, int mode, const void* src, void* dst, size_t bytes,
                                      uint32_t* sink, size_t sink_words) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (mode < 0 || mode > 2 || bytes % 16 != 0) return to_public_status(MCSP_STATUS_INVALID_VALUE);
    if ((mode != 1 && src == nullptr) || (mode != 0 && dst == nullptr) || (mode == 0 && sink == nullptr))
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) != 0)
        return to_public_status(MCSP_STATUS_INVALID_VALUE);
    if ((mode == 0 && sink_words == 0) || bytes >= (size_t(1) << 44)) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    mcsp::launch_stream_probe(handle->stream, mode, src, dst, bytes, sink,
                              static_cast<uint32_t>(sink_words < 0xffffffffu ? sink_words : 0xffffffffu));
    return MCSPARSE_STATUS_SUCCESS;
}

}  // extern "C"
