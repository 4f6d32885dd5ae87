// Legacy typed entry points (csrmv, CsrmvEx, csrmm, csrmm2) and the matrix descriptor they
// take.  They are thin adapters onto the kernels of the generic path, with the argument checks
// of the reference's templates.
#include <cstring>
#include <new>

#include "internal.h"

using mcsp::idx_t;

namespace {

template <typename T>
bool legacy_scalar(mcsparseHandle_t h, const T* p, T* out) {
    if (h->ptr_mode == MCSPARSE_POINTER_MODE_HOST) {
        *out = *p;
        return true;
    }
    if (hipMemcpyAsync(out, p, sizeof(T), hipMemcpyDeviceToHost, h->stream) != hipSuccess) return false;
    return hipStreamSynchronize(h->stream) == hipSuccess;
}

bool descr_is_plain(const mcsparseMatDescr* d) {
    return d->type == MCSPARSE_MATRIX_TYPE_GENERAL && d->fill_mode == MCSPARSE_FILL_MODE_FULL &&
           d->diag_type == MCSPARSE_DIAG_TYPE_NON_UNIT;
}

// reference: mcspSpmvCsrVectorTemplate, src/kernels/level2/spmv/mcsp_spmv_gpu.cpp:203-259.
// `workspace` non-null selects the merge-path kernel.
template <typename T>
mcspStatus_t csrmv_impl(mcsparseHandle_t handle, int m, int n, int nnz, const T* alpha, const mcsparseMatDescr* descr,
                        const T* val, const int* row_ptr, const int* col, const T* x, const T* beta, T* y) {
    if (handle == nullptr) return MCSP_STATUS_INVALID_HANDLE;
    if (nnz < 0 || m < 0 || n < 0) return MCSP_STATUS_INVALID_SIZE;  // dead in the reference (uint32 casts)
    if (alpha == nullptr || beta == nullptr || row_ptr == nullptr || col == nullptr || val == nullptr ||
        x == nullptr || y == nullptr || descr == nullptr)
        return MCSP_STATUS_INVALID_POINTER;
    if (!descr_is_plain(descr)) return MCSP_STATUS_NOT_IMPLEMENTED;
    T h_alpha, h_beta;
    if (!legacy_scalar(handle, beta, &h_beta) || !legacy_scalar(handle, alpha, &h_alpha))
        return MCSP_STATUS_INTERNAL_ERROR;
    if (nnz == 0 || (h_alpha == T(0) && h_beta == T(0))) return MCSP_STATUS_SUCCESS;  // :235-237
    mcsp::SpmvArgs a;
    a.m = static_cast<idx_t>(m);
    a.n = static_cast<idx_t>(n);
    a.nnz = static_cast<idx_t>(nnz);
    a.base = static_cast<idx_t>(descr->base);
    a.row_ptr = reinterpret_cast<const idx_t*>(row_ptr);
    a.col = reinterpret_cast<const idx_t*>(col);
    a.val = val;
    a.x = x;
    a.y = y;
    // the typed entry points have no buffer whose size is known (csrmv has none, CsrmvEx's is the
    // reference's constant 128 bytes and is never touched there, :905-944): row-per-lane-group kernel
    mcsp::launch_spmv_vector<T>(handle->stream, a, h_alpha, h_beta, mcsp::spmv_pick_lanes(a.m, a.nnz));
    return MCSP_STATUS_SUCCESS;
}

// reference: mcspCsrSpmmTemplate, src/kernels/level3/spmm/mcsp_spmm_gpu.cpp:19-80
template <typename T>
mcspStatus_t csrmm2_impl(mcsparseHandle_t handle, mcsparseOperation_t trans_a, mcsparseOperation_t trans_b, int m,
                         int n, int k, int nnz, const T* alpha, const mcsparseMatDescr* descr, const T* val,
                         const int* row_ptr, const int* col, const T* B, int ldb, const T* beta, T* C, int ldc) {
    if (handle == nullptr) return MCSP_STATUS_INVALID_HANDLE;
    if (m < 0 || n < 0 || k < 0 || nnz < 0) return MCSP_STATUS_INVALID_SIZE;
    if (alpha == nullptr || beta == nullptr || val == nullptr || row_ptr == nullptr || col == nullptr ||
        B == nullptr || C == nullptr || descr == nullptr)
        return MCSP_STATUS_INVALID_POINTER;
    if (trans_a != MCSPARSE_OPERATION_NON_TRANSPOSE || !descr_is_plain(descr)) return MCSP_STATUS_NOT_IMPLEMENTED;
    // leading dimensions the reference never checks and then reads out of bounds on
    const bool b_t = trans_b != MCSPARSE_OPERATION_NON_TRANSPOSE;
    if (ldb < (b_t ? n : k) || ldc < m) return MCSP_STATUS_INVALID_SIZE;
    T h_alpha, h_beta;
    if (!legacy_scalar(handle, beta, &h_beta) || !legacy_scalar(handle, alpha, &h_alpha))
        return MCSP_STATUS_INTERNAL_ERROR;
    if (nnz == 0 && h_beta == T(1)) return MCSP_STATUS_SUCCESS;  // :46-48
    mcsp::SpmmArgs a;
    a.m = static_cast<idx_t>(m);
    a.n = static_cast<idx_t>(n);
    a.k = static_cast<idx_t>(k);
    a.nnz = static_cast<idx_t>(nnz);
    a.base = static_cast<idx_t>(descr->base);
    a.row_ptr = reinterpret_cast<const idx_t*>(row_ptr);
    a.col = reinterpret_cast<const idx_t*>(col);
    a.val = val;
    a.B = B;
    a.ldb = ldb;
    // B is column-major: transB = N gives op(B)(kk, j) at j*ldb + kk; transB = T stores the n x k
    // matrix, whose image is op(B) row-major -- read in place instead of the reference's copy (:50-63)
    a.b_row_major = b_t;
    a.C = C;
    a.ldc = ldc;
    a.c_row_major = false;
    mcsp::launch_spmm<T>(handle->stream, a, h_alpha, h_beta);
    return MCSP_STATUS_SUCCESS;
}

}  // namespace

extern "C" {

// ---- matrix descriptor: src/common/mcsp_helper.cpp:90-112, :200-292 ----------------------

mcsparseStatus_t mcsparseCreateMatDescr(mcsparseMatDescr_t* descr) {
    if (descr == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *descr = new (std::nothrow) mcsparseMatDescr();
    return to_public_status(*descr == nullptr ? MCSP_STATUS_INTERNAL_ERROR : MCSP_STATUS_SUCCESS);
}

mcsparseStatus_t mcsparseDestroyMatDescr(mcsparseMatDescr_t descr) {
    delete descr;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseCopyMatDescr(mcsparseMatDescr_t, const mcsparseMatDescr_t) {
    return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);  // :127-129
}

mcsparseStatus_t mcsparseSetMatIndexBase(mcsparseMatDescr_t descr, mcsparseIndexBase_t index_base) {
    if (descr == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (index_base != MCSPARSE_INDEX_BASE_ZERO && index_base != MCSPARSE_INDEX_BASE_ONE)
        return to_public_status(MCSP_STATUS_INVALID_VALUE);
    descr->base = index_base;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseIndexBase_t mcsparseGetMatIndexBase(const mcsparseMatDescr_t descr) {
    return descr == nullptr ? static_cast<mcsparseIndexBase_t>(-1) : descr->base;
}

mcsparseStatus_t mcsparseSetMatType(mcsparseMatDescr_t descr, mcsparseMatrixType_t t) {
    if (descr == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (t != MCSPARSE_MATRIX_TYPE_GENERAL && t != MCSPARSE_MATRIX_TYPE_HERMITIAN &&
        t != MCSPARSE_MATRIX_TYPE_SYMMETRIC && t != MCSPARSE_MATRIX_TYPE_TRIANGULAR)
        return to_public_status(MCSP_STATUS_INVALID_VALUE);
    descr->type = t;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseMatrixType_t mcsparseGetMatType(const mcsparseMatDescr_t descr) {
    return descr == nullptr ? static_cast<mcsparseMatrixType_t>(-1) : descr->type;
}

mcsparseStatus_t mcsparseSetMatFillMode(mcsparseMatDescr_t descr, mcsparseFillMode_t mode) {
    if (descr == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (mode != MCSPARSE_FILL_MODE_FULL && mode != MCSPARSE_FILL_MODE_LOWER && mode != MCSPARSE_FILL_MODE_UPPER)
        return to_public_status(MCSP_STATUS_INVALID_VALUE);
    descr->fill_mode = mode;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseFillMode_t mcsparseGetMatFillMode(const mcsparseMatDescr_t descr) {
    return descr == nullptr ? static_cast<mcsparseFillMode_t>(-1) : descr->fill_mode;
}

mcsparseStatus_t mcsparseSetMatDiagType(mcsparseMatDescr_t descr, mcsparseDiagType_t diag_type) {
    if (descr == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (diag_type != MCSPARSE_DIAG_TYPE_NON_UNIT && diag_type != MCSPARSE_DIAG_TYPE_UNIT)
        return to_public_status(MCSP_STATUS_INVALID_VALUE);
    descr->diag_type = diag_type;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseDiagType_t mcsparseGetMatDiagType(const mcsparseMatDescr_t descr) {
    return descr == nullptr ? static_cast<mcsparseDiagType_t>(-1) : descr->diag_type;
}

mcsparseStatus_t mcsparseSetStorageMode(mcsparseMatDescr_t descr, mcsparseStorageMode_t storage_mode) {
    if (descr == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (storage_mode != MCSPARSE_STORAGE_MODE_SORTED && storage_mode != MCSPARSE_STORAGE_MODE_UNSORTED)
        return to_public_status(MCSP_STATUS_INVALID_VALUE);
    descr->storage_mode = storage_mode;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseGetStorageMode(const mcsparseMatDescr_t descr, mcsparseStorageMode_t* storage_mode) {
    if (descr == nullptr || storage_mode == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *storage_mode = descr->storage_mode;
    return MCSPARSE_STATUS_SUCCESS;
}

// ---- csrmv: src/kernels/level2/spmv/mcsp_spmv_gpu.cpp:946-953, :1190-1202 ------------------

mcsparseStatus_t mcsparseScsrmv(mcsparseHandle_t handle, mcsparseOperation_t /*transA*/, int m, int n, int nnz,
                                const float* alpha, const mcsparseMatDescr_t descrA, const float* csrValA,
                                const int* csrRowPtrA, const int* csrColIndA, const float* x, const float* beta,
                                float* y) {
    return to_public_status(
        csrmv_impl<float>(handle, m, n, nnz, alpha, descrA, csrValA, csrRowPtrA, csrColIndA, x, beta, y));
}

mcsparseStatus_t mcsparseDcsrmv(mcsparseHandle_t handle, mcsparseOperation_t /*transA*/, int m, int n, int nnz,
                                const double* alpha, const mcsparseMatDescr_t descrA, const double* csrValA,
                                const int* csrRowPtrA, const int* csrColIndA, const double* x, const double* beta,
                                double* y) {
    return to_public_status(
        csrmv_impl<double>(handle, m, n, nnz, alpha, descrA, csrValA, csrRowPtrA, csrColIndA, x, beta, y));
}

// reference: :1149-1158 writes 128 without looking at any argument; the same constant here, so
// that a caller with the reference's size compiled in stays inside its buffer
mcsparseStatus_t mcsparseCsrmvEx_bufferSize(mcsparseHandle_t handle, mcsparseAlgMode_t, mcsparseOperation_t, int m,
                                            int /*n*/, int nnz, const void*, macaDataType, const mcsparseMatDescr_t,
                                            const void*, macaDataType, const int*, const int*, const void*,
                                            macaDataType, const void*, macaDataType, void*, macaDataType, macaDataType,
                                            size_t* bufferSizeInBytes) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (bufferSizeInBytes == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (m < 0 || nnz < 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    *bufferSizeInBytes = kMinBuffer;
    return MCSPARSE_STATUS_SUCCESS;
}

// reference: mcspCsrmvExImpl, :905-944
mcsparseStatus_t mcsparseCsrmvEx(mcsparseHandle_t handle, mcsparseAlgMode_t, mcsparseOperation_t /*transA*/, int m,
                                 int n, int nnz, const void* alpha, macaDataType alphatype,
                                 const mcsparseMatDescr_t descrA, const void* csrValA, macaDataType csrValAtype,
                                 const int* csrRowPtrA, const int* csrColIndA, const void* x, macaDataType xtype,
                                 const void* beta, macaDataType betatype, void* y, macaDataType ytype,
                                 macaDataType executiontype, void* /*buffer*/) {
    if (!(alphatype == xtype && csrValAtype == xtype && betatype == xtype && ytype == xtype &&
          executiontype == xtype))
        return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);
    // the buffer is neither checked nor used, as in the reference
    switch (csrValAtype) {
        case MACA_R_32F:
            return to_public_status(csrmv_impl<float>(
                handle, m, n, nnz, static_cast<const float*>(alpha), descrA, static_cast<const float*>(csrValA),
                csrRowPtrA, csrColIndA, static_cast<const float*>(x), static_cast<const float*>(beta),
                static_cast<float*>(y)));
        case MACA_R_64F:
            return to_public_status(csrmv_impl<double>(
                handle, m, n, nnz, static_cast<const double*>(alpha), descrA, static_cast<const double*>(csrValA),
                csrRowPtrA, csrColIndA, static_cast<const double*>(x), static_cast<const double*>(beta),
                static_cast<double*>(y)));
        default:
            return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);  // complex types are not built
    }
}

// ---- csrmm / csrmm2: src/kernels/level3/spmm/mcsp_spmm_gpu.cpp:878-948 ----------------------

mcsparseStatus_t mcsparseScsrmm2(mcsparseHandle_t handle, mcsparseOperation_t transA, mcsparseOperation_t transB, int m,
                                 int n, int k, int nnz, const float* alpha, const mcsparseMatDescr_t descrA,
                                 const float* csrValA, const int* csrRowPtrA, const int* csrColIndA, const float* B,
                                 int ldb, const float* beta, float* C, int ldc) {
    return to_public_status(csrmm2_impl<float>(handle, transA, transB, m, n, k, nnz, alpha, descrA, csrValA, csrRowPtrA,
                                               csrColIndA, B, ldb, beta, C, ldc));
}

mcsparseStatus_t mcsparseDcsrmm2(mcsparseHandle_t handle, mcsparseOperation_t transA, mcsparseOperation_t transB, int m,
                                 int n, int k, int nnz, const double* alpha, const mcsparseMatDescr_t descrA,
                                 const double* csrValA, const int* csrRowPtrA, const int* csrColIndA, const double* B,
                                 int ldb, const double* beta, double* C, int ldc) {
    return to_public_status(csrmm2_impl<double>(handle, transA, transB, m, n, k, nnz, alpha, descrA, csrValA,
                                                csrRowPtrA, csrColIndA, B, ldb, beta, C, ldc));
}

// the wrapper forwards csrmm to csrmm2 with transB = N (src/wrapper/mcsp_interface_wrapper.cpp:3743-3758)
mcsparseStatus_t mcsparseScsrmm(mcsparseHandle_t handle, mcsparseOperation_t transA, int m, int n, int k, int nnz,
                                const float* alpha, const mcsparseMatDescr_t descrA, const float* csrValA,
                                const int* csrRowPtrA, const int* csrColIndA, const float* B, int ldb,
                                const float* beta, float* C, int ldc) {
    return mcsparseScsrmm2(handle, transA, MCSPARSE_OPERATION_NON_TRANSPOSE, m, n, k, nnz, alpha, descrA, csrValA,
                           csrRowPtrA, csrColIndA, B, ldb, beta, C, ldc);
}

mcsparseStatus_t mcsparseDcsrmm(mcsparseHandle_t handle, mcsparseOperation_t transA, int m, int n, int k, int nnz,
                                const double* alpha, const mcsparseMatDescr_t descrA, const double* csrValA,
                                const int* csrRowPtrA, const int* csrColIndA, const double* B, int ldb,
                                const double* beta, double* C, int ldc) {
    return mcsparseDcsrmm2(handle, transA, MCSPARSE_OPERATION_NON_TRANSPOSE, m, n, k, nnz, alpha, descrA, csrValA,
                           csrRowPtrA, csrColIndA, B, ldb, beta, C, ldc);
}

}  // extern "C"
