// Index sorts, the identity permutation and the dense gather: what a caller needs to turn an
// unsorted CSR / CSC / COO structure into the sorted form the SpMV / SpMM kernels expect
// (sort the indices with a permutation, then gather the values through it).
//
// The reference builds every sort from two radix sorts of (key, permutation) pairs and three
// gathers through the result (src/kernels/conversion/mcsp_csrsort.cpp:43-121,
// mcsp_coosort.cpp:41-110).  Here the (major, minor, permutation) triples travel through the
// sort passes themselves, so no gather and no copy back follows.  One defect of the reference
// is not reproduced: with a one-based descriptor its gathers subtract the index base from
// zero-based permutation entries (mcsp_csrsort.cpp:95-104 with gthr_device.hpp:8-14), which
// reads one element before the arrays.
#include "internal.h"

using mcsp::idx_t;

namespace {

mcspStatus_t sort_buffer_size(mcsparseHandle_t handle, int m, int n, int nnz, const int* a, const int* b,
                              size_t* buffer_size) {
    // reference: mcsp_csrsort.cpp:13-40, mcsp_coosort.cpp:12-38
    if (handle == nullptr) return MCSP_STATUS_INVALID_HANDLE;
    if (n < 0 || m < 0 || nnz < 0) return MCSP_STATUS_INVALID_SIZE;
    if (a == nullptr || b == nullptr || buffer_size == nullptr) return MCSP_STATUS_INVALID_POINTER;
    if (n == 0 || m == 0 || nnz == 0) {
        *buffer_size = kMinBuffer;
        return MCSP_STATUS_SUCCESS;
    }
    *buffer_size = mcsp::index_sort_workspace_bytes(static_cast<idx_t>(nnz));
    return MCSP_STATUS_SUCCESS;
}

// rows/cols here are the arrays of a CSR structure; the CSC sort passes them swapped.
mcspStatus_t csrsort(mcsparseHandle_t handle, int m, int n, int nnz, mcsparseMatDescr_t descr, const int* offsets,
                     int* indices, int* perm, void* buffer) {
    // reference: mcsp_csrsort.cpp:43-64
    if (handle == nullptr) return MCSP_STATUS_INVALID_HANDLE;
    if (n < 0 || m < 0 || nnz < 0) return MCSP_STATUS_INVALID_SIZE;
    if (n == 0 || m == 0 || nnz == 0) return MCSP_STATUS_SUCCESS;
    if (descr == nullptr || offsets == nullptr || indices == nullptr || buffer == nullptr)
        return MCSP_STATUS_INVALID_POINTER;
    mcsp::launch_csrsort(handle->stream, m, n, nnz, static_cast<idx_t>(descr->base),
                         reinterpret_cast<const idx_t*>(offsets), reinterpret_cast<idx_t*>(indices),
                         reinterpret_cast<idx_t*>(perm), buffer);
    return MCSP_STATUS_SUCCESS;
}

mcspStatus_t coosort(mcsparseHandle_t handle, int major_extent, int minor_extent, int nnz, int* major, int* minor,
                     int* perm, void* buffer) {
    // reference: mcsp_coosort.cpp:41-61
    if (handle == nullptr) return MCSP_STATUS_INVALID_HANDLE;
    if (major_extent < 0 || minor_extent < 0 || nnz < 0) return MCSP_STATUS_INVALID_SIZE;
    if (major_extent == 0 || minor_extent == 0 || nnz == 0) return MCSP_STATUS_SUCCESS;
    if (major == nullptr || minor == nullptr || buffer == nullptr) return MCSP_STATUS_INVALID_POINTER;
    mcsp::launch_coosort(handle->stream, major_extent, minor_extent, nnz, reinterpret_cast<idx_t*>(major),
                         reinterpret_cast<idx_t*>(minor), reinterpret_cast<idx_t*>(perm), buffer);
    return MCSP_STATUS_SUCCESS;
}

template <typename T>
mcspStatus_t gthr(mcsparseHandle_t handle, int nnz, const T* y, T* x_val, const int* x_ind, mcsparseIndexBase_t base) {
    // reference: src/kernels/level1/mcsp_gthr.cpp:7-31
    if (handle == nullptr) return MCSP_STATUS_INVALID_HANDLE;
    if (nnz < 0) return MCSP_STATUS_INVALID_SIZE;
    if (nnz == 0) return MCSP_STATUS_SUCCESS;
    if (y == nullptr || x_val == nullptr || x_ind == nullptr) return MCSP_STATUS_INVALID_POINTER;
    mcsp::launch_gather<T>(handle->stream, nnz, y, x_val, reinterpret_cast<const idx_t*>(x_ind),
                           static_cast<idx_t>(base));
    return MCSP_STATUS_SUCCESS;
}

}  // namespace

extern "C" {

mcsparseStatus_t mcsparseXcsrsort_bufferSizeExt(mcsparseHandle_t handle, int m, int n, int nnz, const int* csr_rows,
                                                const int* csr_cols, size_t* buffer_size) {
    return to_public_status(sort_buffer_size(handle, m, n, nnz, csr_rows, csr_cols, buffer_size));
}

mcsparseStatus_t mcsparseXcsrsort(mcsparseHandle_t handle, int m, int n, int nnz, mcsparseMatDescr_t descr,
                                  const int* csr_rows, int* csr_cols, int* perm, void* temp_buffer) {
    return to_public_status(csrsort(handle, m, n, nnz, descr, csr_rows, csr_cols, perm, temp_buffer));
}

// reference: src/kernels/conversion/mcsp_cscsort.cpp:8-16 (the CSR sort with m and n exchanged)
mcsparseStatus_t mcsparseXcscsort_bufferSizeExt(mcsparseHandle_t handle, int m, int n, int nnz, const int* csc_cols,
                                                const int* csc_rows, size_t* buffer_size) {
    return to_public_status(sort_buffer_size(handle, n, m, nnz, csc_cols, csc_rows, buffer_size));
}

mcsparseStatus_t mcsparseXcscsort(mcsparseHandle_t handle, int m, int n, int nnz, mcsparseMatDescr_t descr,
                                  const int* csc_cols, int* csc_rows, int* perm, void* temp_buffer) {
    return to_public_status(csrsort(handle, n, m, nnz, descr, csc_cols, csc_rows, perm, temp_buffer));
}

mcsparseStatus_t mcsparseXcoosort_bufferSizeExt(mcsparseHandle_t handle, int m, int n, int nnz, const int* coo_rows,
                                                const int* coo_cols, size_t* buffer_size) {
    return to_public_status(sort_buffer_size(handle, m, n, nnz, coo_rows, coo_cols, buffer_size));
}

mcsparseStatus_t mcsparseXcoosortByRow(mcsparseHandle_t handle, int m, int n, int nnz, int* coo_rows, int* coo_cols,
                                       int* perm, void* temp_buffer) {
    return to_public_status(coosort(handle, m, n, nnz, coo_rows, coo_cols, perm, temp_buffer));
}

// reference: mcsp_coosort.cpp:112-116 (the row sort with the roles of the arrays exchanged)
mcsparseStatus_t mcsparseXcoosortByColumn(mcsparseHandle_t handle, int m, int n, int nnz, int* coo_rows, int* coo_cols,
                                          int* perm, void* temp_buffer) {
    return to_public_status(coosort(handle, n, m, nnz, coo_cols, coo_rows, perm, temp_buffer));
}

// reference: src/kernels/conversion/mcsp_create_identity.cpp:6-30
mcsparseStatus_t mcsparseCreateIdentityPermutation(mcsparseHandle_t handle, int n, int* p) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (n < 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    if (p == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    mcsp::launch_identity(handle->stream, n, reinterpret_cast<idx_t*>(p));
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSgthr(mcsparseHandle_t handle, int nnz, const float* y, float* x_val, const int* x_ind,
                               mcsparseIndexBase_t idx_base) {
    return to_public_status(gthr<float>(handle, nnz, y, x_val, x_ind, idx_base));
}

mcsparseStatus_t mcsparseDgthr(mcsparseHandle_t handle, int nnz, const double* y, double* x_val, const int* x_ind,
                               mcsparseIndexBase_t idx_base) {
    return to_public_status(gthr<double>(handle, nnz, y, x_val, x_ind, idx_base));
}

}  // extern "C"
