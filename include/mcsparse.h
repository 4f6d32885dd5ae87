/*
 * mcsparse.h -- C ABI of the CSR SpMV / SpMM / csr2csc / csr2coo path, MI355X (gfx950) build.
 *
 * This is the drop-in boundary: every enum value, opaque handle name and prototype below
 * is the one a program written against MetaX mcSparse already uses for this path, so that
 * program relinks against libmcsparse.so from this repository unchanged.  Each block cites
 * the reference declaration it stands in for (paths relative to the reference checkout,
 * mcsparse/...).  Functions marked EXTENSION have no counterpart in the reference.
 *
 * The stream type of the reference is a build-time substitution
 * (include/interface/mcsp_helper.h.in:21); here it is HIP's stream handle.
 */
#ifndef MCSPARSE_H__
#define MCSPARSE_H__

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The library is built with hidden visibility; what this header declares is its exported surface. */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

/* HIP stream handle.  Re-declaring the typedef is legal when <hip/hip_runtime_api.h>
 * is also included; mcStream_t is kept as the name the reference's users spell. */
struct ihipStream_t;
typedef struct ihipStream_t* hipStream_t;
typedef hipStream_t mcStream_t;

/* ---- value types: include/common/internal/mcsp_datatype.h:5-41 ------------------- */
typedef enum libraryPropertyType_t { MAJOR_VERSION, MINOR_VERSION, PATCH_LEVEL } libraryPropertyType;

typedef enum macaDataType_t {
    MACA_R_32F = 0,
    MACA_R_64F = 1,
    MACA_R_16F = 2,
    MACA_R_8I = 3,
    MACA_C_32F = 4,
    MACA_C_64F = 5,
    MACA_C_16F = 6,
    MACA_C_8I = 7,
    MACA_R_8U = 8,
    MACA_C_8U = 9,
    MACA_R_32I = 10,
    MACA_C_32I = 11,
    MACA_R_32U = 12,
    MACA_C_32U = 13,
    MACA_R_16BF = 14,
    MACA_C_16BF = 15,
    MACA_R_4I = 16,
    MACA_C_4I = 17,
    MACA_R_4U = 18,
    MACA_C_4U = 19,
    MACA_R_16I = 20,
    MACA_C_16I = 21,
    MACA_R_16U = 22,
    MACA_C_16U = 23,
    MACA_R_64I = 24,
    MACA_C_64I = 25,
    MACA_R_64U = 26,
    MACA_C_64U = 27
} macaDataType;

/* ---- enums: include/common/mcsp_types.h.in --------------------------------------- */
/* :18-31 */
typedef enum {
    MCSPARSE_STATUS_SUCCESS = 0,
    MCSPARSE_STATUS_NOT_INITIALIZED = 1,
    MCSPARSE_STATUS_ALLOC_FAILED = 2,
    MCSPARSE_STATUS_INVALID_VALUE = 3,
    MCSPARSE_STATUS_ARCH_MISMATCH = 4,
    MCSPARSE_STATUS_MAPPING_ERROR = 5,
    MCSPARSE_STATUS_EXECUTION_FAILED = 6,
    MCSPARSE_STATUS_INTERNAL_ERROR = 7,
    MCSPARSE_STATUS_MATRIX_TYPE_NOT_SUPPORTED = 8,
    MCSPARSE_STATUS_ZERO_PIVOT = 9,
    MCSPARSE_STATUS_NOT_SUPPORTED = 10,
    MCSPARSE_STATUS_INSUFFICIENT_RESOURCES = 11
} mcsparseStatus_t;

/* :12-16 */
typedef enum {
    MCSPARSE_OPERATION_NON_TRANSPOSE = 0,
    MCSPARSE_OPERATION_TRANSPOSE = 1,
    MCSPARSE_OPERATION_CONJUGATE_TRANSPOSE = 2
} mcsparseOperation_t;

/* :33-38, :52-62 -- matrix descriptor attributes of the legacy typed entry points */
typedef enum {
    MCSPARSE_MATRIX_TYPE_GENERAL = 0,
    MCSPARSE_MATRIX_TYPE_SYMMETRIC = 1,
    MCSPARSE_MATRIX_TYPE_HERMITIAN = 2,
    MCSPARSE_MATRIX_TYPE_TRIANGULAR = 3
} mcsparseMatrixType_t;
typedef enum { MCSPARSE_DIAG_TYPE_NON_UNIT = 0, MCSPARSE_DIAG_TYPE_UNIT = 1 } mcsparseDiagType_t;
typedef enum {
    MCSPARSE_FILL_MODE_LOWER = 0,
    MCSPARSE_FILL_MODE_UPPER = 1,
    MCSPARSE_FILL_MODE_FULL = 2
} mcsparseFillMode_t;
/* :46-49 */
typedef enum { MCSPARSE_STORAGE_MODE_SORTED = 0, MCSPARSE_STORAGE_MODE_UNSORTED = 1 } mcsparseStorageMode_t;
/* :91-93 -- accepted and ignored by mcsparseCsrmvEx, as in the reference */
typedef enum { MCSPARSE_ALG_MERGE_PATH } mcsparseAlgMode_t;

/* :40-44 */
typedef enum { MCSPARSE_INDEX_BASE_ZERO = 0, MCSPARSE_INDEX_BASE_ONE = 1 } mcsparseIndexBase_t;

/* :76-79 */
typedef enum { MCSPARSE_POINTER_MODE_HOST = 0, MCSPARSE_POINTER_MODE_DEVICE = 1 } mcsparsePointerMode_t;

/* :81-84 -- SYMBOLIC converts indices only, NUMERIC converts indices and values */
typedef enum { MCSPARSE_ACTION_SYMBOLIC = 0, MCSPARSE_ACTION_NUMERIC = 1 } mcsparseAction_t;

/* :99-105 */
typedef enum {
    MCSPARSE_FORMAT_CSR = 1,
    MCSPARSE_FORMAT_CSC = 2,
    MCSPARSE_FORMAT_COO = 3,
    MCSPARSE_FORMAT_COO_AOS = 4,
    MCSPARSE_FORMAT_BLOCKED_ELL = 5
} mcsparseFormat_t;

/* :107-110 */
typedef enum { MCSPARSE_ORDER_COL = 1, MCSPARSE_ORDER_ROW = 2 } mcsparseOrder_t;

/* :112-116 -- 32I arrays are processed as unsigned 32-bit (src/include/mcsp_internal_types.h:4) */
typedef enum { MCSPARSE_INDEX_16U = 1, MCSPARSE_INDEX_32I = 2, MCSPARSE_INDEX_64I = 3 } mcsparseIndexType_t;

/* :124-134 -- the reference accepts and ignores them on this path.  Here MCSPARSE_SPMV_CSR_ALG2 (= CSRMV_ALG2)
 * selects the variants whose sums are added in a fixed order, so that two runs give the same bits; every other
 * value the faster ones (see mcsparseSpMV and mcsparseSpMV_preprocess).  The error bound is the same. */
typedef enum {
    MCSPARSE_MV_ALG_DEFAULT = 0,
    MCSPARSE_COOMV_ALG = 1,
    MCSPARSE_CSRMV_ALG1 = 2,
    MCSPARSE_CSRMV_ALG2 = 3,
    MCSPARSE_SPMV_ALG_DEFAULT = 0,
    MCSPARSE_SPMV_CSR_ALG1 = 2,
    MCSPARSE_SPMV_CSR_ALG2 = 3,
    MCSPARSE_SPMV_COO_ALG1 = 1,
    MCSPARSE_SPMV_COO_ALG2 = 4
} mcsparseSpMVAlg_t;

/* :140-155 -- accepted and ignored on this path, as in the reference */
typedef enum {
    MCSPARSE_MM_ALG_DEFAULT = 0,
    MCSPARSE_COOMM_ALG1 = 1,
    MCSPARSE_COOMM_ALG2 = 2,
    MCSPARSE_COOMM_ALG3 = 3,
    MCSPARSE_CSRMM_ALG1 = 4,
    MCSPARSE_SPMM_ALG_DEFAULT = 0,
    MCSPARSE_SPMM_COO_ALG1 = 1,
    MCSPARSE_SPMM_COO_ALG2 = 2,
    MCSPARSE_SPMM_COO_ALG3 = 3,
    MCSPARSE_SPMM_COO_ALG4 = 5,
    MCSPARSE_SPMM_CSR_ALG1 = 4,
    MCSPARSE_SPMM_CSR_ALG2 = 6,
    MCSPARSE_SPMM_CSR_ALG3 = 12,
    MCSPARSE_SPMM_BLOCKED_ELL_ALG1 = 13
} mcsparseSpMMAlg_t;

/* :167-170 -- accepted and ignored (mcsp_csr2csc.cpp:293-310 never reads alg) */
typedef enum { MCSPARSE_CSR2CSC_ALG1 = 1, MCSPARSE_CSR2CSC_ALG2 = 2 } mcsparseCsr2CscAlg_t;

/* ---- opaque handles: include/common/mcsp_types.h.in:190-242 ---------------------- */
struct mcsparseContext;
typedef struct mcsparseContext* mcsparseHandle_t;
struct mcsparseMatDescr;
typedef struct mcsparseMatDescr* mcsparseMatDescr_t;
struct mcsparseSpMatDescr;
typedef struct mcsparseSpMatDescr* mcsparseSpMatDescr_t;
struct mcsparseDnVecDescr;
typedef struct mcsparseDnVecDescr* mcsparseDnVecDescr_t;
struct mcsparseDnMatDescr;
typedef struct mcsparseDnMatDescr* mcsparseDnMatDescr_t;

/* ---- library handle: include/interface/mcsp_helper.h.in:12-29 --------------------- */
/* Unlike src/common/mcsp_handle.cpp:5-22 no device memory pool is reserved: the pool only
 * serves COO SpMV (mcsp_spmv_gpu.cpp:69-75), which is outside this path.  Creating a handle
 * therefore touches no device and succeeds on a host without a GPU. */
mcsparseStatus_t mcsparseCreate(mcsparseHandle_t* handle);                                   /* :12 */
mcsparseStatus_t mcsparseDestroy(mcsparseHandle_t handle);                                   /* :13 */
mcsparseStatus_t mcsparseGetVersion(mcsparseHandle_t handle, int* version);                  /* :15 */
mcsparseStatus_t mcsparseGetProperty(libraryPropertyType type, int* value);                  /* :16 */
const char* mcsparseGetErrorName(mcsparseStatus_t status);                                   /* :18 */
const char* mcsparseGetErrorString(mcsparseStatus_t status);                                 /* :19 */
mcsparseStatus_t mcsparseSetStream(mcsparseHandle_t handle, hipStream_t sid);                /* :21 */
mcsparseStatus_t mcsparseGetStream(const mcsparseHandle_t handle, hipStream_t* sid);         /* :22 */
mcsparseStatus_t mcsparseSetPointerMode(mcsparseHandle_t handle, mcsparsePointerMode_t m);   /* :28 */
mcsparseStatus_t mcsparseGetPointerMode(const mcsparseHandle_t handle, mcsparsePointerMode_t* m); /* :29 */

/* ---- legacy matrix descriptor: mcsp_helper.h.in:24-44 ------------------------------ */
/* Defaults: GENERAL, FULL, NON_UNIT, SORTED, base 0 (src/include/mcsp_internal_types.h:86-94).
 * The getters return (enum)-1 for a NULL descriptor, as the reference does. */
mcsparseStatus_t mcsparseCreateMatDescr(mcsparseMatDescr_t* descr);
mcsparseStatus_t mcsparseDestroyMatDescr(mcsparseMatDescr_t descr);
mcsparseStatus_t mcsparseCopyMatDescr(mcsparseMatDescr_t dest, const mcsparseMatDescr_t src); /* NOT_SUPPORTED there too */
mcsparseStatus_t mcsparseSetMatIndexBase(mcsparseMatDescr_t descr, mcsparseIndexBase_t index_base);
mcsparseIndexBase_t mcsparseGetMatIndexBase(const mcsparseMatDescr_t descr);
mcsparseStatus_t mcsparseSetMatType(mcsparseMatDescr_t descr, mcsparseMatrixType_t matrix_type);
mcsparseMatrixType_t mcsparseGetMatType(const mcsparseMatDescr_t descr);
mcsparseStatus_t mcsparseSetMatFillMode(mcsparseMatDescr_t descr, mcsparseFillMode_t mode);
mcsparseFillMode_t mcsparseGetMatFillMode(const mcsparseMatDescr_t descr);
mcsparseStatus_t mcsparseSetMatDiagType(mcsparseMatDescr_t descr, mcsparseDiagType_t diag_type);
mcsparseDiagType_t mcsparseGetMatDiagType(const mcsparseMatDescr_t descr);
mcsparseStatus_t mcsparseSetStorageMode(mcsparseMatDescr_t descr, mcsparseStorageMode_t storage_mode);
mcsparseStatus_t mcsparseGetStorageMode(const mcsparseMatDescr_t descr, mcsparseStorageMode_t* storage_mode);

/* ---- dense vector descriptor: mcsp_helper.h.in:46-50 ------------------------------ */
mcsparseStatus_t mcsparseCreateDnVec(mcsparseDnVecDescr_t* dnVecDescr, int64_t size, void* values,
                                     macaDataType valueType);
mcsparseStatus_t mcsparseDestroyDnVec(mcsparseDnVecDescr_t dnVecDescr);
mcsparseStatus_t mcsparseDnVecGet(mcsparseDnVecDescr_t dnVecDescr, int64_t* size, void** values,
                                  macaDataType* valueType);
mcsparseStatus_t mcsparseDnVecGetValues(mcsparseDnVecDescr_t dnVecDescr, void** values);
mcsparseStatus_t mcsparseDnVecSetValues(mcsparseDnVecDescr_t dnVecDescr, void* values);

/* ---- sparse matrix descriptor: mcsp_helper.h.in:60-86 ------------------------------ */
/* Descriptors borrow the device pointers; nothing is copied or owned. */
mcsparseStatus_t mcsparseCreateCsr(mcsparseSpMatDescr_t* spMatDescr, int64_t rows, int64_t cols, int64_t nnz,
                                   void* csrRowOffsets, void* csrColInd, void* csrValues,
                                   mcsparseIndexType_t csrRowOffsetsType, mcsparseIndexType_t csrColIndType,
                                   mcsparseIndexBase_t idxBase, macaDataType valueType);    /* :60 */
mcsparseStatus_t mcsparseCsrGet(mcsparseSpMatDescr_t spMatDescr, int64_t* rows, int64_t* cols, int64_t* nnz,
                                void** csrRowOffsets, void** csrColInd, void** csrValues,
                                mcsparseIndexType_t* csrRowOffsetsType, mcsparseIndexType_t* csrColIndType,
                                mcsparseIndexBase_t* idxBase, macaDataType* valueType);     /* :63 */
mcsparseStatus_t mcsparseCsrSetPointers(mcsparseSpMatDescr_t spMatDescr, void* csrRowOffsets, void* csrColInd,
                                        void* csrValues);                                   /* :66 */
mcsparseStatus_t mcsparseCreateCsc(mcsparseSpMatDescr_t* spMatDescr, int64_t rows, int64_t cols, int64_t nnz,
                                   void* cscColOffsets, void* cscRowInd, void* cscValues,
                                   mcsparseIndexType_t cscColOffsetsType, mcsparseIndexType_t cscRowIndType,
                                   mcsparseIndexBase_t idxBase, macaDataType valueType);    /* :69 */
mcsparseStatus_t mcsparseCscSetPointers(mcsparseSpMatDescr_t spMatDescr, void* cscColOffsets, void* cscRowInd,
                                        void* cscValues);                                   /* :72 */
/* COO (structure of arrays) with entries sorted by row, the order the reference's COO kernels
 * assume as well (src/kernels/level2/spmv/coo_flat_device.hpp:65-171 adds partial sums of
 * adjacent equal rows without atomics).  SpMV and SpMM build the row offsets in the scratch
 * buffer and run the CSR kernels.                                                :52-58 */
mcsparseStatus_t mcsparseCreateCoo(mcsparseSpMatDescr_t* spMatDescr, int64_t rows, int64_t cols, int64_t nnz,
                                   void* cooRowInd, void* cooColInd, void* cooValues,
                                   mcsparseIndexType_t cooIdxType, mcsparseIndexBase_t idxBase,
                                   macaDataType valueType);
mcsparseStatus_t mcsparseCooGet(mcsparseSpMatDescr_t spMatDescr, int64_t* rows, int64_t* cols, int64_t* nnz,
                                void** cooRowInd, void** cooColInd, void** cooValues, mcsparseIndexType_t* idxType,
                                mcsparseIndexBase_t* idxBase, macaDataType* valueType);
mcsparseStatus_t mcsparseCooSetPointers(mcsparseSpMatDescr_t spMatDescr, void* cooRows, void* cooColumns,
                                        void* cooValues);
mcsparseStatus_t mcsparseDestroySpMat(mcsparseSpMatDescr_t spMatDescr);                     /* :81 */
mcsparseStatus_t mcsparseSpMatGetSize(mcsparseSpMatDescr_t spMatDescr, int64_t* rows, int64_t* cols,
                                      int64_t* nnz);                                        /* :82 */
mcsparseStatus_t mcsparseSpMatGetFormat(mcsparseSpMatDescr_t spMatDescr, mcsparseFormat_t* format);      /* :83 */
mcsparseStatus_t mcsparseSpMatGetIndexBase(mcsparseSpMatDescr_t spMatDescr, mcsparseIndexBase_t* idxBase); /* :84 */
mcsparseStatus_t mcsparseSpMatGetValues(mcsparseSpMatDescr_t spMatDescr, void** values);    /* :85 */
mcsparseStatus_t mcsparseSpMatSetValues(mcsparseSpMatDescr_t spMatDescr, void* values);     /* :86 */

/* ---- dense matrix descriptor: mcsp_helper.h.in:92-98 ------------------------------- */
mcsparseStatus_t mcsparseCreateDnMat(mcsparseDnMatDescr_t* dnMatDescr, int64_t rows, int64_t cols, int64_t ld,
                                     void* values, macaDataType valueType, mcsparseOrder_t order);
mcsparseStatus_t mcsparseDestroyDnMat(mcsparseDnMatDescr_t dnMatDescr);
mcsparseStatus_t mcsparseDnMatGet(mcsparseDnMatDescr_t dnMatDescr, int64_t* rows, int64_t* cols, int64_t* ld,
                                  void** values, macaDataType* type, mcsparseOrder_t* order);
mcsparseStatus_t mcsparseDnMatGetValues(mcsparseDnMatDescr_t dnMatDescr, void** values);
mcsparseStatus_t mcsparseDnMatSetValues(mcsparseDnMatDescr_t dnMatDescr, void* values);

/* ---- strided batches for SpMM: include/interface/mcsp_generic.h:178-185 ------------- */
/* Batch b of a call uses the arrays moved on by b strides (in elements); all three operands
 * of an SpMM must carry the same batch count (src/kernels/level3/spmm/mcsp_spmm_gpu.cpp:96-98).
 * A stride of 0 shares the array between the batches. */
mcsparseStatus_t mcsparseCooSetStridedBatch(mcsparseSpMatDescr_t spMatDescr, int batchCount, int64_t batchStride);
mcsparseStatus_t mcsparseCsrSetStridedBatch(mcsparseSpMatDescr_t spMatDescr, int batchCount, int64_t offsetsBatchStride,
                                            int64_t columnsValuesBatchStride);
mcsparseStatus_t mcsparseDnMatSetStridedBatch(mcsparseDnMatDescr_t dnMatDescr, int batchCount, int64_t batchStride);
mcsparseStatus_t mcsparseDnMatGetStridedBatch(mcsparseDnMatDescr_t dnMatDescr, int* batchCount, int64_t* batchStride);

/* ---- y = alpha*op(A)*x + beta*y : include/interface/mcsp_generic.h:43-51 ---------- */
/* externalBuffer is caller-allocated device scratch of at least *bufferSize bytes and must be
 * non-NULL even for op N (src/kernels/level2/spmv/mcsp_spmv_gpu.cpp:703-705).  Work is
 * enqueued on the handle's stream.  With MCSPARSE_POINTER_MODE_DEVICE the scalars are read
 * with a blocking copy, as the reference does (src/include/mcsp_internal_host_utils.hpp:34-63).
 *
 * DIFFERENT FROM THE REFERENCE: the buffer is used, and is larger.  The reference returns 128
 * bytes for CSR op N and never writes to the buffer (mcsp_spmv_gpu.cpp:1136-1147); here the
 * buffer holds the row-length histogram and the workspace of the merge-path kernel even for op N
 * (a few bytes per 1024 rows + nonzeros).  A caller that hard-codes the reference's 128 bytes
 * would be written past: always allocate what mcsparseSpMV_bufferSize returns.
 *
 * alg (ignored by the reference): the direct kernels of the non-transposing directions give the same
 * bits on every run whatever alg is.  A transposing call (CSR or COO with op T, CSC with op N) orders the
 * products value * x[row] by column in the buffer: completely under MCSPARSE_SPMV_CSR_ALG2, whose sums
 * then add in row order and repeat their bits; with any other value, for 2^14 to 2^22 columns, only into
 * buckets of neighbouring columns whose sums are formed in the order the products arrive (and for fewer
 * columns with many nonzeros each, not at all: the sums are formed as the nonzeros lie), which is more
 * than twice as fast and stays within the same error bound, but the last bits can differ between runs. */
mcsparseStatus_t mcsparseSpMV(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha,
                              mcsparseSpMatDescr_t matA, mcsparseDnVecDescr_t vecX, const void* beta,
                              mcsparseDnVecDescr_t vecY, macaDataType computeType, mcsparseSpMVAlg_t alg,
                              void* externalBuffer);
mcsparseStatus_t mcsparseSpMV_bufferSize(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha,
                                         mcsparseSpMatDescr_t matA, mcsparseDnVecDescr_t vecX, const void* beta,
                                         mcsparseDnVecDescr_t vecY, macaDataType computeType,
                                         mcsparseSpMVAlg_t alg, size_t* bufferSize);

/* ---- C = alpha*A*op(B) + beta*C : include/interface/mcsp_generic.h:54-67 ---------- */
/* opA must be NON_TRANSPOSE for CSR (src/kernels/level3/spmm/mcsp_spmm_gpu.cpp:105-108).
 * The first mcsparseSpMM on a CSR structure reads the row lengths back once (136 bytes, kept on the descriptor and
 * shared with mcsparseSpMV; not on a stream under graph capture); later calls only enqueue kernels.  Rows of more
 * than 1024 nonzeros are cut into pieces of 4096 that a workgroup each takes, their partial sums kept in
 * externalBuffer and added in the order of the pieces: results repeat bit for bit from run to run. */
mcsparseStatus_t mcsparseSpMM_bufferSize(mcsparseHandle_t handle, mcsparseOperation_t opA, mcsparseOperation_t opB,
                                         const void* alpha, mcsparseSpMatDescr_t matA, mcsparseDnMatDescr_t matB,
                                         const void* beta, mcsparseDnMatDescr_t matC, macaDataType computeType,
                                         mcsparseSpMMAlg_t alg, size_t* bufferSize);
mcsparseStatus_t mcsparseSpMM_preprocess(mcsparseHandle_t handle, mcsparseOperation_t opA, mcsparseOperation_t opB,
                                         const void* alpha, mcsparseSpMatDescr_t matA, mcsparseDnMatDescr_t matB,
                                         const void* beta, mcsparseDnMatDescr_t matC, macaDataType computeType,
                                         mcsparseSpMMAlg_t alg, void* externalBuffer);
mcsparseStatus_t mcsparseSpMM(mcsparseHandle_t handle, mcsparseOperation_t opA, mcsparseOperation_t opB,
                              const void* alpha, mcsparseSpMatDescr_t matA, mcsparseDnMatDescr_t matB,
                              const void* beta, mcsparseDnMatDescr_t matC, macaDataType computeType,
                              mcsparseSpMMAlg_t alg, void* externalBuffer);

/* ---- legacy typed entry points onto the same kernels ------------------------------- */
/* y = alpha*A*x + beta*y: include/interface/mcsp_level2.h:11-36.  transA is accepted and
 * ignored, exactly as in the reference (src/kernels/level2/spmv/mcsp_spmv_gpu.cpp:946-953 hands it
 * to a template that never reads it), so these always apply A itself.  The index base comes from
 * descrA.  Neither call has a scratch buffer of known size (csrmv has none; CsrmvEx_bufferSize
 * returns the reference's constant 128 and CsrmvEx never touches its buffer, as in the reference,
 * mcsp_spmv_gpu.cpp:905-944,1149-1158), so both run the kernel that gives a group of lanes to each
 * row.  The kernels that need scratch are reached through mcsparseSpMV, whose buffer size is NOT
 * the reference's 128 bytes: see mcsparseSpMV_bufferSize. */
mcsparseStatus_t mcsparseScsrmv(mcsparseHandle_t handle, mcsparseOperation_t transA, int m, int n, int nnz,
                                const float* alpha, const mcsparseMatDescr_t descrA, const float* csrValA,
                                const int* csrRowPtrA, const int* csrColIndA, const float* x, const float* beta,
                                float* y);
mcsparseStatus_t mcsparseDcsrmv(mcsparseHandle_t handle, mcsparseOperation_t transA, int m, int n, int nnz,
                                const double* alpha, const mcsparseMatDescr_t descrA, const double* csrValA,
                                const int* csrRowPtrA, const int* csrColIndA, const double* x, const double* beta,
                                double* y);
mcsparseStatus_t mcsparseCsrmvEx_bufferSize(mcsparseHandle_t handle, mcsparseAlgMode_t alg, mcsparseOperation_t transA,
                                            int m, int n, int nnz, const void* alpha, macaDataType alphatype,
                                            const mcsparseMatDescr_t descrA, const void* csrValA,
                                            macaDataType csrValAtype, const int* csrRowPtrA, const int* csrColIndA,
                                            const void* x, macaDataType xtype, const void* beta, macaDataType betatype,
                                            void* y, macaDataType ytype, macaDataType executiontype,
                                            size_t* bufferSizeInBytes);
mcsparseStatus_t mcsparseCsrmvEx(mcsparseHandle_t handle, mcsparseAlgMode_t alg, mcsparseOperation_t transA, int m,
                                 int n, int nnz, const void* alpha, macaDataType alphatype,
                                 const mcsparseMatDescr_t descrA, const void* csrValA, macaDataType csrValAtype,
                                 const int* csrRowPtrA, const int* csrColIndA, const void* x, macaDataType xtype,
                                 const void* beta, macaDataType betatype, void* y, macaDataType ytype,
                                 macaDataType executiontype, void* buffer);
/* C = alpha*A*op(B) + beta*C with column-major B and C: include/interface/mcsp_level3.h:139-169.
 * A is m x k, C is m x n; B is k x n (transB = N) or n x k (transB = T).  transA must be N
 * (src/kernels/level3/spmm/mcsp_spmm_gpu.cpp:39-42).  csrmm is csrmm2 with transB = N. */
mcsparseStatus_t mcsparseScsrmm2(mcsparseHandle_t handle, mcsparseOperation_t transA, mcsparseOperation_t transB, int m,
                                 int n, int k, int nnz, const float* alpha, const mcsparseMatDescr_t descrA,
                                 const float* csrValA, const int* csrRowPtrA, const int* csrColIndA, const float* B,
                                 int ldb, const float* beta, float* C, int ldc);
mcsparseStatus_t mcsparseDcsrmm2(mcsparseHandle_t handle, mcsparseOperation_t transA, mcsparseOperation_t transB, int m,
                                 int n, int k, int nnz, const double* alpha, const mcsparseMatDescr_t descrA,
                                 const double* csrValA, const int* csrRowPtrA, const int* csrColIndA, const double* B,
                                 int ldb, const double* beta, double* C, int ldc);
mcsparseStatus_t mcsparseScsrmm(mcsparseHandle_t handle, mcsparseOperation_t transA, int m, int n, int k, int nnz,
                                const float* alpha, const mcsparseMatDescr_t descrA, const float* csrValA,
                                const int* csrRowPtrA, const int* csrColIndA, const float* B, int ldb,
                                const float* beta, float* C, int ldc);
mcsparseStatus_t mcsparseDcsrmm(mcsparseHandle_t handle, mcsparseOperation_t transA, int m, int n, int k, int nnz,
                                const double* alpha, const mcsparseMatDescr_t descrA, const double* csrValA,
                                const int* csrRowPtrA, const int* csrColIndA, const double* B, int ldb,
                                const double* beta, double* C, int ldc);

/* ---- index conversions: include/interface/mcsp_conversion.h:11-28 ------------------ */
/* coo_rows must be sorted; csr_rows receives m+1 offsets.                       :11 */
mcsparseStatus_t mcsparseXcoo2csr(mcsparseHandle_t handle, const int* coo_rows, int nnz, int m, int* csr_rows,
                                  mcsparseIndexBase_t idx_base);
/* coo_rows[j] = row of nonzero j (+ idx_base).                                  :15 */
mcsparseStatus_t mcsparseXcsr2coo(mcsparseHandle_t handle, const int* csr_rows, int nnz, int m, int* coo_rows,
                                  mcsparseIndexBase_t idx_base);
/* Note the output order: csc_val, csc_cols (= n+1 column offsets), csc_rows (= nnz row indices).
 * Entries of one column keep their CSR order (a stable sort by column).         :19 */
mcsparseStatus_t mcsparseCsr2cscEx2(mcsparseHandle_t handle, int m, int n, int nnz, const void* csr_val,
                                    const int* csr_rows, const int* csr_cols, void* csc_val, int* csc_cols,
                                    int* csc_rows, macaDataType val_type, mcsparseAction_t csc_action,
                                    mcsparseIndexBase_t idx_base, mcsparseCsr2CscAlg_t alg, void* temp_buffer);
/*                                                                               :24 */
mcsparseStatus_t mcsparseCsr2cscEx2_bufferSize(mcsparseHandle_t handle, int m, int n, int nnz, const void* csr_val,
                                               const int* csr_rows, const int* csr_cols, void* csc_val,
                                               int* csc_cols, int* csc_rows, macaDataType val_type,
                                               mcsparseAction_t csc_action, mcsparseIndexBase_t idx_base,
                                               mcsparseCsr2CscAlg_t alg, size_t* buffer_size);

/* ---- index sorts: include/interface/mcsp_conversion.h:65-107 ------------------------ *
 * All sorts are stable and in place.  perm may be NULL; otherwise it holds nnz entries that
 * move with their nonzeros, so after `mcsparseCreateIdentityPermutation` followed by a sort
 * perm[i] is the old position of the entry now at i, and `mcsparse{S,D}gthr` through it puts
 * the values in the new order.  The scratch size depends on nnz only. */
/* Sorts the column indices inside every row.                                     :66, :69 */
mcsparseStatus_t mcsparseXcsrsort_bufferSizeExt(mcsparseHandle_t handle, int m, int n, int nnz, const int* csr_rows,
                                                const int* csr_cols, size_t* buffer_size);
mcsparseStatus_t mcsparseXcsrsort(mcsparseHandle_t handle, int m, int n, int nnz, mcsparseMatDescr_t mcsp_descr_A,
                                  const int* csr_rows, int* csr_cols, int* perm, void* temp_buffer);
/* Sorts the row indices inside every column.                                     :90, :93 */
mcsparseStatus_t mcsparseXcscsort_bufferSizeExt(mcsparseHandle_t handle, int m, int n, int nnz, const int* csc_cols,
                                                const int* csc_rows, size_t* buffer_size);
mcsparseStatus_t mcsparseXcscsort(mcsparseHandle_t handle, int m, int n, int nnz, mcsparseMatDescr_t mcsp_descr_A,
                                  const int* csc_cols, int* csc_rows, int* perm, void* temp_buffer);
/* Sort COO entries by (row, column) or by (column, row); indices may be zero- or one-based.
 *                                                                           :97, :100, :103 */
mcsparseStatus_t mcsparseXcoosort_bufferSizeExt(mcsparseHandle_t handle, int m, int n, int nnz, const int* coo_rows,
                                                const int* coo_cols, size_t* buffer_size);
mcsparseStatus_t mcsparseXcoosortByRow(mcsparseHandle_t handle, int m, int n, int nnz, int* coo_rows, int* coo_cols,
                                       int* perm, void* temp_buffer);
mcsparseStatus_t mcsparseXcoosortByColumn(mcsparseHandle_t handle, int m, int n, int nnz, int* coo_rows,
                                          int* coo_cols, int* perm, void* temp_buffer);
/* p[i] = i for i < n.                                                            :107 */
mcsparseStatus_t mcsparseCreateIdentityPermutation(mcsparseHandle_t handle, int n, int* p);
/* x_val[i] = y[x_ind[i] - idx_base]: include/interface/mcsp_level1.h:25-29 */
mcsparseStatus_t mcsparseSgthr(mcsparseHandle_t handle, int nnz, const float* y, float* x_val, const int* x_ind,
                               mcsparseIndexBase_t idx_base);
mcsparseStatus_t mcsparseDgthr(mcsparseHandle_t handle, int nnz, const double* y, double* x_val, const int* x_ind,
                               mcsparseIndexBase_t idx_base);

/* ---- EXTENSIONS (no counterpart in the reference) ---------------------------------- */

/* Number of row-length classes: class 0 holds empty rows, class b >= 1 holds rows whose
 * length lies in [2^(b-1), 2^b). */
#define MCSPARSE_ROW_BIN_COUNT 33

/* Row-length binning that steers the SpMV kernel choice.  All arrays are device memory.
 *   row_bins  : m bytes, class of every row (may be NULL)
 *   bin_hist  : MCSPARSE_ROW_BIN_COUNT uint32 counters + 1 trailing uint32 = longest row
 *               (34 uint32 in all; must not be NULL)
 * The result is a pure function of csr_rows, so it can be checked bit for bit on the host. */
mcsparseStatus_t mcsparseXcsrRowBins(mcsparseHandle_t handle, int m, const int* csr_rows,
                                     mcsparseIndexBase_t idx_base, uint8_t* row_bins, uint32_t* bin_hist);

/* The kernel choice mcsparseSpMV derives from such a histogram (host arrays, no GPU work): family and
 * lanes_per_row as mcsparseSpMatGetSpMVPlan reports them.  m rows, nnz nonzeros, x_bytes = bytes of
 * the dense vector.  The dispatch is per matrix: the bins say how well rows of this spread fill the
 * lanes of the sub-wavefront kernel, and the merge-path kernel takes over when they fill under half. */
mcsparseStatus_t mcsparseXcsrRowBinsPlan(const uint32_t* bin_hist, int64_t m, int64_t nnz, int64_t x_bytes, int* family,
                                         int* lanes_per_row);

/* Which SpMV kernel family a CSR op-N call on this descriptor runs:
 * 0 = not analysed yet, 1 = sub-wavefront vector kernel, 2 = merge-path kernel.
 * lanes_per_row is the sub-wavefront width for family 1; for family 2 it is 1 when the tiles of
 * the merge path run in the order of their first column (chosen for matrices with rows longer
 * than a tile and an x too large for an L2) and 0 when they run in storage order. */
mcsparseStatus_t mcsparseSpMatGetSpMVPlan(mcsparseSpMatDescr_t spMatDescr, int* family, int* lanes_per_row);

/* Forces the SpMV kernel family for a descriptor (0 = automatic).  For tests and benchmarks. */
mcsparseStatus_t mcsparseSpMatSetSpMVPlan(mcsparseSpMatDescr_t spMatDescr, int family, int lanes_per_row);

/* What mcsparseSpMM_preprocess left on a CSR descriptor:
 * state 0 = no schedule, 1 = built but the rows share too few columns for it to pay off
 * (SpMM ignores it); 2, 3, 4 = SpMM uses it when called with the same buffer and CSR arrays:
 * 2 = merged column lists of groups of four rows, 3 = diagonal blocks over groups of eight consecutive rows,
 * 4 = diagonal blocks over groups of four strips of four rows a fixed distance (a grid line) apart.
 * merged_entries = total length of the merged column lists of all row groups (compare with nnz), or the
 * number of blocks. */
mcsparseStatus_t mcsparseSpMatGetSpMMSchedule(mcsparseSpMatDescr_t spMatDescr, int* state, int64_t* merged_entries);

/* Optional preparation of y = alpha*op(A)*x + beta*y for a matrix that is multiplied many times (the
 * reference has no such step: include/interface/mcsp_generic.h:43-51).  It copies A into externalBuffer
 * in a column-banded layout in which the reads of x hit in cache; mcsparseSpMV then uses that copy
 * whenever it is called with the same externalBuffer, the same three arrays and extents and the same opA.
 *   - externalBuffer needs mcsparseSpMV_preprocess_bufferSize bytes (about three times the matrix), is
 *     passed to both calls, and must be left alone in between, like the structure of A.  It also holds
 *     the partial sums of the call in flight: two mcsparseSpMV calls that use the same copy must not
 *     overlap in time (one stream, or an event between them).
 *   - The copy includes the values.  After changing values in place call mcsparseSpMV_preprocess
 *     again; mcsparseSpMatSetValues and mcsparseCsrSetPointers drop the copy.
 *   - A copy serves the direction it was prepared for (the opA of the preprocess call).  For the
 *     transposing directions (CSR with op T, CSC with op N) the copy is of the transpose, so that such
 *     calls stop sorting the nonzeros by column on every call; externalBuffer then also needs room
 *     for the conversion (about five times the matrix in all).
 *   - CSR, CSC and COO descriptors with 32- or 64-bit indices can be prepared (64-bit indices are
 *     narrowed and COO row indices turned into offsets once, inside externalBuffer).  Calls the layout
 *     cannot help (x fits in cache as it is, a matrix too small to fill the GPU) are left to the
 *     ordinary kernels; the call still returns SUCCESS.  mcsparseSpMatGetSpMVPreprocess tells which
 *     case applies.
 *   - For a direction that does not transpose (CSR and COO with op N, CSC with op T) the call ends with a
 *     trial: the product is run from the caller's arrays and from the copy, one to three times each, on the
 *     handle's stream, and the copy is kept only if it was the faster by more than a twentieth (a banded
 *     matrix, whose rows read x line by line as it is, or long rows over an x that fits in cache, run
 *     faster from the arrays).  The trial reads vecX, whose memory must be there but whose contents do not
 *     matter, and writes a y of its own inside externalBuffer, never vecY.  mcsparseSetSpMVPreprocessTrial
 *     turns it off; a descriptor whose band width or kernel family the caller has set is not tried either.
 *   - alg chooses between two layouts (the reference ignores alg; the meanings are those APIs of this
 *     family give the values).  MCSPARSE_SPMV_CSR_ALG2, the algorithm that promises the same bits on
 *     every run, builds the banded copy described above: row sums are formed in a fixed order.  Every
 *     other value builds the copy with its tiles in column order: the lanes of a wavefront then read
 *     neighbouring elements of x, and the products are added to the row sums in LDS in the order the
 *     wavefronts reach them.  That is faster by a quarter to a third on the benchmark matrices and stays
 *     within the same error bound, but the last bits can differ between two calls.  Its buffer is larger
 *     (about seven times the matrix: the build sorts the nonzeros by column first); shapes it does not
 *     fit (more than 64 bands of x) get the banded copy.
 *   - mcsparseSpMV called with MCSPARSE_SPMV_CSR_ALG2 never uses a copy in column order: it runs the
 *     ordinary kernels, whose results are reproducible.
 * The call blocks the host until the copy is built. */
mcsparseStatus_t mcsparseSpMV_preprocess_bufferSize(mcsparseHandle_t handle, mcsparseOperation_t opA,
                                                    const void* alpha, mcsparseSpMatDescr_t matA,
                                                    mcsparseDnVecDescr_t vecX, const void* beta,
                                                    mcsparseDnVecDescr_t vecY, macaDataType computeType,
                                                    mcsparseSpMVAlg_t alg, size_t* bufferSize);
mcsparseStatus_t mcsparseSpMV_preprocess(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha,
                                         mcsparseSpMatDescr_t matA, mcsparseDnVecDescr_t vecX, const void* beta,
                                         mcsparseDnVecDescr_t vecY, macaDataType computeType, mcsparseSpMVAlg_t alg,
                                         void* externalBuffer);
/* Whether mcsparseSpMV_preprocess ends with the trial described above (trial != 0, the default) or keeps every
 * copy it can build.  For tests and benchmarks of the copies by themselves. */
mcsparseStatus_t mcsparseSetSpMVPreprocessTrial(mcsparseHandle_t handle, int trial);
mcsparseStatus_t mcsparseGetSpMVPreprocessTrial(const mcsparseHandle_t handle, int* trial);
/* state 0 = not preprocessed, 1 = preprocessed and left to the ordinary kernels, 2 = banded copy in
 * use, 3 = the copy in column order (MCSPARSE_SPMV_CSR_ALG1) in use; bands and rows_per_tile describe
 * the copy (0 unless state is 2 or 3). */
mcsparseStatus_t mcsparseSpMatGetSpMVPreprocess(mcsparseSpMatDescr_t spMatDescr, int* state, int* bands,
                                                int* rows_per_tile);

/* Width, in bytes of x, of the column bands mcsparseSpMV_preprocess cuts (0 = the default: 2 MiB, or, for
 * the copy in column order, all of x where the call finds that a few lines of x take most of the gathers;
 * rounded down to a power of two).  Drops a banded copy already built.  For tests and benchmarks. */
mcsparseStatus_t mcsparseSpMatSetSpMVBandBytes(mcsparseSpMatDescr_t spMatDescr, size_t band_bytes);

/* What the device's memory takes by itself, measured with kernels as plain as this library's can be (16-byte
 * accesses, a contiguous 16 KB per workgroup): mode 0 reads `bytes` of src, mode 1 writes `bytes` of dst, mode 2
 * copies src to dst.  bytes must be a multiple of 16 and both arrays 16-byte aligned; mode 0 needs `sink`, device
 * memory of sink_words >= 1 uint32 (a word of it is written only if a thread's data adds up to one particular
 * value, which keeps the loads from being optimised away).  A yardstick for benchmarks: the rates the kernels of
 * the path are held against besides the published 8 TB/s. */
mcsparseStatus_t mcsparseXstreamProbe(mcsparseHandle_t handle, int mode, const void* src, void* dst, size_t bytes,
                                      uint32_t* sink, size_t sink_words);

/* The reference's SpMV adds the products of a row in a fixed order, so two runs of a call give the same bits
 * whatever `alg` is.  In this library only MCSPARSE_SPMV_CSR_ALG2 promises that: the other values take the faster
 * paths that add products in LDS in the order the wavefronts reach them (a transposing call without preprocess,
 * every call after mcsparseSpMV_preprocess), within the same error bound but not bit for bit the same between runs.
 * deterministic != 0 makes every mcsparseSpMV, mcsparseSpMV_preprocess(_bufferSize) and mcsparseSpMV_staticBuffer
 * call of the handle run as MCSPARSE_SPMV_CSR_ALG2, for callers that compare runs and cannot change the `alg` they
 * pass.  Off by default. */
mcsparseStatus_t mcsparseSetSpMVDeterministic(mcsparseHandle_t handle, int deterministic);
mcsparseStatus_t mcsparseGetSpMVDeterministic(const mcsparseHandle_t handle, int* deterministic);

/* How many XCDs (dies with an L2 of their own, which take the workgroups of a launch in turn) the library
 * assumes behind a device that shows `computeUnits` compute units: computeUnits / 32 where that is a whole
 * number up to 8 (256 -> 8, 128 -> 4, 64 -> 2, 32 -> 1), else 1, in which case the orders that keep
 * neighbouring work in one L2 turn into the plain order.  A pure host function; the library asks the device for
 * its compute units at the first launch that needs them.  For tests. */
mcsparseStatus_t mcsparseXtopologyOfCuCount(int computeUnits, int* xcds);

/* mcsparseSpMV without an externalBuffer, for callers that cannot allocate device memory: code
 * under HIP graph capture, serving loops and harnesses that forbid hipMalloc.  No counterpart in
 * the reference.  The scratch lives in a device array of MCSPARSE_SPMV_STATIC_BUFFER_BYTES inside
 * the library (one copy per GPU the library runs on, held until the process ends); a call whose
 * scratch need (what mcsparseSpMV_bufferSize reports) exceeds it returns
 * MCSPARSE_STATUS_INSUFFICIENT_RESOURCES and launches nothing.  The call allocates nothing and
 * copies nothing to the host: it needs MCSPARSE_POINTER_MODE_HOST (NOT_SUPPORTED otherwise), and a
 * structure that has no SpMV plan yet runs the merge-path family instead of being analysed.
 * Results are those of mcsparseSpMV with the same kernel family.  All calls on one GPU share the
 * array: calls that overlap in time on one GPU (different streams or threads) race.  The first call
 * on a GPU looks the array's address up, which a stream under graph capture cannot hold: that call
 * must come before the capture (under capture it returns NOT_SUPPORTED and enqueues nothing). */
#define MCSPARSE_SPMV_STATIC_BUFFER_BYTES (4u << 20)
mcsparseStatus_t mcsparseSpMV_staticBuffer(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha,
                                           mcsparseSpMatDescr_t matA, mcsparseDnVecDescr_t vecX, const void* beta,
                                           mcsparseDnVecDescr_t vecY, macaDataType computeType,
                                           mcsparseSpMVAlg_t alg);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif

#ifdef __cplusplus
}
#endif

#endif /* MCSPARSE_H__ */
