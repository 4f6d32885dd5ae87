// Handle, status strings and descriptor objects of the C ABI.  Pure host code: nothing in
// this file touches a device, so every entry point here also works on a host without a GPU.
#include <new>

#include "internal.h"

// reference: src/wrapper/mcsp_interface_wrapper.cpp:5-42
mcsparseStatus_t to_public_status(mcspStatus_t s) {
    switch (s) {
        case MCSP_STATUS_SUCCESS: return MCSPARSE_STATUS_SUCCESS;
        case MCSP_STATUS_INVALID_HANDLE: return MCSPARSE_STATUS_NOT_INITIALIZED;
        case MCSP_STATUS_NOT_IMPLEMENTED: return MCSPARSE_STATUS_NOT_SUPPORTED;
        case MCSP_STATUS_INVALID_POINTER: return MCSPARSE_STATUS_INVALID_VALUE;
        case MCSP_STATUS_INVALID_SIZE: return MCSPARSE_STATUS_INVALID_VALUE;
        case MCSP_STATUS_MEMORY_ERROR: return MCSPARSE_STATUS_ALLOC_FAILED;
        case MCSP_STATUS_INTERNAL_ERROR: return MCSPARSE_STATUS_INTERNAL_ERROR;
        case MCSP_STATUS_INVALID_VALUE: return MCSPARSE_STATUS_INVALID_VALUE;
        case MCSP_STATUS_ARCH_MISMATCH: return MCSPARSE_STATUS_ARCH_MISMATCH;
        case MCSP_STATUS_ZERO_PIVOT: return MCSPARSE_STATUS_ZERO_PIVOT;
        case MCSP_STATUS_NOT_INITIALIZED: return MCSPARSE_STATUS_NOT_INITIALIZED;
        case MCSP_STATUS_TYPE_MISMATCH: return MCSPARSE_STATUS_INVALID_VALUE;
        case MCSP_STATUS_MAPPING_ERROR: return MCSPARSE_STATUS_MAPPING_ERROR;
        case MCSP_STATUS_EXECUTION_FAILED: return MCSPARSE_STATUS_EXECUTION_FAILED;
        case MCSP_STATUS_MATRIX_TYPE_NOT_SUPPORTED: return MCSPARSE_STATUS_MATRIX_TYPE_NOT_SUPPORTED;
        case MCSP_STATUS_INSUFFICIENT_RESOURCES: return MCSPARSE_STATUS_INSUFFICIENT_RESOURCES;
    }
    return MCSPARSE_STATUS_INTERNAL_ERROR;
}

namespace {

// reference: src/common/mcsp_helper.cpp:7-9
constexpr int kVerMajor = 1, kVerMinor = 0, kVerPatch = 0;

struct StatusText {
    mcsparseStatus_t code;
    const char* name;
    const char* text;
};
// reference: src/wrapper/mcsp_interface_wrapper.cpp:48-108
const StatusText kStatusText[] = {
    {MCSPARSE_STATUS_SUCCESS, "MCSPARSE_STATUS_SUCCESS", "success"},
    {MCSPARSE_STATUS_NOT_INITIALIZED, "MCSPARSE_STATUS_NOT_INITIALIZED", "initialization error"},
    {MCSPARSE_STATUS_ALLOC_FAILED, "MCSPARSE_STATUS_ALLOC_FAILED", "out of memory"},
    {MCSPARSE_STATUS_INVALID_VALUE, "MCSPARSE_STATUS_INVALID_VALUE", "invalid value"},
    {MCSPARSE_STATUS_ARCH_MISMATCH, "MCSPARSE_STATUS_ARCH_MISMATCH", "architecture mismatch"},
    {MCSPARSE_STATUS_MAPPING_ERROR, "MCSPARSE_STATUS_MAPPING_ERROR", "texture memory mapping error"},
    {MCSPARSE_STATUS_EXECUTION_FAILED, "MCSPARSE_STATUS_EXECUTION_FAILED", "kernel launch failure"},
    {MCSPARSE_STATUS_INTERNAL_ERROR, "MCSPARSE_STATUS_INTERNAL_ERROR", "internal error"},
    {MCSPARSE_STATUS_MATRIX_TYPE_NOT_SUPPORTED, "MCSPARSE_STATUS_MATRIX_TYPE_NOT_SUPPORTED",
     "matrix type not supported"},
    {MCSPARSE_STATUS_ZERO_PIVOT, "MCSPARSE_STATUS_ZERO_PIVOT", "zero pivot"},
    {MCSPARSE_STATUS_NOT_SUPPORTED, "MCSPARSE_STATUS_NOT_SUPPORTED", "operation not supported"},
    {MCSPARSE_STATUS_INSUFFICIENT_RESOURCES, "MCSPARSE_STATUS_INSUFFICIENT_RESOURCES", "insufficient resources"},
};
const char* const kUnknownStatus = "unrecognized error code";

// Value types a dense vector may carry (src/common/mcsp_helper.cpp:335-339).
bool dnvec_type_ok(macaDataType t) {
    switch (t) {
        case MACA_R_32F: case MACA_R_64F: case MACA_C_32F: case MACA_C_64F: case MACA_R_16F:
        case MACA_R_16BF: case MACA_C_16F: case MACA_C_16BF: case MACA_R_8I: case MACA_R_32I:
            return true;
        default:
            return false;
    }
}

// Value types a sparse matrix may carry (src/common/mcsp_helper.cpp:397-404): as above minus R_32I.
bool spmat_type_ok(macaDataType t) { return t != MACA_R_32I && dnvec_type_ok(t); }

mcspStatus_t create_spmat(mcsparseSpMatDescr_t* out, int64_t row_num, int64_t col_num, int64_t nnz, void* rows,
                          void* cols, void* vals, mcsparseIndexType_t row_t, mcsparseIndexType_t col_t,
                          mcsparseIndexBase_t base, macaDataType vt, mcsparseFormat_t format) {
    // check order of src/common/mcsp_helper.cpp:392-409: sizes, then type, then the out pointer
    if (row_num < 0 || col_num < 0 || nnz < 0) return MCSP_STATUS_INVALID_SIZE;
    if (!spmat_type_ok(vt)) return MCSP_STATUS_NOT_IMPLEMENTED;
    if (out == nullptr) return MCSP_STATUS_INVALID_POINTER;
    // the reference creates the descriptor and then rejects a bad base (:427-430, :204-206),
    // leaking it; here the base is checked before anything is allocated
    if (base != MCSPARSE_INDEX_BASE_ZERO && base != MCSPARSE_INDEX_BASE_ONE) return MCSP_STATUS_INVALID_VALUE;
    mcsparseSpMatDescr* d = new (std::nothrow) mcsparseSpMatDescr();
    if (d == nullptr) return MCSP_STATUS_INTERNAL_ERROR;
    d->format = format;
    d->row_num = row_num;
    d->col_num = col_num;
    d->nnz = nnz;
    d->rows = rows;
    d->cols = cols;
    d->vals = vals;
    d->rowIdxType = row_t;
    d->colIdxType = col_t;
    d->idxBase = base;
    d->valueType = vt;
    *out = d;
    return MCSP_STATUS_SUCCESS;
}

}  // namespace

extern "C" {

// ---- handle: src/common/mcsp_helper.cpp:69-88, :154-198, :294-322 ----------------------

mcsparseStatus_t mcsparseCreate(mcsparseHandle_t* handle) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *handle = new (std::nothrow) mcsparseContext();
    if (*handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDestroy(mcsparseHandle_t handle) {
    delete handle;  // NULL is accepted (:82-85)
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseGetVersion(mcsparseHandle_t handle, int* version) {
    if (version == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);  // pointer first (:295-301)
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    *version = kVerMajor * 1000000 + kVerMinor * 1000 + kVerPatch;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseGetProperty(libraryPropertyType type, int* value) {
    if (value == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    switch (type) {
        case MAJOR_VERSION: *value = kVerMajor; break;
        case MINOR_VERSION: *value = kVerMinor; break;
        case PATCH_LEVEL: *value = kVerPatch; break;
        default: return to_public_status(MCSP_STATUS_TYPE_MISMATCH);
    }
    return MCSPARSE_STATUS_SUCCESS;
}

const char* mcsparseGetErrorName(mcsparseStatus_t status) {
    for (const StatusText& s : kStatusText)
        if (s.code == status) return s.name;
    return kUnknownStatus;
}

const char* mcsparseGetErrorString(mcsparseStatus_t status) {
    for (const StatusText& s : kStatusText)
        if (s.code == status) return s.text;
    return kUnknownStatus;
}

mcsparseStatus_t mcsparseSetStream(mcsparseHandle_t handle, hipStream_t sid) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    handle->stream = sid;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseGetStream(const mcsparseHandle_t handle, hipStream_t* sid) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (sid == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *sid = handle->stream;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSetPointerMode(mcsparseHandle_t handle, mcsparsePointerMode_t m) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    handle->ptr_mode = m;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseGetPointerMode(const mcsparseHandle_t handle, mcsparsePointerMode_t* m) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (m == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *m = handle->ptr_mode;
    return MCSPARSE_STATUS_SUCCESS;
}

// EXTENSION.  The reference's SpMV adds every row in a fixed order (csr_vector_device.hpp:40-75), so two runs give
// the same bits whatever `alg` says.  Here only MCSPARSE_SPMV_CSR_ALG2 promises that; with this switch on, every
// mcsparseSpMV / mcsparseSpMV_preprocess / mcsparseSpMV_staticBuffer call of the handle runs as that algorithm.
mcsparseStatus_t mcsparseSetSpMVDeterministic(mcsparseHandle_t handle, int deterministic) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    handle->spmv_deterministic = deterministic != 0;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseGetSpMVDeterministic(const mcsparseHandle_t handle, int* deterministic) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (deterministic == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *deterministic = handle->spmv_deterministic ? 1 : 0;
    return MCSPARSE_STATUS_SUCCESS;
}

// EXTENSION.  Whether mcsparseSpMV_preprocess, having built its copy for a direction that does not transpose, runs
// the call both ways and keeps the copy only where it is the faster one (the default), or keeps every copy it
// can build.
mcsparseStatus_t mcsparseSetSpMVPreprocessTrial(mcsparseHandle_t handle, int trial) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    handle->spmv_preprocess_trial = trial != 0;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseGetSpMVPreprocessTrial(const mcsparseHandle_t handle, int* trial) {
    if (handle == nullptr) return to_public_status(MCSP_STATUS_INVALID_HANDLE);
    if (trial == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *trial = handle->spmv_preprocess_trial ? 1 : 0;
    return MCSPARSE_STATUS_SUCCESS;
}

// ---- dense vector: src/common/mcsp_helper.cpp:325-387 ------------------------------------

mcsparseStatus_t mcsparseCreateDnVec(mcsparseDnVecDescr_t* dnVecDescr, int64_t size, void* values,
                                     macaDataType valueType) {
    if (size < 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    if (dnVecDescr == nullptr || values == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (!dnvec_type_ok(valueType)) return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);
    mcsparseDnVecDescr* d = new (std::nothrow) mcsparseDnVecDescr();
    if (d == nullptr) return to_public_status(MCSP_STATUS_INTERNAL_ERROR);
    d->valueType = valueType;
    d->size = size;
    d->values = values;
    *dnVecDescr = d;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDestroyDnVec(mcsparseDnVecDescr_t dnVecDescr) {
    delete dnVecDescr;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDnVecGet(mcsparseDnVecDescr_t d, int64_t* size, void** values, macaDataType* valueType) {
    if (d == nullptr || size == nullptr || values == nullptr || valueType == nullptr)
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *size = d->size;
    *values = d->values;
    *valueType = d->valueType;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDnVecGetValues(mcsparseDnVecDescr_t d, void** values) {
    if (d == nullptr || values == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *values = d->values;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDnVecSetValues(mcsparseDnVecDescr_t d, void* values) {
    if (d == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    d->values = values;  // NULL is not rejected (:380-386)
    return MCSPARSE_STATUS_SUCCESS;
}

// ---- sparse matrix: src/common/mcsp_helper.cpp:389-452, :503-524, :587-683 ---------------

mcsparseStatus_t mcsparseCreateCsr(mcsparseSpMatDescr_t* spMatDescr, int64_t rows, int64_t cols, int64_t nnz,
                                   void* csrRowOffsets, void* csrColInd, void* csrValues,
                                   mcsparseIndexType_t csrRowOffsetsType, mcsparseIndexType_t csrColIndType,
                                   mcsparseIndexBase_t idxBase, macaDataType valueType) {
    return to_public_status(create_spmat(spMatDescr, rows, cols, nnz, csrRowOffsets, csrColInd, csrValues,
                                         csrRowOffsetsType, csrColIndType, idxBase, valueType,
                                         MCSPARSE_FORMAT_CSR));
}

mcsparseStatus_t mcsparseCreateCsc(mcsparseSpMatDescr_t* spMatDescr, int64_t rows, int64_t cols, int64_t nnz,
                                   void* cscColOffsets, void* cscRowInd, void* cscValues,
                                   mcsparseIndexType_t cscColOffsetsType, mcsparseIndexType_t cscRowIndType,
                                   mcsparseIndexBase_t idxBase, macaDataType valueType) {
    // rows <- row indices, cols <- column offsets (:447-452)
    return to_public_status(create_spmat(spMatDescr, rows, cols, nnz, cscRowInd, cscColOffsets, cscValues,
                                         cscRowIndType, cscColOffsetsType, idxBase, valueType,
                                         MCSPARSE_FORMAT_CSC));
}

mcsparseStatus_t mcsparseCreateCoo(mcsparseSpMatDescr_t* spMatDescr, int64_t rows, int64_t cols, int64_t nnz,
                                   void* cooRowInd, void* cooColInd, void* cooValues,
                                   mcsparseIndexType_t cooIdxType, mcsparseIndexBase_t idxBase,
                                   macaDataType valueType) {
    return to_public_status(create_spmat(spMatDescr, rows, cols, nnz, cooRowInd, cooColInd, cooValues, cooIdxType,
                                         cooIdxType, idxBase, valueType, MCSPARSE_FORMAT_COO));
}

mcsparseStatus_t mcsparseCooGet(mcsparseSpMatDescr_t d, int64_t* rows, int64_t* cols, int64_t* nnz, void** cooRowInd,
                                void** cooColInd, void** cooValues, mcsparseIndexType_t* idxType,
                                mcsparseIndexBase_t* idxBase, macaDataType* valueType) {
    if (d == nullptr || rows == nullptr || cols == nullptr || nnz == nullptr || cooRowInd == nullptr ||
        cooColInd == nullptr || cooValues == nullptr || idxType == nullptr || idxBase == nullptr ||
        valueType == nullptr)
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *rows = d->row_num;
    *cols = d->col_num;
    *nnz = d->nnz;
    *cooRowInd = d->rows;
    *cooColInd = d->cols;
    *cooValues = d->vals;
    *idxType = d->rowIdxType;
    *idxBase = d->idxBase;
    *valueType = d->valueType;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseCooSetPointers(mcsparseSpMatDescr_t d, void* cooRows, void* cooColumns, void* cooValues) {
    if (d == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    d->rows = cooRows;
    d->cols = cooColumns;
    d->vals = cooValues;
    d->plan.valid = false;
    d->banded.valid = false;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseCsrGet(mcsparseSpMatDescr_t d, int64_t* rows, int64_t* cols, int64_t* nnz,
                                void** csrRowOffsets, void** csrColInd, void** csrValues,
                                mcsparseIndexType_t* csrRowOffsetsType, mcsparseIndexType_t* csrColIndType,
                                mcsparseIndexBase_t* idxBase, macaDataType* valueType) {
    if (d == nullptr || rows == nullptr || cols == nullptr || nnz == nullptr || csrRowOffsets == nullptr ||
        csrColInd == nullptr || csrValues == nullptr || csrRowOffsetsType == nullptr || csrColIndType == nullptr ||
        idxBase == nullptr || valueType == nullptr)
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *rows = d->row_num;
    *cols = d->col_num;
    *nnz = d->nnz;
    *csrRowOffsets = d->rows;
    *csrColInd = d->cols;
    *csrValues = d->vals;
    *csrRowOffsetsType = d->rowIdxType;
    *csrColIndType = d->colIdxType;
    *idxBase = d->idxBase;
    *valueType = d->valueType;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseCsrSetPointers(mcsparseSpMatDescr_t d, void* csrRowOffsets, void* csrColInd,
                                        void* csrValues) {
    if (d == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    d->rows = csrRowOffsets;
    d->cols = csrColInd;
    d->vals = csrValues;
    d->plan.valid = false;  // new structure, new analysis
    d->schedule.valid = false;
    d->banded.valid = false;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseCscSetPointers(mcsparseSpMatDescr_t d, void* cscColOffsets, void* cscRowInd,
                                        void* cscValues) {
    if (d == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    d->rows = cscRowInd;
    d->cols = cscColOffsets;
    d->vals = cscValues;
    d->plan.valid = false;
    d->banded.valid = false;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDestroySpMat(mcsparseSpMatDescr_t d) {
    delete d;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSpMatGetSize(mcsparseSpMatDescr_t d, int64_t* rows, int64_t* cols, int64_t* nnz) {
    if (d == nullptr || rows == nullptr || cols == nullptr || nnz == nullptr)
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *rows = d->row_num;
    *cols = d->col_num;
    *nnz = d->nnz;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSpMatGetFormat(mcsparseSpMatDescr_t d, mcsparseFormat_t* format) {
    if (d == nullptr || format == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *format = d->format;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSpMatGetIndexBase(mcsparseSpMatDescr_t d, mcsparseIndexBase_t* idxBase) {
    if (d == nullptr || idxBase == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *idxBase = d->idxBase;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSpMatGetValues(mcsparseSpMatDescr_t d, void** values) {
    if (d == nullptr || values == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *values = d->vals;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSpMatSetValues(mcsparseSpMatDescr_t d, void* values) {
    if (d == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    d->vals = values;
    d->banded.valid = false;  // the banded copy holds the old values
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSpMatGetSpMVPlan(mcsparseSpMatDescr_t d, int* family, int* lanes_per_row) {
    if (d == nullptr || family == nullptr || lanes_per_row == nullptr)
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *family = d->plan.valid ? d->plan.family : kFamilyAuto;
    *lanes_per_row = d->plan.valid ? d->plan.lanes : 0;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSpMatGetSpMMSchedule(mcsparseSpMatDescr_t d, int* state, int64_t* merged_entries) {
    if (d == nullptr || state == nullptr || merged_entries == nullptr)
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *state = !d->schedule.valid ? 0 : (!d->schedule.useful ? 1 : (d->schedule.blocks ? (d->schedule.stride != 0 ? 4 : 3) : 2));
    *merged_entries = d->schedule.valid ? static_cast<int64_t>(d->schedule.entries) : 0;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSpMatGetSpMVPreprocess(mcsparseSpMatDescr_t d, int* state, int* bands, int* rows_per_tile) {
    if (d == nullptr || state == nullptr || bands == nullptr || rows_per_tile == nullptr)
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *state = !d->banded.valid ? 0 : (!d->banded.useful ? 1 : (d->banded.shape.by_column ? 3 : 2));
    *bands = d->banded.valid && d->banded.useful ? static_cast<int>(d->banded.shape.bands) : 0;
    *rows_per_tile = d->banded.valid && d->banded.useful ? static_cast<int>(d->banded.shape.rows_per_tile) : 0;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSpMatSetSpMVBandBytes(mcsparseSpMatDescr_t d, size_t band_bytes) {
    if (d == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (band_bytes != 0 && (band_bytes < 16 || band_bytes > (size_t(1) << 30)))
        return to_public_status(MCSP_STATUS_INVALID_VALUE);
    d->banded.band_bytes = band_bytes;
    d->banded.valid = false;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseSpMatSetSpMVPlan(mcsparseSpMatDescr_t d, int family, int lanes_per_row) {
    if (d == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (family < kFamilyAuto || family > kFamilyMerge) return to_public_status(MCSP_STATUS_INVALID_VALUE);
    if (lanes_per_row != 0 && (lanes_per_row < 1 || lanes_per_row > 64 || (lanes_per_row & (lanes_per_row - 1))))
        return to_public_status(MCSP_STATUS_INVALID_VALUE);
    d->plan.forced_family = family;
    d->plan.forced_lanes = lanes_per_row;
    d->plan.valid = false;
    return MCSPARSE_STATUS_SUCCESS;
}

// ---- dense matrix: src/common/mcsp_helper.cpp:715-760 -------------------------------------

mcsparseStatus_t mcsparseCreateDnMat(mcsparseDnMatDescr_t* dnMatDescr, int64_t rows, int64_t cols, int64_t ld,
                                     void* values, macaDataType valueType, mcsparseOrder_t order) {
    if (rows < 0 || cols < 0 || ld < 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    if (!dnvec_type_ok(valueType)) return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);
    if (dnMatDescr == nullptr || values == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    mcsparseDnMatDescr* d = new (std::nothrow) mcsparseDnMatDescr();
    if (d == nullptr) return to_public_status(MCSP_STATUS_INTERNAL_ERROR);
    d->valueType = valueType;
    d->order = order;
    d->row_num = rows;
    d->col_num = cols;
    d->ld = ld;
    d->values = values;
    *dnMatDescr = d;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDestroyDnMat(mcsparseDnMatDescr_t dnMatDescr) {
    delete dnMatDescr;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDnMatGet(mcsparseDnMatDescr_t d, int64_t* rows, int64_t* cols, int64_t* ld, void** values,
                                  macaDataType* type, mcsparseOrder_t* order) {
    if (d == nullptr || rows == nullptr || cols == nullptr || ld == nullptr || values == nullptr ||
        type == nullptr || order == nullptr)
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *rows = d->row_num;
    *cols = d->col_num;
    *ld = d->ld;
    *values = d->values;
    *type = d->valueType;
    *order = d->order;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDnMatGetValues(mcsparseDnMatDescr_t d, void** values) {
    if (d == nullptr || values == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *values = d->values;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDnMatSetValues(mcsparseDnMatDescr_t d, void* values) {
    if (d == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    d->values = values;
    return MCSPARSE_STATUS_SUCCESS;
}

// ---- strided batches: src/kernels/generic/mcsp_generic.cpp:686-743, :787-802 -----------------

mcsparseStatus_t mcsparseCooSetStridedBatch(mcsparseSpMatDescr_t d, int batchCount, int64_t batchStride) {
    if (d == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (batchCount <= 0 || batchStride < 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    d->batchCount = batchCount;
    d->batchStride = batchStride;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseCsrSetStridedBatch(mcsparseSpMatDescr_t d, int batchCount, int64_t offsetsBatchStride,
                                            int64_t columnsValuesBatchStride) {
    if (d == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (batchCount <= 0 || offsetsBatchStride < 0 || columnsValuesBatchStride < 0)
        return to_public_status(MCSP_STATUS_INVALID_SIZE);
    d->batchCount = batchCount;
    d->offsetsBatchStride = offsetsBatchStride;
    d->batchStride = columnsValuesBatchStride;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDnMatSetStridedBatch(mcsparseDnMatDescr_t d, int batchCount, int64_t batchStride) {
    if (d == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (batchCount <= 0 || batchStride < 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    d->batchCount = batchCount;
    d->batchStride = batchStride;
    return MCSPARSE_STATUS_SUCCESS;
}

mcsparseStatus_t mcsparseDnMatGetStridedBatch(mcsparseDnMatDescr_t d, int* batchCount, int64_t* batchStride) {
    if (d == nullptr || batchCount == nullptr || batchStride == nullptr)
        return to_public_status(MCSP_STATUS_INVALID_POINTER);
    *batchCount = static_cast<int>(d->batchCount);
    *batchStride = d->batchStride;
    return MCSPARSE_STATUS_SUCCESS;
}

}  // extern "C"
