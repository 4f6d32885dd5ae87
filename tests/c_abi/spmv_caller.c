/* A caller written against mcSparse's C API, compiled as C99 against include/mcsparse.h and linked
 * with libmcsparse.so.  It walks the descriptor life cycle and the argument checks of the SpMV /
 * SpMM / conversion entry points, all of which return before anything is launched, so it runs
 * without a GPU.  Prints "ok" and exits 0 when every status is the expected one. */
#include <stdio.h>
#include <stdint.h>

#include "mcsparse.h"

#define EXPECT(call, want)                                                                    \
    do {                                                                                      \
        mcsparseStatus_t got_ = (call);                                                       \
        if (got_ != (want)) {                                                                 \
            printf("%s:%d: %s returned %s, expected %s\n", __FILE__, __LINE__, #call,         \
                   mcsparseGetErrorName(got_), mcsparseGetErrorName(want));                   \
            return 1;                                                                         \
        }                                                                                     \
    } while (0)

int main(void) {
    /* device pointers are never dereferenced on these paths: any non-null address will do */
    void* fake = (void*)(uintptr_t)0x1000;
    const int64_t m = 5, n = 7, nnz = 11;
    double alpha = 1.5, beta = 0.5;
    size_t bytes = 0;
    int version = 0;

    mcsparseHandle_t h = NULL;
    EXPECT(mcsparseCreate(&h), MCSPARSE_STATUS_SUCCESS);
    EXPECT(mcsparseGetVersion(h, &version), MCSPARSE_STATUS_SUCCESS);
    EXPECT(mcsparseSetPointerMode(h, MCSPARSE_POINTER_MODE_HOST), MCSPARSE_STATUS_SUCCESS);

    mcsparseSpMatDescr_t A = NULL;
    mcsparseDnVecDescr_t X = NULL, Y = NULL;
    EXPECT(mcsparseCreateCsr(&A, m, n, nnz, fake, fake, fake, MCSPARSE_INDEX_32I, MCSPARSE_INDEX_32I,
                             MCSPARSE_INDEX_BASE_ZERO, MACA_R_64F),
           MCSPARSE_STATUS_SUCCESS);
    EXPECT(mcsparseCreateDnVec(&X, n, fake, MACA_R_64F), MCSPARSE_STATUS_SUCCESS);
    EXPECT(mcsparseCreateDnVec(&Y, m, fake, MACA_R_64F), MCSPARSE_STATUS_SUCCESS);

    EXPECT(mcsparseSpMV_bufferSize(h, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, A, X, &beta, Y, MACA_R_64F,
                                   MCSPARSE_SPMV_ALG_DEFAULT, &bytes),
           MCSPARSE_STATUS_SUCCESS);
    if (bytes < 128 || bytes % 128 != 0) {
        printf("unexpected SpMV buffer size %zu\n", bytes);
        return 1;
    }
    /* the argument checks of mcsparseSpMV, in the reference's order */
    EXPECT(mcsparseSpMV(NULL, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, A, X, &beta, Y, MACA_R_64F,
                        MCSPARSE_SPMV_ALG_DEFAULT, fake),
           MCSPARSE_STATUS_NOT_INITIALIZED);
    EXPECT(mcsparseSpMV(h, MCSPARSE_OPERATION_NON_TRANSPOSE, NULL, A, X, &beta, Y, MACA_R_64F,
                        MCSPARSE_SPMV_ALG_DEFAULT, fake),
           MCSPARSE_STATUS_INVALID_VALUE);
    EXPECT(mcsparseSpMV(h, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, A, X, &beta, Y, MACA_R_64F,
                        MCSPARSE_SPMV_ALG_DEFAULT, NULL),
           MCSPARSE_STATUS_INVALID_VALUE);
    /* x and y swapped: sizes do not fit op N */
    EXPECT(mcsparseSpMV(h, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, A, Y, &beta, X, MACA_R_64F,
                        MCSPARSE_SPMV_ALG_DEFAULT, fake),
           MCSPARSE_STATUS_INVALID_VALUE);
    EXPECT(mcsparseSpMV(h, MCSPARSE_OPERATION_CONJUGATE_TRANSPOSE, &alpha, A, Y, &beta, X, MACA_R_64F,
                        MCSPARSE_SPMV_ALG_DEFAULT, fake),
           MCSPARSE_STATUS_INVALID_VALUE);
    /* compute type differs from the value types: outside the path */
    EXPECT(mcsparseSpMV(h, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, A, X, &beta, Y, MACA_R_32F,
                        MCSPARSE_SPMV_ALG_DEFAULT, fake),
           MCSPARSE_STATUS_NOT_SUPPORTED);
    /* NULL arrays are handed back, not launched on */
    EXPECT(mcsparseCsrSetPointers(A, fake, NULL, fake), MCSPARSE_STATUS_SUCCESS);
    EXPECT(mcsparseSpMV(h, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, A, X, &beta, Y, MACA_R_64F,
                        MCSPARSE_SPMV_ALG_DEFAULT, fake),
           MCSPARSE_STATUS_INVALID_VALUE);
    EXPECT(mcsparseCsrSetPointers(A, fake, fake, fake), MCSPARSE_STATUS_SUCCESS);

    /* the preparation step (an extension): sizes depend on the algorithm, arguments are checked like SpMV's */
    {
        const int64_t big = 1 << 20;
        size_t plain = 0, banded = 0, by_column = 0;
        int state = -1, bands = -1, rows_per_tile = -1;
        mcsparseSpMatDescr_t W = NULL;
        mcsparseDnVecDescr_t WX = NULL, WY = NULL;
        EXPECT(mcsparseCreateCsr(&W, big, big, 16 * big, fake, fake, fake, MCSPARSE_INDEX_32I, MCSPARSE_INDEX_32I,
                                 MCSPARSE_INDEX_BASE_ZERO, MACA_R_64F),
               MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseCreateDnVec(&WX, big, fake, MACA_R_64F), MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseCreateDnVec(&WY, big, fake, MACA_R_64F), MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseSpMV_bufferSize(h, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, W, WX, &beta, WY, MACA_R_64F,
                                       MCSPARSE_SPMV_ALG_DEFAULT, &plain),
               MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseSpMV_preprocess_bufferSize(h, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, W, WX, &beta, WY,
                                                  MACA_R_64F, MCSPARSE_SPMV_CSR_ALG2, &banded),
               MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseSpMV_preprocess_bufferSize(h, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, W, WX, &beta, WY,
                                                  MACA_R_64F, MCSPARSE_SPMV_ALG_DEFAULT, &by_column),
               MCSPARSE_STATUS_SUCCESS);
        if (!(plain < banded && banded < by_column)) {
            printf("unexpected preprocess buffer sizes %zu %zu %zu\n", plain, banded, by_column);
            return 1;
        }
        EXPECT(mcsparseSpMV_preprocess(h, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, W, WX, &beta, WY, MACA_R_64F,
                                       MCSPARSE_SPMV_ALG_DEFAULT, NULL),
               MCSPARSE_STATUS_INVALID_VALUE);
        EXPECT(mcsparseSpMV_preprocess(NULL, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, W, WX, &beta, WY, MACA_R_64F,
                                       MCSPARSE_SPMV_ALG_DEFAULT, fake),
               MCSPARSE_STATUS_NOT_INITIALIZED);
        EXPECT(mcsparseSpMatGetSpMVPreprocess(W, &state, &bands, &rows_per_tile), MCSPARSE_STATUS_SUCCESS);
        if (state != 0 || bands != 0 || rows_per_tile != 0) {
            printf("a descriptor that was never prepared reports state %d\n", state);
            return 1;
        }
        EXPECT(mcsparseSpMatSetSpMVBandBytes(W, 8), MCSPARSE_STATUS_INVALID_VALUE);
        EXPECT(mcsparseSpMatSetSpMVBandBytes(W, 1 << 20), MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseSpMV_staticBuffer(h, MCSPARSE_OPERATION_NON_TRANSPOSE, NULL, W, WX, &beta, WY, MACA_R_64F,
                                         MCSPARSE_SPMV_ALG_DEFAULT),
               MCSPARSE_STATUS_INVALID_VALUE);
        EXPECT(mcsparseDestroyDnVec(WX), MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseDestroyDnVec(WY), MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseDestroySpMat(W), MCSPARSE_STATUS_SUCCESS);
    }

    /* SpMM: op(A) = T is not supported for CSR; shapes are checked */
    {
        mcsparseDnMatDescr_t B = NULL, C = NULL;
        EXPECT(mcsparseCreateDnMat(&B, n, 4, 4, fake, MACA_R_64F, MCSPARSE_ORDER_ROW), MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseCreateDnMat(&C, m, 4, 4, fake, MACA_R_64F, MCSPARSE_ORDER_ROW), MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseSpMM_bufferSize(h, MCSPARSE_OPERATION_NON_TRANSPOSE, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha,
                                       A, B, &beta, C, MACA_R_64F, MCSPARSE_SPMM_ALG_DEFAULT, &bytes),
               MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseSpMM(h, MCSPARSE_OPERATION_TRANSPOSE, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, A, B, &beta, C,
                            MACA_R_64F, MCSPARSE_SPMM_ALG_DEFAULT, fake),
               MCSPARSE_STATUS_NOT_SUPPORTED);
        EXPECT(mcsparseSpMM(h, MCSPARSE_OPERATION_NON_TRANSPOSE, MCSPARSE_OPERATION_NON_TRANSPOSE, &alpha, A, C, &beta,
                            B, MACA_R_64F, MCSPARSE_SPMM_ALG_DEFAULT, fake),
               MCSPARSE_STATUS_INVALID_VALUE);
        EXPECT(mcsparseDestroyDnMat(B), MCSPARSE_STATUS_SUCCESS);
        EXPECT(mcsparseDestroyDnMat(C), MCSPARSE_STATUS_SUCCESS);
    }

    /* conversions: sizes first, then pointers; nnz == 0 is a success that touches nothing */
    EXPECT(mcsparseCsr2cscEx2_bufferSize(h, 5, 7, 11, fake, fake, fake, fake, fake, fake, MACA_R_32F,
                                         MCSPARSE_ACTION_NUMERIC, MCSPARSE_INDEX_BASE_ZERO, MCSPARSE_CSR2CSC_ALG1,
                                         &bytes),
           MCSPARSE_STATUS_SUCCESS);
    EXPECT(mcsparseCsr2cscEx2(h, 5, 7, 11, fake, fake, fake, fake, fake, fake, MACA_R_32F, MCSPARSE_ACTION_NUMERIC,
                              MCSPARSE_INDEX_BASE_ZERO, MCSPARSE_CSR2CSC_ALG1, NULL),
           MCSPARSE_STATUS_INVALID_VALUE);
    EXPECT(mcsparseXcsr2coo(h, NULL, 0, 5, NULL, MCSPARSE_INDEX_BASE_ZERO), MCSPARSE_STATUS_SUCCESS);
    EXPECT(mcsparseXcoo2csr(h, NULL, 3, 5, NULL, MCSPARSE_INDEX_BASE_ZERO), MCSPARSE_STATUS_INVALID_VALUE);

    EXPECT(mcsparseDestroyDnVec(X), MCSPARSE_STATUS_SUCCESS);
    EXPECT(mcsparseDestroyDnVec(Y), MCSPARSE_STATUS_SUCCESS);
    EXPECT(mcsparseDestroySpMat(A), MCSPARSE_STATUS_SUCCESS);
    EXPECT(mcsparseDestroy(h), MCSPARSE_STATUS_SUCCESS);
    printf("ok\n");
    return 0;
}
