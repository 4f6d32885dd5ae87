/*
 * CPU oracle for the CSR SpMV / SpMM / csr2csc / csr2coo path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, what the reference computes on
 * this path; the GPU library is checked against it.  Nothing that ships (the mcsparse_amd
 * package, libmcsparse.so) may call, link or load it -- only tests/, the smoke check and the
 * cpu_baseline leg of bench.py do.
 *
 * The reference (MetaX mcSparse) is MACA device code that needs the MetaX compiler and
 * runtime, so it cannot be built or run here; it also ships no tests or golden vectors.  Each
 * function below therefore follows the reference's source (cited per function, paths relative
 * to the reference checkout, mcsparse/...) and is pinned by tests/test_oracle.py against
 * independent checks: scipy.sparse results, dense brute force, closed forms and round trips.
 *
 * Floating point: the reference's result depends on its summation order (64 lane partials,
 * then a halving tree), which is not part of the contract.  The oracle accumulates in
 * long double (x87 80-bit, 64-bit mantissa) and also returns the bound sum_j |a_ij||x_j| that
 * the acceptance test |y - y_ref| <= 8u(...) is stated in.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef uint32_t idx_t;
typedef long double acc_t;

/* ------------------------------------------------------------------------------------------
 * SpMV  y = alpha*op(A)*x + beta*y
 * reference: src/kernels/level2/spmv/csr_vector_device.hpp:22-79 (row sum, then
 * y[row] = beta*y[row] + alpha*sum at :75), op T = the same on the transpose
 * (src/kernels/level2/spmv/mcsp_spmv_gpu.cpp:797-851).
 * y_ref[i]   = beta*y[i] + alpha*sum_j a_ij x_j          (long double)
 * bound[i]   = |alpha| * sum_j |a_ij||x_j| + |beta*y[i]|  (long double)
 * y may be NULL when beta == 0.
 * ------------------------------------------------------------------------------------------ */
#define DEFINE_SPMV(NAME, T)                                                                                      \
    void NAME(int op_t, int64_t m, int64_t n, int base, const idx_t* ptr, const idx_t* col, const T* val,        \
              double alpha, double beta, const T* x, const T* y, acc_t* y_ref, acc_t* bound) {                    \
        const int64_t out_len = op_t ? n : m;                                                                     \
        for (int64_t i = 0; i < out_len; ++i) {                                                                   \
            y_ref[i] = 0;                                                                                         \
            bound[i] = 0;                                                                                         \
        }                                                                                                         \
        for (int64_t r = 0; r < m; ++r) {                                                                         \
            for (idx_t j = ptr[r] - base; j < ptr[r + 1] - base; ++j) {                                           \
                const int64_t c = (int64_t)col[j] - base;                                                         \
                if (!op_t) {                                                                                      \
                    const acc_t p = (acc_t)val[j] * (acc_t)x[c];                                                  \
                    y_ref[r] += p;                                                                                \
                    bound[r] += fabsl(p);                                                                         \
                } else {                                                                                          \
                    const acc_t p = (acc_t)val[j] * (acc_t)x[r];                                                  \
                    y_ref[c] += p;                                                                                \
                    bound[c] += fabsl(p);                                                                         \
                }                                                                                                 \
            }                                                                                                     \
        }                                                                                                         \
        for (int64_t i = 0; i < out_len; ++i) {                                                                   \
            const acc_t by = (beta != 0.0 && y != NULL) ? (acc_t)beta * (acc_t)y[i] : 0;                          \
            y_ref[i] = by + (acc_t)alpha * y_ref[i];                                                              \
            bound[i] = fabsl((acc_t)alpha) * bound[i] + fabsl(by);                                                \
        }                                                                                                         \
    }
DEFINE_SPMV(orc_spmv_f32, float)
DEFINE_SPMV(orc_spmv_f64, double)

/* ------------------------------------------------------------------------------------------
 * SpMM  C = alpha*A*op(B) + beta*C, A m x k CSR, op(B) k x n
 * reference: src/kernels/level3/spmm/csr_spmm_device.hpp:91-167.  There op(B) has already been
 * brought to column-major (mcsp_spmm_gpu.cpp:119-133); here the element (kk, j) of op(B) is
 * addressed directly: b_row_major -> B[kk*ldb + j], else B[j*ldb + kk].  C likewise (:150,:163).
 * ------------------------------------------------------------------------------------------ */
#define DEFINE_SPMM(NAME, T)                                                                                      \
    void NAME(int64_t m, int64_t n, int base, const idx_t* ptr, const idx_t* col, const T* val, double alpha,    \
              double beta, const T* B, int64_t ldb, int b_row_major, const T* C, int64_t ldc, int c_row_major,    \
              acc_t* c_ref, acc_t* bound) {                                                                       \
        /* c_ref and bound are dense m x n, row-major, ld = n */                                                  \
        for (int64_t r = 0; r < m; ++r) {                                                                         \
            for (int64_t j = 0; j < n; ++j) {                                                                     \
                acc_t s = 0, b = 0;                                                                               \
                for (idx_t e = ptr[r] - base; e < ptr[r + 1] - base; ++e) {                                       \
                    const int64_t kk = (int64_t)col[e] - base;                                                    \
                    const T bv = b_row_major ? B[kk * ldb + j] : B[j * ldb + kk];                                 \
                    const acc_t p = (acc_t)val[e] * (acc_t)bv;                                                    \
                    s += p;                                                                                       \
                    b += fabsl(p);                                                                                \
                }                                                                                                 \
                const int64_t off = c_row_major ? r * ldc + j : j * ldc + r;                                      \
                const acc_t bc = (beta != 0.0 && C != NULL) ? (acc_t)beta * (acc_t)C[off] : 0;                    \
                c_ref[r * n + j] = bc + (acc_t)alpha * s;                                                         \
                bound[r * n + j] = fabsl((acc_t)alpha) * b + fabsl(bc);                                           \
            }                                                                                                     \
        }                                                                                                         \
    }
DEFINE_SPMM(orc_spmm_f32, float)
DEFINE_SPMM(orc_spmm_f64, double)

/* ------------------------------------------------------------------------------------------
 * csr2coo: coo_rows[j] = r + base for every j in [ptr[r]-base, ptr[r+1]-base)
 * reference: src/kernels/conversion/coo2csr_device.hpp:26-41
 * ------------------------------------------------------------------------------------------ */
void orc_csr2coo(int64_t m, int base, const idx_t* ptr, idx_t* coo_rows) {
    for (int64_t r = 0; r < m; ++r)
        for (idx_t j = ptr[r] - base; j < ptr[r + 1] - base; ++j) coo_rows[j] = (idx_t)(r + base);
}

/* ------------------------------------------------------------------------------------------
 * coo2csr from sorted row indices.  The reference's thread t (0 <= t <= nnz) writes
 * ptr[i] = t + base for every i from (row of entry t-1) + 1 up to (row of entry t), with 0 and
 * m + 1 at the two ends -- src/kernels/conversion/coo2csr_device.hpp:8-24.  Run over t in order.
 * ------------------------------------------------------------------------------------------ */
void orc_coo2csr(int64_t nnz, int64_t m, int base, const idx_t* coo_rows, idx_t* ptr) {
    for (int64_t t = 0; t <= nnz; ++t) {
        const int64_t first = t == 0 ? 0 : (int64_t)coo_rows[t - 1] - base + 1;
        const int64_t last = t == nnz ? m + 1 : (int64_t)coo_rows[t] - base + 1;
        for (int64_t i = first; i < last; ++i) ptr[i] = (idx_t)(t + base);
    }
}

static uint32_t bit_length_u32(uint32_t v) { /* src/include/mcsp_internal_host_utils.hpp:25-32 */
    uint32_t b = 0;
    while (v) {
        ++b;
        v >>= 1;
    }
    return b;
}

/* ------------------------------------------------------------------------------------------
 * csr2csc, literal restatement of src/kernels/conversion/mcsp_csr2csc.cpp:43-132 (NUMERIC
 * branch; the SYMBOLIC branch sorts the row indices as payload and gives the same indices):
 *   perm = identity                                                       (:91)
 *   stable LSD radix sort of (key = csr_cols, payload = perm), 2 bits per pass over bits
 *   [0, bit_length(n))                     (:84-85, :97-98; device_radix_sort.hpp:283-306)
 *   col_ptr = coo2csr(sorted keys)                                        (:100)
 *   coo_rows = csr2coo(row_ptr)                                           (:101)
 *   row_ind[i] = coo_rows[perm[i]], csc_val[i] = csr_val[perm[i]]         (:108, csr2csc_device.hpp)
 * value_bytes == 0 skips the values.  Returns 0, or -1 if out of memory.
 * Keys keep their index base, as in the reference, so the sort covers bit_length(n) bits.
 * ------------------------------------------------------------------------------------------ */
int orc_csr2csc_radix2(int64_t m, int64_t n, int64_t nnz, int base, const idx_t* ptr, const idx_t* col,
                       const void* val, int64_t value_bytes, idx_t* col_ptr, idx_t* row_ind, void* csc_val) {
    if (m == 0 || n == 0 || nnz == 0) return 0; /* :56-58, outputs untouched */
    idx_t* key_a = (idx_t*)malloc(sizeof(idx_t) * nnz);
    idx_t* key_b = (idx_t*)malloc(sizeof(idx_t) * nnz);
    idx_t* perm_a = (idx_t*)malloc(sizeof(idx_t) * nnz);
    idx_t* perm_b = (idx_t*)malloc(sizeof(idx_t) * nnz);
    idx_t* coo = (idx_t*)malloc(sizeof(idx_t) * nnz);
    if (!key_a || !key_b || !perm_a || !perm_b || !coo) {
        free(key_a); free(key_b); free(perm_a); free(perm_b); free(coo);
        return -1;
    }
    for (int64_t i = 0; i < nnz; ++i) {
        key_a[i] = col[i];
        perm_a[i] = (idx_t)i;
    }
    const uint32_t end_bit = bit_length_u32((uint32_t)n);
    for (uint32_t bit = 0; bit < end_bit; bit += 2) {
        int64_t count[4] = {0, 0, 0, 0}, start[4];
        for (int64_t i = 0; i < nnz; ++i) ++count[(key_a[i] >> bit) & 3u];
        start[0] = 0;
        for (int d = 1; d < 4; ++d) start[d] = start[d - 1] + count[d - 1];
        for (int64_t i = 0; i < nnz; ++i) { /* in input order => stable */
            const int64_t dst = start[(key_a[i] >> bit) & 3u]++;
            key_b[dst] = key_a[i];
            perm_b[dst] = perm_a[i];
        }
        idx_t* t = key_a; key_a = key_b; key_b = t;
        t = perm_a; perm_a = perm_b; perm_b = t;
    }
    orc_coo2csr(nnz, n, base, key_a, col_ptr);
    orc_csr2coo(m, base, ptr, coo);
    for (int64_t i = 0; i < nnz; ++i) {
        row_ind[i] = coo[perm_a[i]];
        if (value_bytes)
            memcpy((char*)csc_val + i * value_bytes, (const char*)val + (int64_t)perm_a[i] * value_bytes,
                   (size_t)value_bytes);
    }
    free(key_a); free(key_b); free(perm_a); free(perm_b); free(coo);
    return 0;
}

/* The same conversion as one stable counting sort by column (what the 2-bit passes add up to):
 * fast enough for 10^8 nonzeros; tests pin it against orc_csr2csc_radix2 on smaller inputs. */
int orc_csr2csc_counting(int64_t m, int64_t n, int64_t nnz, int base, const idx_t* ptr, const idx_t* col,
                         const void* val, int64_t value_bytes, idx_t* col_ptr, idx_t* row_ind, void* csc_val) {
    if (m == 0 || n == 0 || nnz == 0) return 0;
    int64_t* next = (int64_t*)calloc((size_t)n + 1, sizeof(int64_t));
    if (!next) return -1;
    for (int64_t j = 0; j < nnz; ++j) ++next[(int64_t)col[j] - base + 1];
    for (int64_t c = 0; c < n; ++c) next[c + 1] += next[c];
    for (int64_t c = 0; c <= n; ++c) col_ptr[c] = (idx_t)(next[c] + base);
    for (int64_t r = 0; r < m; ++r) {
        for (idx_t j = ptr[r] - base; j < ptr[r + 1] - base; ++j) { /* row-major order => stable */
            const int64_t dst = next[(int64_t)col[j] - base]++;
            row_ind[dst] = (idx_t)(r + base);
            if (value_bytes)
                memcpy((char*)csc_val + dst * value_bytes, (const char*)val + (int64_t)j * value_bytes,
                       (size_t)value_bytes);
        }
    }
    free(next);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Index sorts.  The reference sorts (minor key, permutation) pairs, gathers the major keys
 * through the result, sorts (major key, permutation) pairs and gathers again
 * (src/kernels/conversion/mcsp_coosort.cpp:63-106, mcsp_csrsort.cpp:66-115): two stable sorts,
 * minor key first.  Restated with stable counting sorts.  perm may be NULL.
 * keys are compared as stored (an index base is simply part of the key).
 * ------------------------------------------------------------------------------------------ */
static int stable_counting_pass(int64_t nnz, int64_t extent, const idx_t* key, const int64_t* order_in,
                                int64_t* order_out) {
    int64_t* next = (int64_t*)calloc((size_t)extent + 2, sizeof(int64_t));
    if (!next) return -1;
    for (int64_t j = 0; j < nnz; ++j) ++next[(int64_t)key[j] + 1];
    for (int64_t k = 0; k <= extent; ++k) next[k + 1] += next[k];
    for (int64_t j = 0; j < nnz; ++j) {
        const int64_t src = order_in[j];
        order_out[next[key[src]]++] = src;
    }
    free(next);
    return 0;
}

int orc_coosort(int64_t major_extent, int64_t minor_extent, int64_t nnz, idx_t* major, idx_t* minor, idx_t* perm) {
    if (nnz == 0) return 0;
    int64_t* o0 = (int64_t*)malloc((size_t)nnz * sizeof(int64_t));
    int64_t* o1 = (int64_t*)malloc((size_t)nnz * sizeof(int64_t));
    idx_t* tmp = (idx_t*)malloc((size_t)nnz * sizeof(idx_t));
    if (!o0 || !o1 || !tmp) return -1;
    for (int64_t j = 0; j < nnz; ++j) o0[j] = j;
    if (stable_counting_pass(nnz, minor_extent, minor, o0, o1)) return -1;
    if (stable_counting_pass(nnz, major_extent, major, o1, o0)) return -1;
    idx_t* arrays[3] = {major, minor, perm};
    for (int a = 0; a < 3; ++a) {
        if (!arrays[a]) continue;
        for (int64_t j = 0; j < nnz; ++j) tmp[j] = arrays[a][o0[j]];
        memcpy(arrays[a], tmp, (size_t)nnz * sizeof(idx_t));
    }
    free(o0);
    free(o1);
    free(tmp);
    return 0;
}

/* mcsp_csrsort.cpp:43-121: csr2coo, then the two-key sort; the sorted row indices are dropped. */
int orc_csrsort(int64_t m, int64_t n, int64_t nnz, int base, const idx_t* ptr, idx_t* col, idx_t* perm) {
    if (m == 0 || n == 0 || nnz == 0) return 0;
    idx_t* rows = (idx_t*)malloc((size_t)nnz * sizeof(idx_t));
    if (!rows) return -1;
    orc_csr2coo(m, base, ptr, rows);
    const int rc = orc_coosort(m + base, n + base, nnz, rows, col, perm);
    free(rows);
    return rc;
}

/* ------------------------------------------------------------------------------------------
 * Row-length classes used by the GPU library's SpMV dispatch (no counterpart in the
 * reference): class 0 = empty row, class b >= 1 = length in [2^(b-1), 2^b).
 * hist: 33 class counters followed by the longest row length.
 * ------------------------------------------------------------------------------------------ */
void orc_row_bins(int64_t m, const idx_t* ptr, uint8_t* row_bins, uint32_t* hist) {
    for (int i = 0; i < 34; ++i) hist[i] = 0;
    for (int64_t r = 0; r < m; ++r) {
        const uint32_t len = ptr[r + 1] - ptr[r];
        const uint32_t b = bit_length_u32(len);
        if (row_bins) row_bins[r] = (uint8_t)b;
        ++hist[b];
        if (len > hist[33]) hist[33] = len;
    }
}

/* ------------------------------------------------------------------------------------------
 * CPU baseline: the same SpMV / SpMM semantics in working precision with OpenMP over rows,
 * timed by bench.py on the GPU box's host cores.  Not used for parity.
 * ------------------------------------------------------------------------------------------ */
#define DEFINE_SPMV_OMP(NAME, T)                                                                                  \
    void NAME(int64_t m, int base, const idx_t* ptr, const idx_t* col, const T* val, T alpha, T beta,             \
              const T* x, T* y, int dynamic) {                                                                    \
        if (dynamic) {                                                                                            \
            _Pragma("omp parallel for schedule(dynamic, 1024)") for (int64_t r = 0; r < m; ++r) {                 \
                T s = 0;                                                                                          \
                for (idx_t j = ptr[r] - base; j < ptr[r + 1] - base; ++j) s += val[j] * x[col[j] - base];         \
                y[r] = beta * y[r] + alpha * s;                                                                   \
            }                                                                                                     \
        } else {                                                                                                  \
            _Pragma("omp parallel for schedule(static)") for (int64_t r = 0; r < m; ++r) {                        \
                T s = 0;                                                                                          \
                for (idx_t j = ptr[r] - base; j < ptr[r + 1] - base; ++j) s += val[j] * x[col[j] - base];         \
                y[r] = beta * y[r] + alpha * s;                                                                   \
            }                                                                                                     \
        }                                                                                                         \
    }
DEFINE_SPMV_OMP(orc_spmv_omp_f32, float)
DEFINE_SPMV_OMP(orc_spmv_omp_f64, double)

/* row-major B and C, ld = n */
void orc_spmm_omp_f32(int64_t m, int64_t n, int base, const idx_t* ptr, const idx_t* col, const float* val,
                      float alpha, float beta, const float* B, float* C) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < m; ++r) {
        float* c = C + r * n;
        for (int64_t j = 0; j < n; ++j) c[j] *= beta;
        for (idx_t e = ptr[r] - base; e < ptr[r + 1] - base; ++e) {
            const float a = alpha * val[e];
            const float* b = B + ((int64_t)col[e] - base) * n;
#pragma omp simd
            for (int64_t j = 0; j < n; ++j) c[j] += a * b[j];
        }
    }
}

/* dst <- src in pages of 4 KiB dealt to the OpenMP threads as schedule(static) deals rows: a page
 * of a freshly mapped dst is then first touched, and so placed, next to the thread that will
 * read it in the loops above. */
void orc_first_touch_copy(void* dst, const void* src, int64_t bytes) {
    const int64_t page = 4096;
    const int64_t pages = (bytes + page - 1) / page;
#pragma omp parallel for schedule(static)
    for (int64_t p = 0; p < pages; ++p) {
        const int64_t off = p * page;
        const int64_t len = bytes - off < page ? bytes - off : page;
        memcpy((char*)dst + off, (const char*)src + off, (size_t)len);
    }
}

int orc_max_threads(void) {
#ifdef _OPENMP
    extern int omp_get_max_threads(void);
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* csr2csc for the CPU baseline: the rows are cut into one block per thread (equal numbers of
 * nonzeros), every block counts its columns, the counts become each block's first slot in every
 * column (blocks in row order, so the order inside a column is the input order), then every block
 * places its nonzeros.  Same result as orc_csr2csc_counting; tests pin them equal. */
int orc_csr2csc_omp(int64_t m, int64_t n, int64_t nnz, int base, const idx_t* ptr, const idx_t* col, const void* val,
                    int64_t value_bytes, idx_t* col_ptr, idx_t* row_ind, void* csc_val) {
    if (m == 0 || n == 0 || nnz == 0) return 0;
    const int blocks = orc_max_threads();
    int64_t* first_row = (int64_t*)malloc(((size_t)blocks + 1) * sizeof(int64_t));
    uint32_t* slot = (uint32_t*)malloc((size_t)blocks * (size_t)n * sizeof(uint32_t));
    int64_t* start = (int64_t*)malloc(((size_t)n + 1) * sizeof(int64_t));
    int64_t* part = (int64_t*)calloc((size_t)blocks + 1, sizeof(int64_t));
    if (!first_row || !slot || !start || !part) {
        free(first_row); free(slot); free(start); free(part);
        return -1;
    }
    for (int b = 0; b <= blocks; ++b) { /* first row whose nonzeros start at or after b/blocks of all */
        const int64_t want = nnz * b / blocks;
        int64_t lo = 0, hi = m;
        while (lo < hi) {
            const int64_t mid = (lo + hi) / 2;
            if ((int64_t)ptr[mid] - base < want) lo = mid + 1; else hi = mid;
        }
        first_row[b] = b == blocks ? m : lo;
    }
#pragma omp parallel for schedule(static, 1)
    for (int b = 0; b < blocks; ++b) {
        uint32_t* mine = slot + (size_t)b * (size_t)n;
        memset(mine, 0, (size_t)n * sizeof(uint32_t));
        for (int64_t j = (int64_t)ptr[first_row[b]] - base; j < (int64_t)ptr[first_row[b + 1]] - base; ++j)
            ++mine[(int64_t)col[j] - base];
    }
#pragma omp parallel for schedule(static, 1)
    for (int t = 0; t < blocks; ++t) { /* a range of columns per thread: counts -> first slots, column totals */
        const int64_t c0 = n * t / blocks, c1 = n * (t + 1) / blocks;
        int64_t sum = 0;
        for (int64_t c = c0; c < c1; ++c) {
            uint32_t running = 0;
            for (int b = 0; b < blocks; ++b) {
                const uint32_t count = slot[(size_t)b * (size_t)n + (size_t)c];
                slot[(size_t)b * (size_t)n + (size_t)c] = running;
                running += count;
            }
            start[c] = running;
            sum += running;
        }
        part[t + 1] = sum;
    }
    for (int t = 0; t < blocks; ++t) part[t + 1] += part[t];
#pragma omp parallel for schedule(static, 1)
    for (int t = 0; t < blocks; ++t) {
        const int64_t c0 = n * t / blocks, c1 = n * (t + 1) / blocks;
        int64_t at = part[t];
        for (int64_t c = c0; c < c1; ++c) {
            const int64_t count = start[c];
            start[c] = at;
            col_ptr[c] = (idx_t)(at + base);
            at += count;
        }
    }
    start[n] = nnz;
    col_ptr[n] = (idx_t)(nnz + base);
#pragma omp parallel for schedule(static, 1)
    for (int b = 0; b < blocks; ++b) {
        uint32_t* mine = slot + (size_t)b * (size_t)n;
        for (int64_t r = first_row[b]; r < first_row[b + 1]; ++r) {
            for (int64_t j = (int64_t)ptr[r] - base; j < (int64_t)ptr[r + 1] - base; ++j) {
                const int64_t c = (int64_t)col[j] - base;
                const int64_t dst = start[c] + mine[c]++;
                row_ind[dst] = (idx_t)(r + base);
                if (value_bytes == 4) ((uint32_t*)csc_val)[dst] = ((const uint32_t*)val)[j];
                else if (value_bytes == 8) ((uint64_t*)csc_val)[dst] = ((const uint64_t*)val)[j];
            }
        }
    }
    free(first_row); free(slot); free(start); free(part);
    return 0;
}

void orc_csr2coo_omp(int64_t m, int base, const idx_t* ptr, idx_t* coo_rows) {
#pragma omp parallel for schedule(dynamic, 4096)
    for (int64_t r = 0; r < m; ++r)
        for (int64_t j = (int64_t)ptr[r] - base; j < (int64_t)ptr[r + 1] - base; ++j) coo_rows[j] = (idx_t)(r + base);
}
