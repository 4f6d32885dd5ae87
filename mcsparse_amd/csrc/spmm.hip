// CSR SpMM for gfx950: C = alpha*A*op(B) + beta*C, A is m x k CSR, op(B) is k x n dense.
//
// The reference (src/kernels/level3/spmm/csr_spmm_device.hpp:91-167) runs one wavefront per
// (row, output column) and therefore re-reads the CSR row n times, after transposing a
// row-major B into a freshly allocated column-major copy (mcsp_spmm_gpu.cpp:119-133).  Here a
// row-major op(B) is read in place: a lane group owns one row of A and each lane a few adjacent
// columns of C, so every nonzero pulls one contiguous stretch of a row of B with wide loads and
// A is read once per column panel.  A column-major op(B) is handled by a gather kernel with the
// lanes spread over the nonzeros of the row.  With beta == 0, C is never read.
#include "device_util.h"
#include "internal.h"

namespace mcsp {

namespace {

constexpr int kBlock = 256;

template <typename T, int V>
struct Vec {
    T v[V];
};

template <typename T, int V>
__device__ __forceinline__ Vec<T, V> load_vec(const T* p) {
    Vec<T, V> r;
    if constexpr (V == 1) {
        r.v[0] = p[0];
    } else if constexpr (sizeof(T) * V == 16) {
        typedef T Native __attribute__((ext_vector_type(V)));
        const Native n = *reinterpret_cast<const Native*>(p);
#pragma unroll
        for (int i = 0; i < V; ++i) r.v[i] = n[i];
    } else {
        static_assert(sizeof(T) * V == 8, "unsupported vector width");
        typedef T Native __attribute__((ext_vector_type(V)));
        const Native n = *reinterpret_cast<const Native*>(p);
#pragma unroll
        for (int i = 0; i < V; ++i) r.v[i] = n[i];
    }
    return r;
}

template <typename T, int V>
__device__ __forceinline__ void store_vec(T* p, const Vec<T, V>& r) {
    if constexpr (V == 1) {
        p[0] = r.v[0];
    } else {
        typedef T Native __attribute__((ext_vector_type(V)));
        Native n;
#pragma unroll
        for (int i = 0; i < V; ++i) n[i] = r.v[i];
        *reinterpret_cast<Native*>(p) = n;
    }
}

// op(B) row-major.  LR lanes per row of A, V adjacent columns per lane; blockIdx.y walks the
// column panels of LR*V columns.  V > 1 requires n, ldb (and ldc when C is row-major) to be
// multiples of V and 16-byte aligned base pointers, which the launcher checks.
template <typename T, int LR, int V, bool BETA0, bool C_ROW>
__global__ __launch_bounds__(kBlock) void spmm_rowb_kernel(idx_t m, idx_t n, idx_t base,
                                                           const idx_t* __restrict__ row_ptr,
                                                           const idx_t* __restrict__ col, const T* __restrict__ val,
                                                           const T* __restrict__ B, int64_t ldb, T* __restrict__ C,
                                                           int64_t ldc, T alpha, T beta) {
    constexpr int kRowsPerBlock = kBlock / LR;
    const idx_t lane = threadIdx.x % LR;
    const uint64_t row = static_cast<uint64_t>(blockIdx.x) * kRowsPerBlock + threadIdx.x / LR;
    const uint64_t c0 = (static_cast<uint64_t>(blockIdx.y) * LR + lane) * V;
    if (row >= m || c0 >= n) return;

    const idx_t start = row_ptr[row] - base;
    const idx_t end = row_ptr[row + 1] - base;
    T acc[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = T(0);

    constexpr int kUnroll = 8;
    const T* Bc = B + c0;
    idx_t j = start;
    for (; j + kUnroll <= end; j += kUnroll) {
        idx_t c[kUnroll];
        T a[kUnroll];
        Vec<T, V> b[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            c[u] = col[j + u] - base;
            a[u] = val[j + u];
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) b[u] = load_vec<T, V>(Bc + static_cast<int64_t>(c[u]) * ldb);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i] += a[u] * b[u].v[i];
        }
    }
    for (; j < end; ++j) {
        const idx_t c = col[j] - base;
        const T a = val[j];
        const Vec<T, V> b = load_vec<T, V>(Bc + static_cast<int64_t>(c) * ldb);
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] += a * b.v[i];
    }

    if constexpr (C_ROW) {
        T* Cp = C + static_cast<int64_t>(row) * ldc + c0;
        Vec<T, V> out;
        if constexpr (BETA0) {
#pragma unroll
            for (int i = 0; i < V; ++i) out.v[i] = alpha * acc[i];
        } else {
            const Vec<T, V> old = load_vec<T, V>(Cp);
#pragma unroll
            for (int i = 0; i < V; ++i) out.v[i] = beta * old.v[i] + alpha * acc[i];
        }
        store_vec<T, V>(Cp, out);
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) {
            T* Cp = C + static_cast<int64_t>(c0 + i) * ldc + row;
            if constexpr (BETA0) {
                *Cp = alpha * acc[i];
            } else {
                *Cp = beta * *Cp + alpha * acc[i];
            }
        }
    }
}

// op(B) column-major: element (kk, j) at j*ldb + kk.  One wavefront per row of A, lanes strided
// over its nonzeros, JB output columns accumulated at once so the row of A is re-read only
// n/JB times.
template <typename T, int JB, bool BETA0>
__global__ __launch_bounds__(kBlock) void spmm_colb_kernel(idx_t m, idx_t n, idx_t base,
                                                           const idx_t* __restrict__ row_ptr,
                                                           const idx_t* __restrict__ col, const T* __restrict__ val,
                                                           const T* __restrict__ B, int64_t ldb, T* __restrict__ C,
                                                           int64_t c_row_stride, int64_t c_col_stride, T alpha,
                                                           T beta) {
    const unsigned lane = threadIdx.x % kWave;
    const uint64_t row = static_cast<uint64_t>(blockIdx.x) * (kBlock / kWave) + threadIdx.x / kWave;
    const bool live = row < m;  // dead waves still run the reductions with zero work
    const idx_t start = live ? row_ptr[row] - base : 0;
    const idx_t end = live ? row_ptr[row + 1] - base : 0;

    for (idx_t j0 = 0; j0 < n; j0 += JB) {
        T s[JB];
#pragma unroll
        for (int jj = 0; jj < JB; ++jj) s[jj] = T(0);
        for (idx_t e = start + lane; e < end; e += kWave) {
            const idx_t c = col[e] - base;
            const T a = val[e];
#pragma unroll
            for (int jj = 0; jj < JB; ++jj) {
                if (j0 + jj < n) s[jj] += a * B[static_cast<int64_t>(j0 + jj) * ldb + c];
            }
        }
#pragma unroll
        for (int jj = 0; jj < JB; ++jj) s[jj] = group_sum<kWave>(s[jj]);
        if (live && lane == 0) {
#pragma unroll
            for (int jj = 0; jj < JB; ++jj) {
                if (j0 + jj < n) {
                    T* Cp = C + static_cast<int64_t>(row) * c_row_stride + static_cast<int64_t>(j0 + jj) * c_col_stride;
                    if constexpr (BETA0) {
                        *Cp = alpha * s[jj];
                    } else {
                        *Cp = beta * *Cp + alpha * s[jj];
                    }
                }
            }
        }
    }
}

template <typename T, int LR, int V>
void launch_rowb(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    const uint64_t row_blocks = (static_cast<uint64_t>(a.m) + (kBlock / LR) - 1) / (kBlock / LR);
    const uint64_t panels = (static_cast<uint64_t>(a.n) + LR * V - 1) / (LR * V);
    const dim3 grid(static_cast<uint32_t>(row_blocks), static_cast<uint32_t>(panels));
    const T* val = static_cast<const T*>(a.val);
    const T* B = static_cast<const T*>(a.B);
    T* C = static_cast<T*>(a.C);
    const bool beta0 = beta == T(0);
#define MCSP_LAUNCH_ROWB(B0, CR)                                                                                   \
    hipLaunchKernelGGL((spmm_rowb_kernel<T, LR, V, B0, CR>), grid, dim3(kBlock), 0, stream, a.m, a.n, a.base,       \
                       a.row_ptr, a.col, val, B, a.ldb, C, a.ldc, alpha, beta)
    if (beta0 && a.c_row_major) MCSP_LAUNCH_ROWB(true, true);
    else if (beta0) MCSP_LAUNCH_ROWB(true, false);
    else if (a.c_row_major) MCSP_LAUNCH_ROWB(false, true);
    else MCSP_LAUNCH_ROWB(false, false);
#undef MCSP_LAUNCH_ROWB
}

template <typename T, int V>
void launch_rowb_v(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    const uint64_t lanes_needed = (static_cast<uint64_t>(a.n) + V - 1) / V;
    if (lanes_needed <= 1) launch_rowb<T, 1, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 2) launch_rowb<T, 2, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 4) launch_rowb<T, 4, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 8) launch_rowb<T, 8, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 16) launch_rowb<T, 16, V>(stream, a, alpha, beta);
    else if (lanes_needed <= 32) launch_rowb<T, 32, V>(stream, a, alpha, beta);
    else launch_rowb<T, 64, V>(stream, a, alpha, beta);
}


}  // namespace

template <typename T>
void launch_spmm(hipStream_t stream, const SpmmArgs& a, T alpha, T beta) {
    if (a.m == 0 || a.n == 0) return;
    if (a.b_row_major) {
        constexpr int kWide = 16 / sizeof(T);  // elements per 128-bit access
        const bool aligned = (reinterpret_cast<uintptr_t>(a.B) % 16 == 0) && (a.ldb % kWide == 0) &&
                             (a.n % kWide == 0) &&
                             (!a.c_row_major || ((reinterpret_cast<uintptr_t>(a.C) % 16 == 0) && (a.ldc % kWide == 0)));
        if (aligned) launch_rowb_v<T, kWide>(stream, a, alpha, beta);
        else launch_rowb_v<T, 1>(stream, a, alpha, beta);
    } else {
        constexpr int kJB = 4;
        const uint64_t blocks = (static_cast<uint64_t>(a.m) + (kBlock / kWave) - 1) / (kBlock / kWave);
        const int64_t rs = a.c_row_major ? a.ldc : 1;
        const int64_t cs = a.c_row_major ? 1 : a.ldc;
        const T* val = static_cast<const T*>(a.val);
        const T* B = static_cast<const T*>(a.B);
        T* C = static_cast<T*>(a.C);
        if (beta == T(0)) {
            hipLaunchKernelGGL((spmm_colb_kernel<T, kJB, true>), dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0,
                               stream, a.m, a.n, a.base, a.row_ptr, a.col, val, B, a.ldb, C, rs, cs, alpha, beta);
        } else {
            hipLaunchKernelGGL((spmm_colb_kernel<T, kJB, false>), dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0,
                               stream, a.m, a.n, a.base, a.row_ptr, a.col, val, B, a.ldb, C, rs, cs, alpha, beta);
        }
    }
}

template void launch_spmm<float>(hipStream_t, const SpmmArgs&, float, float);
template void launch_spmm<double>(hipStream_t, const SpmmArgs&, double, double);

}  // namespace mcsp
