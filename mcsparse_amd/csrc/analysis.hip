// Row-length binning of a CSR structure.  Class 0 = empty row, class b >= 1 = length in
// [2^(b-1), 2^b).  The histogram (and the longest row) steer the SpMV kernel choice; the
// per-row classes are exported for inspection.  Integer work only, so the result does not
// depend on the order in which workgroups finish.
#include "device_util.h"
#include "internal.h"

namespace mcsp {

namespace {

constexpr int kBinsBlock = 256;
constexpr int kBinsMaxGrid = 1024;

__global__ __launch_bounds__(kBinsBlock) void row_bins_kernel(idx_t m, const idx_t* __restrict__ row_ptr,
                                                              uint8_t* __restrict__ row_bins,
                                                              uint32_t* __restrict__ hist_out) {
    __shared__ uint32_t s_hist[MCSPARSE_ROW_BIN_COUNT + 1];
    if (threadIdx.x <= MCSPARSE_ROW_BIN_COUNT) s_hist[threadIdx.x] = 0;
    __syncthreads();

    uint32_t local_max = 0;
    // row_ptr differences do not depend on the index base
    for (uint64_t r = static_cast<uint64_t>(blockIdx.x) * kBinsBlock + threadIdx.x; r < m;
         r += static_cast<uint64_t>(gridDim.x) * kBinsBlock) {
        const uint32_t len = row_ptr[r + 1] - row_ptr[r];
        const uint32_t bin = len == 0 ? 0u : 32u - static_cast<uint32_t>(__clz(static_cast<int>(len)));
        if (row_bins != nullptr) row_bins[r] = static_cast<uint8_t>(bin);
        atomicAdd(&s_hist[bin], 1u);
        local_max = max(local_max, len);
    }
    atomicMax(&s_hist[MCSPARSE_ROW_BIN_COUNT], local_max);
    __syncthreads();

    if (threadIdx.x < MCSPARSE_ROW_BIN_COUNT) {
        const uint32_t c = s_hist[threadIdx.x];
        if (c != 0) atomicAdd(&hist_out[threadIdx.x], c);
    } else if (threadIdx.x == MCSPARSE_ROW_BIN_COUNT) {
        const uint32_t c = s_hist[threadIdx.x];
        if (c != 0) atomicMax(&hist_out[MCSPARSE_ROW_BIN_COUNT], c);
    }
}

// ---- what the memory takes by itself ----------------------------------------------------------------------
// Three streaming kernels over 16-byte pieces, as plain as the kernels of this library can be made: the yardstick
// their achieved bytes per second are held against (mcsparseXstreamProbe).  A workgroup takes a contiguous 16 KB:
// four pieces per thread, asked for together.  (A grid of a few workgroups per compute unit striding through the
// array with eight pieces in flight per thread wrote 4.5 TB/s and copied 4.6 TB/s where this shape writes and
// copies what a plain device fill and copy reach.)
constexpr int kProbeBlock = 256;
constexpr int kProbeAhead = 4;
typedef uint32_t piece_t __attribute__((ext_vector_type(4)));

// mode 0: read src (every thread's pieces are summed and the sum kept in sink[thread % sink_words] when it is
// not zero, which the contents of a benchmark buffer never add up to, so that the loads stay and nothing is
// written), 1: write dst, 2: copy src to dst.
template <int MODE>
__global__ __launch_bounds__(kProbeBlock) void stream_probe_kernel(const piece_t* __restrict__ src,
                                                                   piece_t* __restrict__ dst, uint64_t pieces,
                                                                   uint32_t* __restrict__ sink, uint32_t sink_words) {
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * (kProbeBlock * kProbeAhead) + threadIdx.x;
    piece_t got[kProbeAhead];
    const piece_t fill = {static_cast<uint32_t>(first), 1u, 2u, 3u};
    if constexpr (MODE != 1) {
#pragma unroll
        for (int a = 0; a < kProbeAhead; ++a) {
            const uint64_t p = first + static_cast<uint64_t>(a) * kProbeBlock;
            got[a] = src[p < pieces ? p : pieces - 1];
        }
    }
    piece_t sum = {0, 0, 0, 0};
#pragma unroll
    for (int a = 0; a < kProbeAhead; ++a) {
        const uint64_t p = first + static_cast<uint64_t>(a) * kProbeBlock;
        if constexpr (MODE == 0) sum += got[a];
        if constexpr (MODE == 1) { if (p < pieces) dst[p] = fill; }
        if constexpr (MODE == 2) { if (p < pieces) dst[p] = got[a]; }
    }
    if constexpr (MODE == 0) {
        const uint32_t folded = sum[0] + sum[1] + sum[2] + sum[3];
        if (folded == 0x9e3779b9u) sink[first % sink_words] = folded;
    }
}

__global__ void zero_u32_kernel(uint32_t* p, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

}  // namespace

void launch_row_bins(hipStream_t stream, idx_t m, const idx_t* row_ptr, idx_t /*base*/, uint8_t* row_bins,
                     uint32_t* hist_out) {
    // a fill kernel rather than a memset node, so that the sequence can be captured in a HIP graph
    hipLaunchKernelGGL(zero_u32_kernel, dim3(1), dim3(64), 0, stream, hist_out,
                       static_cast<uint32_t>(MCSPARSE_ROW_BIN_COUNT + 1));
    if (m == 0) return;
    const uint64_t blocks = (static_cast<uint64_t>(m) + kBinsBlock - 1) / kBinsBlock;
    const uint32_t grid = static_cast<uint32_t>(blocks < kBinsMaxGrid ? blocks : kBinsMaxGrid);
    hipLaunchKernelGGL(row_bins_kernel, dim3(grid), dim3(kBinsBlock), 0, stream, m, row_ptr, row_bins, hist_out);
}

// bytes: a multiple of 16, both arrays 16-byte aligned; sink: at least one uint32 (mode 0).
void launch_stream_probe(hipStream_t stream, int mode, const void* src, void* dst, uint64_t bytes, uint32_t* sink,
                         uint32_t sink_words) {
    const uint64_t pieces = bytes / 16;
    if (pieces == 0) return;
    const uint64_t per_block = static_cast<uint64_t>(kProbeBlock) * kProbeAhead;
    const dim3 grid(static_cast<uint32_t>((pieces + per_block - 1) / per_block));
    const piece_t* s = static_cast<const piece_t*>(src);
    piece_t* d = static_cast<piece_t*>(dst);
    if (mode == 0)
        hipLaunchKernelGGL((stream_probe_kernel<0>), grid, dim3(kProbeBlock), 0, stream, s, d, pieces, sink, sink_words);
    else if (mode == 1)
        hipLaunchKernelGGL((stream_probe_kernel<1>), grid, dim3(kProbeBlock), 0, stream, s, d, pieces, sink, sink_words);
    else
        hipLaunchKernelGGL((stream_probe_kernel<2>), grid, dim3(kProbeBlock), 0, stream, s, d, pieces, sink, sink_words);
}

}  // namespace mcsp
