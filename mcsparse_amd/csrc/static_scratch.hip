// mcsparseSpMV_staticBuffer: mcsparseSpMV for callers that cannot allocate device memory (code under
// HIP graph capture, serving loops and harnesses that forbid hipMalloc).  The scratch that
// mcsparseSpMV takes as externalBuffer lives here in a device array of fixed size that is part of the
// library's code object, so every GPU the library runs on holds one copy until the process ends.
#include <hip/hip_runtime.h>

#include <mutex>

#include "internal.h"

namespace {

constexpr size_t kScratchBytes = MCSPARSE_SPMV_STATIC_BUFFER_BYTES;
constexpr int kMaxDevices = 64;

// In host code this name only stands for the symbol; the memory is reached through the address
// that hipGetSymbolAddress reports for the current device.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

std::mutex g_lock;
void* g_scratch_of_device[kMaxDevices] = {nullptr};

// Address of the current device's copy of `scratch`, looked up once per device.  The lookup may load the
// library's code object, which is not stream work: while `stream` is being captured into a graph it is not
// attempted (hipErrorStreamCaptureUnsupported), so the first call on a device must come before the capture.
hipError_t scratch_of_current_device(hipStream_t stream, void** out) {
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return err;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(g_lock);
    if (g_scratch_of_device[device] == nullptr) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone)
            return hipErrorStreamCaptureUnsupported;
        void* ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return err;
        if (ptr == nullptr) return hipErrorInvalidSymbol;
        g_scratch_of_device[device] = ptr;
    }
    *out = g_scratch_of_device[device];
    return hipSuccess;
}

}  // namespace

extern "C" {

// EXTENSION
mcsparseStatus_t mcsparseSpMV_staticBuffer(mcsparseHandle_t handle, mcsparseOperation_t opA, const void* alpha,
                                           mcsparseSpMatDescr_t matA, mcsparseDnVecDescr_t vecX, const void* beta,
                                           mcsparseDnVecDescr_t vecY, macaDataType computeType,
                                           mcsparseSpMVAlg_t alg) {
    // Every argument check, the size check included, comes before the device is touched; the checks
    // only need a buffer pointer that is not null.
    static unsigned char placeholder;
    const mcspStatus_t st =
        mcsp::spmv_check(handle, opA, alpha, matA, vecX, beta, vecY, computeType, &placeholder, kScratchBytes, false);
    if (st != MCSP_STATUS_SUCCESS) return to_public_status(st);
    void* buffer = nullptr;
    const hipError_t found = scratch_of_current_device(handle->stream, &buffer);
    // the first call on a device under graph capture: NOT_SUPPORTED, as for everything a capture cannot hold
    if (found == hipErrorStreamCaptureUnsupported) return to_public_status(MCSP_STATUS_NOT_IMPLEMENTED);
    if (found != hipSuccess) return to_public_status(MCSP_STATUS_INTERNAL_ERROR);
    return to_public_status(
        mcsp::spmv_call(handle, opA, alpha, matA, vecX, beta, vecY, computeType, buffer, kScratchBytes, false, alg));
}

}  // extern "C"
