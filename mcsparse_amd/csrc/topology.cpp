// What the kernels' launch shapes assume about the chip, read from the device instead of written into them.
#include <mutex>

#include "internal.h"

namespace mcsp {

// A gfx950 accelerator complex die (XCD) holds 32 compute units with an L2 of their own, and the hardware hands
// consecutive workgroups of a launch to the XCDs of a device in turn.  An MI355X shows all eight XCDs (256 compute
// units) as one device; partitioned, a device is four, two or one XCD.  A compute-unit count that is not a whole
// number of XCDs (another part, a harvested one) gives one "XCD": the orders that keep neighbouring work in one L2
// then turn into the plain order, which is correct everywhere and merely not tuned.
Topology topology_of_cu_count(int cus) {
    Topology t;
    t.cus = cus > 0 ? static_cast<uint32_t>(cus) : 1u;
    const uint32_t per_xcd = 32;
    t.xcds = (t.cus % per_xcd == 0 && t.cus / per_xcd <= kMaxXcds) ? t.cus / per_xcd : 1u;
    return t;
}

// Of the current device, asked once per device at the first launch that needs it (mcsparseCreate touches no device).
Topology device_topology() {
    constexpr int kMaxDevices = 64;
    static std::mutex lock;
    static Topology known[kMaxDevices];
    static bool have[kMaxDevices] = {false};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return topology_of_cu_count(256);
    std::lock_guard<std::mutex> guard(lock);
    if (!have[device]) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) cus = 256;
        known[device] = topology_of_cu_count(cus);
        have[device] = true;
    }
    return known[device];
}

}  // namespace mcsp

extern "C" {

// EXTENSION
mcsparseStatus_t mcsparseXtopologyOfCuCount(int computeUnits, int* xcds) {
    if (xcds == nullptr) return to_public_status(MCSP_STATUS_INVALID_POINTER);
    if (computeUnits <= 0) return to_public_status(MCSP_STATUS_INVALID_SIZE);
    *xcds = static_cast<int>(mcsp::topology_of_cu_count(computeUnits).xcds);
    return MCSPARSE_STATUS_SUCCESS;
}

}  // extern "C"
