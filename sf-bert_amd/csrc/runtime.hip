// Small runtime queries of libsfbert_hip.
#include <hip/hip_runtime.h>

#include "../../include/sfbert_hip.h"

extern "C" int sfb_device_available(void) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return count > 0 ? 1 : 0;
}

// Work-groups of the fused attention kernels that the current device keeps resident at once (4 per compute unit:
// 2 waves of up to 256 registers each, 32-36 KiB of LDS), i.e. the number of lists sfb_build_plan should make.
// 0 when no device is usable.
extern "C" uint32_t sfb_resident_work_groups(void) {
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) {
        (void)hipGetLastError();
        return 0;
    }
    return 4u * (uint32_t)cus;
}
