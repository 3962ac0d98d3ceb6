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
