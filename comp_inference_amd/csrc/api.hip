// Library-wide entry points: error text, ABI version, device check.
#include "ci_common.h"

#include <string.h>

namespace ci {
thread_local char g_err[512] = "";
}

extern "C" const char *ci_last_error(void) { return ci::g_err; }

extern "C" int ci_abi_version(void) { return 3; }

extern "C" int ci_check_device(void) {
    int dev = 0;
    CI_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    CI_HIP(hipGetDeviceProperties(&prop, dev));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return ci::fail(CI_ERR_DEVICE, "device %d is %s; this library holds gfx950 code only", dev,
                        prop.gcnArchName);
    // per-device set-up that must not happen for the first time inside a graph capture
    return ci_fused_linear_noalloc_init();
}
