// Library-level entry points of the C ABI: version, error strings, device check.
#include <string.h>

#include "mx_common.h"

extern "C" int mx_abi_version(void) { return MX_ABI_VERSION; }

extern "C" const char *mx_strerror(int status) {
    switch (status) {
    case MX_OK: return "ok";
    case MX_EINVAL: return "invalid argument: a size, stride or alignment contract is violated";
    case MX_EUNSUPPORTED: return "unsupported: no kernel in this build covers the request";
    case MX_ELAUNCH: return "the HIP runtime refused the kernel launch";
    case MX_ENODEV: return "the device is not a gfx950 (MI355X-class) GPU";
    case MX_ECAPTURE:
        return "the stream is being captured into a graph: this library refuses to be recorded (run it eagerly)";
    case MX_ETOOBIG:
        return "the request needs more scratch than the fixed array of this no-allocation entry point holds; use the "
               "variant that takes a caller workspace";
    default: return "unknown status";
    }
}

extern "C" int mx_device_supported(int dev) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return MX_ENODEV;
    return strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? MX_OK : MX_ENODEV;
}
