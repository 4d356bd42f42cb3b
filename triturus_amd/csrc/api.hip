// Library identity and status text of the C ABI.
#include "common.hpp"

extern "C" int trt_version(void) { return TRT_ABI_VERSION; }

extern "C" const char *trt_error_string(int status) {
    switch (status) {
        case TRT_OK: return "success";
        case TRT_E_INVALID: return "invalid argument (null pointer, non-positive size or unknown enum)";
        case TRT_E_LAYOUT: return "unsupported layout (unit trailing stride where required, strides non-negative, pointers element-aligned)";
        case TRT_E_WORKSPACE: return "workspace missing or too small";
        case TRT_E_RANGE: return "size exceeds the supported index range";
        case TRT_E_SCRATCH: return "the call needs more scratch memory than the library's static array holds";
        default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown status";
}
