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
        case TRT_E_STATE: return "the arrival counters of a max workspace are not idle (never prepared with trt_max_workspace_init, written over, or in use by another stream)";
        default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown status";
}

// Is `stream` being captured into a HIP graph, and into which capture?  *capture_id is 0 when it
// is not.  Host only.
extern "C" int trt_stream_capture_id(void *stream, unsigned long long *capture_id) {
    if (!capture_id) return TRT_E_INVALID;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long id = 0;
    const hipError_t err = hipStreamGetCaptureInfo(static_cast<hipStream_t>(stream), &status, &id);
    if (err != hipSuccess) return (int)err;
    *capture_id = status == hipStreamCaptureStatusActive ? (id ? id : 1) : 0;
    return TRT_OK;
}
