// Library-level entry points: version and error text.
#include "tk3d_common.h"

extern "C" {

int tk3d_version(void) { return TK3D_VERSION; }

const char *tk3d_error_string(int code)
{
    switch (code) {
    case TK3D_OK:
        return "success";
    case TK3D_ERR_NULL_POINTER:
        return "a required pointer argument is NULL";
    case TK3D_ERR_BAD_SIZE:
        return "a size argument is negative";
    case TK3D_ERR_BAD_K:
        return "k / num_samples is outside the legal range";
    case TK3D_ERR_BAD_VERSION:
        return "Invalid version";
    case TK3D_ERR_WORKSPACE:
        return "workspace is missing or too small";
    case TK3D_ERR_UNSUPPORTED:
        return "shape is larger than the kernels can index";
    default:
        break;
    }
    if (code > 0)
        return hipGetErrorString((hipError_t)code);
    return "unknown tk3d error code";
}

}  // extern "C"
