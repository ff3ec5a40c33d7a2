// Library-level entry points of the C ABI: version and error strings.
#include "common.h"

REPDL_API int repdl_hip_abi_version(void) { return 1; }

REPDL_API const char *repdl_hip_error_string(int code)
{
    switch (code)
    {
    case REPDL_OK:
        return "success";
    case REPDL_E_ARG:
        return "repdl_hip: invalid argument (null pointer, negative or oversized extent)";
    case REPDL_E_UNSUPPORTED:
        return "repdl_hip: unsupported combination of arguments";
    case REPDL_E_WORKSPACE:
        return "repdl_hip: workspace missing or too small";
    case REPDL_E_TOO_LARGE:
        return "repdl_hip: input exceeds the fixed capacity of this entry point (it allocates nothing; see its *_max_n)";
    default:
        break;
    }
    if (code > 0)
        return hipGetErrorString((hipError_t)code);
    return "repdl_hip: unknown error code";
}
