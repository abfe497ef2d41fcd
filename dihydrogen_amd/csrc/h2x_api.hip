// Library-level entry points: ABI version and status strings.
#include "h2x_device.hpp"

extern "C" int h2x_abi_version(void)
{
    return 1;
}

extern "C" const char* h2x_status_string(int status)
{
    switch (status)
    {
    case H2X_SUCCESS: return "success";
    case H2X_ERR_INVALID_ARGUMENT: return "invalid argument";
    case H2X_ERR_UNSUPPORTED: return "unsupported element type, size or operation";
    case H2X_ERR_TOO_LARGE: return "size exceeds what one launch can address";
    case H2X_ERR_SCRATCH_LIMIT:
        return "input exceeds the fixed capacity of the library's static scratch array "
               "(use the entry point that takes a workspace)";
    default: break;
    }
    if (status > 0)
        return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown h2x status";
}
