// Version and status text of the C ABI.
#include "tpk_device.h"

extern "C" int tpk_version(void)
{
    return 200; // 0.2.0: three_nn, the Chamfer forward and the packed ball query take a workspace
}

extern "C" const char* tpk_status_string(int status)
{
    switch (status)
    {
    case TPK_OK:
        return "ok";
    case TPK_ERR_INVALID_ARG:
        return "invalid argument (negative size or missing pointer)";
    case TPK_ERR_UNSUPPORTED:
        return "size outside the supported range";
    case TPK_ERR_WORKSPACE:
        return "workspace missing or too small";
    case TPK_ERR_TOO_LARGE:
        return "problem needs more scratch memory than the library's fixed array holds";
    default:
        break;
    }
    if (status > 0)
        return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown status";
}
