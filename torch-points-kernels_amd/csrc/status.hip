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

#ifdef TPK_COUNT_WORK
// Counting build only: the per-translation-unit work counters (tpk_device.h) and their sum.
#include <vector>

namespace {
std::vector<int (*)(unsigned long long*)>& work_readers()
{
    static std::vector<int (*)(unsigned long long*)> readers;
    return readers;
}
} // namespace

extern "C" void tpk_work_register(int (*read_reset)(unsigned long long*))
{
    work_readers().push_back(read_reset);
}

// Waits for the device, returns the pair evaluations counted since the last call in *pairs and
// sets the counters back to zero.
extern "C" int tpk_work_read_reset(unsigned long long* pairs)
{
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess)
        return static_cast<int>(e);
    unsigned long long total = 0;
    for (auto reader : work_readers())
    {
        unsigned long long part = 0;
        const int st = reader(&part);
        if (st != 0)
            return st;
        total += part;
    }
    *pairs = total;
    return TPK_OK;
}
#endif
