// Library-level entry points of the C ABI (status strings, version, chunk size).
#include "common.h"

extern "C" const char *mrx_status_string(int status)
{
    switch (status) {
    case MRX_OK: return "ok";
    case MRX_ERR_INVALID_ARG: return "invalid argument";
    case MRX_ERR_UNSUPPORTED: return "unsupported configuration";
    case MRX_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown status";
    }
}

extern "C" int mrx_version(void) { return 100; }

#ifdef MRX_PHASE_TIMING
__device__ unsigned long long mrx_phase_ticks[64];
__device__ unsigned long long mrx_wg_trace[4096 * 3];
extern "C" int mrx_wg_trace_read(unsigned long long *host)
{
    return hipMemcpyFromSymbol(host, HIP_SYMBOL(mrx_wg_trace), sizeof(unsigned long long) * 4096 * 3) == hipSuccess ? 0 : -1;
}
extern "C" int mrx_phase_read(unsigned long long *host, int reset)
{
    if (hipMemcpyFromSymbol(host, HIP_SYMBOL(mrx_phase_ticks), sizeof(unsigned long long) * 64) != hipSuccess) return -1;
    if (reset) {
        unsigned long long z[64] = {0};
        if (hipMemcpyToSymbol(HIP_SYMBOL(mrx_phase_ticks), z, sizeof(z)) != hipSuccess) return -1;
    }
    return 0;
}
#endif
