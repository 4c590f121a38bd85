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
