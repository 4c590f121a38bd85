// Library-level entry points of the C ABI: status strings, version, per-device set-up.
#include <atomic>
#include <mutex>

#include "common.h"

namespace mrx {

namespace {
KernelNode *g_kernels = nullptr;               // filled while the library is loaded, read-only afterwards
std::atomic<unsigned long long> g_ready{0ull};  // bit d: device d has been set up
std::mutex g_setup;
int g_cus[64] = {0};
}  // namespace

void register_kernel(KernelNode *node)
{
    node->next = g_kernels;
    g_kernels = node;
}

int prepare_device(int *cus, int *dev_out)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return MRX_ERR_LAUNCH;
    if (dev < 0 || dev >= 64) return MRX_ERR_UNSUPPORTED;
    const unsigned long long bit = 1ull << dev;
    if (!(g_ready.load(std::memory_order_acquire) & bit)) {
        std::lock_guard<std::mutex> lock(g_setup);
        if (!(g_ready.load(std::memory_order_relaxed) & bit)) {
            // a refused set-up call is reported through the return value and taken off the runtime's
            // record, as a refused launch is (launch_kernel)
            auto failed = [](hipError_t e) {
                if (e == hipSuccess) return false;
                (void)hipGetLastError();
                return true;
            };
            for (const KernelNode *n = g_kernels; n; n = n->next)
                if (failed(hipFuncSetAttribute(n->fn, hipFuncAttributeMaxDynamicSharedMemorySize, n->lds_bytes)))
                    return MRX_ERR_LAUNCH;
            int n_cu = 0;
            if (failed(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev))) return MRX_ERR_LAUNCH;
            g_cus[dev] = n_cu;
            if (const int rc = resolve_scratch(dev); rc != MRX_OK) return rc;
            g_ready.fetch_or(bit, std::memory_order_release);
        }
    }
    if (cus) *cus = g_cus[dev];
    if (dev_out) *dev_out = dev;
    return MRX_OK;
}

}  // namespace mrx

extern "C" const char *mrx_status_string(int status)
{
    switch (status) {
    case MRX_OK: return "ok";
    case MRX_ERR_INVALID_ARG: return "invalid argument";
    case MRX_ERR_UNSUPPORTED: return "unsupported configuration";
    case MRX_ERR_LAUNCH: return "kernel launch failed";
    case MRX_ERR_SCRATCH: return "problem exceeds the library's static scratch buffer";
    default: return "unknown status";
    }
}

extern "C" int mrx_version(void) { return 400; }

extern "C" int mrx_init(int device)
{
    int prev = 0;
    if (hipGetDevice(&prev) != hipSuccess) return MRX_ERR_LAUNCH;
    if (device < 0 || device >= 64) return MRX_ERR_INVALID_ARG;
    if (device != prev && hipSetDevice(device) != hipSuccess) return MRX_ERR_INVALID_ARG;
    const int rc = mrx::prepare_device();
    if (device != prev && hipSetDevice(prev) != hipSuccess) return MRX_ERR_LAUNCH;
    return rc;
}
