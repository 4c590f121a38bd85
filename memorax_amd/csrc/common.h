// Shared host/device helpers for the gfx950 sequence kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <tuple>
#include <utility>

#include "memorax_amd.h"

namespace mrx {

// done flag at flat index i; `is_f32` selects float32 storage, else uint8.
__device__ __forceinline__ bool done_at(const void *done, int is_f32, int64_t i)
{
    return is_f32 ? (reinterpret_cast<const float *>(done)[i] != 0.0f)
                  : (reinterpret_cast<const uint8_t *>(done)[i] != 0);
}

// Raw (unconverted) load of a done flag / test of a raw value.  Keeping the loaded
// bits untouched until the next chunk lets the load stay in flight: any arithmetic
// on the value right after the load would force a wait on the whole prefetch.
__device__ __forceinline__ uint32_t done_raw(const void *done, int is_f32, int64_t i)
{
    return is_f32 ? reinterpret_cast<const uint32_t *>(done)[i]
                  : (uint32_t) reinterpret_cast<const uint8_t *>(done)[i];
}
__device__ __forceinline__ bool done_test(uint32_t raw, int is_f32)
{
    return is_f32 ? (__uint_as_float(raw) != 0.0f) : (raw != 0u);
}

// Launches `kern` and returns MRX_OK or MRX_ERR_LAUNCH from the launch call's own return code.
// The runtime's sticky "last error" is not consulted, so an error left behind by other code in the
// process is not mistaken for this launch's, and is still there for its owner.  When the launch
// itself is refused, the error it has just recorded is this call's own and is reported through the
// return value: it is taken off the runtime's record, or the next runtime call of the host
// framework would report it a second time as its own.
template <typename... KArgs, size_t... I>
inline int launch_impl(void (*kern)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t st,
                       std::tuple<KArgs...> &vals, std::index_sequence<I...>)
{
    void *ptrs[] = {static_cast<void *>(&std::get<I>(vals))...};
    if (hipLaunchKernel(reinterpret_cast<const void *>(kern), grid, block, ptrs, lds_bytes, st) == hipSuccess) return MRX_OK;
    (void)hipGetLastError();
    return MRX_ERR_LAUNCH;
}
template <typename... KArgs, typename... Args>
inline int launch_kernel(void (*kern)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t st, Args... args)
{
    static_assert(sizeof...(KArgs) == sizeof...(Args), "one argument per kernel parameter");
    std::tuple<KArgs...> vals(static_cast<KArgs>(args)...);
    return launch_impl(kern, grid, block, lds_bytes, st, vals, std::index_sequence_for<KArgs...>{});
}

// Per-device set-up, done once per device by mrx_init() or by the first launch on it: every kernel
// that needs more than the default 64 KB of dynamic LDS gets its limit raised (the attribute belongs
// to the device's copy of the kernel), the number of compute units is cached, and the address of the
// library's static scratch array on that device is resolved.  Kernels enter the list through a
// KernelRegistrar with static storage, i.e. while the library is being loaded; after that the list
// is read-only.
struct KernelNode {
    const void *fn;
    int lds_bytes;
    KernelNode *next;
};
void register_kernel(KernelNode *node);
struct KernelRegistrar {
    KernelNode node;
    KernelRegistrar(const void *fn, int lds_bytes) : node{fn, lds_bytes, nullptr} { register_kernel(&node); }
};
// Makes the current device ready (see above).  Returns an MRX_* status; *cus (if given) receives the
// device's compute-unit count, *dev its index.
int prepare_device(int *cus = nullptr, int *dev = nullptr);
// Defined beside the scratch array (chunk_fwd.hip): resolves its address on the current device.
int resolve_scratch(int dev);

inline bool aligned(const void *p, size_t n)
{
    return (reinterpret_cast<uintptr_t>(p) % n) == 0;
}

}  // namespace mrx
