// Shared host/device helpers for the gfx950 sequence kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

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

inline int launch_status()
{
    return hipGetLastError() == hipSuccess ? MRX_OK : MRX_ERR_LAUNCH;
}

// Raises a kernel's dynamic LDS limit once per device (the attribute belongs to the device's
// copy of the kernel).  `done` is a per-kernel bit mask indexed by device id; setting it twice
// from racing threads only repeats an idempotent call.
template <typename K> inline int ensure_lds_limit(K kern, int bytes, unsigned long long &done)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return MRX_ERR_LAUNCH;
    const unsigned long long bit = 1ull << (dev & 63);
    if (!(done & bit)) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                bytes) != hipSuccess)
            return MRX_ERR_LAUNCH;
        done |= bit;
    }
    return MRX_OK;
}

inline bool aligned(const void *p, size_t n)
{
    return (reinterpret_cast<uintptr_t>(p) % n) == 0;
}

}  // namespace mrx

// Phase timing for kernel tuning: compiled in only with -DMRX_PHASE_TIMING (never in
// the shipped library).  Workgroup 0 / thread 0 accumulates the shader-clock ticks
// spent between consecutive MRX_PHASE marks; MRX_PHASE_FLUSH adds them to mrx_phase_ticks[].
#ifdef MRX_PHASE_TIMING
extern __device__ unsigned long long mrx_phase_ticks[64];
extern __device__ unsigned long long mrx_wg_trace[4096 * 3];
#define MRX_WG_BEGIN()                                                                    \
    do {                                                                                  \
        if (threadIdx.x == 0 && blockIdx.x < 4096) {                                      \
            mrx_wg_trace[blockIdx.x * 3 + 0] = wall_clock64();                            \
            mrx_wg_trace[blockIdx.x * 3 + 2] = __builtin_amdgcn_s_getreg((4) | (0 << 6) | (31 << 11)) \
                | ((unsigned long long)__builtin_amdgcn_s_getreg((20) | (0 << 6) | (31 << 11)) << 32); \
        }                                                                                 \
    } while (0)
#define MRX_WG_END()                                                                      \
    do {                                                                                  \
        if (threadIdx.x == 0 && blockIdx.x < 4096) mrx_wg_trace[blockIdx.x * 3 + 1] = wall_clock64(); \
    } while (0)
// marks (i < 32; thread 0 -> slot i, thread 256 -> slot 32 + i) accumulate in LDS
// (fire-and-forget ds_add) so that a mark never waits on global memory
#define MRX_PHASE_INIT()                                                    \
    __shared__ unsigned long long mrx_lds_ticks[64];                        \
    if (threadIdx.x < 64) mrx_lds_ticks[threadIdx.x] = 0;                   \
    unsigned long long mrx_t_last = clock64()
#define MRX_PHASE(i)                                                        \
    do {                                                                    \
        if (blockIdx.x == 0 && (threadIdx.x == 0 || threadIdx.x == 256)) {  \
            const unsigned long long mrx_t_now = clock64();                 \
            __hip_atomic_fetch_add(&mrx_lds_ticks[(i) + (threadIdx.x ? 32 : 0)], mrx_t_now - mrx_t_last, __ATOMIC_RELAXED, \
                                   __HIP_MEMORY_SCOPE_WORKGROUP);           \
            mrx_t_last = mrx_t_now;                                         \
        }                                                                   \
    } while (0)
#define MRX_PHASE_FLUSH()                                                   \
    do {                                                                    \
        if (blockIdx.x == 0 && threadIdx.x < 64) mrx_phase_ticks[threadIdx.x] += mrx_lds_ticks[threadIdx.x]; \
    } while (0)
#else
#define MRX_WG_BEGIN() do { } while (0)
#define MRX_WG_END() do { } while (0)
#define MRX_PHASE_INIT() do { } while (0)
#define MRX_PHASE(i) do { } while (0)
#define MRX_PHASE_FLUSH() do { } while (0)
#endif
