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

inline int launch_status()
{
    return hipGetLastError() == hipSuccess ? MRX_OK : MRX_ERR_LAUNCH;
}

inline bool aligned(const void *p, size_t n)
{
    return (reinterpret_cast<uintptr_t>(p) % n) == 0;
}

}  // namespace mrx
