// kvcm_internal.h -- shared by the translation units of libkvcm_hip.so (not installed).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kvcm_hip.h"

namespace kvcm {

constexpr uint64_t kGolden = 0x9e3779b97f4a7c15ULL;

inline int32_t launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? KVCM_OK : static_cast<int32_t>(e);
}

// One hashInt64Func step (kv_cache_manager/manager/hash_util.h:8-12) with the token term pre-added:
// a = value + 0x9e3779b97f4a7c15. Unsigned arithmetic wraps mod 2^64; the right shift is arithmetic.
__host__ __device__ inline uint64_t hash_step_preadded(uint64_t h, uint64_t a) {
    return h ^ (a + (h << 12) + static_cast<uint64_t>(static_cast<int64_t>(h) >> 32));
}

}  // namespace kvcm
