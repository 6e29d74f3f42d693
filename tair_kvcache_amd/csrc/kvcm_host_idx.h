// kvcm_host_idx.h -- the host side of the gather/scatter entry points that take their index lists in host memory
// (kvcm_hip_batch_gather_host_idx / kvcm_hip_batch_scatter_host_idx): the one pass over the lists, and the packing of a
// launch's tables into the block that rides in the kernel's arguments. Plain C++, no HIP: kvcm_copy.hip includes it, and
// so do the host sanitizer runs (tests/cpp/sanitize).
#pragma once

#include <stdint.h>

#include "kvcm_hip.h"

namespace kvcm {

// Index tables of one launch, copied into the kernel's argument block: run starts from entry 0, the staging slots
// behind them. 3328 bytes of the 4 KiB an argument block may have.
constexpr int kEmbedInts = 832;
struct EmbeddedIdx {
    int32_t v[kEmbedInts];
};

// Walks the lists once. Checks every token slot against pool_slots (0 = unchecked) and every staging slot against
// staging_slots (0 = only "not negative"), and finds the largest r that divides T such that every block's T slots are
// runs of r consecutive slots: r = gcd(T, every position inside a block where the slot is not its predecessor's + 1).
// A negative slot means "skip this row" and never joins a run, so that nothing but that row is skipped.
inline int32_t walk_host_idx(const int32_t *h_token_idx, const int32_t *h_staging_idx, int32_t B, int32_t T,
                             int64_t pool_slots, int64_t staging_slots, int32_t *run_tokens) {
    const auto gcd = [](uint32_t x, uint32_t y) {
        while (y) {
            const uint32_t t = x % y;
            x = y;
            y = t;
        }
        return x;
    };
    uint32_t r = static_cast<uint32_t>(T);
    const int64_t pool_limit = pool_slots > 0 ? pool_slots : (int64_t{1} << 31);
    for (int32_t b = 0; b < B; ++b) {
        const int32_t *row = h_token_idx + static_cast<int64_t>(b) * T;
        if (row[0] >= pool_limit) {
            return KVCM_ERR_OUT_OF_RANGE;
        }
        for (int32_t j = 1; j < T; ++j) {
            if (row[j] >= pool_limit) {
                return KVCM_ERR_OUT_OF_RANGE;
            }
            // (the sum is formed in 64 bits: a slot of INT32_MAX has no successor)
            if (r > 1 && (row[j - 1] < 0 || row[j] != static_cast<int64_t>(row[j - 1]) + 1)) {
                r = gcd(r, static_cast<uint32_t>(j));
            }
        }
        if (h_staging_idx) {
            const int64_t sb = h_staging_idx[b];
            if (sb < 0 || (staging_slots > 0 && sb >= staging_slots)) {
                return KVCM_ERR_OUT_OF_RANGE;
            }
        } else if (staging_slots > 0 && b >= staging_slots) {
            return KVCM_ERR_OUT_OF_RANGE;
        }
    }
    *run_tokens = static_cast<int32_t>(r);
    return KVCM_OK;
}

// Tables of blocks [b0, b0 + nb) with runs of r slots: emb->v[i * (T / r) + k] = first slot of run k of block b0 + i,
// emb->v[nb * (T / r) + i] = its staging slot. The caller has made sure that nb * (T / r + 1) <= kEmbedInts.
inline void fill_embedded(EmbeddedIdx *emb, const int32_t *h_token_idx, const int32_t *h_staging_idx, int32_t b0,
                          int32_t nb, int32_t T, int32_t r) {
    const int32_t runs = T / r;
    for (int32_t i = 0; i < nb; ++i) {
        const int32_t *row = h_token_idx + static_cast<int64_t>(b0 + i) * T;
        for (int32_t k = 0; k < runs; ++k) {
            emb->v[i * runs + k] = row[k * r];
        }
        emb->v[nb * runs + i] = h_staging_idx ? h_staging_idx[b0 + i] : b0 + i;
    }
}

}  // namespace kvcm
