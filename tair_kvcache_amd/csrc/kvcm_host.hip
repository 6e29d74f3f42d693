// kvcm_host.hip -- the entry points of libkvcm_hip.so that are host code and nothing else: version, error text and the
// per-block hash over iov CRCs. Kept apart from the kernels so that a plain host compiler can build this file (and
// kvcm_file.hip, kvcm_host_idx.h) for the sanitizer runs of tests/cpp/sanitize.
#include "kvcm_internal.h"

extern "C" {

int32_t kvcm_hip_version(void) { return 200; }  // 0.2.0: host-index gather/scatter added, test hook gone

const char *kvcm_hip_error_string(int32_t code) {
    switch (code) {
        case KVCM_OK:
            return "ok";
        case KVCM_ERR_INVALID_ARG:
            return "invalid argument";
        case KVCM_ERR_ALIGNMENT:
            return "misaligned address or stride";
        case KVCM_ERR_TOO_LARGE:
            return "size exceeds the launch geometry";
        case KVCM_ERR_IO:
            return "file input/output error";
        case KVCM_ERR_OUT_OF_RANGE:
            return "index out of range";
        default:
            return code > 0 ? hipGetErrorString(static_cast<hipError_t>(code)) : "unknown kvcm error";
    }
}

int32_t kvcm_blocks_hash_from_crcs(const uint32_t *crcs, int64_t n_crcs, int32_t iovs_per_block, int64_t *out_hashes) {
    if (iovs_per_block <= 0 || n_crcs < 0 || (n_crcs > 0 && (!crcs || !out_hashes))) {
        return KVCM_ERR_INVALID_ARG;
    }
    int64_t nb = 0;
    for (int64_t off = 0; off + iovs_per_block <= n_crcs; off += iovs_per_block) {
        uint64_t h = 0;
        for (int32_t i = 0; i < iovs_per_block; ++i) {
            h = kvcm::hash_step_preadded(h, static_cast<uint64_t>(crcs[off + i]) + kvcm::kGolden);
        }
        out_hashes[nb++] = static_cast<int64_t>(h);
    }
    return KVCM_OK;
}

}  // extern "C"
