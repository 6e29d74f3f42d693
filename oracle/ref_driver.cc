// ref_driver.cc -- extern "C" doors onto the REFERENCE's own hash headers, compiled where they lie.
//
// TEST INFRASTRUCTURE ONLY. Built by oracle/Makefile into oracle/_ref/libkvcm_refhash.so when the
// reference tree is present; nothing here restates the hash step: every state update below is a call
// into kv_cache_manager/manager/hash_util.h or kv_cache_manager/common/hash_util.h.
//
// The two loops around those calls restate code that cannot be compiled on its own:
//   GenKeyVector    kv_cache_manager/manager/cache_manager.cc:76-87   (anonymous namespace of a .cc whose
//                   includes need the whole manager build)
//   ApplyPrefixHash kv_cache_manager/optimizer/trace_converter/trace_util.cc:47-56 (same reason)
#include <cstddef>
#include <cstdint>
#include <functional>
#include <vector>

#include "kv_cache_manager/common/hash_util.h"
#include "kv_cache_manager/manager/hash_util.h"

extern "C" {

int64_t kvcm_refsrc_hash_step(int64_t hash, int64_t value) {
    std::hash<int64_t> hasher;
    return kv_cache_manager::hashInt64Func(hasher, hash, value);
}

int64_t kvcm_refsrc_hash_array(int64_t hash, const int64_t *begin, const int64_t *end) {
    return kv_cache_manager::hashInt64Array(hash, begin, end);
}

// cache_manager.cc:76-87 around the real hashInt64Array.
int64_t kvcm_refsrc_gen_key_vector(const int64_t *tokens, int64_t n, int64_t block_size, int64_t *keys) {
    std::vector<int64_t> v(tokens, tokens + n);
    size_t total_blocks = v.size() / block_size;
    int64_t hash = 0;
    for (size_t index = 0; index < total_blocks; index++) {
        auto pos = index * block_size;
        hash = kv_cache_manager::hashInt64Array(hash, v.data() + pos, v.data() + pos + block_size);
        keys[index] = hash;
    }
    return (int64_t)total_blocks;
}

// One request after another, as the manager serves one RPC at a time on a thread.
int32_t kvcm_refsrc_hash_tokens(const int64_t *tokens, const int64_t *token_offsets, int32_t R,
                                int32_t block_size, int64_t *keys, const int64_t *key_offsets) {
    for (int32_t r = 0; r < R; r++) {
        const int64_t *t = tokens + token_offsets[r];
        int64_t n = token_offsets[r + 1] - token_offsets[r];
        int64_t *out = keys + key_offsets[r];
        int64_t hash = 0;
        for (int64_t b = 0; b < n / block_size; b++) {
            hash = kv_cache_manager::hashInt64Array(hash, t + b * block_size, t + (b + 1) * block_size);
            out[b] = hash;
        }
    }
    return 0;
}

// trace_util.cc:47-56 around the real hashInt64Func.
void kvcm_refsrc_prefix_chain(const int64_t *ids, int64_t n, int64_t *keys) {
    int64_t hash = 0;
    std::hash<int64_t> hasher = std::hash<int64_t>();
    for (int64_t i = 0; i < n; i++) {
        hash = kv_cache_manager::hashInt64Func(hasher, hash, ids[i]);
        keys[i] = hash;
    }
}

// sdk_buffer_check_util.cc:58 calls exactly this instantiation.
int64_t kvcm_refsrc_hash_u32_array(uint32_t *begin, uint32_t *end, int64_t hash) {
    return kv_cache_manager::HashUtil::HashIntArray<uint32_t>(begin, end, hash);
}

}  // extern "C"
