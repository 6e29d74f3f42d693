/*
 * kvcm_oracle.h -- CPU restatement of the reference's algorithms for the save/load hot path.
 *
 * TEST INFRASTRUCTURE ONLY. This library is the checker that the HIP path is compared with and the
 * CPU baseline that bench.py times next to it. Nothing in the product (the HIP library, the Python
 * package) may link, load or call it.
 *
 * Each function cites the reference file:line it follows (paths relative to the reference root).
 * Pinning (what makes each function trustworthy) is listed in kvcm_oracle.c's header.
 */
#ifndef KVCM_ORACLE_H
#define KVCM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* hashInt64Func: kv_cache_manager/manager/hash_util.h:8-12 (std::hash<int64_t> is the identity). */
int64_t kvcm_ref_hash_step(int64_t hash, int64_t value);

/* hashInt64Array: kv_cache_manager/manager/hash_util.h:14-24. */
int64_t kvcm_ref_hash_array(int64_t hash, const int64_t *begin, const int64_t *end);

/* GenKeyVector for one request: kv_cache_manager/manager/cache_manager.cc:76-87.
 * Writes n / block_size keys, returns that count. */
int64_t kvcm_ref_gen_key_vector(const int64_t *tokens, int64_t n, int64_t block_size, int64_t seed,
                                int64_t *keys);

/* GenKeyVector over R ragged requests, same argument meaning as kvcm_hip_hash_tokens. */
int32_t kvcm_ref_hash_tokens(const int64_t *tokens, const int64_t *token_offsets, int32_t R,
                             int32_t block_size, int64_t seed, int64_t *keys, const int64_t *key_offsets);
int32_t kvcm_ref_hash_tokens_i32(const int32_t *tokens, const int64_t *token_offsets, int32_t R,
                                 int32_t block_size, int64_t seed, int64_t *keys,
                                 const int64_t *key_offsets);
/* The same, requests split statically over `threads` pthreads (one request per core at a time). */
int32_t kvcm_ref_hash_tokens_mt(const int64_t *tokens, const int64_t *token_offsets, int32_t R,
                                int32_t block_size, int64_t seed, int64_t *keys,
                                const int64_t *key_offsets, int32_t threads);

/* ApplyPrefixHash: kv_cache_manager/optimizer/trace_converter/trace_util.cc:47-56. */
int32_t kvcm_ref_prefix_chain(const int64_t *digests, const int64_t *offsets, int32_t R, int64_t *keys);

/* _sha256_to_int64: kv_cache_manager/py_connector/sglang/connector.py:397-401. */
void kvcm_ref_sha256(const uint8_t *msg, size_t len, uint8_t digest[32]);
int32_t kvcm_ref_sha256_first8_be(const uint8_t *bytes, const int64_t *offsets, int32_t N, int64_t *out);

/* Mirror of kvcm_copy_desc with host pointers everywhere. */
typedef struct kvcm_ref_copy_desc {
    const void *const *ptr_table;
    int32_t P;
    int32_t ptrs_per_entry;
    int64_t entry_stride_bytes;
    void *staging;
    int64_t staging_block_stride_bytes;
    int64_t staging_tile_stride_bytes;
    const int32_t *run_start;
    const int32_t *staging_idx;
    int32_t B;
    int32_t T;
    int32_t run_tokens;
    int32_t slot_limit;
    int64_t row_bytes;
    const void *const *trailer_ptr_table;
    const int32_t *trailer_idx;
    int32_t trailer_bytes;
    int32_t max_workgroups; /* ignored */
} kvcm_ref_copy_desc;

/* kv_cache_batch_gather_kernel / kv_cache_batch_scatter_kernel index algebra
 * (kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:49-98,155-205) and the legacy
 * kernels (gather_scatter_helper.py:10-107), as nested loops with one memcpy per contiguous run --
 * which is also how the reference's CPU copy path moves data: one memcpy per Iov
 * (kv_cache_manager/client/src/internal/sdk/local_file_sdk.cc:326-351,
 *  kv_cache_manager/client/src/internal/sdk/hf3fs_usrbio_client.cc:478-505). */
int32_t kvcm_ref_gather_ex(const kvcm_ref_copy_desc *d);
int32_t kvcm_ref_scatter_ex(const kvcm_ref_copy_desc *d);
/* Work blocks split statically over `threads` pthreads. */
int32_t kvcm_ref_gather_ex_mt(const kvcm_ref_copy_desc *d, int32_t threads);
int32_t kvcm_ref_scatter_ex_mt(const kvcm_ref_copy_desc *d, int32_t threads);

int32_t kvcm_ref_batch_gather(const void *const *ptr_table, int32_t P, void *staging,
                              int64_t staging_block_stride_bytes, const int32_t *token_idx,
                              const int32_t *staging_idx, int32_t B, int32_t T, int64_t row_bytes);
int32_t kvcm_ref_batch_scatter(const void *const *ptr_table, int32_t P, const void *staging,
                               int64_t staging_block_stride_bytes, const int32_t *token_idx,
                               const int32_t *staging_idx, int32_t B, int32_t T, int64_t row_bytes);

/* generate_blocks_idx: kv_cache_manager/py_connector/vllm/v1_connector.py:308-320.
 * Returns 0, or 1 if some token fell beyond n_local blocks (those entries are written as -1). */
int32_t kvcm_ref_generate_blocks_idx(const int32_t *manager_block_idxes, int32_t B,
                                     const int32_t *local_block_ids, int32_t n_local, int32_t T_mgr,
                                     int32_t T_eng, int32_t *out);

typedef struct kvcm_ref_iov {
    const void *base;
    size_t size;
} kvcm_ref_iov;

/* GetIovsCrcDevice: kv_cache_manager/client/src/internal/sdk/sdk_buffer_check_util.cu:10-44. */
int32_t kvcm_ref_iov_crc32(const kvcm_ref_iov *iovs, int32_t n, uint32_t *crc, size_t cal_bytes);

/* GetBlocksHash's fold: kv_cache_manager/client/src/internal/sdk/sdk_buffer_check_util.cc:56-60. */
int32_t kvcm_ref_blocks_hash_from_crcs(const uint32_t *crcs, int64_t n_crcs, int32_t iovs_per_block,
                                       int64_t *out_hashes);

/* In-batch first occurrence of every key (no reference counterpart; the manager's per-request filter is
 * kv_cache_manager/manager/cache_manager.cc:589-635). is_repeat may be NULL. */
int32_t kvcm_ref_first_occurrence(const int64_t *keys, int64_t n, int32_t *first_idx, uint8_t *is_repeat);

/* parse_block_mask_to_save_indices, bool_masks branch: kv_cache_manager/py_connector/vllm/v1_connector.py:835-850. */
int64_t kvcm_ref_mask_to_indices(const uint8_t *mask, const uint8_t *mask2, int64_t n, int32_t *indices);

/* Iov (kv_cache_manager/client/include/common.h:102-110) for the block-file functions; host memory only here. */
typedef struct kvcm_ref_fiov {
    uint8_t type;
    uint8_t ignore;
    void *base;
    size_t size;
} kvcm_ref_fiov;

/* LocalFileSdk::DoPut / DoGet on host iovs: kv_cache_manager/client/src/internal/sdk/local_file_sdk.cc:161-364. */
int32_t kvcm_ref_file_put(const char *path, int64_t bsz, const uint64_t *blkids, const uint64_t *sizes,
                          const int32_t *iov_counts, const kvcm_ref_fiov *iovs, int32_t n_blocks);
int32_t kvcm_ref_file_get(const char *path, int64_t bsz, const uint64_t *blkids, const uint64_t *sizes,
                          const int32_t *iov_counts, const kvcm_ref_fiov *iovs, int32_t n_blocks);

/* Hf3fsUsrbioClient::CopyIovs on host iovs: kv_cache_manager/client/src/internal/sdk/hf3fs_usrbio_client.cc:478-505.
 * Returns the number of bytes the iovs take in the buffer. */
int64_t kvcm_ref_copy_iovs(void *host_buffer, const kvcm_ref_fiov *iovs, int32_t n, int32_t load);

#ifdef __cplusplus
}
#endif
#endif
