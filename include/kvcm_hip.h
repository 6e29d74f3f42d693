/*
 * kvcm_hip.h -- C-ABI of libkvcm_hip.so: the MI355X (gfx950) save/load hot path of the
 * Tair KVCache Manager connector.
 *
 * Two families of entry points:
 *   - block-key hashing of token-ID sequences (the manager's GenKeyVector / hashInt64Array and its
 *     siblings), batched over requests;
 *   - gather/scatter of paged KV blocks between an engine's per-layer paged cache ("pool") and the
 *     contiguous block-major staging buffers that the storage SDKs read and write.
 *
 * Conventions
 *   - every pointer whose name starts with d_ is DEVICE memory, readable/writable by kernels on the
 *     current HIP device; everything else is host memory;
 *   - all kvcm_hip_* entry points are asynchronous on `stream` (a hipStream_t passed as void*; NULL = null stream),
 *     never synchronise, never allocate and never switch device. With ONE exception they keep no mutable state
 *     inside the library, so they can be called concurrently from many host threads (the reference calls its
 *     kernels from a 32-thread pool: kv_cache_manager/py_connector/vllm/data_transfer.py:80-93). The exception is
 *     kvcm_hip_first_occurrence_static: its table is a device array owned by the library, one per GPU, shared by
 *     every call on that GPU -- calls that overlap on one GPU race (see its prototype);
 *   - the library reads no environment variable per call and exports no switch: the one tuning knob,
 *     KVCM_COPY_XCD_REMAP, is read once when the first copy is launched;
 *   - device buffers passed in must stay alive until `stream` has executed the call;
 *   - the kvcm_file_store_* family at the end is host-side file I/O: it blocks, and it owns streams and pinned
 *     buffers between create and destroy;
 *   - return value: 0 = OK, negative = KVCM_ERR_* (argument rejected, nothing launched),
 *     positive = a hipError_t reported by the launch.
 *
 * Every prototype cites the reference interface it replaces (paths relative to the reference root).
 */
#ifndef KVCM_HIP_H
#define KVCM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *kvcm_stream_t;

#define KVCM_OK 0
#define KVCM_ERR_INVALID_ARG (-1) /* null pointer, non-positive size, inconsistent shape */
#define KVCM_ERR_ALIGNMENT (-2)   /* an address or stride is not aligned as the entry point requires */
#define KVCM_ERR_TOO_LARGE (-3)   /* a size exceeds what the launch geometry can express */
#define KVCM_ERR_IO (-4)          /* a file could not be created, opened, grown, read or written */
#define KVCM_ERR_OUT_OF_RANGE (-5) /* an index in a HOST index list names a slot beyond the size the caller stated */

/* Library version: major*10000 + minor*100 + patch. */
int32_t kvcm_hip_version(void);

/* Text for a return code of this library (negative codes) or of HIP (positive codes). */
const char *kvcm_hip_error_string(int32_t code);

/* ------------------------------------------------------------------------------------------------
 * Block-key hashing
 * ------------------------------------------------------------------------------------------------ */

/*
 * Parent-chained block keys of R token sequences in one launch.
 * Replaces: GenKeyVector(tokens, block_size)  kv_cache_manager/manager/cache_manager.cc:76-87
 *           over hashInt64Array / hashInt64Func kv_cache_manager/manager/hash_util.h:8-24
 * (one call per request in the reference; here R requests per launch).
 *
 * Request r owns tokens d_tokens[d_token_offsets[r] .. d_token_offsets[r+1]) and produces
 * n_r = len_r / block_size keys (floor; a trailing partial block yields no key), written to
 * d_keys[d_key_offsets[r] .. d_key_offsets[r] + n_r). Key i is the running 64-bit state, started at
 * `seed` (the reference uses 0), after folding tokens [0, (i+1)*block_size) with
 *   h <- h XOR (v + 0x9e3779b97f4a7c15 + (h << 12) + (h >> 32))   (int64, arithmetic >>, mod 2^64).
 * d_key_offsets may be NULL when every request has the same length L = token_offsets[1]-[0]; keys of
 * request r then start at r * (L / block_size).
 */
int32_t kvcm_hip_hash_tokens(const int64_t *d_tokens, const int64_t *d_token_offsets, int32_t R,
                             int32_t block_size, int64_t seed, int64_t *d_keys,
                             const int64_t *d_key_offsets, kvcm_stream_t stream);

/* Same function for int32 token IDs (sign-extended to int64 before hashing): engines hold token IDs as
 * int32, the wire format widens them (kv_cache_manager/protocol/protobuf/meta_service.proto:199). */
int32_t kvcm_hip_hash_tokens_i32(const int32_t *d_tokens, const int64_t *d_token_offsets, int32_t R,
                                 int32_t block_size, int64_t seed, int64_t *d_keys,
                                 const int64_t *d_key_offsets, kvcm_stream_t stream);

/*
 * Prefix-chained keys from per-block digests: keys[i] = fold of digests[0..i].
 * Replaces: ApplyPrefixHash  kv_cache_manager/optimizer/trace_converter/trace_util.cc:47-56.
 * Sequence r owns d_digests[d_offsets[r] .. d_offsets[r+1]) and writes the same index range of d_keys.
 */
int32_t kvcm_hip_prefix_chain(const int64_t *d_digests, const int64_t *d_offsets, int32_t R,
                              int64_t *d_keys, kvcm_stream_t stream);

/*
 * int64 keys from strings: big-endian signed value of the first 8 bytes of SHA-256(bytes).
 * Replaces: HiCacheKVCM._sha256_to_int64 / _prepare_block_keys
 *           kv_cache_manager/py_connector/sglang/connector.py:397-415.
 * String i is d_bytes[d_offsets[i] .. d_offsets[i+1]) (already UTF-8 encoded).
 */
int32_t kvcm_hip_sha256_first8_be(const uint8_t *d_bytes, const int64_t *d_offsets, int32_t N,
                                  int64_t *d_out, kvcm_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * Paged-KV gather / scatter
 * ------------------------------------------------------------------------------------------------
 * Pool: P separate arrays ("one per layer and K/V"), array p = rows of `row_bytes` bytes, row s at
 *       d_ptr_table[p] + s * row_bytes (s = token slot). Order of p: layer-major, K before V
 *       (kv_cache_manager/py_connector/vllm/v1_connector.py:405-413).
 * Staging: slots of staging_block_stride_bytes; slot k holds one block as [P][T][row_bytes]
 *       (kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:104), the exact bytes the
 *       storage SDKs put at file offset blkid * location_spec_size.
 * Work block b (b < B) names T token slots and one staging slot d_staging_idx[b]
 * (NULL = slot b). Staging slots not named are left untouched; so are pool rows not named.
 * Scatter with two work blocks that name the same pool row is a data race: callers must not do that.
 * Data are moved as raw bytes; the element type never matters.
 */

/*
 * gather:  staging[sb[b]][p][t][:] <- pool_p[idx[b][t]][:]      for all b < B, p < P, t < T
 * Replaces: batch_gather_kv_caches + kv_cache_batch_gather_kernel
 *           kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:33-136.
 * d_token_idx is int32 [B][T] (token slot numbers), as the reference uploads it (:118).
 * max_workgroups <= 0 fills the device; a positive value caps the grid (the reference's sm_count, :110).
 */
int32_t kvcm_hip_batch_gather(const void *const *d_ptr_table, int32_t P, void *d_staging,
                              int64_t staging_block_stride_bytes, const int32_t *d_token_idx,
                              const int32_t *d_staging_idx, int32_t B, int32_t T, int64_t row_bytes,
                              int32_t max_workgroups, kvcm_stream_t stream);

/*
 * scatter: pool_p[idx[b][t]][:] <- staging[sb[b]][p][t][:]
 * Replaces: batch_scatter_kv_caches + kv_cache_batch_scatter_kernel
 *           kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:139-248.
 */
int32_t kvcm_hip_batch_scatter(const void *const *d_ptr_table, int32_t P, const void *d_staging,
                               int64_t staging_block_stride_bytes, const int32_t *d_token_idx,
                               const int32_t *d_staging_idx, int32_t B, int32_t T, int64_t row_bytes,
                               int32_t max_workgroups, kvcm_stream_t stream);

/*
 * gather / scatter with the index lists in HOST memory -- the form in which the reference's operators receive them
 * (Python lists, turned into tensors and uploaded per call:
 * kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:116-121,223-228; call sites
 * kv_cache_manager/py_connector/vllm/data_transfer.py:139-146,206-213). Same results as kvcm_hip_batch_gather /
 * kvcm_hip_batch_scatter on the uploaded lists. Nothing is uploaded and nothing is allocated: the lists are walked once
 * on the calling thread and travel to the kernel inside its argument block, so they may be freed or overwritten as soon
 * as the call returns, and the call can be captured into a HIP graph. During that walk
 *   - every token slot is checked against pool_slots (the number of token slots of each pool array; 0 = not checked)
 *     and every staging slot against staging_slots (0 = only "not negative" is checked): KVCM_ERR_OUT_OF_RANGE, and
 *     nothing is launched, when one is out of range. A NEGATIVE token slot is not an error: that row is skipped, as in
 *     the device-index entry points;
 *   - when the T slots of every work block turn out to be runs of r consecutive slots (r = T whenever a manager block
 *     is a whole number of engine blocks) the launch takes the block-table form below with run_tokens = r.
 * A call is split into several launches when its tables exceed one argument block (3328 bytes: 416 blocks per launch
 * in block-table form, 48 with 16 unrelated slots per block). KVCM_ERR_TOO_LARGE when a single block has more than
 * 831 runs: upload the list and use the device-index entry points then. h_staging_idx may be NULL (slot b).
 */
int32_t kvcm_hip_batch_gather_host_idx(const void *const *d_ptr_table, int32_t P, void *d_staging,
                                       int64_t staging_block_stride_bytes, int64_t staging_slots,
                                       const int32_t *h_token_idx, const int32_t *h_staging_idx, int32_t B, int32_t T,
                                       int64_t row_bytes, int64_t pool_slots, int32_t max_workgroups,
                                       kvcm_stream_t stream);
int32_t kvcm_hip_batch_scatter_host_idx(const void *const *d_ptr_table, int32_t P, const void *d_staging,
                                        int64_t staging_block_stride_bytes, int64_t staging_slots,
                                        const int32_t *h_token_idx, const int32_t *h_staging_idx, int32_t B, int32_t T,
                                        int64_t row_bytes, int64_t pool_slots, int32_t max_workgroups,
                                        kvcm_stream_t stream);

/*
 * Block-table fast path: the T tokens of work block b are T / run_tokens runs of `run_tokens`
 * consecutive slots; d_run_start is int32 [B][T / run_tokens] and holds the first slot of every run
 * (engine_block_id * engine_block_size + offset). Equal to kvcm_hip_batch_gather on the expanded
 * per-token index that generate_blocks_idx builds
 * (kv_cache_manager/py_connector/vllm/v1_connector.py:308-320), without building it.
 */
int32_t kvcm_hip_paged_gather(const void *const *d_ptr_table, int32_t P, void *d_staging,
                              int64_t staging_block_stride_bytes, const int32_t *d_run_start,
                              int32_t run_tokens, const int32_t *d_staging_idx, int32_t B, int32_t T,
                              int64_t row_bytes, int32_t max_workgroups, kvcm_stream_t stream);

int32_t kvcm_hip_paged_scatter(const void *const *d_ptr_table, int32_t P, const void *d_staging,
                               int64_t staging_block_stride_bytes, const int32_t *d_run_start,
                               int32_t run_tokens, const int32_t *d_staging_idx, int32_t B, int32_t T,
                               int64_t row_bytes, int32_t max_workgroups, kvcm_stream_t stream);

/*
 * General form behind all gather/scatter entry points.
 *
 *  - pool array p lives at d_ptr_table[p / ptrs_per_entry] + (p % ptrs_per_entry) * entry_stride_bytes:
 *    ptrs_per_entry = 1 for a table of P pointers; ptrs_per_entry = 2 with entry_stride_bytes =
 *    total_slots * row_bytes for one [2, total_slots, H] tensor per layer, K then V
 *    (legacy layout, kv_cache_manager/py_connector/kernel/gather_scatter_helper.py:91-97);
 *  - slot_limit > 0: runs whose first slot is >= slot_limit are skipped in both directions
 *    (gather_scatter_helper.py:37-38,88-89); 0 = no limit;
 *  - staging_tile_stride_bytes: distance between tile p and tile p+1 inside a staging slot;
 *    T * row_bytes + trailer_bytes for the packed record;
 *  - trailer: trailer_bytes > 0 appends to every (b, p) tile the bytes
 *    d_trailer_ptr_table[p][d_trailer_idx[b] * trailer_bytes ..] (per-block quantisation scales of an
 *    fp8 cache); on scatter they are written back. d_trailer_idx[b] < 0 skips block b's trailers in both directions
 *    (the staging bytes and the trailer arrays stay as they are). No counterpart in the reference, which has only the
 *    one-pointer-per-layer MLA branch (kv_cache_manager/py_connector/vllm/v1_connector.py:398-403).
 */
typedef struct kvcm_copy_desc {
    const void *const *d_ptr_table;
    int32_t P;
    int32_t ptrs_per_entry;
    int64_t entry_stride_bytes;
    void *d_staging;
    int64_t staging_block_stride_bytes;
    int64_t staging_tile_stride_bytes;
    const int32_t *d_run_start;
    const int32_t *d_staging_idx;
    int32_t B;
    int32_t T;
    int32_t run_tokens;
    int32_t slot_limit;
    int64_t row_bytes;
    const void *const *d_trailer_ptr_table;
    const int32_t *d_trailer_idx;
    int32_t trailer_bytes;
    int32_t max_workgroups;
} kvcm_copy_desc;

int32_t kvcm_hip_gather_ex(const kvcm_copy_desc *desc, kvcm_stream_t stream);
int32_t kvcm_hip_scatter_ex(const kvcm_copy_desc *desc, kvcm_stream_t stream);

/*
 * Token-slot indices of manager blocks on device:
 *   out[b][i] = block_ids[(m_b*T_mgr + i) / T_eng] * T_eng + (m_b*T_mgr + i) % T_eng,  i < T_mgr
 * Replaces: TairKvCacheConnector.generate_blocks_idx
 *           kv_cache_manager/py_connector/vllm/v1_connector.py:308-320 (a Python double loop).
 * n_local = length of d_local_block_ids; a token that falls beyond it (the reference asserts) makes
 * the kernel write -1 for that entry and raise *d_error_flag (int32, may be NULL) to 1.
 */
int32_t kvcm_hip_generate_blocks_idx(const int32_t *d_manager_block_idxes, int32_t B,
                                     const int32_t *d_local_block_ids, int32_t n_local, int32_t T_mgr,
                                     int32_t T_eng, int32_t *d_out, int32_t *d_error_flag,
                                     kvcm_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * Which blocks of a batch have to be saved
 * ------------------------------------------------------------------------------------------------ */

/*
 * In-batch duplicate detection on block keys: d_first_idx[i] = the smallest j with d_keys[j] == d_keys[i]
 * (so d_first_idx[i] == i marks the first occurrence); d_is_repeat (uint8 [n], may be NULL) gets 1 where a smaller
 * index holds the same key, 0 otherwise -- the polarity of the manager's block mask, "true = nothing to save".
 * No counterpart in the reference: there a block that several requests share is filtered by the manager, one
 * StartWriteCache call per request against the metadata index (FilterWriteCache,
 * kv_cache_manager/manager/cache_manager.cc:589-635); this is the batched, client-side form for connectors that
 * compute block_keys themselves (kvcm_hip_hash_tokens) and save a whole batch of requests at once.
 * d_workspace: device scratch of at least kvcm_hip_first_occurrence_workspace_bytes(n) bytes, 4-byte aligned,
 * contents irrelevant before and undefined after. n <= 2^30. The result does not depend on scheduling.
 */
int64_t kvcm_hip_first_occurrence_workspace_bytes(int64_t n);
int32_t kvcm_hip_first_occurrence(const int64_t *d_keys, int64_t n, void *d_workspace, int64_t workspace_bytes,
                                  int32_t *d_first_idx, uint8_t *d_is_repeat, kvcm_stream_t stream);

/*
 * kvcm_hip_first_occurrence without a workspace argument and without any allocation: the table lives in a device
 * array that is part of the library's code object (8 MiB per GPU the library is used on, held until the process
 * ends). No counterpart in the reference. It is for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc. Same results as kvcm_hip_first_occurrence.
 * n <= kvcm_hip_first_occurrence_static_max_keys() = 2^20, KVCM_ERR_TOO_LARGE beyond. The device that is current at
 * the call is the one whose table is used; its address is looked up on the first call per device (a call with n = 0
 * does just that and launches nothing: make it before a capture starts). All calls on one GPU share that GPU's table:
 * calls that overlap on one GPU (two streams, or two threads) race and give undefined results; serialise them, or use
 * kvcm_hip_first_occurrence with a workspace per call.
 */
int64_t kvcm_hip_first_occurrence_static_max_keys(void);
int32_t kvcm_hip_first_occurrence_static(const int64_t *d_keys, int64_t n, int32_t *d_first_idx, uint8_t *d_is_repeat,
                                         kvcm_stream_t stream);

/*
 * Indices of the blocks to save, ascending: every i < n with d_mask[i] == 0 (and d_mask2[i] == 0 when d_mask2 is
 * not NULL) is appended to d_indices (int32, room for n entries); their number goes to *d_count (device int32).
 * Replaces: TairKvCacheConnector.parse_block_mask_to_save_indices, bool_masks branch
 *           kv_cache_manager/py_connector/vllm/v1_connector.py:835-850 ("False = has to be saved"); the offset
 *           branch (:839-842) is the mask that is 1 below the offset.
 * d_mask2 lets the caller combine the manager's mask with d_is_repeat of kvcm_hip_first_occurrence.
 * d_workspace: at least kvcm_hip_mask_to_indices_workspace_bytes(n) bytes, 4-byte aligned. n <= 2^30.
 */
int64_t kvcm_hip_mask_to_indices_workspace_bytes(int64_t n);
int32_t kvcm_hip_mask_to_indices(const uint8_t *d_mask, const uint8_t *d_mask2, int64_t n, void *d_workspace,
                                 int64_t workspace_bytes, int32_t *d_indices, int32_t *d_count,
                                 kvcm_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * Buffer check (debug aid of the transfer client)
 * ------------------------------------------------------------------------------------------------ */

typedef struct kvcm_iov_device {
    const void *base;
    size_t size;
} kvcm_iov_device;

/*
 * Per iov: reflected CRC-32 (poly 0xEDB88320, init 0xFFFFFFFF, final NOT) over the first cal_bytes and
 * then the last cal_bytes bytes of the iov, one running CRC.
 * Replaces: GetIovsCrcDevice  kv_cache_manager/client/src/internal/sdk/sdk_buffer_check_util.cu:21-44
 * (the caller picks cal_bytes = min(KVCM_CHECK_IOV_BYTE_SIZE, iovs[0].size / 2) and skips the launch
 * when it is 0, as sdk_buffer_check_util.cu:50-55 does).
 * Contract for an iov with base == NULL or size < cal_bytes (the reference reads out of bounds there, so there is no
 * behaviour to match): the kernel reads nothing of it and writes d_crc[i] = 0. Because 0 is also a valid CRC, a
 * caller that cannot rule such iovs out validates them on the host before the launch: kvcm::IovCheckBytes
 * (kvcm_hip.hpp) returns 0 = "check nothing" for the whole call, the Python layer raises ValueError.
 */
int32_t kvcm_hip_iov_crc32(const kvcm_iov_device *d_iovs, int32_t n, uint32_t *d_crc,
                           size_t cal_bytes, kvcm_stream_t stream);

/*
 * Host helper, no device work: per block, the hashInt64 chain (seed 0) over the block's
 * `iovs_per_block` CRCs, each zero-extended to 64 bits.
 * Replaces: the loop at kv_cache_manager/client/src/internal/sdk/sdk_buffer_check_util.cc:56-60 over
 * HashUtil::HashIntArray<uint32_t>  kv_cache_manager/common/hash_util.h:17-25.
 */
int32_t kvcm_blocks_hash_from_crcs(const uint32_t *crcs, int64_t n_crcs, int32_t iovs_per_block,
                                   int64_t *out_hashes);

/* ------------------------------------------------------------------------------------------------
 * Staging slots <-> block files (host code; the step after gather and before scatter)
 * ------------------------------------------------------------------------------------------------ */

#define KVCM_MEMORY_CPU 0
#define KVCM_MEMORY_GPU 1

/* One contiguous piece of a block, in host or device memory.
 * Mirrors: struct Iov  kv_cache_manager/client/include/common.h:102-110 (MemoryType :94-97). */
typedef struct kvcm_iov {
    uint8_t type;   /* KVCM_MEMORY_CPU or KVCM_MEMORY_GPU */
    uint8_t ignore; /* non-zero: skip the bytes, still advance the file offset */
    void *base;     /* NULL is skipped like an ignored iov */
    size_t size;
} kvcm_iov;

typedef struct kvcm_file_store kvcm_file_store;

/*
 * Replaces: LocalFileSdk::Init  kv_cache_manager/client/src/internal/sdk/local_file_sdk.cc:68-85.
 * byte_size_per_block must be positive. bounce_bytes = size of each pinned bounce buffer for device iovs (0 = 8 MiB);
 * they, and a stream, are created on the first call that meets a device iov, per concurrent caller (at most 64), and
 * live until the store is destroyed. sync_on_put != 0 ends every put with fdatasync, the counterpart of the
 * reference's msync(MS_SYNC) (:362). io_threads (0 = 4, at most 32) = threads that share the device iovs of ONE
 * get, each with its own stream and buffers: a single thread is bound by pread, not by the link (a put stays on the
 * calling thread: more writers to one new file gain nothing inside the kernel). A store may be used from many threads
 * at once. This family of entry points does allocate and does block: it is file I/O.
 */
int32_t kvcm_file_store_create(int64_t byte_size_per_block, int64_t bounce_bytes, int32_t sync_on_put,
                               int32_t io_threads, kvcm_file_store **out);
/* Waits for puts and gets that are still running on other threads to hand back their streams and buffers, then frees
 * everything. No call may START on a store once its destruction has begun. */
void kvcm_file_store_destroy(kvcm_file_store *store);

/*
 * Writes n_blocks blocks into ONE file: block b goes to byte offset blkids[b] * byte_size_per_block, its
 * iov_counts[b] iovs (consecutive entries of `iovs`) back to back from there. The file and its parent directories
 * are created when missing and the file is grown to (max blkid + 1) * byte_size_per_block, never shrunk.
 * sizes[b] is the `size` parameter of the block's URI and must equal byte_size_per_block; an iov that would reach
 * beyond the grown size is refused. Everything is checked before the first byte moves.
 * Replaces: LocalFileSdk::Alloc + DoPut  local_file_sdk.cc:136-159,262-364 for one path group of Put (:115-133).
 * Returns KVCM_OK, KVCM_ERR_INVALID_ARG (the reference's ER_INVALID_PARAMS cases), KVCM_ERR_IO
 * (ER_FILE_IO_ERROR cases) or a positive hipError_t.
 */
int32_t kvcm_file_store_put(kvcm_file_store *store, const char *path, const uint64_t *blkids, const uint64_t *sizes,
                            const int32_t *iov_counts, const kvcm_iov *iovs, int32_t n_blocks);

/*
 * Reads n_blocks blocks of ONE file into their iovs; the inverse of put. The file must exist; an iov that would reach
 * beyond its end is refused (local_file_sdk.cc:221-224). Returns when the data are in place (device iovs included).
 * Replaces: LocalFileSdk::DoGet  local_file_sdk.cc:161-260 for one path group of Get (:89-103).
 */
int32_t kvcm_file_store_get(kvcm_file_store *store, const char *path, const uint64_t *blkids, const uint64_t *sizes,
                            const int32_t *iov_counts, const kvcm_iov *iovs, int32_t n_blocks);

/*
 * iovs <-> one contiguous host buffer (the I/O buffer a storage client reads from or writes into): the pieces lie back
 * to back in the buffer in iov order; IGNORED iovs take no room in it (unlike in a block file).
 * load = 0 packs the iovs into the buffer, load != 0 unpacks the buffer into the iovs. Device iovs are copied
 * asynchronously on `stream` and the call returns after the stream has been synchronised, as the reference does; host
 * iovs are memcpy'd. A pinned host buffer gives full-speed copies; a pageable one works.
 * Replaces: Hf3fsUsrbioClient::CopyIovs  kv_cache_manager/client/src/internal/sdk/hf3fs_usrbio_client.cc:478-505
 *           over Hf3fsCudaUtil            kv_cache_manager/client/src/internal/sdk/hf3fs_cuda_util.h:21-79.
 * Returns KVCM_ERR_INVALID_ARG when the pieces do not fit into host_buffer_size (nothing is copied then).
 */
int32_t kvcm_copy_iovs(void *host_buffer, size_t host_buffer_size, const kvcm_iov *iovs, int32_t n, int32_t load,
                       kvcm_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* KVCM_HIP_H */
