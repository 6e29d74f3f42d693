"""MI355X-native save/load hot path of the Tair KVCache Manager connector.

Operators (same names and argument order as the reference's Python operator modules):
    tair_kvcache_amd.kernel.batch_gather_scatter_helper  batch_gather_kv_caches, batch_scatter_kv_caches
    tair_kvcache_amd.kernel.gather_scatter_helper        gather_kv_caches, scatter_kv_caches, CopyBufferAllocator
    tair_kvcache_amd.hashing                             gen_key_vector, hash_tokens, apply_prefix_hash, ...
    tair_kvcache_amd.buffer_check                        get_iovs_crc, get_blocks_hash
    tair_kvcache_amd.connector                           generate_blocks_idx, register_kv_caches, KVCacheInfo,
                                                         MultiResult, DataTransferManager
    tair_kvcache_amd.save_selection                      first_occurrence, mask_to_indices, select_save_indices
    tair_kvcache_amd.local_file_sdk                      StandardUri, LocalFileSdk, LocalFileTransferClient

All device work goes through libkvcm_hip.so (include/kvcm_hip.h); there is no CPU fallback.
"""

__version__ = "0.2.0"
