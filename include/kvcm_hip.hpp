// kvcm_hip.hpp -- header-only C++ convenience layer over the C-ABI of libkvcm_hip.so, for host code that holds its
// data in std::vector the way the reference's manager and client do. Function names and argument meaning follow the
// reference interfaces cited below (paths relative to the reference root).
//
// Unlike the C-ABI underneath, these helpers allocate device memory, copy and WAIT for the stream: they are for
// call sites that want a value back (a server thread answering one RPC, a trace converter, a test), not for the
// asynchronous data path, which calls kvcm_hip_* directly on device buffers.
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <condition_variable>
#include <cstdint>
#include <cstdlib>
#include <mutex>
#include <vector>

#include "kvcm_hip.h"

namespace kvcm {

using TokenIdsVector = std::vector<int64_t>;  // kv_cache_manager/manager/cache_manager.h:55-56
using KeyVector = std::vector<int64_t>;

namespace detail {
// Device buffer that frees itself; empty when the allocation failed.
template <typename T>
struct DeviceArray {
    T *ptr = nullptr;
    explicit DeviceArray(size_t n) {
        if (n > 0 && hipMalloc(reinterpret_cast<void **>(&ptr), n * sizeof(T)) != hipSuccess) {
            ptr = nullptr;
        }
    }
    ~DeviceArray() {
        if (ptr) {
            (void)hipFree(ptr);
        }
    }
    DeviceArray(const DeviceArray &) = delete;
    DeviceArray &operator=(const DeviceArray &) = delete;
};
}  // namespace detail

// GenKeyVector for a batch of requests in one launch: (*keys)[r] == GenKeyVector(requests[r], block_size) of
// kv_cache_manager/manager/cache_manager.cc:76-87. Returns KVCM_OK, a KVCM_ERR_* code or a hipError_t.
inline int32_t GenKeyVectors(const std::vector<TokenIdsVector> &requests, int64_t block_size,
                             std::vector<KeyVector> *keys, hipStream_t stream = nullptr) {
    if (!keys || block_size <= 0 || block_size > INT32_MAX || requests.size() > static_cast<size_t>(INT32_MAX)) {
        return KVCM_ERR_INVALID_ARG;
    }
    const int32_t R = static_cast<int32_t>(requests.size());
    keys->assign(requests.size(), KeyVector());
    std::vector<int64_t> token_offsets(R + 1, 0), key_offsets(R + 1, 0);
    for (int32_t r = 0; r < R; ++r) {
        token_offsets[r + 1] = token_offsets[r] + static_cast<int64_t>(requests[r].size());
        key_offsets[r + 1] = key_offsets[r] + static_cast<int64_t>(requests[r].size()) / block_size;
    }
    const int64_t n_tokens = token_offsets[R], n_keys = key_offsets[R];
    if (n_keys == 0) {
        return KVCM_OK;
    }
    std::vector<int64_t> flat(static_cast<size_t>(n_tokens));
    for (int32_t r = 0; r < R; ++r) {
        std::copy(requests[r].begin(), requests[r].end(), flat.begin() + token_offsets[r]);
    }
    detail::DeviceArray<int64_t> d_tokens(flat.size()), d_toff(token_offsets.size()), d_koff(key_offsets.size()),
        d_keys(static_cast<size_t>(n_keys));
    if (!d_tokens.ptr || !d_toff.ptr || !d_koff.ptr || !d_keys.ptr) {
        return static_cast<int32_t>(hipErrorOutOfMemory);
    }
    hipError_t e = hipMemcpyAsync(d_tokens.ptr, flat.data(), flat.size() * 8, hipMemcpyHostToDevice, stream);
    if (e == hipSuccess) {
        e = hipMemcpyAsync(d_toff.ptr, token_offsets.data(), token_offsets.size() * 8, hipMemcpyHostToDevice, stream);
    }
    if (e == hipSuccess) {
        e = hipMemcpyAsync(d_koff.ptr, key_offsets.data(), key_offsets.size() * 8, hipMemcpyHostToDevice, stream);
    }
    if (e != hipSuccess) {
        return static_cast<int32_t>(e);
    }
    const int32_t rc = kvcm_hip_hash_tokens(d_tokens.ptr, d_toff.ptr, R, static_cast<int32_t>(block_size), 0,
                                            d_keys.ptr, d_koff.ptr, stream);
    if (rc != KVCM_OK) {
        (void)hipStreamSynchronize(stream);
        return rc;
    }
    std::vector<int64_t> flat_keys(static_cast<size_t>(n_keys));
    e = hipMemcpyAsync(flat_keys.data(), d_keys.ptr, flat_keys.size() * 8, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) {
        e = hipStreamSynchronize(stream);
    }
    if (e != hipSuccess) {
        return static_cast<int32_t>(e);
    }
    for (int32_t r = 0; r < R; ++r) {
        (*keys)[r].assign(flat_keys.begin() + key_offsets[r], flat_keys.begin() + key_offsets[r + 1]);
    }
    return KVCM_OK;
}

// One request, the reference's own signature; an empty vector on error or when tokens is shorter than a block.
inline KeyVector GenKeyVector(const TokenIdsVector &tokens, int64_t block_size) {
    std::vector<KeyVector> out;
    if (GenKeyVectors({tokens}, block_size, &out) != KVCM_OK || out.empty()) {
        return {};
    }
    return out[0];
}

// kv_cache_manager/optimizer/trace_converter/trace_util.cc:47-56: one key per element, every key chained on the
// one before.
inline std::vector<int64_t> ApplyPrefixHash(const std::vector<int64_t> &hash_ids) {
    return GenKeyVector(hash_ids, 1);
}

// Number of bytes hashed at each end of an iov: min(min_cal_byte_size, iovs[0].size / 2) -- from the FIRST iov, as
// kv_cache_manager/client/src/internal/sdk/sdk_buffer_check_util.cu:52 takes it. 0 = nothing to do. Also 0 when any
// iov has no base address or is shorter than that: the reference would read out of bounds there.
inline size_t IovCheckBytes(const kvcm_iov_device *iovs_h, size_t n, size_t min_cal_byte_size) {
    if (n == 0 || !iovs_h) {
        return 0;
    }
    const size_t cal = std::min(min_cal_byte_size, iovs_h[0].size / 2);
    for (size_t i = 0; i < n && cal > 0; ++i) {
        if (!iovs_h[i].base || iovs_h[i].size < cal) {
            return 0;
        }
    }
    return cal;
}

// SdkBufferCheckUtil::GetIovsCrc on the caller's buffers (sdk_buffer_check_util.cu:50-69, the five-argument form):
// iovs_d and crcs_d are device arrays with room for iovs_size entries; iovs_h_ptr should be pinned memory (it is
// read by an asynchronous copy). Allocates nothing on the device. Empty result when there is nothing to hash or on
// error.
inline std::vector<uint32_t> GetIovsCrc(const kvcm_iov_device *iovs_h_ptr, size_t iovs_size, kvcm_iov_device *iovs_d,
                                        uint32_t *crcs_d, hipStream_t stream, size_t min_cal_byte_size = 4) {
    const size_t cal = IovCheckBytes(iovs_h_ptr, iovs_size, min_cal_byte_size);
    if (cal == 0 || !iovs_d || !crcs_d || iovs_size > static_cast<size_t>(INT32_MAX)) {
        return {};
    }
    if (hipMemcpyAsync(iovs_d, iovs_h_ptr, iovs_size * sizeof(kvcm_iov_device), hipMemcpyHostToDevice, stream) !=
        hipSuccess) {
        return {};
    }
    if (kvcm_hip_iov_crc32(iovs_d, static_cast<int32_t>(iovs_size), crcs_d, cal, stream) != KVCM_OK) {
        (void)hipStreamSynchronize(stream);
        return {};
    }
    std::vector<uint32_t> crcs(iovs_size);
    if (hipMemcpyAsync(crcs.data(), crcs_d, crcs.size() * 4, hipMemcpyDeviceToHost, stream) != hipSuccess ||
        hipStreamSynchronize(stream) != hipSuccess) {
        return {};
    }
    return crcs;
}

// The one-argument form (sdk_buffer_check_util.cu:71-87): allocates its device buffers for the call. Call sites that
// check every transfer take a cell of SdkBufferCheckPool instead.
inline std::vector<uint32_t> GetIovsCrc(const std::vector<kvcm_iov_device> &iovs_h, size_t min_cal_byte_size = 4,
                                        hipStream_t stream = nullptr) {
    if (IovCheckBytes(iovs_h.data(), iovs_h.size(), min_cal_byte_size) == 0) {
        return {};
    }
    detail::DeviceArray<kvcm_iov_device> d_iovs(iovs_h.size());
    detail::DeviceArray<uint32_t> d_crc(iovs_h.size());
    if (!d_iovs.ptr || !d_crc.ptr) {
        return {};
    }
    return GetIovsCrc(iovs_h.data(), iovs_h.size(), d_iovs.ptr, d_crc.ptr, stream, min_cal_byte_size);
}

// SdkBufferCheckUtil::GetBlocksHash (sdk_buffer_check_util.cc:11-28): one hash per block of iovs_per_block iovs.
inline std::vector<int64_t> GetBlocksHash(const std::vector<kvcm_iov_device> &iovs_h, int32_t iovs_per_block,
                                          size_t min_cal_byte_size = 4, hipStream_t stream = nullptr) {
    const std::vector<uint32_t> crcs = GetIovsCrc(iovs_h, min_cal_byte_size, stream);
    if (crcs.empty() || iovs_per_block <= 0) {
        return {};
    }
    std::vector<int64_t> out(crcs.size() / iovs_per_block);
    if (kvcm_blocks_hash_from_crcs(crcs.data(), static_cast<int64_t>(crcs.size()), iovs_per_block, out.data()) !=
        KVCM_OK) {
        return {};
    }
    return out;
}

// In-batch duplicate detection on block keys: (*first_idx)[i] = smallest j with keys[j] == keys[i]. The batched,
// client-side counterpart of the manager's per-request filter (kv_cache_manager/manager/cache_manager.cc:589-635).
inline int32_t FirstOccurrence(const KeyVector &keys, std::vector<int32_t> *first_idx, hipStream_t stream = nullptr) {
    if (!first_idx) {
        return KVCM_ERR_INVALID_ARG;
    }
    first_idx->assign(keys.size(), 0);
    if (keys.empty()) {
        return KVCM_OK;
    }
    const int64_t n = static_cast<int64_t>(keys.size());
    const int64_t ws_bytes = kvcm_hip_first_occurrence_workspace_bytes(n);
    if (ws_bytes < 0) {
        return static_cast<int32_t>(ws_bytes);
    }
    detail::DeviceArray<int64_t> d_keys(keys.size());
    detail::DeviceArray<int32_t> d_first(keys.size()), d_ws(static_cast<size_t>(ws_bytes / 4));
    if (!d_keys.ptr || !d_first.ptr || !d_ws.ptr) {
        return static_cast<int32_t>(hipErrorOutOfMemory);
    }
    hipError_t e = hipMemcpyAsync(d_keys.ptr, keys.data(), keys.size() * 8, hipMemcpyHostToDevice, stream);
    if (e != hipSuccess) {
        return static_cast<int32_t>(e);
    }
    const int32_t rc = kvcm_hip_first_occurrence(d_keys.ptr, n, d_ws.ptr, ws_bytes, d_first.ptr, nullptr, stream);
    if (rc != KVCM_OK) {
        (void)hipStreamSynchronize(stream);
        return rc;
    }
    e = hipMemcpyAsync(first_idx->data(), d_first.ptr, keys.size() * 4, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) {
        e = hipStreamSynchronize(stream);
    }
    return e == hipSuccess ? KVCM_OK : static_cast<int32_t>(e);
}

// Block files with the reference's layout (kv_cache_manager/client/src/internal/sdk/local_file_sdk.cc:161-364):
// owns a kvcm_file_store. One BlockBuffer per block, as kv_cache_manager/client/include/common.h:116-118.
struct BlockBuffer {
    std::vector<kvcm_iov> iovs;
};
using BlockBuffers = std::vector<BlockBuffer>;

// SdkBufferCheckUtil::GetBlocksHash on the caller's buffers (sdk_buffer_check_util.cc:35-61): whole blocks are taken
// while their iovs fit into max_iov_num (the rest is not checked, :45-47); iovs_h_to_save is host room for
// max_iov_num entries, pinned in a pool cell. All blocks must hold as many iovs as the first.
inline std::vector<int64_t> GetBlocksHash(const BlockBuffers &block_buffers, kvcm_iov_device *iovs_d, uint32_t *crcs_d,
                                          kvcm_iov_device *iovs_h_to_save, size_t max_iov_num, hipStream_t stream,
                                          size_t min_cal_byte_size = 4) {
    if (block_buffers.empty() || block_buffers.front().iovs.empty() || !iovs_h_to_save) {
        return {};
    }
    const size_t iov_num = block_buffers.front().iovs.size();
    size_t n = 0;
    for (const BlockBuffer &b : block_buffers) {
        if (b.iovs.size() != iov_num) {
            return {};
        }
        if (n + iov_num > max_iov_num) {
            break;
        }
        for (const kvcm_iov &iov : b.iovs) {
            iovs_h_to_save[n++] = kvcm_iov_device{iov.base, iov.size};
        }
    }
    const std::vector<uint32_t> crcs = GetIovsCrc(iovs_h_to_save, n, iovs_d, crcs_d, stream, min_cal_byte_size);
    if (crcs.empty()) {
        return {};
    }
    std::vector<int64_t> out(crcs.size() / iov_num);
    if (kvcm_blocks_hash_from_crcs(crcs.data(), static_cast<int64_t>(crcs.size()), static_cast<int32_t>(iov_num),
                                   out.data()) != KVCM_OK) {
        return {};
    }
    return out;
}

// Reusable buffers for the buffer check, so that checking a transfer allocates nothing:
// SdkBufferCheckPool (kv_cache_manager/client/src/internal/sdk/sdk_buffer_check_util.h:43-93, .cc:65-132; used at
// kv_cache_manager/client/src/transfer_client_impl.cc:85-88,129-131,146-148). cell_num cells, each with a pinned host
// table, a device table, a device CRC array (room for max_check_iov_num iovs) and a non-blocking stream of its own at
// the default priority. GetCell() blocks until a cell is free; the handle gives the cell back when it goes out of
// scope.
class SdkBufferCheckPool {
public:
    struct Cell {
        kvcm_iov_device *h_iovs = nullptr;
        kvcm_iov_device *d_iovs = nullptr;
        uint32_t *d_crcs = nullptr;
        hipStream_t stream = nullptr;
    };

    class CellHandle {
    public:
        CellHandle(SdkBufferCheckPool *pool, Cell *cell) : pool_(pool), cell_(cell) {}
        CellHandle(CellHandle &&o) noexcept : pool_(o.pool_), cell_(o.cell_) { o.pool_ = nullptr, o.cell_ = nullptr; }
        CellHandle(const CellHandle &) = delete;
        CellHandle &operator=(const CellHandle &) = delete;
        ~CellHandle() {
            if (pool_ && cell_) {
                pool_->PutCell(cell_);
            }
        }
        Cell *operator->() { return cell_; }
        Cell &operator*() { return *cell_; }
        explicit operator bool() const { return cell_ != nullptr; }

    private:
        SdkBufferCheckPool *pool_;
        Cell *cell_;
    };

    explicit SdkBufferCheckPool(size_t cell_num = 4) : cells_(cell_num) {}
    SdkBufferCheckPool(const SdkBufferCheckPool &) = delete;
    SdkBufferCheckPool &operator=(const SdkBufferCheckPool &) = delete;
    ~SdkBufferCheckPool() {
        for (Cell &c : cells_) {
            if (c.stream) {
                (void)hipStreamSynchronize(c.stream);
                (void)hipStreamDestroy(c.stream);
            }
            if (c.h_iovs) {
                (void)hipHostFree(c.h_iovs);
            }
            if (c.d_iovs) {
                (void)hipFree(c.d_iovs);
            }
            if (c.d_crcs) {
                (void)hipFree(c.d_crcs);
            }
        }
    }

    // Allocates every cell on the current device. false = some allocation failed (what exists is freed by the
    // destructor); the pool then hands out no cells it could not fill.
    bool Init(size_t max_check_iov_num) {
        if (max_check_iov_num == 0 || !free_.empty()) {
            return false;
        }
        max_iov_num_ = max_check_iov_num;
        const size_t iov_bytes = max_check_iov_num * sizeof(kvcm_iov_device), crc_bytes = max_check_iov_num * 4;
        for (Cell &c : cells_) {
            if (hipHostMalloc(reinterpret_cast<void **>(&c.h_iovs), iov_bytes, hipHostMallocDefault) != hipSuccess ||
                hipMalloc(reinterpret_cast<void **>(&c.d_iovs), iov_bytes) != hipSuccess ||
                hipMalloc(reinterpret_cast<void **>(&c.d_crcs), crc_bytes) != hipSuccess ||
                hipStreamCreateWithFlags(&c.stream, hipStreamNonBlocking) != hipSuccess) {
                free_.clear();
                return false;
            }
            free_.push_back(&c);
        }
        return true;
    }

    CellHandle GetCell() {
        std::unique_lock<std::mutex> lock(mutex_);
        cv_.wait(lock, [this] { return !free_.empty(); });
        Cell *c = free_.back();
        free_.pop_back();
        return CellHandle(this, c);
    }

    // GetBlocksHash of `block_buffers` on a cell of this pool: what the transfer client does around every transfer
    // when KVCM_SDK_CHECK is set (transfer_client_impl.cc:127-133).
    std::vector<int64_t> GetBlocksHash(const BlockBuffers &block_buffers, size_t min_cal_byte_size = 4) {
        CellHandle cell = GetCell();
        return kvcm::GetBlocksHash(block_buffers, cell->d_iovs, cell->d_crcs, cell->h_iovs, max_iov_num_, cell->stream,
                                   min_cal_byte_size);
    }

    size_t FreeCells() {
        std::lock_guard<std::mutex> lock(mutex_);
        return free_.size();
    }
    size_t MaxCheckIovNum() const { return max_iov_num_; }

private:
    void PutCell(Cell *c) {
        {
            std::lock_guard<std::mutex> lock(mutex_);
            free_.push_back(c);
        }
        cv_.notify_one();
    }

    std::mutex mutex_;
    std::condition_variable cv_;
    std::vector<Cell> cells_;
    std::vector<Cell *> free_;
    size_t max_iov_num_ = 0;
};

class LocalFileStore {
public:
    explicit LocalFileStore(int64_t byte_size_per_block, int64_t bounce_bytes = 0, bool sync_on_put = true,
                            int32_t io_threads = 0) {
        if (kvcm_file_store_create(byte_size_per_block, bounce_bytes, sync_on_put ? 1 : 0, io_threads, &store_) !=
            KVCM_OK) {
            store_ = nullptr;
        }
        size_ = static_cast<uint64_t>(byte_size_per_block);
    }
    ~LocalFileStore() { kvcm_file_store_destroy(store_); }
    LocalFileStore(const LocalFileStore &) = delete;
    LocalFileStore &operator=(const LocalFileStore &) = delete;
    bool Valid() const { return store_ != nullptr; }

    // All blocks go to the one file `path`; blkids[b] and uri_sizes[b] are the URI parameters of block b
    // (uri_sizes empty = the store's block size).
    int32_t Put(const char *path, const std::vector<uint64_t> &blkids, const std::vector<BlockBuffer> &buffers,
                const std::vector<uint64_t> &uri_sizes = {}) {
        return Call(kvcm_file_store_put, path, blkids, buffers, uri_sizes);
    }
    int32_t Get(const char *path, const std::vector<uint64_t> &blkids, const std::vector<BlockBuffer> &buffers,
                const std::vector<uint64_t> &uri_sizes = {}) {
        return Call(kvcm_file_store_get, path, blkids, buffers, uri_sizes);
    }

private:
    template <typename Fn>
    int32_t Call(Fn fn, const char *path, const std::vector<uint64_t> &blkids, const std::vector<BlockBuffer> &buffers,
                 const std::vector<uint64_t> &uri_sizes) {
        if (!store_ || blkids.size() != buffers.size() || (!uri_sizes.empty() && uri_sizes.size() != blkids.size()) ||
            blkids.size() > static_cast<size_t>(INT32_MAX)) {
            return KVCM_ERR_INVALID_ARG;
        }
        std::vector<uint64_t> sizes = uri_sizes.empty() ? std::vector<uint64_t>(blkids.size(), size_) : uri_sizes;
        std::vector<int32_t> counts;
        std::vector<kvcm_iov> flat;
        for (const BlockBuffer &b : buffers) {
            counts.push_back(static_cast<int32_t>(b.iovs.size()));
            flat.insert(flat.end(), b.iovs.begin(), b.iovs.end());
        }
        return fn(store_, path, blkids.data(), sizes.data(), counts.data(), flat.data(),
                  static_cast<int32_t>(blkids.size()));
    }

    kvcm_file_store *store_ = nullptr;
    uint64_t size_ = 0;
};

}  // namespace kvcm
