// kvcm_file.hip -- the hop between staging slots and block files, host code only (no kernels).
//
// Follows LocalFileSdk (kv_cache_manager/client/src/internal/sdk/local_file_sdk.cc): block `blkid` of a file lives at
// byte offset blkid * byte_size_per_block, a block's iovs lie back to back from there, ignored or null iovs advance the
// offset without moving bytes, Put grows the file to (max blkid + 1) * byte_size_per_block, Get refuses iovs that
// reach past the end of the file.
//
// What is different is how bytes of a DEVICE iov reach the file. The reference maps the file, registers the mapping
// with the GPU runtime and issues one asynchronous copy per iov into it (:237, :345). Registering memory that already
// exists is not available on the MI355X hosts this library targets, so device iovs go through pinned bounce buffers
// allocated as such: neighbouring iovs that are contiguous both in HBM and in the file are merged into segments (a
// staging slot is one segment, a run of slots with consecutive blkids too), every segment is cut into bounce-sized
// chunks, and the copy engine fills one bounce buffer while the host writes the other one out with pwrite (or, on
// Get, pread fills one while the other is copied up). Host iovs are written and read in place.
#include <errno.h>
#include <string.h>
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <condition_variable>
#include <mutex>
#include <string>
#include <vector>

#include "kvcm_internal.h"

namespace kvcm {
namespace {

constexpr int kMaxLanes = 64;

// One caller at a time: a stream, two pinned bounce buffers and the events that say when each one is free again.
struct Lane {
    int device = -1;
    hipStream_t stream = nullptr;
    void *bounce[2] = {nullptr, nullptr};
    hipEvent_t done[2] = {nullptr, nullptr};
};

struct Segment {
    bool on_device;
    char *base;
    uint64_t file_offset;
    size_t size;
};

int32_t hip_code(hipError_t e) { return e == hipSuccess ? KVCM_OK : static_cast<int32_t>(e); }

bool write_all(int fd, const char *src, size_t size, uint64_t offset) {
    while (size > 0) {
        ssize_t w = pwrite(fd, src, size, static_cast<off_t>(offset));
        if (w < 0) {
            if (errno == EINTR) {
                continue;
            }
            return false;
        }
        src += w;
        offset += static_cast<uint64_t>(w);
        size -= static_cast<size_t>(w);
    }
    return true;
}

bool read_all(int fd, char *dst, size_t size, uint64_t offset) {
    while (size > 0) {
        ssize_t r = pread(fd, dst, size, static_cast<off_t>(offset));
        if (r < 0) {
            if (errno == EINTR) {
                continue;
            }
            return false;
        }
        if (r == 0) {
            return false;  // the file shrank under us
        }
        dst += r;
        offset += static_cast<uint64_t>(r);
        size -= static_cast<size_t>(r);
    }
    return true;
}

bool make_parent_dirs(const std::string &path) {
    for (size_t pos = path.find('/', 1); pos != std::string::npos; pos = path.find('/', pos + 1)) {
        std::string dir = path.substr(0, pos);
        if (mkdir(dir.c_str(), 0755) != 0 && errno != EEXIST) {
            return false;
        }
    }
    return true;
}

}  // namespace
}  // namespace kvcm

struct kvcm_file_store {
    int64_t byte_size_per_block = 0;
    size_t bounce_bytes = 0;
    int32_t sync_on_put = 1;
    std::mutex mu;
    std::condition_variable lane_freed;
    std::vector<kvcm::Lane *> idle;
    int lanes_alive = 0;

    // A lane of the current device; created on first need, so a store that only ever sees host iovs never touches HIP.
    int32_t acquire(kvcm::Lane **out) {
        int device = -1;
        hipError_t e = hipGetDevice(&device);
        if (e != hipSuccess) {
            return kvcm::hip_code(e);
        }
        std::unique_lock<std::mutex> lock(mu);
        for (;;) {
            for (size_t i = 0; i < idle.size(); i++) {
                if (idle[i]->device == device) {
                    *out = idle[i];
                    idle.erase(idle.begin() + static_cast<long>(i));
                    return KVCM_OK;
                }
            }
            if (lanes_alive < kvcm::kMaxLanes) {
                break;
            }
            lane_freed.wait(lock);
        }
        lanes_alive++;
        lock.unlock();
        kvcm::Lane *lane = new kvcm::Lane();
        lane->device = device;
        e = hipStreamCreateWithFlags(&lane->stream, hipStreamNonBlocking);
        for (int k = 0; k < 2 && e == hipSuccess; k++) {
            e = hipHostMalloc(&lane->bounce[k], bounce_bytes, hipHostMallocDefault);
            if (e == hipSuccess) {
                e = hipEventCreateWithFlags(&lane->done[k], hipEventDisableTiming);
            }
        }
        if (e != hipSuccess) {
            destroy(lane);
            lock.lock();
            lanes_alive--;
            lane_freed.notify_one();
            return kvcm::hip_code(e);
        }
        *out = lane;
        return KVCM_OK;
    }

    void release(kvcm::Lane *lane) {
        std::lock_guard<std::mutex> lock(mu);
        idle.push_back(lane);
        lane_freed.notify_one();
    }

    static void destroy(kvcm::Lane *lane) {
        for (int k = 0; k < 2; k++) {
            if (lane->done[k]) {
                (void)hipEventDestroy(lane->done[k]);
            }
            if (lane->bounce[k]) {
                (void)hipHostFree(lane->bounce[k]);
            }
        }
        if (lane->stream) {
            (void)hipStreamDestroy(lane->stream);
        }
        delete lane;
    }
};

namespace kvcm {
namespace {

// Validation and layout shared by Put and Get (local_file_sdk.cc:197-252, 317-359): returns the byte ranges to
// move, merged where both sides are contiguous. `limit` is the size no iov may reach beyond.
int32_t plan_segments(const kvcm_file_store *store, const uint64_t *blkids, const uint64_t *sizes,
                      const int32_t *iov_counts, const kvcm_iov *iovs, int32_t n_blocks, uint64_t limit,
                      std::vector<Segment> *out) {
    const uint64_t bsz = static_cast<uint64_t>(store->byte_size_per_block);
    int64_t first = 0;
    for (int32_t b = 0; b < n_blocks; b++) {
        if (sizes[b] != bsz || iov_counts[b] < 0 || (iov_counts[b] > 0 && !iovs)) {
            return KVCM_ERR_INVALID_ARG;
        }
        if (blkids[b] >= (uint64_t{1} << 62) / bsz) {
            return KVCM_ERR_TOO_LARGE;
        }
        uint64_t offset = blkids[b] * bsz;
        for (int32_t k = 0; k < iov_counts[b]; k++) {
            const kvcm_iov &iov = iovs[first + k];
            if (offset + iov.size > limit) {
                return KVCM_ERR_INVALID_ARG;
            }
            if (!iov.ignore && iov.base && iov.size > 0) {
                if (iov.type != KVCM_MEMORY_CPU && iov.type != KVCM_MEMORY_GPU) {
                    return KVCM_ERR_INVALID_ARG;
                }
                const bool dev = iov.type == KVCM_MEMORY_GPU;
                char *base = static_cast<char *>(iov.base);
                if (!out->empty() && out->back().on_device == dev && out->back().base + out->back().size == base &&
                    out->back().file_offset + out->back().size == offset) {
                    out->back().size += iov.size;
                } else {
                    out->push_back(Segment{dev, base, offset, iov.size});
                }
            }
            offset += iov.size;
        }
        first += iov_counts[b];
    }
    return KVCM_OK;
}

// Device segments -> file. Chunk k is copied down into bounce[k % 2] while chunk k-1 is being written out.
int32_t put_device_segments(kvcm_file_store *store, Lane *lane, int fd, const std::vector<Segment> &segs) {
    struct Pending {
        bool valid = false;
        int slot = 0;
        uint64_t file_offset = 0;
        size_t size = 0;
    } prev;
    int k = 0;
    auto flush = [&](const Pending &p) -> int32_t {
        hipError_t e = hipEventSynchronize(lane->done[p.slot]);
        if (e != hipSuccess) {
            return hip_code(e);
        }
        return write_all(fd, static_cast<const char *>(lane->bounce[p.slot]), p.size, p.file_offset) ? KVCM_OK
                                                                                                     : KVCM_ERR_IO;
    };
    for (const Segment &s : segs) {
        if (!s.on_device) {
            continue;
        }
        for (size_t done = 0; done < s.size; done += store->bounce_bytes, k++) {
            Pending cur;
            cur.valid = true;
            cur.slot = k & 1;
            cur.size = std::min(store->bounce_bytes, s.size - done);
            cur.file_offset = s.file_offset + done;
            hipError_t e = hipMemcpyAsync(lane->bounce[cur.slot], s.base + done, cur.size, hipMemcpyDeviceToHost,
                                          lane->stream);
            if (e == hipSuccess) {
                e = hipEventRecord(lane->done[cur.slot], lane->stream);
            }
            if (e != hipSuccess) {
                (void)hipStreamSynchronize(lane->stream);
                return hip_code(e);
            }
            if (prev.valid) {
                int32_t rc = flush(prev);
                if (rc != KVCM_OK) {
                    (void)hipStreamSynchronize(lane->stream);
                    return rc;
                }
            }
            prev = cur;
        }
    }
    return prev.valid ? flush(prev) : KVCM_OK;
}

// File -> device segments. Chunk k is read into bounce[k % 2] while chunk k-1 is on its way up.
int32_t get_device_segments(kvcm_file_store *store, Lane *lane, int fd, const std::vector<Segment> &segs) {
    int k = 0;
    int32_t rc = KVCM_OK;
    for (const Segment &s : segs) {
        if (!s.on_device) {
            continue;
        }
        for (size_t done = 0; done < s.size && rc == KVCM_OK; done += store->bounce_bytes, k++) {
            const int slot = k & 1;
            const size_t size = std::min(store->bounce_bytes, s.size - done);
            if (k >= 2) {
                rc = hip_code(hipEventSynchronize(lane->done[slot]));  // the copy that last used this buffer
                if (rc != KVCM_OK) {
                    break;
                }
            }
            if (!read_all(fd, static_cast<char *>(lane->bounce[slot]), size, s.file_offset + done)) {
                rc = KVCM_ERR_IO;
                break;
            }
            hipError_t e = hipMemcpyAsync(s.base + done, lane->bounce[slot], size, hipMemcpyHostToDevice, lane->stream);
            if (e == hipSuccess) {
                e = hipEventRecord(lane->done[slot], lane->stream);
            }
            rc = hip_code(e);
        }
        if (rc != KVCM_OK) {
            break;
        }
    }
    int32_t tail = hip_code(hipStreamSynchronize(lane->stream));
    return rc != KVCM_OK ? rc : tail;
}

bool any_device(const std::vector<Segment> &segs) {
    for (const Segment &s : segs) {
        if (s.on_device) {
            return true;
        }
    }
    return false;
}

}  // namespace
}  // namespace kvcm

extern "C" {

int32_t kvcm_file_store_create(int64_t byte_size_per_block, int64_t bounce_bytes, int32_t sync_on_put,
                               kvcm_file_store **out) {
    if (!out || byte_size_per_block <= 0 || bounce_bytes < 0) {
        return KVCM_ERR_INVALID_ARG;
    }
    kvcm_file_store *s = new kvcm_file_store();
    s->byte_size_per_block = byte_size_per_block;
    s->bounce_bytes = bounce_bytes > 0 ? static_cast<size_t>(bounce_bytes) : (size_t{8} << 20);
    s->sync_on_put = sync_on_put;
    *out = s;
    return KVCM_OK;
}

void kvcm_file_store_destroy(kvcm_file_store *store) {
    if (!store) {
        return;
    }
    for (kvcm::Lane *lane : store->idle) {
        kvcm_file_store::destroy(lane);
    }
    delete store;
}

int32_t kvcm_file_store_put(kvcm_file_store *store, const char *path, const uint64_t *blkids, const uint64_t *sizes,
                            const int32_t *iov_counts, const kvcm_iov *iovs, int32_t n_blocks) {
    if (!store || !path || !*path || n_blocks <= 0 || !blkids || !sizes || !iov_counts) {
        return KVCM_ERR_INVALID_ARG;
    }
    const uint64_t bsz = static_cast<uint64_t>(store->byte_size_per_block);
    uint64_t required = 0;
    for (int32_t b = 0; b < n_blocks; b++) {
        if (blkids[b] >= (uint64_t{1} << 62) / bsz) {
            return KVCM_ERR_TOO_LARGE;
        }
        required = std::max(required, (blkids[b] + 1) * bsz);
    }
    std::vector<kvcm::Segment> segs;
    int32_t rc = kvcm::plan_segments(store, blkids, sizes, iov_counts, iovs, n_blocks, required, &segs);
    if (rc != KVCM_OK) {
        return rc;
    }
    if (!kvcm::make_parent_dirs(path)) {
        return KVCM_ERR_IO;
    }
    int fd = open(path, O_RDWR | O_CREAT, 0644);
    if (fd < 0) {
        return KVCM_ERR_IO;
    }
    int fa = posix_fallocate(fd, 0, static_cast<off_t>(required));  // grows, never shrinks
    if (fa != 0) {
        struct stat st;
        if (fstat(fd, &st) != 0 ||
            (static_cast<uint64_t>(st.st_size) < required && ftruncate(fd, static_cast<off_t>(required)) != 0)) {
            close(fd);
            return KVCM_ERR_IO;
        }
    }
    for (const kvcm::Segment &s : segs) {
        if (!s.on_device && !kvcm::write_all(fd, s.base, s.size, s.file_offset)) {
            rc = KVCM_ERR_IO;
            break;
        }
    }
    if (rc == KVCM_OK && kvcm::any_device(segs)) {
        kvcm::Lane *lane = nullptr;
        rc = store->acquire(&lane);
        if (rc == KVCM_OK) {
            rc = kvcm::put_device_segments(store, lane, fd, segs);
            store->release(lane);
        }
    }
    if (rc == KVCM_OK && store->sync_on_put && fdatasync(fd) != 0) {
        rc = KVCM_ERR_IO;
    }
    close(fd);
    return rc;
}

int32_t kvcm_file_store_get(kvcm_file_store *store, const char *path, const uint64_t *blkids, const uint64_t *sizes,
                            const int32_t *iov_counts, const kvcm_iov *iovs, int32_t n_blocks) {
    if (!store || !path || !*path || n_blocks <= 0 || !blkids || !sizes || !iov_counts) {
        return KVCM_ERR_INVALID_ARG;
    }
    int fd = open(path, O_RDONLY);
    if (fd < 0) {
        return KVCM_ERR_IO;
    }
    struct stat st;
    if (fstat(fd, &st) != 0) {
        close(fd);
        return KVCM_ERR_IO;
    }
    std::vector<kvcm::Segment> segs;
    int32_t rc = kvcm::plan_segments(store, blkids, sizes, iov_counts, iovs, n_blocks,
                                     static_cast<uint64_t>(st.st_size), &segs);
    for (size_t i = 0; rc == KVCM_OK && i < segs.size(); i++) {
        const kvcm::Segment &s = segs[i];
        if (!s.on_device && !kvcm::read_all(fd, s.base, s.size, s.file_offset)) {
            rc = KVCM_ERR_IO;
        }
    }
    if (rc == KVCM_OK && kvcm::any_device(segs)) {
        kvcm::Lane *lane = nullptr;
        rc = store->acquire(&lane);
        if (rc == KVCM_OK) {
            rc = kvcm::get_device_segments(store, lane, fd, segs);
            store->release(lane);
        }
    }
    close(fd);
    return rc;
}

int32_t kvcm_copy_iovs(void *host_buffer, size_t host_buffer_size, const kvcm_iov *iovs, int32_t n, int32_t load,
                       kvcm_stream_t stream) {
    if (n < 0 || (n > 0 && (!iovs || !host_buffer))) {
        return KVCM_ERR_INVALID_ARG;
    }
    size_t total = 0;
    for (int32_t i = 0; i < n; i++) {
        if (iovs[i].ignore) {
            continue;
        }
        if (iovs[i].type != KVCM_MEMORY_CPU && iovs[i].type != KVCM_MEMORY_GPU) {
            return KVCM_ERR_INVALID_ARG;
        }
        if (iovs[i].size > host_buffer_size - total) {
            return KVCM_ERR_INVALID_ARG;
        }
        total += iovs[i].size;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    char *buffer = static_cast<char *>(host_buffer);
    size_t offset = 0;
    bool device = false;
    hipError_t e = hipSuccess;
    for (int32_t i = 0; i < n && e == hipSuccess; i++) {
        const kvcm_iov &iov = iovs[i];
        if (iov.ignore) {
            continue;
        }
        if (iov.base && iov.size > 0) {
            if (iov.type == KVCM_MEMORY_GPU) {
                device = true;
                e = load ? hipMemcpyAsync(iov.base, buffer + offset, iov.size, hipMemcpyHostToDevice, s)
                         : hipMemcpyAsync(buffer + offset, iov.base, iov.size, hipMemcpyDeviceToHost, s);
            } else if (load) {
                memcpy(iov.base, buffer + offset, iov.size);
            } else {
                memcpy(buffer + offset, iov.base, iov.size);
            }
        }
        offset += iov.size;
    }
    if (device) {
        hipError_t sync = hipStreamSynchronize(s);
        if (e == hipSuccess) {
            e = sync;
        }
    }
    return kvcm::hip_code(e);
}

}  // extern "C"
