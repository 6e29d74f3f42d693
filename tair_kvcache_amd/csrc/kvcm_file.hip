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
// Get, pread fills one while the other is copied up); a big transfer is shared among a few threads, each with its
// own pair of buffers. Host iovs are written and read in place.
#include <errno.h>
#include <string.h>
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <deque>
#include <functional>
#include <mutex>
#include <string>
#include <thread>
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

// A bounce-buffer-sized piece of a device segment.
struct Chunk {
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
    int32_t io_threads = 1;
    std::mutex mu;
    std::condition_variable lane_freed;
    std::vector<kvcm::Lane *> idle;
    int lanes_alive = 0;
    // puts and gets between entry and return, under `mu`: what kvcm_file_store_destroy waits for before it touches
    // the helper threads or the lanes
    int calls_running = 0;
    std::condition_variable calls_done;

    // Helper threads for big reads: started on first need, at most io_threads - 1, alive until the store is destroyed
    // (a thread's first HIP call costs far more than a 256 MiB read, so they are not started per call).
    std::mutex pool_mu;
    std::condition_variable pool_wake;
    std::deque<std::function<void()>> pool_jobs;
    std::vector<std::thread> pool;
    int pool_idle = 0;
    bool pool_stop = false;
    std::atomic<int> transfers_in_flight{0};

    void submit(std::function<void()> job) {
        {
            std::lock_guard<std::mutex> lock(pool_mu);
            if (!pool_stop) {
                pool_jobs.push_back(std::move(job));
                if (pool_idle == 0 && static_cast<int32_t>(pool.size()) < io_threads - 1) {
                    pool.emplace_back([this] { pool_loop(); });
                }
                pool_wake.notify_one();
                return;
            }
        }
        job();  // the helper threads are being joined: nobody would take the job, so the caller does it itself
    }

    void pool_loop() {
        std::unique_lock<std::mutex> lock(pool_mu);
        for (;;) {
            pool_idle++;
            pool_wake.wait(lock, [this] { return pool_stop || !pool_jobs.empty(); });
            pool_idle--;
            if (pool_jobs.empty()) {
                return;  // pool_stop
            }
            std::function<void()> job = std::move(pool_jobs.front());
            pool_jobs.pop_front();
            lock.unlock();
            job();
            lock.lock();
        }
    }

    void stop_pool() {
        {
            std::lock_guard<std::mutex> lock(pool_mu);
            pool_stop = true;
        }
        pool_wake.notify_all();
        for (std::thread &t : pool) {
            t.join();
        }
        pool.clear();
    }

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
            lane_freed.notify_all();
            return kvcm::hip_code(e);
        }
        *out = lane;
        return KVCM_OK;
    }

    void release(kvcm::Lane *lane) {
        std::lock_guard<std::mutex> lock(mu);
        idle.push_back(lane);
        lane_freed.notify_all();  // a caller waiting for a lane, and the destroyer waiting for all of them
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

// Marks a put or get as running from its first look at the store to its return.
struct CallGuard {
    kvcm_file_store *store;
    explicit CallGuard(kvcm_file_store *s) : store(s) {
        std::lock_guard<std::mutex> lock(store->mu);
        store->calls_running++;
    }
    ~CallGuard() {
        std::lock_guard<std::mutex> lock(store->mu);
        if (--store->calls_running == 0) {
            store->calls_done.notify_all();
        }
    }
    CallGuard(const CallGuard &) = delete;
    CallGuard &operator=(const CallGuard &) = delete;
};

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
            if (offset > limit || iov.size > limit - offset) {  // written so that a huge size cannot wrap around
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

// Device chunks [begin, end) -> file. Chunk k is copied down into bounce[k % 2] while chunk k-1 is being written out.
int32_t put_chunks(Lane *lane, int fd, const Chunk *begin, const Chunk *end) {
    const Chunk *prev = nullptr;
    int prev_slot = 0;
    auto flush = [&](const Chunk *c, int slot) -> int32_t {
        hipError_t e = hipEventSynchronize(lane->done[slot]);
        if (e != hipSuccess) {
            return hip_code(e);
        }
        return write_all(fd, static_cast<const char *>(lane->bounce[slot]), c->size, c->file_offset) ? KVCM_OK
                                                                                                     : KVCM_ERR_IO;
    };
    int k = 0;
    for (const Chunk *c = begin; c != end; ++c, ++k) {
        const int slot = k & 1;
        hipError_t e = hipMemcpyAsync(lane->bounce[slot], c->base, c->size, hipMemcpyDeviceToHost, lane->stream);
        if (e == hipSuccess) {
            e = hipEventRecord(lane->done[slot], lane->stream);
        }
        int32_t rc = hip_code(e);
        if (rc == KVCM_OK && prev) {
            rc = flush(prev, prev_slot);
        }
        if (rc != KVCM_OK) {
            (void)hipStreamSynchronize(lane->stream);
            return rc;
        }
        prev = c;
        prev_slot = slot;
    }
    return prev ? flush(prev, prev_slot) : KVCM_OK;
}

// File -> device chunks [begin, end). Chunk k is read into bounce[k % 2] while chunk k-1 is on its way up.
int32_t get_chunks(Lane *lane, int fd, const Chunk *begin, const Chunk *end) {
    int32_t rc = KVCM_OK;
    int k = 0;
    for (const Chunk *c = begin; c != end && rc == KVCM_OK; ++c, ++k) {
        const int slot = k & 1;
        if (k >= 2) {
            rc = hip_code(hipEventSynchronize(lane->done[slot]));  // the copy that last used this buffer
            if (rc != KVCM_OK) {
                break;
            }
        }
        if (!read_all(fd, static_cast<char *>(lane->bounce[slot]), c->size, c->file_offset)) {
            rc = KVCM_ERR_IO;
            break;
        }
        hipError_t e = hipMemcpyAsync(c->base, lane->bounce[slot], c->size, hipMemcpyHostToDevice, lane->stream);
        if (e == hipSuccess) {
            e = hipEventRecord(lane->done[slot], lane->stream);
        }
        rc = hip_code(e);
    }
    const int32_t tail = hip_code(hipStreamSynchronize(lane->stream));
    return rc != KVCM_OK ? rc : tail;
}

// Moves every device segment, cut into bounce-sized chunks. A big read is shared among up to io_threads threads, each
// with a lane of its own and a contiguous range of the chunks: one thread's pread tops out near 31-36 GiB/s out of the
// page cache, four reach 47-49. A write stays on the calling thread: filling ONE new file is bound inside the kernel
// (page allocation under the file's lock, 9 GiB/s on tmpfs and 18 GiB/s on a disk-backed page cache here) and more
// writers to the same file, through pwrite or a shared mapping, measure the same or lower. Writers of different files
// do scale, which is what concurrent callers give.
int32_t move_device_segments(kvcm_file_store *store, int fd, const std::vector<Segment> &segs, bool put) {
    std::vector<Chunk> chunks;
    for (const Segment &s : segs) {
        if (!s.on_device) {
            continue;
        }
        for (size_t done = 0; done < s.size; done += store->bounce_bytes) {
            chunks.push_back(Chunk{s.base + done, s.file_offset + done, std::min(store->bounce_bytes, s.size - done)});
        }
    }
    if (chunks.empty()) {
        return KVCM_OK;
    }
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) {
        return hip_code(e);
    }
    // Transfers that run at the same time share the helper threads: eight callers are eight movers already.
    struct InFlight {
        std::atomic<int> &n;
        int now;
        explicit InFlight(std::atomic<int> &counter) : n(counter), now(++counter) {}
        ~InFlight() { --n; }
    } in_flight(store->transfers_in_flight);
    const size_t workers =
        put ? 1
            : std::max<size_t>(1, std::min<size_t>(static_cast<size_t>(store->io_threads / in_flight.now),
                                                   chunks.size() / 2));
    std::vector<int32_t> codes(workers, KVCM_OK);
    auto work = [&](size_t w) {
        if (w != 0 && hipSetDevice(device) != hipSuccess) {  // worker 0 is the caller: its device is current
            codes[w] = static_cast<int32_t>(hipErrorInvalidDevice);
            return;
        }
        const size_t lo = chunks.size() * w / workers, hi = chunks.size() * (w + 1) / workers;
        Lane *lane = nullptr;
        int32_t rc = store->acquire(&lane);
        if (rc == KVCM_OK) {
            rc = put ? put_chunks(lane, fd, chunks.data() + lo, chunks.data() + hi)
                     : get_chunks(lane, fd, chunks.data() + lo, chunks.data() + hi);
            store->release(lane);
        }
        codes[w] = rc;
    };
    std::mutex done_mu;
    std::condition_variable done_cv;
    size_t pending = workers - 1;
    for (size_t w = 1; w < workers; w++) {
        store->submit([&, w] {
            work(w);
            std::lock_guard<std::mutex> lock(done_mu);
            if (--pending == 0) {
                done_cv.notify_one();
            }
        });
    }
    work(0);
    {
        std::unique_lock<std::mutex> lock(done_mu);
        done_cv.wait(lock, [&] { return pending == 0; });
    }
    for (int32_t rc : codes) {
        if (rc != KVCM_OK) {
            return rc;
        }
    }
    return KVCM_OK;
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
                               int32_t io_threads, kvcm_file_store **out) {
    if (!out || byte_size_per_block <= 0 || bounce_bytes < 0 || io_threads < 0 || io_threads > 32) {
        return KVCM_ERR_INVALID_ARG;
    }
    kvcm_file_store *s = new kvcm_file_store();
    s->byte_size_per_block = byte_size_per_block;
    s->bounce_bytes = bounce_bytes > 0 ? static_cast<size_t>(bounce_bytes) : (size_t{8} << 20);
    s->sync_on_put = sync_on_put;
    s->io_threads = io_threads > 0 ? io_threads : 4;
    *out = s;
    return KVCM_OK;
}

void kvcm_file_store_destroy(kvcm_file_store *store) {
    if (!store) {
        return;
    }
    {
        // Puts and gets that other threads are still inside of finish first: they may yet hand work to the helper
        // threads and take lanes. (A call that has not reached its first line when this wait ends is the caller's
        // bug: no call may start once destruction has begun.)
        std::unique_lock<std::mutex> lock(store->mu);
        store->calls_done.wait(lock, [store] { return store->calls_running == 0; });
    }
    store->stop_pool();
    {
        std::unique_lock<std::mutex> lock(store->mu);
        // every lane is back by now (a call returns its lanes before it ends); the wait is a second line of defence
        store->lane_freed.wait(lock, [store] { return static_cast<int>(store->idle.size()) == store->lanes_alive; });
        for (kvcm::Lane *lane : store->idle) {
            kvcm_file_store::destroy(lane);
        }
        store->idle.clear();
        store->lanes_alive = 0;
    }
    delete store;
}

int32_t kvcm_file_store_put(kvcm_file_store *store, const char *path, const uint64_t *blkids, const uint64_t *sizes,
                            const int32_t *iov_counts, const kvcm_iov *iovs, int32_t n_blocks) {
    if (!store || !path || !*path || n_blocks <= 0 || !blkids || !sizes || !iov_counts) {
        return KVCM_ERR_INVALID_ARG;
    }
    kvcm::CallGuard running(store);
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
        rc = kvcm::move_device_segments(store, fd, segs, true);
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
    kvcm::CallGuard running(store);
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
        rc = kvcm::move_device_segments(store, fd, segs, false);
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
