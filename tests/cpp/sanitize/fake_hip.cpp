// fake_hip.cpp -- a HOST stand-in for the handful of HIP runtime calls that the library's host code makes
// (tair_kvcache_amd/csrc/kvcm_file.hip, kvcm_host.hip, include/kvcm_hip.hpp), for sanitizer runs on a machine without
// a GPU. Test infrastructure: linked into tests/cpp/sanitize binaries only, never into the library.
//
// "Device" memory is malloc'd host memory. Streams are real queues with a worker thread each: hipMemcpyAsync returns
// at once and the copy happens later, on the stream's thread, in order; hipEventRecord marks a point in that order;
// hipEventSynchronize / hipStreamSynchronize wait for it. So code that touches a bounce buffer before the copy it is
// waiting for has finished is a data race that ThreadSanitizer sees, and a use after free that AddressSanitizer sees --
// which is the point.
#include <hip/hip_runtime_api.h>

#include <atomic>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <mutex>
#include <thread>

#include "fake_hip.h"

namespace {

struct FakeStream {
    std::mutex mu;
    std::condition_variable wake, idle_cv;
    std::deque<std::function<void()>> jobs;
    bool stop = false, busy = false;
    std::thread worker;

    FakeStream() : worker([this] { loop(); }) {}
    ~FakeStream() {
        {
            std::lock_guard<std::mutex> lock(mu);
            stop = true;
        }
        wake.notify_all();
        worker.join();
    }
    void loop() {
        std::unique_lock<std::mutex> lock(mu);
        for (;;) {
            wake.wait(lock, [this] { return stop || !jobs.empty(); });
            if (jobs.empty()) {
                return;
            }
            std::function<void()> job = std::move(jobs.front());
            jobs.pop_front();
            busy = true;
            lock.unlock();
            job();
            lock.lock();
            busy = false;
            if (jobs.empty()) {
                idle_cv.notify_all();
            }
        }
    }
    void push(std::function<void()> job) {
        {
            std::lock_guard<std::mutex> lock(mu);
            jobs.push_back(std::move(job));
        }
        wake.notify_one();
    }
    void drain() {
        std::unique_lock<std::mutex> lock(mu);
        idle_cv.wait(lock, [this] { return jobs.empty() && !busy; });
    }
};

struct FakeEvent {
    std::mutex mu;
    std::condition_variable cv;
    uint64_t recorded = 0, completed = 0;
};

FakeStream *null_stream() {
    static FakeStream *s = new FakeStream();  // lives as long as the process, like the real one
    return s;
}
FakeStream *as_stream(hipStream_t s) { return s ? reinterpret_cast<FakeStream *>(s) : null_stream(); }

std::atomic<int> g_devices{1};
std::atomic<long> g_live_allocs{0};
thread_local int t_device = 0;
std::mutex g_hook_mu;
std::function<void()> g_on_get_device;

}  // namespace

void fake_hip_set_device_count(int n) { g_devices = n; }
long fake_hip_live_allocations() { return g_live_allocs.load(); }
void fake_hip_on_get_device(std::function<void()> fn) {
    std::lock_guard<std::mutex> lock(g_hook_mu);
    g_on_get_device = std::move(fn);
}

void fake_hip_enqueue(void *stream, std::function<void()> job) {
    as_stream(static_cast<hipStream_t>(stream))->push(std::move(job));
}

extern "C" {

hipError_t hipGetDevice(int *device) {
    std::function<void()> hook;
    {
        std::lock_guard<std::mutex> lock(g_hook_mu);
        hook = g_on_get_device;
    }
    if (hook) {
        hook();
    }
    if (g_devices.load() <= 0) {
        return hipErrorNoDevice;
    }
    *device = t_device;
    return hipSuccess;
}

hipError_t hipSetDevice(int device) {
    if (device < 0 || device >= g_devices.load()) {
        return hipErrorInvalidDevice;
    }
    t_device = device;
    return hipSuccess;
}

hipError_t hipGetLastError(void) { return hipSuccess; }
const char *hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "fake hip error"; }

hipError_t hipMalloc(void **ptr, size_t size) {
    *ptr = std::malloc(size ? size : 1);
    if (!*ptr) {
        return hipErrorOutOfMemory;
    }
    g_live_allocs++;
    return hipSuccess;
}
hipError_t hipFree(void *ptr) {
    if (ptr) {
        g_live_allocs--;
    }
    std::free(ptr);
    return hipSuccess;
}
hipError_t hipHostMalloc(void **ptr, size_t size, unsigned int) { return hipMalloc(ptr, size); }
hipError_t hipHostFree(void *ptr) { return hipFree(ptr); }

hipError_t hipStreamCreateWithFlags(hipStream_t *stream, unsigned int) {
    *stream = reinterpret_cast<hipStream_t>(new FakeStream());
    g_live_allocs++;
    return hipSuccess;
}
hipError_t hipStreamDestroy(hipStream_t stream) {
    if (stream) {
        delete reinterpret_cast<FakeStream *>(stream);
        g_live_allocs--;
    }
    return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t stream) {
    as_stream(stream)->drain();
    return hipSuccess;
}

hipError_t hipEventCreateWithFlags(hipEvent_t *event, unsigned int) {
    *event = reinterpret_cast<hipEvent_t>(new FakeEvent());
    g_live_allocs++;
    return hipSuccess;
}
hipError_t hipEventDestroy(hipEvent_t event) {
    if (event) {
        FakeEvent *ev = reinterpret_cast<FakeEvent *>(event);
        {
            // the real runtime keeps a destroyed event alive until its last record has been reached
            std::unique_lock<std::mutex> lock(ev->mu);
            ev->cv.wait(lock, [ev] { return ev->completed >= ev->recorded; });
        }
        delete ev;
        g_live_allocs--;
    }
    return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream) {
    FakeEvent *ev = reinterpret_cast<FakeEvent *>(event);
    uint64_t ticket;
    {
        std::lock_guard<std::mutex> lock(ev->mu);
        ticket = ++ev->recorded;
    }
    as_stream(stream)->push([ev, ticket] {
        std::lock_guard<std::mutex> lock(ev->mu);  // notified under the lock: once it is released the stream's
        if (ticket > ev->completed) {               // thread does not touch the event again, so it may be destroyed
            ev->completed = ticket;
        }
        ev->cv.notify_all();
    });
    return hipSuccess;
}
hipError_t hipEventSynchronize(hipEvent_t event) {
    FakeEvent *ev = reinterpret_cast<FakeEvent *>(event);
    std::unique_lock<std::mutex> lock(ev->mu);
    const uint64_t want = ev->recorded;  // the latest record, as the real call does
    ev->cv.wait(lock, [&] { return ev->completed >= want; });
    return hipSuccess;
}

hipError_t hipMemcpyAsync(void *dst, const void *src, size_t size, hipMemcpyKind, hipStream_t stream) {
    if (!dst || !src) {
        return hipErrorInvalidValue;
    }
    as_stream(stream)->push([dst, src, size] { std::memcpy(dst, src, size); });
    return hipSuccess;
}

}  // extern "C"
