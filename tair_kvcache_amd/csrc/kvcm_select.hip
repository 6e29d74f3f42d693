// kvcm_select.hip -- which blocks of a batch have to be moved: first occurrences of block keys inside a
// batch of requests, and the ascending index list of the blocks a mask leaves to save.
//
// The reference decides this on the host: the manager answers StartWriteCache with a block mask and the connector
// turns it into a Python list (kv_cache_manager/py_connector/vllm/v1_connector.py:835-850); requests of one batch that
// share a prefix are not compared with each other at all. Here both steps stay on the device, next to the keys
// (kvcm_hip_hash_tokens) and to the index kernels that consume the list.
//
// Small integer kernels, nowhere near a bandwidth bound: n is the number of block keys of a batch (thousands).
#include <atomic>
#include <mutex>

#include "kvcm_internal.h"

namespace kvcm {
namespace {

// Table of kvcm_hip_first_occurrence_static: room for 2^20 keys (capacity 2 n, one int32 per slot = 8 MiB).
// Every device that the library runs on holds its own copy, at its own address, until the process ends.
constexpr int64_t kStaticMaxKeys = int64_t{1} << 20;
constexpr int64_t kStaticCapacity = 2 * kStaticMaxKeys;
static __device__ __align__(256) int32_t scratch[kStaticCapacity];

// Device address of `scratch` per device: in host code the array's name is only a handle for the runtime's symbol
// calls, never an address a kernel may be given.
constexpr int kMaxDevices = 64;
std::atomic<int32_t *> g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

// The current device's copy of `scratch`; looked up once per device. Returns a kvcm / HIP code.
int32_t static_scratch(int32_t **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        return static_cast<int32_t>(e);
    }
    if (dev < 0 || dev >= kMaxDevices) {
        return KVCM_ERR_TOO_LARGE;
    }
    int32_t *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> guard(g_scratch_mutex);
        p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (!p) {
            void *addr = nullptr;
            e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
            if (e != hipSuccess) {
                return static_cast<int32_t>(e);
            }
            if (!addr) {
                return static_cast<int32_t>(hipErrorInvalidSymbol);
            }
            p = static_cast<int32_t *>(addr);
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return KVCM_OK;
}

constexpr int kSelThreads = 1024;  // 16 waves: one workgroup scans 1024 flags or counts per pass
constexpr int kSelWaves = kSelThreads / 64;

__device__ inline int32_t table_load(const int32_t *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t *__restrict__ p, int64_t n, int32_t v) {
    int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

// Open addressing, linear probing, one int32 per slot: -1 = empty, otherwise an index whose key owns the slot.
// A slot claimed for key K is only ever lowered (atomicMin) by indices that hold the same K, so whatever index a
// probe reads from a slot names that slot's key; after the launch the slot holds the smallest such index.
__global__ __launch_bounds__(256) void insert_kernel(const int64_t *__restrict__ keys, int32_t n,
                                                     int32_t *table, uint32_t mask, int shift,
                                                     int32_t *__restrict__ slot_of) {
    int32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) {
        return;
    }
    const int64_t k = keys[i];
    uint32_t s = static_cast<uint32_t>((static_cast<uint64_t>(k) * kGolden) >> shift) & mask;
    for (;;) {
        int32_t o = table_load(table + s);
        if (o < 0) {
            o = atomicCAS(table + s, -1, i);
            if (o < 0) {
                break;  // claimed
            }
        }
        if (keys[o] == k) {
            atomicMin(table + s, i);
            break;
        }
        s = (s + 1) & mask;
    }
    slot_of[i] = static_cast<int32_t>(s);
}

__global__ __launch_bounds__(256) void resolve_kernel(int32_t *__restrict__ first_idx, const int32_t *__restrict__ table,
                                                      int32_t n, uint8_t *__restrict__ is_repeat) {
    int32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) {
        return;
    }
    int32_t f = table[first_idx[i]];
    first_idx[i] = f;
    if (is_repeat) {
        is_repeat[i] = f != i;
    }
}

__device__ inline bool wanted(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b, int32_t i) {
    return a[i] == 0 && (b == nullptr || b[i] == 0);
}

// Rank of this thread among the workgroup's set flags, and the workgroup's total. All threads call.
__device__ inline int32_t flag_rank(bool flag, int32_t *wave_totals, int32_t *total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint64_t ballot = __ballot(flag);
    if (lane == 0) {
        wave_totals[wave] = __popcll(ballot);
    }
    __syncthreads();
    int32_t before = 0, all = 0;
    for (int w = 0; w < kSelWaves; w++) {
        int32_t c = wave_totals[w];
        before += w < wave ? c : 0;
        all += c;
    }
    *total = all;
    return before + __popcll(ballot & ((1ull << lane) - 1));
}

__global__ __launch_bounds__(kSelThreads) void count_kernel(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b,
                                                            int32_t n, int32_t *__restrict__ group_count) {
    __shared__ int32_t wave_totals[kSelWaves];
    int32_t i = blockIdx.x * kSelThreads + threadIdx.x, total;
    flag_rank(i < n && wanted(a, b, i), wave_totals, &total);
    if (threadIdx.x == 0) {
        group_count[blockIdx.x] = total;
    }
}

// One workgroup: counts[0..G) -> exclusive prefix sums in place, grand total to *d_total.
__global__ __launch_bounds__(kSelThreads) void scan_kernel(int32_t *__restrict__ counts, int32_t G,
                                                           int32_t *__restrict__ d_total) {
    __shared__ int32_t wave_totals[kSelWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int32_t carry = 0;
    for (int32_t base = 0; base < G; base += kSelThreads) {
        const int32_t i = base + threadIdx.x;
        const int32_t v = i < G ? counts[i] : 0;
        int32_t incl = v;
        for (int d = 1; d < 64; d <<= 1) {
            int32_t up = __shfl_up(incl, d, 64);
            incl += lane >= d ? up : 0;
        }
        if (lane == 63) {
            wave_totals[wave] = incl;
        }
        __syncthreads();
        int32_t before = 0, all = 0;
        for (int w = 0; w < kSelWaves; w++) {
            int32_t c = wave_totals[w];
            before += w < wave ? c : 0;
            all += c;
        }
        if (i < G) {
            counts[i] = carry + before + incl - v;
        }
        carry += all;
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        *d_total = carry;
    }
}

__global__ __launch_bounds__(kSelThreads) void write_kernel(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b,
                                                            int32_t n, const int32_t *__restrict__ group_offset,
                                                            int32_t *__restrict__ indices) {
    __shared__ int32_t wave_totals[kSelWaves];
    int32_t i = blockIdx.x * kSelThreads + threadIdx.x, total;
    const bool flag = i < n && wanted(a, b, i);
    const int32_t rank = flag_rank(flag, wave_totals, &total);
    if (flag) {
        indices[group_offset[blockIdx.x] + rank] = i;
    }
}

constexpr int64_t kMaxKeys = int64_t{1} << 30;

int64_t table_capacity(int64_t n) {
    int64_t cap = 1024;
    while (cap < 2 * n) {
        cap <<= 1;
    }
    return cap;
}

// fill / insert / resolve on a table of `cap` slots (a power of two, >= 2 n); the fill is a kernel, so the
// sequence may be recorded into a graph.
int32_t launch_first_occurrence(const int64_t *d_keys, int64_t n, int32_t *table, int64_t cap, int32_t *d_first_idx,
                                uint8_t *d_is_repeat, hipStream_t s) {
    int log2cap = 0;
    while ((int64_t{1} << log2cap) < cap) {
        log2cap++;
    }
    const int32_t n32 = static_cast<int32_t>(n);
    const unsigned groups = static_cast<unsigned>((n + 255) / 256);
    fill_i32_kernel<<<static_cast<unsigned>(cap / 256), 256, 0, s>>>(table, cap, -1);
    insert_kernel<<<groups, 256, 0, s>>>(d_keys, n32, table, static_cast<uint32_t>(cap - 1), 64 - log2cap, d_first_idx);
    resolve_kernel<<<groups, 256, 0, s>>>(d_first_idx, table, n32, d_is_repeat);
    return launch_status();
}

}  // namespace
}  // namespace kvcm

extern "C" {

int64_t kvcm_hip_first_occurrence_workspace_bytes(int64_t n) {
    if (n < 0 || n > kvcm::kMaxKeys) {
        return KVCM_ERR_TOO_LARGE;
    }
    return kvcm::table_capacity(n) * 4;
}

int32_t kvcm_hip_first_occurrence(const int64_t *d_keys, int64_t n, void *d_workspace, int64_t workspace_bytes,
                                  int32_t *d_first_idx, uint8_t *d_is_repeat, kvcm_stream_t stream) {
    if (n < 0) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (n == 0) {
        return KVCM_OK;
    }
    if (n > kvcm::kMaxKeys) {
        return KVCM_ERR_TOO_LARGE;
    }
    if (!d_keys || !d_workspace || !d_first_idx) {
        return KVCM_ERR_INVALID_ARG;
    }
    const int64_t cap = kvcm::table_capacity(n);
    if (workspace_bytes < cap * 4) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (reinterpret_cast<uintptr_t>(d_workspace) % 4 != 0) {
        return KVCM_ERR_ALIGNMENT;
    }
    return kvcm::launch_first_occurrence(d_keys, n, static_cast<int32_t *>(d_workspace), cap, d_first_idx, d_is_repeat,
                                         static_cast<hipStream_t>(stream));
}

int64_t kvcm_hip_first_occurrence_static_max_keys(void) { return kvcm::kStaticMaxKeys; }

int32_t kvcm_hip_first_occurrence_static(const int64_t *d_keys, int64_t n, int32_t *d_first_idx, uint8_t *d_is_repeat,
                                         kvcm_stream_t stream) {
    if (n < 0) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (n > kvcm::kStaticMaxKeys) {
        return KVCM_ERR_TOO_LARGE;
    }
    if (n > 0 && (!d_keys || !d_first_idx)) {
        return KVCM_ERR_INVALID_ARG;
    }
    // also for n == 0: a call with no keys is how a caller does the per-device set-up ahead of time
    int32_t *table = nullptr;
    const int32_t rc = kvcm::static_scratch(&table);
    if (rc != KVCM_OK) {
        return rc;
    }
    if (n == 0) {
        return KVCM_OK;
    }
    // the table keeps the last call's contents: the fill kernel clears the slots this call probes
    return kvcm::launch_first_occurrence(d_keys, n, table, kvcm::table_capacity(n), d_first_idx, d_is_repeat,
                                         static_cast<hipStream_t>(stream));
}

int64_t kvcm_hip_mask_to_indices_workspace_bytes(int64_t n) {
    if (n < 0 || n > kvcm::kMaxKeys) {
        return KVCM_ERR_TOO_LARGE;
    }
    return ((n + kvcm::kSelThreads - 1) / kvcm::kSelThreads + 1) * 4;
}

int32_t kvcm_hip_mask_to_indices(const uint8_t *d_mask, const uint8_t *d_mask2, int64_t n, void *d_workspace,
                                 int64_t workspace_bytes, int32_t *d_indices, int32_t *d_count,
                                 kvcm_stream_t stream) {
    if (n < 0 || !d_count) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (n > kvcm::kMaxKeys) {
        return KVCM_ERR_TOO_LARGE;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (n == 0) {
        kvcm::fill_i32_kernel<<<1, 256, 0, s>>>(d_count, 1, 0);
        return kvcm::launch_status();
    }
    if (!d_mask || !d_workspace || !d_indices) {
        return KVCM_ERR_INVALID_ARG;
    }
    const int64_t G = (n + kvcm::kSelThreads - 1) / kvcm::kSelThreads;
    if (workspace_bytes < (G + 1) * 4) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (reinterpret_cast<uintptr_t>(d_workspace) % 4 != 0) {
        return KVCM_ERR_ALIGNMENT;
    }
    int32_t *counts = static_cast<int32_t *>(d_workspace);
    const int32_t n32 = static_cast<int32_t>(n), G32 = static_cast<int32_t>(G);
    kvcm::count_kernel<<<G32, kvcm::kSelThreads, 0, s>>>(d_mask, d_mask2, n32, counts);
    kvcm::scan_kernel<<<1, kvcm::kSelThreads, 0, s>>>(counts, G32, d_count);
    kvcm::write_kernel<<<G32, kvcm::kSelThreads, 0, s>>>(d_mask, d_mask2, n32, counts, d_indices);
    return kvcm::launch_status();
}

}  // extern "C"
