// kvcm_copy.hip -- gather/scatter of paged KV blocks between per-layer pools and block-major staging.
//
// Semantics follow kv_cache_batch_gather_kernel / kv_cache_batch_scatter_kernel
// (kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:33-98,139-205) and the legacy
// single-block kernels (kv_cache_manager/py_connector/kernel/gather_scatter_helper.py:10-107); the
// launch shape does not: the reference runs 3 programs that walk all blocks serially because its staging
// buffer sits behind PCIe, here staging is HBM and the device is filled.
//
// Work decomposition (gfx950, wave64):
//   tile   = one (pool array p, work block b): T rows, contiguous in staging, `runs` contiguous runs in
//            the pool. One wavefront moves one tile with 16-byte accesses, 8 loads in flight per lane
//            before the first store.
//   unit   = one work block b and a group of `tiles_per_wg` consecutive p: one workgroup of 4 waves.
//            The block's run-start slots are read once per workgroup into LDS; the four waves then
//            take p = first, first+4, ...
//   The layer-major -> block-major transposition is only address arithmetic: a lane's 16 bytes go
//   from pool_p + slot*row_bytes + off to staging + sb*block_stride + p*tile_stride + run*run_bytes + off
//   through registers; nothing is reshaped in memory.
//
// Roofline: HBM. Algorithmic bytes per tile = 2 * T * row_bytes (+ trailer), index bytes are negligible.
#include "kvcm_internal.h"

#include <atomic>
#include <cstdlib>

namespace kvcm {
namespace {

#ifndef KVCM_COPY_THREADS
#define KVCM_COPY_THREADS 256
#endif
#ifndef KVCM_COPY_UNROLL
#define KVCM_COPY_UNROLL 8
#endif
// Every byte is touched once, so loads and stores carry the non-temporal hint (streaming policy in L2):
// measured +10 % on gather at the Llama-3-8B layout against plain accesses.
#ifndef KVCM_COPY_NT_LOAD
#define KVCM_COPY_NT_LOAD 1
#endif
#ifndef KVCM_COPY_NT_STORE
#define KVCM_COPY_NT_STORE 1
#endif

constexpr int kThreads = KVCM_COPY_THREADS;
constexpr int kWaves = kThreads / 64;
constexpr int kMaxRuns = 2048;          // run-start slots of one work block staged in LDS (8 KiB)
constexpr int kUnroll = KVCM_COPY_UNROLL;  // 16-byte accesses in flight per lane

struct CopyArgs {
    const void *const *ptr_table;
    const void *const *trailer_table;
    unsigned char *staging;
    const int32_t *run_start;
    const int32_t *staging_idx;
    const int32_t *trailer_idx;
    int64_t entry_stride;
    int64_t block_stride;
    int64_t tile_stride;
    int64_t row_bytes;
    int64_t run_bytes;
    int32_t P;
    int32_t ptrs_per_entry;
    int32_t runs;
    int32_t slot_limit;
    int32_t trailer_bytes;
    int32_t tiles_per_wg;
    uint32_t pgroups;
    uint32_t n_units;
    int32_t host_align;   // 16, 4 or 1: alignment shared by staging base, all strides and row_bytes
    int32_t xcd_remap;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// 16 bytes at dword alignment: still one dwordx4 access (global memory accepts dword-aligned wide
// accesses); used when a 4-byte trailer shifts every staging tile off the 16-byte grid.
typedef u32x4 u32x4_dword_aligned __attribute__((aligned(4)));

// Access descriptors: the register type V and the pointer type P the memory access goes through.
struct Acc16 {
    using V = u32x4;
    using P = u32x4;
};
struct Acc16U {
    using V = u32x4;
    using P = u32x4_dword_aligned;
};
struct Acc4 {
    using V = uint32_t;
    using P = uint32_t;
};
struct Acc1 {
    using V = uint8_t;
    using P = uint8_t;
};

// The access goes through A::P so that its alignment (not the register type's) is what the compiler assumes.
template <typename A>
__device__ __forceinline__ typename A::V load_chunk(const unsigned char *p) {
#if KVCM_COPY_NT_LOAD
    return __builtin_nontemporal_load(reinterpret_cast<const typename A::P *>(p));
#else
    return *reinterpret_cast<const typename A::P *>(p);
#endif
}

template <typename A>
__device__ __forceinline__ void store_chunk(unsigned char *p, typename A::V v) {
#if KVCM_COPY_NT_STORE
    __builtin_nontemporal_store(v, reinterpret_cast<typename A::P *>(p));
#else
    *reinterpret_cast<typename A::P *>(p) = v;
#endif
}

// Moves one tile. `runs_lds` holds the first slot of every run. Chunks (sizeof(V) bytes) are numbered
// along the staging tile; chunk c belongs to run c / cpr at offset c % cpr. A lane visits chunks
// lane, lane + 64, ... and keeps (run, offset) up to date incrementally, so the loop has no division.
template <typename A, bool SCATTER>
__device__ __forceinline__ void move_tile(unsigned char *pool, unsigned char *tile, const int32_t *runs_lds,
                                          const CopyArgs &a, uint32_t lane) {
    using V = typename A::V;
    const uint32_t cpr = static_cast<uint32_t>(a.run_bytes / static_cast<int64_t>(sizeof(V)));
    const uint32_t total = static_cast<uint32_t>(a.runs) * cpr;
    const uint32_t step_r = 64u / cpr;
    const uint32_t step_off = 64u - step_r * cpr;
    const int64_t limit = a.slot_limit > 0 ? a.slot_limit : INT64_MAX;
    uint32_t r = lane / cpr;
    uint32_t off = lane - r * cpr;
    for (uint32_t c0 = lane; c0 < total; c0 += 64u * kUnroll) {
        V v[kUnroll];
        unsigned char *pp[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            pp[u] = nullptr;
            if (c0 + 64u * u < total) {
                const int64_t slot = runs_lds[r];
                if (slot >= 0 && slot < limit) {
                    pp[u] = pool + slot * a.row_bytes + static_cast<int64_t>(off) * sizeof(V);
                }
            }
            off += step_off;
            r += step_r;
            if (off >= cpr) {
                off -= cpr;
                r += 1;
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (pp[u]) {
                const unsigned char *sp = tile + static_cast<int64_t>(c0 + 64u * u) * sizeof(V);
                v[u] = load_chunk<A>(SCATTER ? sp : pp[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (pp[u]) {
                unsigned char *sp = tile + static_cast<int64_t>(c0 + 64u * u) * sizeof(V);
                store_chunk<A>(SCATTER ? pp[u] : sp, v[u]);
            }
        }
    }
}

template <bool SCATTER>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 8))) void copy_tiles_kernel(const CopyArgs a) {
    __shared__ int32_t s_runs[kMaxRuns];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    // Consecutive workgroup ids land on consecutive XCDs (8 per device, one L2 each). With the remap
    // every XCD walks one contiguous eighth of the unit range instead of every eighth unit.
    uint32_t first = blockIdx.x;
    if (a.xcd_remap) {
        const uint32_t q = gridDim.x >> 3, rem = gridDim.x & 7u;
        const uint32_t xcd = blockIdx.x & 7u, idx = blockIdx.x >> 3;
        first = xcd * q + (xcd < rem ? xcd : rem) + idx;
    }

    for (uint32_t unit = first; unit < a.n_units; unit += gridDim.x) {
        const uint32_t b = unit / a.pgroups;
        const uint32_t pg = unit - b * a.pgroups;
        __syncthreads();
        for (int32_t i = threadIdx.x; i < a.runs; i += kThreads) {
            s_runs[i] = a.run_start[static_cast<int64_t>(b) * a.runs + i];
        }
        __syncthreads();
        const int64_t slot = a.staging_idx ? a.staging_idx[b] : static_cast<int64_t>(b);
        unsigned char *block = a.staging + slot * a.block_stride;
        const int32_t p_begin = static_cast<int32_t>(pg) * a.tiles_per_wg;
        const int32_t p_end = min(a.P, p_begin + a.tiles_per_wg);
        for (int32_t p = p_begin + static_cast<int32_t>(wave); p < p_end; p += kWaves) {
            const int32_t entry = p / a.ptrs_per_entry;
            const int32_t inner = p - entry * a.ptrs_per_entry;
            unsigned char *pool = static_cast<unsigned char *>(const_cast<void *>(a.ptr_table[entry])) +
                                  static_cast<int64_t>(inner) * a.entry_stride;
            unsigned char *tile = block + static_cast<int64_t>(p) * a.tile_stride;
            const uintptr_t pa = reinterpret_cast<uintptr_t>(pool);
            if (a.host_align == 16 && (pa & 15u) == 0) {
                move_tile<Acc16, SCATTER>(pool, tile, s_runs, a, lane);
            } else if (a.host_align >= 4 && (pa & 3u) == 0 && (a.run_bytes & 15) == 0) {
                move_tile<Acc16U, SCATTER>(pool, tile, s_runs, a, lane);
            } else if (a.host_align >= 4 && (pa & 3u) == 0) {
                move_tile<Acc4, SCATTER>(pool, tile, s_runs, a, lane);
            } else {
                move_tile<Acc1, SCATTER>(pool, tile, s_runs, a, lane);
            }
            if (a.trailer_bytes > 0) {
                unsigned char *tr = static_cast<unsigned char *>(const_cast<void *>(a.trailer_table[p])) +
                                    static_cast<int64_t>(a.trailer_idx[b]) * a.trailer_bytes;
                unsigned char *st = tile + static_cast<int64_t>(a.runs) * a.run_bytes;
                for (int32_t i = lane; i < a.trailer_bytes; i += 64) {
                    if (SCATTER) {
                        tr[i] = st[i];
                    } else {
                        st[i] = tr[i];
                    }
                }
            }
        }
    }
}

// out[b][i] = block_ids[(m_b*T_mgr + i) / T_eng] * T_eng + (m_b*T_mgr + i) % T_eng
// (kv_cache_manager/py_connector/vllm/v1_connector.py:308-320).
__global__ __launch_bounds__(256) void blocks_idx_kernel(const int32_t *mgr, int32_t B, const int32_t *local_ids,
                                                         int32_t n_local, int32_t T_mgr, int32_t T_eng, int32_t *out,
                                                         int32_t *error_flag) {
    const int64_t n = static_cast<int64_t>(B) * T_mgr;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; e < n;
         e += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t b = e / T_mgr;
        const int64_t i = e - b * T_mgr;
        const int64_t tok = static_cast<int64_t>(mgr[b]) * T_mgr + i;
        const int64_t blk = tok / T_eng;
        int32_t v = -1;
        if (tok >= 0 && blk < n_local) {
            v = static_cast<int32_t>(static_cast<int64_t>(local_ids[blk]) * T_eng + (tok - blk * T_eng));
        } else if (error_flag) {
            *error_flag = 1;
        }
        out[e] = v;
    }
}

int env_int(const char *name, int dflt) {
    const char *s = std::getenv(name);
    return s ? std::atoi(s) : dflt;
}

int32_t align_class(uint64_t bits) {
    if ((bits & 15u) == 0) {
        return 16;
    }
    if ((bits & 3u) == 0) {
        return 4;
    }
    return 1;
}

int32_t launch_copy(const kvcm_copy_desc *d, bool scatter, hipStream_t stream) {
    if (!d) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (d->B < 0 || d->P <= 0 || d->T <= 0 || d->run_tokens <= 0 || d->row_bytes <= 0 || d->ptrs_per_entry <= 0 ||
        d->trailer_bytes < 0 || d->slot_limit < 0 || d->entry_stride_bytes < 0) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (d->T % d->run_tokens != 0 || d->P % d->ptrs_per_entry != 0) {
        return KVCM_ERR_INVALID_ARG;
    }
    const int64_t payload = static_cast<int64_t>(d->T) * d->row_bytes;
    if (d->staging_tile_stride_bytes < payload + d->trailer_bytes ||
        d->staging_block_stride_bytes < static_cast<int64_t>(d->P) * d->staging_tile_stride_bytes) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (d->B == 0) {
        return KVCM_OK;
    }
    if (!d->d_ptr_table || !d->d_staging || !d->d_run_start) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (d->trailer_bytes > 0 && (!d->d_trailer_ptr_table || !d->d_trailer_idx)) {
        return KVCM_ERR_INVALID_ARG;
    }
    const int32_t runs = d->T / d->run_tokens;
    if (runs > kMaxRuns || payload >= (int64_t{1} << 31)) {
        return KVCM_ERR_TOO_LARGE;
    }

    CopyArgs a{};
    a.ptr_table = d->d_ptr_table;
    a.trailer_table = d->d_trailer_ptr_table;
    a.staging = static_cast<unsigned char *>(d->d_staging);
    a.run_start = d->d_run_start;
    a.staging_idx = d->d_staging_idx;
    a.trailer_idx = d->d_trailer_idx;
    a.entry_stride = d->entry_stride_bytes;
    a.block_stride = d->staging_block_stride_bytes;
    a.tile_stride = d->staging_tile_stride_bytes;
    a.row_bytes = d->row_bytes;
    a.run_bytes = static_cast<int64_t>(d->run_tokens) * d->row_bytes;
    a.P = d->P;
    a.ptrs_per_entry = d->ptrs_per_entry;
    a.runs = runs;
    a.slot_limit = d->slot_limit;
    a.trailer_bytes = d->trailer_bytes;
    a.host_align = align_class(reinterpret_cast<uint64_t>(d->d_staging) | static_cast<uint64_t>(a.block_stride) |
                               static_cast<uint64_t>(a.tile_stride) | static_cast<uint64_t>(a.row_bytes) |
                               static_cast<uint64_t>(a.entry_stride));

    // Tiles per workgroup: one per wave when tiles are large; more for small tiles so that a workgroup
    // moves at least 64 KiB, as long as enough workgroups remain to fill the device.
    const int cus = device_cu_count();
    int32_t tpw = kWaves;
    while (tpw < d->P && payload * tpw < 65536 &&
           static_cast<int64_t>(d->B) * ((d->P + 2 * tpw - 1) / (2 * tpw)) >= static_cast<int64_t>(cus) * 8) {
        tpw *= 2;
    }
    tpw = env_int("KVCM_COPY_TILES_PER_WG", tpw);
    a.tiles_per_wg = tpw;
    a.pgroups = static_cast<uint32_t>((d->P + tpw - 1) / tpw);
    const int64_t units = static_cast<int64_t>(d->B) * a.pgroups;
    if (units >= (int64_t{1} << 31)) {
        return KVCM_ERR_TOO_LARGE;
    }
    a.n_units = static_cast<uint32_t>(units);
    a.xcd_remap = env_int("KVCM_COPY_XCD_REMAP", 1);

    int64_t grid = units;
    const int per_cu = env_int("KVCM_COPY_WG_PER_CU", 0);
    if (per_cu > 0) {
        grid = std::min<int64_t>(grid, static_cast<int64_t>(cus) * per_cu);
    }
    if (d->max_workgroups > 0) {
        grid = std::min<int64_t>(grid, d->max_workgroups);
    }
    if (scatter) {
        hipLaunchKernelGGL(copy_tiles_kernel<true>, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), 0, stream, a);
    } else {
        hipLaunchKernelGGL(copy_tiles_kernel<false>, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), 0, stream, a);
    }
    return launch_status();
}

kvcm_copy_desc flat_desc(const void *const *d_ptr_table, int32_t P, void *d_staging, int64_t block_stride,
                         const int32_t *d_run_start, int32_t run_tokens, const int32_t *d_staging_idx, int32_t B,
                         int32_t T, int64_t row_bytes, int32_t max_workgroups) {
    kvcm_copy_desc d{};
    d.d_ptr_table = d_ptr_table;
    d.P = P;
    d.ptrs_per_entry = 1;
    d.entry_stride_bytes = 0;
    d.d_staging = d_staging;
    d.staging_block_stride_bytes = block_stride;
    d.staging_tile_stride_bytes = static_cast<int64_t>(T) * row_bytes;
    d.d_run_start = d_run_start;
    d.d_staging_idx = d_staging_idx;
    d.B = B;
    d.T = T;
    d.run_tokens = run_tokens;
    d.slot_limit = 0;
    d.row_bytes = row_bytes;
    d.max_workgroups = max_workgroups;
    return d;
}

}  // namespace

int device_cu_count() {
    static std::atomic<int> cache[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        return 256;
    }
    int v = cache[dev].load(std::memory_order_relaxed);
    if (v == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            n = 256;
        }
        cache[dev].store(n, std::memory_order_relaxed);
        v = n;
    }
    return v;
}

}  // namespace kvcm

extern "C" {

int32_t kvcm_hip_gather_ex(const kvcm_copy_desc *desc, kvcm_stream_t stream) {
    return kvcm::launch_copy(desc, false, static_cast<hipStream_t>(stream));
}

int32_t kvcm_hip_scatter_ex(const kvcm_copy_desc *desc, kvcm_stream_t stream) {
    return kvcm::launch_copy(desc, true, static_cast<hipStream_t>(stream));
}

int32_t kvcm_hip_batch_gather(const void *const *d_ptr_table, int32_t P, void *d_staging,
                              int64_t staging_block_stride_bytes, const int32_t *d_token_idx,
                              const int32_t *d_staging_idx, int32_t B, int32_t T, int64_t row_bytes,
                              int32_t max_workgroups, kvcm_stream_t stream) {
    kvcm_copy_desc d = kvcm::flat_desc(d_ptr_table, P, d_staging, staging_block_stride_bytes, d_token_idx, 1,
                                       d_staging_idx, B, T, row_bytes, max_workgroups);
    return kvcm::launch_copy(&d, false, static_cast<hipStream_t>(stream));
}

int32_t kvcm_hip_batch_scatter(const void *const *d_ptr_table, int32_t P, const void *d_staging,
                               int64_t staging_block_stride_bytes, const int32_t *d_token_idx,
                               const int32_t *d_staging_idx, int32_t B, int32_t T, int64_t row_bytes,
                               int32_t max_workgroups, kvcm_stream_t stream) {
    kvcm_copy_desc d = kvcm::flat_desc(d_ptr_table, P, const_cast<void *>(d_staging), staging_block_stride_bytes,
                                       d_token_idx, 1, d_staging_idx, B, T, row_bytes, max_workgroups);
    return kvcm::launch_copy(&d, true, static_cast<hipStream_t>(stream));
}

int32_t kvcm_hip_paged_gather(const void *const *d_ptr_table, int32_t P, void *d_staging,
                              int64_t staging_block_stride_bytes, const int32_t *d_run_start, int32_t run_tokens,
                              const int32_t *d_staging_idx, int32_t B, int32_t T, int64_t row_bytes,
                              int32_t max_workgroups, kvcm_stream_t stream) {
    kvcm_copy_desc d = kvcm::flat_desc(d_ptr_table, P, d_staging, staging_block_stride_bytes, d_run_start, run_tokens,
                                       d_staging_idx, B, T, row_bytes, max_workgroups);
    return kvcm::launch_copy(&d, false, static_cast<hipStream_t>(stream));
}

int32_t kvcm_hip_paged_scatter(const void *const *d_ptr_table, int32_t P, const void *d_staging,
                               int64_t staging_block_stride_bytes, const int32_t *d_run_start, int32_t run_tokens,
                               const int32_t *d_staging_idx, int32_t B, int32_t T, int64_t row_bytes,
                               int32_t max_workgroups, kvcm_stream_t stream) {
    kvcm_copy_desc d = kvcm::flat_desc(d_ptr_table, P, const_cast<void *>(d_staging), staging_block_stride_bytes,
                                       d_run_start, run_tokens, d_staging_idx, B, T, row_bytes, max_workgroups);
    return kvcm::launch_copy(&d, true, static_cast<hipStream_t>(stream));
}

int32_t kvcm_hip_generate_blocks_idx(const int32_t *d_manager_block_idxes, int32_t B, const int32_t *d_local_block_ids,
                                     int32_t n_local, int32_t T_mgr, int32_t T_eng, int32_t *d_out,
                                     int32_t *d_error_flag, kvcm_stream_t stream) {
    if (B < 0 || n_local < 0 || T_mgr <= 0 || T_eng <= 0) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (B == 0) {
        return KVCM_OK;
    }
    if (!d_manager_block_idxes || !d_local_block_ids || !d_out) {
        return KVCM_ERR_INVALID_ARG;
    }
    const int64_t n = static_cast<int64_t>(B) * T_mgr;
    const int64_t grid = std::min<int64_t>((n + 255) / 256, 65536);
    hipLaunchKernelGGL(kvcm::blocks_idx_kernel, dim3(static_cast<uint32_t>(grid)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_manager_block_idxes, B, d_local_block_ids, n_local, T_mgr,
                       T_eng, d_out, d_error_flag);
    return kvcm::launch_status();
}

}  // extern "C"
