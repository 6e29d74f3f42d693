// kvcm_copy.hip -- gather/scatter of paged KV blocks between per-layer pools and block-major staging.
//
// Semantics follow kv_cache_batch_gather_kernel / kv_cache_batch_scatter_kernel
// (kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:33-98,139-205) and the legacy
// single-block kernels (kv_cache_manager/py_connector/kernel/gather_scatter_helper.py:10-107); the
// launch shape does not: the reference runs 3 programs that walk all blocks serially because its staging
// buffer sits behind PCIe, here staging is HBM and the device is filled.
//
// Work decomposition (gfx950, wave64), chosen by measurement on MI355X:
//   A staging block is a run of 16-byte chunks, tile after tile ([P][T*row_bytes]). A workgroup of 256 threads
//   (4 waves) takes one SPAN of 256 consecutive chunks = 4 KiB of staging and every thread moves exactly one
//   chunk: one 16-byte load, one 16-byte store, done. There is no loop and nothing to unroll; memory-level
//   parallelism comes from the ~32 resident waves per CU, each with one access in flight, and from the
//   dispatcher replacing finished workgroups. For the Llama-3-8B layout a (layer, K/V, block) tile is 8 spans.
//   Measured at that layout (12 416 blocks, 2 x 24.25 GiB per launch, % of the 8 TB/s HBM peak):
//       one wavefront streams a whole 32 KiB tile, 8 loads in flight per lane      gather 74 %   scatter 68 %
//       1024 threads x 2 chunks, one 32 KiB tile per workgroup                      gather 75 %   scatter 74 %
//       256 threads x 1 chunk (this kernel)                                         gather 79 %   scatter 77 %
//   The fine-grained form wins because each 4 KiB piece of a pool block is read or written in one short burst
//   while its DRAM pages are open, instead of trickling out of a long-lived wave that shares the memory
//   controllers with 2000 other half-finished tiles; scattered 32 KiB writes gain the most.
//   Workgroup ids are dealt round-robin to the 8 XCDs; the kernel renumbers them so that every XCD walks one
//   contiguous eighth of the span range (+6 % against leaving consecutive 4 KiB spans on different XCDs).
//   The layer-major -> block-major transposition is only address arithmetic: a thread's 16 bytes go from
//   pool_p + slot*row_bytes + off to staging + sb*block_stride + p*tile_stride + run*run_bytes + off through
//   registers; nothing is reshaped in memory. When a span lies inside one tile (and one run) the tile number,
//   pool pointer and slot are workgroup-uniform: scalar arithmetic and scalar loads, and a thread's own work is
//   two address adds. Otherwise chunk -> (tile, run, offset) is two multiply-shift divisions per thread.
//   Every byte is touched once: loads carry the non-temporal hint (+4 % gather against plain accesses), and so
//   do stores, except where whole tiles move (block-table form): there the staging side of a gather is written
//   through at system scope and the pool side of a scatter carries both bits (see the store site below).
//
// Roofline: HBM. Algorithmic bytes per tile = 2 * T * row_bytes (+ trailer), index bytes are negligible.
#include "kvcm_internal.h"

#include <cstdlib>

#include "kvcm_host_idx.h"

namespace kvcm {
namespace {

#ifndef KVCM_COPY_THREADS
#define KVCM_COPY_THREADS 256
#endif
#ifndef KVCM_COPY_CHUNKS_PER_THREAD
#define KVCM_COPY_CHUNKS_PER_THREAD 1
#endif
#ifndef KVCM_COPY_NT_LOAD
#define KVCM_COPY_NT_LOAD 1
#endif
#ifndef KVCM_COPY_GATHER_STORE_POLICY
#define KVCM_COPY_GATHER_STORE_POLICY 1
#endif
#ifndef KVCM_COPY_SCATTER_STORE_POLICY
#define KVCM_COPY_SCATTER_STORE_POLICY 2
#endif
#ifndef KVCM_COPY_NT_STORE
#define KVCM_COPY_NT_STORE 1
#endif

constexpr int kThreads = KVCM_COPY_THREADS;
constexpr int kCPT = KVCM_COPY_CHUNKS_PER_THREAD;  // chunks per thread per span
constexpr uint32_t kSpan = static_cast<uint32_t>(kThreads) * kCPT;

// n / d for n < 2^31 as a multiply and a shift: mul = ceil(2^(31+L) / d), L = ceil(log2 d).
struct FastDiv {
    uint32_t mul;
    uint32_t shift;
};

FastDiv make_fastdiv(uint32_t d) {
    uint32_t L = 0;
    while ((uint64_t{1} << L) < d) {
        ++L;
    }
    const uint64_t pow = uint64_t{1} << (31 + L);
    return FastDiv{static_cast<uint32_t>((pow + d - 1) / d), 31 + L};
}

__device__ __forceinline__ uint32_t fast_div(uint32_t n, FastDiv f) {
    return static_cast<uint32_t>((static_cast<uint64_t>(n) * f.mul) >> f.shift);
}

struct CopyArgs {
    unsigned char *staging;
    int64_t entry_stride;
    int64_t block_stride;
    int64_t tile_stride;
    int64_t row_bytes;
    int64_t tile_payload;  // T * row_bytes: where the trailer starts inside a staging tile
    uint32_t ptrs_per_entry;
    uint32_t runs;
    int32_t slot_limit;
    int32_t trailer_bytes;
    uint32_t chunks_per_run;
    uint32_t chunks_per_tile;
    uint32_t chunks_per_block;
    uint32_t units_per_block;
    uint32_t n_units;
    FastDiv div_tile;
    FastDiv div_run;
    FastDiv div_entry;
    FastDiv div_units;
    int32_t xcd_remap;
    int32_t staging_on_line_grid;  // staging base, block stride and tile stride are multiples of 128
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// 16 bytes at dword alignment: still ONE dwordx4 instruction (global memory takes dword-aligned wide accesses);
// the alignment only tells the compiler what it may assume. A 4-byte trailer per tile shifts staging tiles off
// the 16-byte grid, so the 16-byte path never promises more than dword alignment.
typedef u32x4 u32x4_dword_aligned __attribute__((aligned(4)));

template <int CS>
struct Chunk;
template <>
struct Chunk<16> {
    using V = u32x4;
    using P = u32x4_dword_aligned;
};
template <>
struct Chunk<4> {
    using V = uint32_t;
    using P = uint32_t;
};
template <>
struct Chunk<1> {
    using V = uint8_t;
    using P = uint8_t;
};

// Pool rows and staging are device (or pinned host) memory: the accesses name the global address space, so the
// compiler emits global_load / global_store rather than flat instructions for pointers it read from a table.
#define KVCM_GLOBAL __attribute__((address_space(1)))

template <int CS>
__device__ __forceinline__ typename Chunk<CS>::V load_chunk(const unsigned char *p) {
    using GP = const KVCM_GLOBAL typename Chunk<CS>::P *;
#if KVCM_COPY_NT_LOAD
    return __builtin_nontemporal_load((GP)(p));
#else
    return *(GP)(p);
#endif
}

template <int CS>
__device__ __forceinline__ void store_chunk(unsigned char *p, typename Chunk<CS>::V v) {
    using GP = KVCM_GLOBAL typename Chunk<CS>::P *;
#if KVCM_COPY_NT_STORE
    __builtin_nontemporal_store(v, (GP)(p));
#else
    *(GP)(p) = v;
#endif
}

// 16-byte chunks, the form every engine layout takes. POLICY 0: non-temporal; 1: written through at system scope
// (sc1); 2: both; 3: sc0 sc1.
template <int POLICY>
__device__ __forceinline__ void store_chunk16(unsigned char *p, u32x4 v) {
    if (POLICY == 1) {
        asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
    } else if (POLICY == 2) {
        asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" : : "v"(p), "v"(v) : "memory");
    } else if (POLICY == 3) {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" : : "v"(p), "v"(v) : "memory");
    } else {
        store_chunk<16>(p, v);
    }
}

// CS = chunk size in bytes (16, 4 or 1), picked on the host from what it can see: staging address, strides,
// row size. Pool base pointers live in device memory; a pool row that is not dword-aligned (CS > 1) is moved
// byte by byte by the one thread that owns the chunk.
//
// UNI_TILE: every span lies inside one tile (chunks_per_tile is a multiple of the span), so the tile number, the
// pool base pointer and the staging tile address are workgroup-uniform: scalar arithmetic and scalar loads.
// RUN = how widely a run of consecutive slots is shared (needs UNI_TILE):
//   kRunPerGroup  every span lies inside one run (block-table fast path, or rows of 4 KiB and more): the run's
//                 first slot is one scalar load per workgroup and a thread's own work is two address adds;
//   kRunPerWave   a run is a whole number of wavefronts' worth of chunks (rows of 1 KiB and more): the slot is a
//                 scalar load per wave;
//   kRunPerThread anything else: the run number is a multiply-shift division per thread and the slot a vector load.
enum RunMode { kRunPerThread = 0, kRunPerWave = 1, kRunPerGroup = 2 };

// Where a launch finds its index tables. PtrIdx: two arrays in device memory (every entry point that takes d_ pointers).
// KernargIdx: the tables travel INSIDE the kernel's argument block, run starts first, staging slots behind them -- the
// form behind the entry points that take host index lists: nothing is uploaded, nothing has to outlive the call, and a
// uniform read of the table is a scalar load from the argument segment like any other kernel argument.
struct PtrIdx {
    const int32_t *run_start;
    const int32_t *staging_idx;
    __device__ __forceinline__ int32_t run(int64_t i) const { return run_start[i]; }
    __device__ __forceinline__ int64_t slot(uint32_t b) const {
        return staging_idx ? staging_idx[b] : static_cast<int64_t>(b);
    }
};
struct KernargIdx {
    const EmbeddedIdx &e;
    uint32_t staging_first;  // index of the first staging slot inside e.v
    __device__ __forceinline__ int32_t run(int64_t i) const { return e.v[i]; }
    __device__ __forceinline__ int64_t slot(uint32_t b) const { return e.v[staging_first + b]; }
};

template <int CS, bool SCATTER, bool UNI_TILE, int RUN, typename Idx>
__device__ __forceinline__ void copy_span_body(const CopyArgs &a, const void *const *__restrict__ ptr_table,
                                               const void *const *__restrict__ trailer_table, const Idx &idx,
                                               const int32_t *__restrict__ trailer_idx) {
    using V = typename Chunk<CS>::V;

    // Consecutive workgroup ids land on consecutive XCDs (8 per device, one L2 each). With the remap every XCD
    // walks one contiguous eighth of the unit range instead of every eighth unit.
    uint32_t first = blockIdx.x;
    if (a.xcd_remap) {
        const uint32_t q = gridDim.x >> 3, rem = gridDim.x & 7u;
        const uint32_t xcd = blockIdx.x & 7u, idx = blockIdx.x >> 3;
        first = xcd * q + (xcd < rem ? xcd : rem) + idx;
    }
    const int64_t limit = a.slot_limit > 0 ? a.slot_limit : INT64_MAX;

    for (uint32_t unit = first; unit < a.n_units; unit += gridDim.x) {
        const uint32_t b = fast_div(unit, a.div_units);
        const uint32_t span = unit - b * a.units_per_block;
        const int64_t runs_b = static_cast<int64_t>(b) * a.runs;  // index of the block's first run
        // workgroup-uniform part: the three table reads below are independent scalar loads in the UNI_* forms
        const uint32_t g_first = span * kSpan;
        const uint32_t p_first = fast_div(g_first, a.div_tile);
        const uint32_t cc_first = g_first - p_first * a.chunks_per_tile;
        const uint32_t r_first = fast_div(cc_first, a.div_run);
        const uint32_t entry_first = fast_div(p_first, a.div_entry);
        int64_t slot_shared = 0;
        uint32_t r_shared = r_first;
        if (RUN == kRunPerGroup) {
            slot_shared = idx.run(runs_b + r_first);
        } else if (RUN == kRunPerWave) {
            // one chunk per thread: a wave's 64 chunks start at a multiple of 64 and lie inside one run
            r_shared = __builtin_amdgcn_readfirstlane(fast_div(cc_first + (threadIdx.x & ~63u), a.div_run));
            slot_shared = idx.run(runs_b + r_shared);
        }
        const void *pool_first = UNI_TILE ? ptr_table[entry_first] : nullptr;
        // the span that starts a tile also moves the tile's trailer: its table entries are workgroup-uniform too
        int32_t trailer_idx_first = -1;
        const void *trailer_base_first = nullptr;
        if (UNI_TILE && a.trailer_bytes > 0 && cc_first == 0) {
            trailer_idx_first = trailer_idx[b];
            trailer_base_first = trailer_table[p_first];
        }
        const int64_t slot_b = idx.slot(b);
        unsigned char *block = a.staging + slot_b * a.block_stride;

        V v[kCPT];
        unsigned char *pp[kCPT];
        unsigned char *sp[kCPT];
        // a 4-byte trailer in flight, and where it goes: one per thread, which is enough because a thread owns one
        // chunk -- with several chunks per thread on the non-uniform path a thread could own the first chunk of two tiles
        static_assert(kCPT == 1, "the 4-byte trailer path keeps one trailer per thread");
        uint32_t tr_word = 0;
        unsigned char *tr_dst = nullptr;
#pragma unroll
        for (int u = 0; u < kCPT; ++u) {
            const uint32_t in_span = threadIdx.x + static_cast<uint32_t>(u) * kThreads;
            const uint32_t g = g_first + in_span;
            pp[u] = nullptr;
            sp[u] = nullptr;
            if (g < a.chunks_per_block) {
                const uint32_t p = UNI_TILE ? p_first : fast_div(g, a.div_tile);
                const uint32_t cc = UNI_TILE ? cc_first + in_span : g - p * a.chunks_per_tile;
                const uint32_t r = RUN != kRunPerThread ? r_shared : fast_div(cc, a.div_run);
                const uint32_t off = cc - r * a.chunks_per_run;
                const int64_t slot = RUN != kRunPerThread ? slot_shared : static_cast<int64_t>(idx.run(runs_b + r));
                unsigned char *tile = block + static_cast<int64_t>(p) * a.tile_stride;
                if (slot >= 0 && slot < limit) {
                    const uint32_t entry = UNI_TILE ? entry_first : fast_div(p, a.div_entry);
                    const uint32_t inner = p - entry * a.ptrs_per_entry;
                    const void *base = UNI_TILE ? pool_first : ptr_table[entry];
                    unsigned char *pool = static_cast<unsigned char *>(const_cast<void *>(base)) +
                                          static_cast<int64_t>(inner) * a.entry_stride;
                    pp[u] = pool + slot * a.row_bytes + static_cast<int64_t>(off) * CS;
                    sp[u] = tile + static_cast<int64_t>(cc) * CS;
                }
                if (a.trailer_bytes > 0 && cc == 0 && (UNI_TILE ? trailer_idx_first : trailer_idx[b]) >= 0) {
                    // the thread that owns a tile's first chunk also moves the tile's trailer (a negative trailer
                    // index means "no trailer for this block": nothing is read or written)
                    const int64_t t_idx = UNI_TILE ? trailer_idx_first : trailer_idx[b];
                    const void *t_base = UNI_TILE ? trailer_base_first : trailer_table[p];
                    unsigned char *tr = static_cast<unsigned char *>(const_cast<void *>(t_base)) + t_idx * a.trailer_bytes;
                    unsigned char *st = tile + a.tile_payload;
                    if (a.trailer_bytes == 4 && ((reinterpret_cast<uintptr_t>(tr) | reinterpret_cast<uintptr_t>(st)) & 3u) == 0) {
                        // one fp32 scale per tile: its load goes out here, next to the load of the thread's own chunk,
                        // and its store follows the chunk's, so the workgroup that holds this thread does not outlive
                        // its neighbours by a chain of byte-sized round trips to memory
                        tr_word = load_chunk<4>(SCATTER ? st : tr);
                        tr_dst = SCATTER ? tr : st;
                    } else {
                        for (int32_t i = 0; i < a.trailer_bytes; ++i) {
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
        // Common case: every chunk of this thread is live and dword-aligned. One straight-line block -- all loads
        // back to back, then all stores -- so that no store waits for an earlier store's acknowledgement (matters
        // when the kernel is built with more than one chunk per thread).
        bool all_fast = true;
#pragma unroll
        for (int u = 0; u < kCPT; ++u) {
            all_fast = all_fast && pp[u] && (CS == 1 || (reinterpret_cast<uintptr_t>(pp[u]) & 3u) == 0);
        }
        if (all_fast) {
#pragma unroll
            for (int u = 0; u < kCPT; ++u) {
                v[u] = load_chunk<CS>(SCATTER ? sp[u] : pp[u]);
            }
#pragma unroll
            for (int u = 0; u < kCPT; ++u) {
                if constexpr (CS == 16) {
                    // Block-table form (whole tiles move): the staging side of a gather is written through at system
                    // scope (sc1), measured +1.5 to +4.6 % over non-temporal stores at the benchmark layouts and +1.6 %
                    // for 128-block tasks; the pool side of a scatter carries sc1 and nt together (+1.3 to +2.5 %, and a
                    // 24 MiB launch that fits the caches finishes 45 % sooner). With token-granular indices either bit
                    // costs 0.5 to 2.5 %: those stores stay non-temporal. Where staging tiles do not start on cache-line
                    // boundaries (a 4-byte scale behind every tile) a wave's kilobyte begins and ends inside a line, and
                    // writing partial lines through costs 15 % (5.2 against 6.0 TB/s): non-temporal there as well.
                    constexpr int kPolicy = RUN != kRunPerGroup ? 0
                                            : (SCATTER ? KVCM_COPY_SCATTER_STORE_POLICY : KVCM_COPY_GATHER_STORE_POLICY);
                    if (kPolicy != 0 && !SCATTER && !a.staging_on_line_grid) {
                        store_chunk16<0>(sp[u], v[u]);
                    } else {
                        store_chunk16<kPolicy>(SCATTER ? pp[u] : sp[u], v[u]);
                    }
                } else {
                    store_chunk<CS>(SCATTER ? pp[u] : sp[u], v[u]);
                }
            }
        } else {
            // Ragged end of a block, skipped rows, or a pool row that is not dword-aligned (never the case for an
            // engine's own allocations): chunk by chunk, bytes where the alignment demands it.
#pragma unroll
            for (int u = 0; u < kCPT; ++u) {
                if (!pp[u]) {
                    continue;
                }
                if (CS > 1 && (reinterpret_cast<uintptr_t>(pp[u]) & 3u) != 0) {
                    for (int i = 0; i < CS; ++i) {
                        if (SCATTER) {
                            pp[u][i] = sp[u][i];
                        } else {
                            sp[u][i] = pp[u][i];
                        }
                    }
                } else {
                    store_chunk<CS>(SCATTER ? pp[u] : sp[u], load_chunk<CS>(SCATTER ? sp[u] : pp[u]));
                }
            }
        }
        if (tr_dst) {
            store_chunk<4>(tr_dst, tr_word);
        }
    }
}

template <int CS, bool SCATTER, bool UNI_TILE, int RUN>
__global__ __launch_bounds__(kThreads) void copy_span_kernel(const CopyArgs a,
                                                             // read-only tables, never written by this kernel:
                                                             // __restrict__ lets uniform reads become scalar loads
                                                             const void *const *__restrict__ ptr_table,
                                                             const void *const *__restrict__ trailer_table,
                                                             const int32_t *__restrict__ run_start,
                                                             const int32_t *__restrict__ staging_idx,
                                                             const int32_t *__restrict__ trailer_idx) {
    copy_span_body<CS, SCATTER, UNI_TILE, RUN>(a, ptr_table, trailer_table, PtrIdx{run_start, staging_idx}, trailer_idx);
}

// The same kernel with its index tables in the argument block (host index lists).
template <int CS, bool SCATTER, bool UNI_TILE, int RUN>
__global__ __launch_bounds__(kThreads) void copy_span_kernarg_kernel(const EmbeddedIdx emb, const CopyArgs a,
                                                                     uint32_t staging_first,
                                                                     const void *const *__restrict__ ptr_table,
                                                                     const void *const *__restrict__ trailer_table,
                                                                     const int32_t *__restrict__ trailer_idx) {
    copy_span_body<CS, SCATTER, UNI_TILE, RUN>(a, ptr_table, trailer_table, KernargIdx{emb, staging_first}, trailer_idx);
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

// emb != nullptr: the index tables are *emb (copied into the kernel's argument block by the launch), run starts from
// entry 0, staging slots from entry `staging_first`; the descriptor's d_run_start / d_staging_idx are not looked at.
template <int CS, bool UNI_TILE, int RUN>
void launch_span(const CopyArgs &a, const kvcm_copy_desc *d, bool scatter, uint32_t grid, hipStream_t stream,
                 const EmbeddedIdx *emb, uint32_t staging_first) {
    if (emb) {
        if (scatter) {
            hipLaunchKernelGGL((copy_span_kernarg_kernel<CS, true, UNI_TILE, RUN>), dim3(grid), dim3(kThreads), 0,
                               stream, *emb, a, staging_first, d->d_ptr_table, d->d_trailer_ptr_table, d->d_trailer_idx);
        } else {
            hipLaunchKernelGGL((copy_span_kernarg_kernel<CS, false, UNI_TILE, RUN>), dim3(grid), dim3(kThreads), 0,
                               stream, *emb, a, staging_first, d->d_ptr_table, d->d_trailer_ptr_table, d->d_trailer_idx);
        }
    } else if (scatter) {
        hipLaunchKernelGGL((copy_span_kernel<CS, true, UNI_TILE, RUN>), dim3(grid), dim3(kThreads), 0, stream, a,
                           d->d_ptr_table, d->d_trailer_ptr_table, d->d_run_start, d->d_staging_idx, d->d_trailer_idx);
    } else {
        hipLaunchKernelGGL((copy_span_kernel<CS, false, UNI_TILE, RUN>), dim3(grid), dim3(kThreads), 0, stream, a,
                           d->d_ptr_table, d->d_trailer_ptr_table, d->d_run_start, d->d_staging_idx, d->d_trailer_idx);
    }
}

int32_t launch_copy(const kvcm_copy_desc *d, bool scatter, hipStream_t stream, const EmbeddedIdx *emb = nullptr,
                    uint32_t staging_first = 0) {
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
    if (!d->d_ptr_table || !d->d_staging || (!emb && !d->d_run_start)) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (d->trailer_bytes > 0 && (!d->d_trailer_ptr_table || !d->d_trailer_idx)) {
        return KVCM_ERR_INVALID_ARG;
    }
    // one staging block must be addressable with 31-bit chunk numbers in every chunk size
    if (payload * d->P >= (int64_t{1} << 31)) {
        return KVCM_ERR_TOO_LARGE;
    }

    CopyArgs a{};
    a.staging = static_cast<unsigned char *>(d->d_staging);
    a.entry_stride = d->entry_stride_bytes;
    a.block_stride = d->staging_block_stride_bytes;
    a.tile_stride = d->staging_tile_stride_bytes;
    a.row_bytes = d->row_bytes;
    a.tile_payload = payload;
    a.ptrs_per_entry = static_cast<uint32_t>(d->ptrs_per_entry);
    a.runs = static_cast<uint32_t>(d->T / d->run_tokens);
    a.slot_limit = d->slot_limit;
    a.trailer_bytes = d->trailer_bytes;

    const int64_t run_bytes = static_cast<int64_t>(d->run_tokens) * d->row_bytes;
    const int32_t cls = align_class(reinterpret_cast<uint64_t>(d->d_staging) | static_cast<uint64_t>(a.block_stride) |
                                    static_cast<uint64_t>(a.tile_stride) | static_cast<uint64_t>(a.row_bytes) |
                                    static_cast<uint64_t>(a.entry_stride));
    const int cs = (cls >= 4 && (run_bytes & 15) == 0) ? 16 : (cls >= 4 ? 4 : 1);
    a.chunks_per_run = static_cast<uint32_t>(run_bytes / cs);
    a.chunks_per_tile = a.runs * a.chunks_per_run;
    a.chunks_per_block = a.chunks_per_tile * static_cast<uint32_t>(d->P);
    a.units_per_block = (a.chunks_per_block + kSpan - 1) / kSpan;
    const int64_t units = static_cast<int64_t>(d->B) * a.units_per_block;
    if (units >= (int64_t{1} << 31)) {
        return KVCM_ERR_TOO_LARGE;
    }
    a.n_units = static_cast<uint32_t>(units);
    a.div_tile = make_fastdiv(a.chunks_per_tile);
    a.div_run = make_fastdiv(a.chunks_per_run);
    a.div_entry = make_fastdiv(a.ptrs_per_entry);
    a.div_units = make_fastdiv(a.units_per_block);
    static const int xcd_remap = env_int("KVCM_COPY_XCD_REMAP", 1);  // tuning knob, read once per process
    a.xcd_remap = xcd_remap;

    int64_t grid = units;
    if (d->max_workgroups > 0) {
        grid = std::min<int64_t>(grid, d->max_workgroups);
    }
    const bool uni_tile = a.chunks_per_tile % kSpan == 0;
    const uint32_t g32 = static_cast<uint32_t>(grid);
    a.staging_on_line_grid = ((reinterpret_cast<uint64_t>(d->d_staging) | static_cast<uint64_t>(a.block_stride) |
                               static_cast<uint64_t>(a.tile_stride)) & 127u) == 0;
    if (cs == 16 && uni_tile && a.chunks_per_run % kSpan == 0) {
        launch_span<16, true, kRunPerGroup>(a, d, scatter, g32, stream, emb, staging_first);
    } else if (cs == 16 && uni_tile && kCPT == 1 && a.chunks_per_run % 64 == 0) {
        launch_span<16, true, kRunPerWave>(a, d, scatter, g32, stream, emb, staging_first);
    } else if (cs == 16 && uni_tile) {
        launch_span<16, true, kRunPerThread>(a, d, scatter, g32, stream, emb, staging_first);
    } else if (cs == 16) {
        launch_span<16, false, kRunPerThread>(a, d, scatter, g32, stream, emb, staging_first);
    } else if (cs == 4) {
        launch_span<4, false, kRunPerThread>(a, d, scatter, g32, stream, emb, staging_first);
    } else {
        launch_span<1, false, kRunPerThread>(a, d, scatter, g32, stream, emb, staging_first);
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

// Host index lists -> launches whose tables ride in the argument block. One pass over the lists does what the callers
// of the device-index entry points do on their side: range checks, and the discovery that the T slots of every block are
// runs of r consecutive slots (r = T when a manager block is k engine blocks: the block-table form, a sixteenth of the
// index reads and workgroup-uniform address arithmetic).
int32_t launch_copy_host_idx(const void *const *d_ptr_table, int32_t P, void *d_staging, int64_t block_stride,
                             int64_t staging_slots, const int32_t *h_token_idx, const int32_t *h_staging_idx, int32_t B,
                             int32_t T, int64_t row_bytes, int64_t pool_slots, int32_t max_workgroups, bool scatter,
                             hipStream_t stream) {
    if (B < 0 || T <= 0 || P <= 0 || row_bytes <= 0 || staging_slots < 0 || pool_slots < 0) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (B == 0) {
        return KVCM_OK;
    }
    if (!h_token_idx || !d_ptr_table || !d_staging) {
        return KVCM_ERR_INVALID_ARG;
    }
    int32_t r = 0;
    const int32_t walked = walk_host_idx(h_token_idx, h_staging_idx, B, T, pool_slots, staging_slots, &r);
    if (walked != KVCM_OK) {
        return walked;
    }
    const int32_t runs = T / r;
    if (runs + 1 > kEmbedInts) {
        return KVCM_ERR_TOO_LARGE;  // one block's table does not fit an argument block: upload it instead
    }
    const int32_t per_launch = kEmbedInts / (runs + 1);
    EmbeddedIdx emb;
    for (int32_t b0 = 0; b0 < B; b0 += per_launch) {
        const int32_t nb = B - b0 < per_launch ? B - b0 : per_launch;
        fill_embedded(&emb, h_token_idx, h_staging_idx, b0, nb, T, r);
        kvcm_copy_desc d = flat_desc(d_ptr_table, P, d_staging, block_stride, nullptr, r, nullptr,
                                     nb, T, row_bytes, max_workgroups);
        const int32_t rc = launch_copy(&d, scatter, stream, &emb, static_cast<uint32_t>(nb * runs));
        if (rc != KVCM_OK) {
            return rc;
        }
    }
    return KVCM_OK;
}

}  // namespace

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

int32_t kvcm_hip_batch_gather_host_idx(const void *const *d_ptr_table, int32_t P, void *d_staging,
                                       int64_t staging_block_stride_bytes, int64_t staging_slots,
                                       const int32_t *h_token_idx, const int32_t *h_staging_idx, int32_t B, int32_t T,
                                       int64_t row_bytes, int64_t pool_slots, int32_t max_workgroups,
                                       kvcm_stream_t stream) {
    return kvcm::launch_copy_host_idx(d_ptr_table, P, d_staging, staging_block_stride_bytes, staging_slots, h_token_idx,
                                      h_staging_idx, B, T, row_bytes, pool_slots, max_workgroups, false,
                                      static_cast<hipStream_t>(stream));
}

int32_t kvcm_hip_batch_scatter_host_idx(const void *const *d_ptr_table, int32_t P, const void *d_staging,
                                        int64_t staging_block_stride_bytes, int64_t staging_slots,
                                        const int32_t *h_token_idx, const int32_t *h_staging_idx, int32_t B, int32_t T,
                                        int64_t row_bytes, int64_t pool_slots, int32_t max_workgroups,
                                        kvcm_stream_t stream) {
    return kvcm::launch_copy_host_idx(d_ptr_table, P, const_cast<void *>(d_staging), staging_block_stride_bytes,
                                      staging_slots, h_token_idx, h_staging_idx, B, T, row_bytes, pool_slots,
                                      max_workgroups, true, static_cast<hipStream_t>(stream));
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
