// kvcm_hash.hip -- block keys of token-ID sequences, batched over requests.
//
// Function: GenKeyVector (kv_cache_manager/manager/cache_manager.cc:76-87) over hashInt64Array
// (kv_cache_manager/manager/hash_util.h:14-24): ONE running 64-bit state per request goes through every
// token, h <- h ^ (v + C + (h << 12) + (h >> 32)), and is emitted at every block boundary. The step mixes
// + and ^, so a request is a serial chain of len dependent steps; the parallelism is across requests.
//
// Design (gfx950, wave64): a workgroup owns 64 requests and is role-split.
//   wave 0      "chain wave": lane = request. Keeps the state in VGPRs and does nothing but the recurrence,
//               reading pre-added terms a = v + C from LDS (one ds_read_b128 per 2 steps, prefetched a whole
//               tile ahead into a second register set). A lone wave issues a dependent VALU instruction 3.5-4 ns
//               after its producer and independent ones 1.75 ns apart (measured), so the step is written for
//               depth: three dependent levels, 5 instructions (see chain_step).
//   waves 1..3  "loader waves": stream the 64 requests' tokens from HBM in [64 requests x 64 tokens] tiles with
//               16-byte buffer loads (512-byte row segments), add C, and write them transposed into a 2-slot LDS
//               ring. Each loader wave owns every third tile and keeps its loads in flight for about three
//               tile periods, so HBM latency stays off the chain. In launches of thousands of requests they also
//               write the keys out: the chain wave leaves them in an LDS buffer, and whole 512-byte rows per
//               request go to memory (kKeysSpread / kKeysBurst) instead of one 8-byte store per key and lane.
//               With 4-byte tokens such launches use tiles of 128 RAW tokens (512-byte row segments here too): the
//               loaders store what they loaded and the chain wave converts, one step ahead of its use.
// Roofline: HBM for many requests (8*block_size + 8 bytes per key); for few requests the bound is the
// dependent-instruction latency of the chain wave, which no amount of bandwidth removes.
#include "kvcm_internal.h"

#include <climits>

namespace kvcm {
namespace {

#ifndef KVCM_HASH_LOADERS
#define KVCM_HASH_LOADERS 3
#endif
#ifndef KVCM_HASH_RAW_AHEAD
#define KVCM_HASH_RAW_AHEAD 1
#endif
#ifndef KVCM_HASH_DRAIN_POLICY
#define KVCM_HASH_DRAIN_POLICY 0
#endif
#ifndef KVCM_HASH_TILE_TOKENS
#define KVCM_HASH_TILE_TOKENS 64
#endif

// Loader waves. Three, so that the four waves of a workgroup sit on the four SIMDs of a CU: the chain wave needs about
// 280 VGPRs (two register sets of 64 pre-added terms) and must not share its SIMD's register file. More loaders were
// measured with 32-token tiles (where the registers fit): no gain at 16 384 requests, 5 % slower for one batch.
constexpr int kLoaders = KVCM_HASH_LOADERS;
constexpr int kThreads = 64 * (1 + kLoaders);
constexpr int kReqs = 64;                     // requests per workgroup = lanes of the chain wave
constexpr int kTT = KVCM_HASH_TILE_TOKENS;    // tokens per request per tile
constexpr int kRing = 2;                      // LDS tiles in the ring: prefetched from, written to (the tile that is
                                              // computed on already sits in the chain wave's registers)
constexpr int kPad = 2;                       // keeps rows 16-byte aligned (b128 reads) and spreads banks
// Raw tiles (4-byte tokens, many requests in flight): a ring slot holds [64 requests x 128 RAW int32 tokens] -- the same
// bytes as 64 pre-added 64-bit terms -- so that a request's share of a tile is 512 contiguous bytes of the token stream
// instead of 256 (the memory system serves 256-byte pieces at little more than half the rate of 512-byte ones), and the
// chain wave sign-extends and adds the constant itself, one instruction per step beside the chain.
constexpr int tile_tokens(bool raw) { return raw ? 2 * kTT : kTT; }
constexpr int kRowVecs = kTT / 2;  // 16-byte pieces of one request's row of a tile, either format
// Staged keys (many requests in flight; block sizes 1, 8, 16, 32, 64 and 128): the keys of a GROUP of tiles collect in LDS
// and leave as whole rows of 512 bytes per request, see hash_tokens_kernel. A group is as many tiles as yield 64 keys per
// request: key_group_tiles(block size), i.e. one tile at block size 1, sixteen at block size 16, 128 at block size 128.
constexpr int kKeysPerGroup = 64;
constexpr int key_group_tiles(int bs, int tok = kTT) { return bs >= 1 && bs <= 2 * kTT ? kKeysPerGroup * bs / tok : 16; }
constexpr int kKeyGroupTiles = key_group_tiles(16);  // the spread form exists for block size 16 only
static_assert(key_group_tiles(1) == 1 && key_group_tiles(16) == 16 && key_group_tiles(128) == 128, "64 keys per group");
constexpr int kKeyPad = 2;
constexpr int kKeyRow = kKeysPerGroup + kKeyPad;  // one request's row of the LDS key buffer

// Workgroup barrier that waits only for this wave's LDS traffic. __syncthreads() would also drain the
// loader waves' outstanding global loads, which must stay in flight across barriers.
// Spelled with builtins so that the compiler's own wait-count bookkeeping sees the LDS wait: after it the chain
// wave's prefetched tile counts as arrived and its steps run without further waits.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0); vmcnt and expcnt left at their maxima
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// One step of the recurrence with the token term pre-added (a = v + C): h ^= a + (h << 12) + sar(h, 32).
// The wave that sets the pace is bound by the LATENCY of dependent VALU instructions (3.5-4 ns each, whatever the
// instruction; measured on a lone wave), so what counts is the depth of the dependence chain, not the instruction
// count. sar(h, 32) is the sign-extended upper half, and v_mad_i64_i32 (hi * 1 + a) adds it to `a` in ONE
// instruction that needs only the upper half of h; the shift runs beside it, and the step is three levels deep:
// {v_mad_i64_i32 | v_lshlrev_b64} -> v_lshl_add_u64 -> 2 x v_xor_b32 (10.9 ns per step against 12.4 ns for the
// four-level form shift -> add -> add -> xor).
__device__ __forceinline__ uint64_t chain_step(uint64_t h, uint64_t a) {
    uint64_t a_plus_sar, carry_out;
    asm("v_mad_i64_i32 %0, %1, %2, 1, %3"
        : "=v"(a_plus_sar), "=s"(carry_out)
        : "v"(static_cast<uint32_t>(h >> 32)), "v"(a));
    return h ^ (a_plus_sar + (h << 12));
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// sign-extended 32-bit token + C in one instruction (the compiler's own form is a shift for the sign and a 64-bit
// add): with 32-bit tokens the loader wave whose turn it is has twice as many tokens to convert per load, and its
// store phase must stay shorter than the chain wave's tile
__device__ __forceinline__ uint64_t pre_add_i32(uint32_t token) {
    uint64_t sum, carry_out;
    asm("v_mad_i64_i32 %0, %1, %2, 1, %3" : "=v"(sum), "=s"(carry_out) : "v"(token), "s"(kGolden));
    return sum;
}

// Maximum / minimum of a 32-bit value over the 64 lanes of a wave, returned as a wave-uniform value. Data-parallel
// primitives within rows of 16 lanes, then across rows: six steps of one or two instructions, against six round trips
// through the LDS crossbar for the shuffle form (0.5 us at the head of a kernel that lasts 50).
template <bool MAX>
__device__ __forceinline__ uint32_t wave_reduce_u32(uint32_t v) {
#define KVCM_DPP_STEP(CTRL)                                                                                       \
    {                                                                                                             \
        const uint32_t o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(static_cast<int>(v), static_cast<int>(v), \
                                                                             CTRL, 0xf, 0xf, false));             \
        v = MAX ? (o > v ? o : v) : (o < v ? o : v);                                                              \
    }
    KVCM_DPP_STEP(0x111)  // row_shr:1   a lane without a source keeps its own value
    KVCM_DPP_STEP(0x112)  // row_shr:2
    KVCM_DPP_STEP(0x114)  // row_shr:4
    KVCM_DPP_STEP(0x118)  // row_shr:8   lane 15 of every row now holds the row's result
    KVCM_DPP_STEP(0x142)  // row_bcast:15
    KVCM_DPP_STEP(0x143)  // row_bcast:31  lane 63 holds the wave's
#undef KVCM_DPP_STEP
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), 63));
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) { return wave_reduce_u32<true>(v); }
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) { return wave_reduce_u32<false>(v); }

// What a loader wave needs to know about its workgroup.
template <typename TokT>
struct LoaderCtx {
    const TokT *tokens;
    const int64_t *s_start;  // LDS: first token of each of the 64 requests
    int64_t last_token;      // index of the last token of the whole batch (clamp target)
    int64_t wg_first_token;  // first token of the workgroup's first request
    uint32_t wg_bytes;       // bytes from there to the end of the batch, saturated at 2^32 - 1
};

// Loader, fast form: 16-byte BUFFER loads. One load instruction covers 64 / kLPR request rows with kLPR lanes
// each, so a tile takes kNL loads per lane (32 for int64 tokens, 16 for int32). The buffer resource spans from the
// workgroup's first token to the end of the batch: the hardware returns zeros past the end instead of faulting, so
// the loads need no clamp, and a load costs two instructions (offset add + buffer_load_dwordx4). Positions past a
// request's own last hashed token read a neighbour's tokens; the chain wave never consumes those entries.
template <typename TokT, bool RAW = false>
struct BufferLoader {
    static_assert(!RAW || sizeof(TokT) == 4, "raw tiles hold 4-byte tokens");
    static constexpr int kEPL = 16 / sizeof(TokT);  // tokens per load
    static constexpr int kLPR = tile_tokens(RAW) / kEPL;  // lanes per request row
    static constexpr int kRPW = 64 / kLPR;          // request rows per load instruction
    static constexpr int kNL = kReqs / kRPW;        // loads per lane per tile
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t rel[kNL];  // byte offset of this lane's piece of row j, tile 0
    u32x4 regs[kNL];
    uint32_t lane;

    __device__ __forceinline__ void setup(const LoaderCtx<TokT> &c, uint32_t lane_) {
        lane = lane_;
        rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<TokT *>(c.tokens + c.wg_first_token), 0, c.wg_bytes,
                                                 0x00020000);
        const uint32_t sub = lane / kLPR, piece = lane % kLPR;
#pragma unroll
        for (int j = 0; j < kNL; ++j) {
            rel[j] = static_cast<uint32_t>((c.s_start[j * kRPW + sub] - c.wg_first_token) * sizeof(TokT)) + piece * 16u;
        }
    }
    __device__ __forceinline__ void issue(int64_t t0) {
        issue_half<0>(t0);
        issue_half<1>(t0);
    }
    template <int HALF>
    __device__ __forceinline__ void issue_half(int64_t t0) {
        const uint32_t tile_off = static_cast<uint32_t>(t0 * sizeof(TokT));
#pragma unroll
        for (int j = HALF * (kNL / 2); j < (HALF + 1) * (kNL / 2); ++j) {
            // aux = 2: the non-temporal bit (sc0, sc1 and both were measured as well: only nt matters). Tokens are
            // read once. Timed the way the kernel is used -- on tokens that are not in the 256 MiB memory-side cache,
            // which holds other dirty data -- the bit is worth 30 to 45 % from 4096 requests up, for either token
            // width (8192 x 4096 8-byte tokens: 68 us against 96; 16 384 x 4096 4-byte tokens: 83 against 125) and
            // 5 % for one batch. Launched over and over on the same 256 MiB or less, the kernel without the bit reads
            // that cache instead of HBM and looks 10 to 25 % faster than with it: a benchmark's artefact.
            regs[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, rel[j] + tile_off, 0, 2);
        }
    }
    // Adds the golden-ratio constant (the token term of the step is v + C) and writes the tile transposed.
    __device__ __forceinline__ void store(uint64_t (*tile)[kTT + kPad]) const {
        const uint32_t sub = lane / kLPR, piece = lane % kLPR;
        // One wait for all the loads of the tile (they were requested two tile periods ago) instead of one in front
        // of every LDS write: this phase has to fit into the chain wave's tile, and every instruction of it counts.
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0); lgkmcnt and expcnt left at their maxima
#pragma unroll
        for (int j = 0; j < kNL; ++j) {
            const u32x4 v = regs[j];
            if (RAW) {
                reinterpret_cast<u32x4 *>(&tile[j * kRPW + sub][0])[piece] = v;  // as it came: the chain wave converts
                continue;
            }
            ulonglong2 *dst = reinterpret_cast<ulonglong2 *>(&tile[j * kRPW + sub][piece * kEPL]);
            if (sizeof(TokT) == 8) {
                dst[0] = make_ulonglong2(((static_cast<uint64_t>(v.y) << 32) | v.x) + kGolden,
                                         ((static_cast<uint64_t>(v.w) << 32) | v.z) + kGolden);
            } else {
                dst[0] = make_ulonglong2(pre_add_i32(v.x), pre_add_i32(v.y));
                dst[1] = make_ulonglong2(pre_add_i32(v.z), pre_add_i32(v.w));
            }
        }
    }
};

// Loader, general form: one element per load through global addresses, positions clamped to the last token of
// the batch. Used when the workgroup's requests span 4 GiB or more, which a 32-bit buffer offset cannot address.
template <typename TokT, bool RAW = false>
struct GlobalLoader {
    static constexpr int kTok = tile_tokens(RAW);
    static constexpr int kPerLane = kReqs * kTok / 64;  // tile elements per loader lane
    LoaderCtx<TokT> c;
    TokT regs[kPerLane];
    uint32_t lane;

    __device__ __forceinline__ void setup(const LoaderCtx<TokT> &c_, uint32_t lane_) {
        c = c_;
        lane = lane_;
    }
    __device__ __forceinline__ void issue(int64_t t0) {
        issue_half<0>(t0);
        issue_half<1>(t0);
    }
    template <int HALF>
    __device__ __forceinline__ void issue_half(int64_t t0) {
#pragma unroll
        for (int j = HALF * (kPerLane / 2); j < (HALF + 1) * (kPerLane / 2); ++j) {
            const uint32_t e = lane + 64u * j;
            const int64_t pos = c.s_start[e / kTok] + t0 + (e % kTok);
            regs[j] = c.tokens[pos < c.last_token ? pos : c.last_token];
        }
    }
    __device__ __forceinline__ void store(uint64_t (*tile)[kTT + kPad]) const {
#pragma unroll
        for (int j = 0; j < kPerLane; ++j) {
            const uint32_t e = lane + 64u * j;
            if (RAW) {
                reinterpret_cast<uint32_t *>(&tile[e / kTok][0])[e % kTok] = static_cast<uint32_t>(regs[j]);
            } else {
                tile[e / kTok][e % kTok] = static_cast<uint64_t>(static_cast<int64_t>(regs[j])) + kGolden;
            }
        }
    }
};

// A loader wave's whole life. Loader lw owns tiles lw, lw + kLoaders, ...; tile t lives in ring slot t % kRing.
// Tiles 0 and 1 are published before the first barrier: the chain wave computes on tile k while its LDS reads of
// tile k+1 are already in flight, so tile k+2 is what gets written during iteration k (its slot held tile k-1,
// which the chain wave pulled into registers an iteration ago). A loader issues the loads of its next tile right
// AFTER the barrier that published its previous one, so they stay in flight for kLoaders - 1 tile periods while the
// data waits in the loader's registers, not in LDS: more loaders = more bytes in flight per CU at no LDS cost.
// What a loader wave needs to write out a group of staged keys (KS kernels only).
struct KeyDrain {
    const uint64_t *s_keys;   // LDS: [2][request][kKeyRow] keys of the group being filled and of the one before
    const int64_t *s_keypos;                                    // LDS: index of each request's first key, -1 = no request
    int64_t *keys;
    int32_t full_tiles;  // tiles in which no request has run out of tokens and whose keys may be staged
};

// One group of staged keys, LDS -> global: every store instruction writes two requests' rows of 512 bytes, whole cache
// lines, non-temporal. Written as 8-byte stores from the chain wave (one line per lane, a sixteenth of it at a time)
// the 32 MiB of keys of a 16 384-request batch cost 20 us of a 107 us launch -- not for their bytes but for what they do
// to the memory system in the middle of the token stream; the same stores into a buffer that stays in the L2 cost
// nothing, and so do they as one burst after the last token. Whole rows at intervals of sixteen tiles recover a third
// of that.
// A group is 32 such store instructions; `step` (0..15) selects two of them, so that the work spreads over the sixteen
// tiles that follow the group instead of holding one loader back from its next barrier.
constexpr int kDrainSteps = kKeyGroupTiles;
constexpr int kDrainPerStep = kReqs * kKeysPerGroup / 128 / kDrainSteps;
__device__ __forceinline__ void drain_keys(const KeyDrain &kd, int32_t group, int32_t step, uint32_t lane) {
    const uint32_t buf = static_cast<uint32_t>(group) & 1u;
#pragma unroll
    for (int j = 0; j < kDrainPerStep; ++j) {
        const uint32_t c = static_cast<uint32_t>(step * kDrainPerStep + j) * 64u + lane;  // 16-byte piece of the group's keys
        const uint32_t row = c / (kKeysPerGroup / 2), piece = c % (kKeysPerGroup / 2);
        const int64_t first = kd.s_keypos[row];
        const u32x4 v = *reinterpret_cast<const u32x4 *>(kd.s_keys + (buf * kReqs + row) * kKeyRow + piece * 2);
        if (first >= 0) {
            typedef u32x4 u32x4_a8 __attribute__((aligned(8)));
            __builtin_nontemporal_store(
                v, reinterpret_cast<u32x4_a8 *>(kd.keys + first + static_cast<int64_t>(group) * kKeysPerGroup + piece * 2));
        }
    }
}

// Half of a closed group (`part` = 0 or 1: every other store instruction), in bursts of eight row pieces: all LDS reads
// of a burst are under way before its first store goes out, so the loader is back at its loads after about 0.2 us.
__device__ __forceinline__ void drain_half(const KeyDrain &kd, int32_t group, int32_t part, uint32_t lane) {
    const uint32_t buf = static_cast<uint32_t>(group) & 1u;
    constexpr int kBurst = 8;
    static_assert((kDrainSteps * kDrainPerStep / 2) % kBurst == 0, "whole bursts");
#pragma unroll 1
    for (int32_t base = 0; base < kDrainSteps * kDrainPerStep / 2; base += kBurst) {
        int64_t first[kBurst];
        u32x4 v[kBurst];
        uint32_t piece[kBurst];
#pragma unroll
        for (int i = 0; i < kBurst; ++i) {
            const uint32_t c = static_cast<uint32_t>((base + i) * 2 + part) * 64u + lane;
            const uint32_t row = c / (kKeysPerGroup / 2);
            piece[i] = c % (kKeysPerGroup / 2);
            first[i] = kd.s_keypos[row];
            v[i] = *reinterpret_cast<const u32x4 *>(kd.s_keys + (buf * kReqs + row) * kKeyRow + piece[i] * 2);
        }
#pragma unroll
        for (int i = 0; i < kBurst; ++i) {
            if (first[i] >= 0) {
                // written through at system scope: 97-99 us for 16 384 x 4096 tokens where the same stores take
                // 101-105 us non-temporal, 104 plain, 100-101 with sc1 alone (65 536 x 4096: 385-388 against 399-403 us)
                int64_t *dst = kd.keys + first[i] + static_cast<int64_t>(group) * kKeysPerGroup + piece[i] * 2;
#if KVCM_HASH_DRAIN_POLICY == 0
                asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" : : "v"(dst), "v"(v[i]) : "memory");
#elif KVCM_HASH_DRAIN_POLICY == 1
                asm volatile("global_store_dwordx4 %0, %1, off nt" : : "v"(dst), "v"(v[i]) : "memory");
#elif KVCM_HASH_DRAIN_POLICY == 2
                asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(dst), "v"(v[i]) : "memory");
#elif KVCM_HASH_DRAIN_POLICY == 3
                asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" : : "v"(dst), "v"(v[i]) : "memory");
#else
                asm volatile("global_store_dwordx4 %0, %1, off" : : "v"(dst), "v"(v[i]) : "memory");
#endif
            }
        }
    }
}

// How a kernel's keys reach memory: from the chain wave, one at a time (kKeysDirect); staged in LDS and written by the
// loaders a sixteenth of a group per tile (kKeysSpread); staged and written a whole group at once, right after the
// barrier that closes it (kKeysBurst); the host chooses by token width and number of requests (the timings stand at
// launch_hash). Writes that all workgroups issue at the same moments disturb the token stream less than writes spread
// evenly through it, as long as the loaders do not fall behind while they issue them.
constexpr int kKeysDirect = 0, kKeysSpread = 1, kKeysBurst = 2;
// A workgroup of a spread kernel whose requests are shorter than this many tiles stores its keys directly: what the last
// group costs after the loop (about 1.5 us) is more than staging saves on 2048 tokens.
constexpr int kSpreadFromTiles = 32;

// The steps [first_step, kDrainSteps) of a group that belong to loader `me` (step % kLoaders == me), all LDS reads
// under way before the first store: nothing else is left to do when this runs, so round trips would add up.
__device__ __forceinline__ void drain_tail(const KeyDrain &kd, int32_t group, int32_t first_step, int32_t me,
                                           uint32_t lane) {
    const uint32_t buf = static_cast<uint32_t>(group) & 1u;
    constexpr int kMaxSteps = (kDrainSteps + kLoaders - 1) / kLoaders;
    constexpr int kN = kMaxSteps * kDrainPerStep;
    typedef u32x4 u32x4_a8 __attribute__((aligned(8)));
    const int32_t s0 = first_step + (me - first_step % kLoaders + kLoaders) % kLoaders;
    int64_t first[kN];
    u32x4 v[kN];
    uint32_t piece[kN];
#pragma unroll
    for (int i = 0; i < kN; ++i) {
        const int32_t step = s0 + (i / kDrainPerStep) * kLoaders;
        first[i] = -1;
        if (step < kDrainSteps) {
            const uint32_t c = static_cast<uint32_t>(step * kDrainPerStep + i % kDrainPerStep) * 64u + lane;
            const uint32_t row = c / (kKeysPerGroup / 2);
            piece[i] = c % (kKeysPerGroup / 2);
            first[i] = kd.s_keypos[row];
            v[i] = *reinterpret_cast<const u32x4 *>(kd.s_keys + (buf * kReqs + row) * kKeyRow + piece[i] * 2);
        }
    }
#pragma unroll
    for (int i = 0; i < kN; ++i) {
        if (first[i] >= 0) {
            __builtin_nontemporal_store(
                v[i], reinterpret_cast<u32x4_a8 *>(kd.keys + first[i] + static_cast<int64_t>(group) * kKeysPerGroup +
                                                  piece[i] * 2));
        }
    }
}

template <typename Loader, typename TokT, int KS, int G, int TOK>
__device__ __forceinline__ void run_loader(const LoaderCtx<TokT> &ctx, uint64_t (*s_tile)[kReqs][kTT + kPad],
                                           int64_t lw, int64_t ntiles, uint32_t lane, const KeyDrain &kd) {
    static_assert(kRing == 2 && kLoaders >= 3, "two ring slots: prefetched from, written to");
    // the burst drain splits a closed group between the kLoaders - 1 loaders whose tile is not due, as halves
    static_assert(KS != kKeysBurst || kLoaders == 3, "drain_half deals a group out to exactly two loaders");
    static_assert((G & (G - 1)) == 0 && (KS != kKeysSpread || G == kKeyGroupTiles), "groups of 2^n tiles; spread: 16");
    Loader ld;
    ld.setup(ctx, lane);
    // 32-bit counters: the loop control stays in scalar registers (there are no ordered 64-bit scalar compares); a
    // request of 2^37 tokens does not fit the memory of the device
    const int32_t nt = static_cast<int32_t>(ntiles), me = static_cast<int32_t>(lw);
    if (me < nt) {
        ld.issue(static_cast<int64_t>(me) * TOK);
    }
    if (me < 2 && me < nt) {
        ld.store(s_tile[me]);
    }
    lds_barrier();
    if (me < 2 && me + kLoaders < nt) {
        ld.issue(static_cast<int64_t>(me + kLoaders) * TOK);
    }
    // tile 2 goes where tile 0 lies: not before the chain wave has pulled tile 0 into its registers
    lds_barrier();
    int32_t turn = 2 % kLoaders;  // loader whose tile is due: (k + 2) % kLoaders
    int slot = 2 % kRing;         // ring slot of that tile: (k + 2) % kRing
    bool was_mine = false;
    for (int32_t k = 0; k < nt; ++k) {
        const int32_t nxt = k + 2;  // tile that must be in LDS when this iteration ends
        const bool my_turn = turn == me;
        const bool mine = my_turn && nxt < nt;
        if (mine) {
            ld.store(s_tile[slot]);
        }
        if (KS == kKeysSpread && k >= kKeyGroupTiles && (k / kKeyGroupTiles) * kKeyGroupTiles <= kd.full_tiles &&
            (turn == 0 ? kLoaders - 1 : turn - 1) == me) {
            // The group of staged keys before the one this tile belongs to was closed by an earlier barrier, and its
            // buffer is not written again before the barrier that ends this group: a sixteenth of it leaves per tile,
            // here, in front of the barrier, through the loader that published a tile an iteration ago and has nothing
            // to do until the barrier (its own next wait for memory is two tiles away, so the stores are not waited for).
            drain_keys(kd, k / kKeyGroupTiles - 1, k & (kKeyGroupTiles - 1), lane);
        }
        turn = turn + 1 == kLoaders ? 0 : turn + 1;
        slot = slot + 1 == kRing ? 0 : slot + 1;
        lds_barrier();
        // the loads of this loader's next tile go out in two halves, one tile period apart: a burst of 32 load
        // instructions sits in the CU's memory pipeline in front of the chain wave's key stores
        // (which of the two forms runs is a compile-time matter: with both in one loop body the compiler waits for
        // all outstanding loads where the paths meet, and a kernel that does so takes 80 us for a batch instead of 58)
        if (KS == kKeysSpread || (KS == kKeysBurst && sizeof(TokT) == 8)) {
            // no key stores of the chain wave to keep out of the way of: 2 to 5 % faster from 4096 requests than in
            // halves (spread form); in the burst form of 8-byte tokens 4 % at 10 240 and 12 288 requests, 7 to 10 % for
            // the prefix chain up to 2048 chains, nothing at 16 384. Raw tiles of 4-byte tokens lose 5 % by it at
            // 16 384 requests (66.8 against 63.6 us) and keep the halves.
            if (mine && nxt + kLoaders < nt) {
                ld.issue(static_cast<int64_t>(nxt + kLoaders) * TOK);
            }
        } else {
            if (mine && nxt + kLoaders < nt) {
                ld.template issue_half<0>(static_cast<int64_t>(nxt + kLoaders) * TOK);
            }
            if (was_mine && nxt - 1 + kLoaders < nt) {
                ld.template issue_half<1>(static_cast<int64_t>(nxt - 1 + kLoaders) * TOK);
            }
        }
        was_mine = mine;
        if (KS == kKeysBurst && (k & (G - 1)) == G - 1 && k < kd.full_tiles && turn != me) {
            // The barrier above closed a group of G tiles. The loader whose tile is due next leaves it alone (its next
            // wait for memory would wait for these stores as well); the other two write half of it each.
            drain_half(kd, k / G, (me - turn + kLoaders) % kLoaders - 1, lane);
        }
    }
    if (KS == kKeysSpread) {
        // What the loop did not reach of the last staged group (all of it when the request ends with the group), the
        // steps dealt out to the loaders; no barrier follows, and nobody writes the buffers any more.
        const int32_t last = kd.full_tiles / kKeyGroupTiles - 1;
        if (last >= 0) {
            const int32_t done = nt - (last + 1) * kKeyGroupTiles;  // steps the loop has taken for this group
            drain_tail(kd, last, done < 0 ? 0 : done, me, lane);
        }
    }
}

// The chain wave's work on one tile: kTT steps from the lane's pre-added terms `a`, a key at every block
// boundary. MASKED = some lane may have run out of tokens inside this tile (ragged batch). Such a lane keeps stepping
// -- on a neighbour's tokens or on zeros, whatever the loaders fetched past its end -- because masking the steps would
// cost the wave a compare, two exec writes and a branch per chunk; its state is dead from there on, and only its KEY
// STORES are masked. The common case of equally long requests takes the unmasked path, which has no per-lane compare.
// BS > 0 = the block size is this compile-time constant (a divisor or a multiple of the tile): the places where a key
// is due are then known when the code is written, and the scalar bookkeeping (add, compare, branch per chunk: one
// instruction slot in sixteen of the wave that sets the pace) disappears from the loop.
// STAGED (unmasked tiles, block size a compile-time constant up to a tile): the tile's keys go to the lane's row of the LDS key buffer, `staged_row`
// pointing at the tile's first key there; a loader wave writes the rows out (drain_keys).
template <int CHUNK, bool MASKED, int BS, bool STAGED = false, bool RAW = false>
__device__ __forceinline__ void run_tile(const ulonglong2 (&a)[kRowVecs], uint64_t &h, int64_t t0, int64_t my_ntok,
                                         int32_t &since_key, int32_t block_size, int64_t *__restrict__ keys,
                                         int64_t &key_pos, uint64_t *staged_row = nullptr) {
    constexpr int TOK = tile_tokens(RAW);  // steps per tile
    static_assert(!STAGED || (!MASKED && BS >= 1 && BS <= 2 * kTT), "keys are staged for whole tiles of blocks up to two tiles");
    static_assert(BS == 0 || (BS % CHUNK == 0 && (TOK % BS == 0 || BS % TOK == 0)), "block size fits the tiling");
    // tokens of this lane that are hashed and lie in this tile or before its end: a block that ends at position p of
    // the tile belongs to the lane iff p <= left (my_ntok is a multiple of the block size)
    const int64_t left64 = my_ntok - t0;
    const int32_t left = MASKED ? static_cast<int32_t>(left64 < TOK ? (left64 > 0 ? left64 : 0) : TOK) : TOK;
    // raw tiles: four 4-byte tokens per 16-byte piece; sign-extension + C is one v_mad_i64_i32 off the chain, issued
    // KVCM_HASH_RAW_AHEAD steps before the step that consumes it
    const auto raw_token = [&](int s) -> uint32_t {
        const uint64_t pair = (s & 2) ? a[s / 4].y : a[s / 4].x;
        return static_cast<uint32_t>((s & 1) ? pair >> 32 : pair);
    };
    constexpr int kAhead = KVCM_HASH_RAW_AHEAD;
    uint64_t pre[kAhead > 0 ? kAhead : 1];
    if (RAW) {
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
            pre[i] = pre_add_i32(raw_token(i));
        }
    }
#pragma unroll
    for (int c = 0; c < TOK; c += CHUNK) {
#pragma unroll
        for (int s = c; s < c + CHUNK; ++s) {
            if (RAW && kAhead > 0) {
                const uint64_t now = pre[s % kAhead];
                if (s + kAhead < TOK) {
                    pre[s % kAhead] = pre_add_i32(raw_token(s + kAhead));
                }
                h = chain_step(h, now);
            } else if (RAW) {
                h = chain_step(h, pre_add_i32(raw_token(s)));
            } else {
                h = chain_step(h, (s & 1) ? a[s / 2].y : a[s / 2].x);
            }
        }
        bool key_due;
        if (BS == 0) {
            since_key += CHUNK;
            key_due = since_key == block_size;
            if (key_due) {
                since_key = 0;
            }
        } else if (BS <= TOK) {
            key_due = (c + CHUNK) % BS == 0;  // tiles start on block boundaries
        } else {
            key_due = c + CHUNK == TOK && (t0 + TOK) % BS == 0;
        }
        if (key_due) {
            if (STAGED) {
                staged_row[BS > TOK ? 0 : (c + CHUNK) / (BS > 0 ? BS : 1) - 1] = h;
            } else if (!MASKED || c + CHUNK <= left) {
                keys[key_pos] = static_cast<int64_t>(h);
            }
            key_pos += 1;
        }
    }
}

__device__ __forceinline__ void read_row(ulonglong2 (&a)[kRowVecs], const uint64_t *row_ptr) {
    const ulonglong2 *row = reinterpret_cast<const ulonglong2 *>(row_ptr);
#pragma unroll
    for (int i = 0; i < kRowVecs; ++i) {
        a[i] = row[i];
    }
}

// CHUNK = steps between two looks at the block boundary: 8 when block_size % 8 == 0 (a lane is then
// active for whole chunks or not at all), otherwise 1. BS = block size when it is 1, 8, 16, 32, 64 or 128, otherwise 0.
// KS != kKeysDirect ("keys staged", block sizes 1 to 64; chosen by the host for batches of many requests, where the launch
// is bound by memory and not by the chain): the chain wave writes its keys into an LDS buffer instead of to memory, and
// after every group of tiles in which every request is whole the loader waves write the group out as rows of 512
// bytes, spread over the next group's tiles (block size 16) or at once.
template <typename TokT, int CHUNK, int BS, int KS = kKeysDirect, bool RAW = false>
__global__ __launch_bounds__(kThreads) void hash_tokens_kernel(const TokT *__restrict__ tokens,
                                                              const int64_t *__restrict__ token_offsets, int32_t R,
                                                              int32_t block_size, uint64_t seed,
                                                              int64_t *__restrict__ keys,
                                                              const int64_t *__restrict__ key_offsets,
                                                              int32_t force_global_loads) {
    __shared__ __attribute__((aligned(16))) uint64_t s_tile[kRing][kReqs][kTT + kPad];
    __shared__ int64_t s_start[kReqs];
    __shared__ int64_t s_ntok[kReqs];
    static_assert(!KS || (BS >= 1 && BS <= 2 * kTT), "keys are staged for block sizes up to two tiles");
    static_assert(KS != kKeysSpread || BS == 16, "the spread form exists for 16-token blocks");
    constexpr int TOK = tile_tokens(RAW);        // tokens per request per tile
    constexpr int G = key_group_tiles(BS, TOK);  // tiles per group of staged keys
    static_assert(!KS || G >= 1, "a group of staged keys is at least one tile");
    constexpr int kDiv = BS > 0 ? BS : 1;  // the first key of tile t of a group lies at position t * TOK / BS of the row
    __shared__ __attribute__((aligned(16))) uint64_t s_keys[KS ? 2 * kReqs * kKeyRow : 2];
    __shared__ int64_t s_keypos[KS ? kReqs : 1];

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t r = static_cast<int64_t>(blockIdx.x) * kReqs + lane;

    // Everything that has to come from memory before the first tile can be requested is asked for here, by all four
    // waves at once: one trip to memory instead of three in a row (a 64 x 4096 batch is only ~50 us long).
    int64_t my_ntok = 0, key_pos = 0;
    LoaderCtx<TokT> ctx;
    bool buffer_loads = false;
    if (wave == 0) {
        int64_t start = token_offsets[static_cast<int64_t>(blockIdx.x) * kReqs];  // rows past R idle at the first row
        if (r < R) {
            start = token_offsets[r];
            const int64_t n = token_offsets[r + 1] - start;
            my_ntok = (n / block_size) * block_size;  // a trailing partial block yields no key
            key_pos = key_offsets ? key_offsets[r] : r * ((token_offsets[1] - token_offsets[0]) / block_size);
        }
        s_start[lane] = start;
        s_ntok[lane] = my_ntok;
        if (KS) {
            s_keypos[lane] = r < R ? key_pos : -1;
        }
    } else {
        ctx.tokens = tokens;
        ctx.s_start = s_start;
        const int64_t total = token_offsets[R];
        ctx.last_token = total - 1;  // >= 0 whenever a tile is loaded: some request has a full block then
        const int64_t r_first = static_cast<int64_t>(blockIdx.x) * kReqs;
        const int64_t r_end = r_first + kReqs < R ? r_first + kReqs : R;
        ctx.wg_first_token = token_offsets[r_first];
        const uint64_t to_end = static_cast<uint64_t>(total - ctx.wg_first_token) * sizeof(TokT);
        ctx.wg_bytes = to_end > 0xFFFFFFFFull ? 0xFFFFFFFFu : static_cast<uint32_t>(to_end);
        const uint64_t wg_span = static_cast<uint64_t>(token_offsets[r_end] - ctx.wg_first_token) * sizeof(TokT);
        buffer_loads = !force_global_loads && wg_span < 0xFFF00000ull;
    }
    __syncthreads();

    // Tiles of the longest request (how long the workgroup runs) and whole tiles of the shortest (from where on some
    // lane has run out): max and min over the 64 lanes of per-lane tile counts, which fit 32 bits (a request of 2^37
    // tokens does not fit the memory of the device). Rows past R in the last workgroup count for neither.
    const int64_t lane_ntok = s_ntok[lane];
    const uint32_t ntiles_u = wave_max_u32(static_cast<uint32_t>((lane_ntok + TOK - 1) / TOK));
    const uint32_t full_u = wave_min_u32(r < R ? static_cast<uint32_t>(lane_ntok / TOK) : 0xFFFFFFFFu);
    const int64_t ntiles = ntiles_u;  // uniform over the workgroup
    if (ntiles == 0) {
        return;
    }
    // tiles [0, n_full) are those in which no request has run out of tokens
    const int32_t n_full = static_cast<int32_t>(full_u < ntiles_u ? full_u : ntiles_u);
    // ... and of those, the ones whose keys may be staged (whole groups of them are)
    const int32_t n_stageable = KS == kKeysSpread && ntiles_u < static_cast<uint32_t>(kSpreadFromTiles) ? 0 : n_full;
    if (wave != 0) {
        // ---------------------------------------------------------------- loader waves
        const KeyDrain kd{s_keys, s_keypos, keys, n_stageable};
        if (buffer_loads) {
            run_loader<BufferLoader<TokT, RAW>, TokT, KS, G, TOK>(ctx, s_tile, wave - 1, ntiles, lane, kd);
        } else {
            run_loader<GlobalLoader<TokT, RAW>, TokT, KS, G, TOK>(ctx, s_tile, wave - 1, ntiles, lane, kd);
        }
        return;
    }

    // -------------------------------------------------------------------- chain wave
    uint64_t h = seed;
    int32_t since_key = 0;  // uniform: all lanes step in lockstep from token 0
    lds_barrier();
    if (r >= R) {
        // A lane without a request leaves here; the wave goes on without it (every workgroup has at least one request,
        // so the wave still meets every barrier). This keeps the unmasked path, whose key stores are unconditional,
        // usable when R is not a multiple of 64.
        return;
    }
    ulonglong2 cur[kRowVecs], nxt[kRowVecs];
    read_row(cur, &s_tile[0][lane][0]);
    lds_barrier();  // tile 0 is in registers: its slot may take tile 2
    // Loop control in 32-bit scalars (there are no ordered 64-bit scalar compares, and every vector compare is an issue
    // slot of this wave). A request of 2^37 tokens does not fit the memory of the device, so the tile count fits 32 bits.
    const int32_t nt = static_cast<int32_t>(ntiles);
    int ring = 0;
    for (int32_t k = 0; k < nt; k += 2) {
        // even tile: compute on `cur`, prefetch the odd tile into `nxt`; then the other way round
        int ring1 = ring + 1 == kRing ? 0 : ring + 1;
        if (k + 1 < nt) {
            read_row(nxt, &s_tile[ring1][lane][0]);
        }
        // a group of G tiles is staged when all of its tiles are whole for every request
        const int32_t group = k / G;
        const bool staged = KS && (group + 1) * G <= n_stageable;
        uint64_t *staged_row = KS ? s_keys + ((group & 1) * kReqs + lane) * kKeyRow + (k & (G - 1)) * TOK / kDiv : nullptr;
        if (KS && staged) {
            run_tile<CHUNK, false, BS, KS != kKeysDirect, RAW>(cur, h, static_cast<int64_t>(k) * TOK, my_ntok, since_key, block_size, keys,
                                           key_pos, staged_row);
        } else if (k < n_full) {
            run_tile<CHUNK, false, BS, false, RAW>(cur, h, static_cast<int64_t>(k) * TOK, my_ntok, since_key, block_size, keys,
                                       key_pos);
        } else {
            run_tile<CHUNK, true, BS, false, RAW>(cur, h, static_cast<int64_t>(k) * TOK, my_ntok, since_key, block_size, keys,
                                      key_pos);
        }
        lds_barrier();
        if (k + 1 >= nt) {
            break;
        }
        ring = ring1 + 1 == kRing ? 0 : ring1 + 1;
        if (k + 2 < nt) {
            read_row(cur, &s_tile[ring][lane][0]);
        }
        const int32_t group1 = (k + 1) / G;  // the same group unless a group is one tile
        const bool staged1 = KS && (group1 + 1) * G <= n_stageable;
        uint64_t *staged_row1 =
            KS ? s_keys + ((group1 & 1) * kReqs + lane) * kKeyRow + ((k + 1) & (G - 1)) * TOK / kDiv : nullptr;
        if (KS && staged1) {
            run_tile<CHUNK, false, BS, KS != kKeysDirect, RAW>(nxt, h, static_cast<int64_t>(k + 1) * TOK, my_ntok, since_key, block_size,
                                           keys, key_pos, staged_row1);
        } else if (k + 1 < n_full) {
            run_tile<CHUNK, false, BS, false, RAW>(nxt, h, static_cast<int64_t>(k + 1) * TOK, my_ntok, since_key, block_size, keys,
                                       key_pos);
        } else {
            run_tile<CHUNK, true, BS, false, RAW>(nxt, h, static_cast<int64_t>(k + 1) * TOK, my_ntok, since_key, block_size, keys,
                                      key_pos);
        }
        lds_barrier();
    }
}

// ------------------------------------------------------------------------------------------- SHA-256

__constant__ uint32_t kShaK[64] = {
    0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5,
    0xd807aa98, 0x12835b01, 0x243185be, 0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174,
    0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa, 0x5cb0a9dc, 0x76f988da,
    0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967,
    0x27b70a85, 0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85,
    0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3, 0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070,
    0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f, 0x682e6ff3,
    0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};

__device__ __forceinline__ uint32_t rotr(uint32_t x, int n) { return __builtin_amdgcn_alignbit(x, x, n); }

// One FIPS 180-4 compression; w holds the 16 big-endian message words and is used as the rolling schedule.
__device__ void sha256_compress(uint32_t (&st)[8], uint32_t (&w)[16]) {
    uint32_t a = st[0], b = st[1], c = st[2], d = st[3], e = st[4], f = st[5], g = st[6], h = st[7];
#pragma unroll
    for (int i = 0; i < 64; ++i) {
        if (i >= 16) {
            const uint32_t w15 = w[(i + 1) & 15], w2 = w[(i + 14) & 15];
            const uint32_t s0 = rotr(w15, 7) ^ rotr(w15, 18) ^ (w15 >> 3);
            const uint32_t s1 = rotr(w2, 17) ^ rotr(w2, 19) ^ (w2 >> 10);
            w[i & 15] = w[i & 15] + s0 + w[(i + 9) & 15] + s1;
        }
        const uint32_t S1 = rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25);
        const uint32_t ch = (e & f) ^ (~e & g);
        const uint32_t t1 = h + S1 + ch + kShaK[i] + w[i & 15];
        const uint32_t S0 = rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22);
        const uint32_t mj = (a & b) ^ (a & c) ^ (b & c);
        const uint32_t t2 = S0 + mj;
        h = g;
        g = f;
        f = e;
        e = d + t1;
        d = c;
        c = b;
        b = a;
        a = t1 + t2;
    }
    st[0] += a;
    st[1] += b;
    st[2] += c;
    st[3] += d;
    st[4] += e;
    st[5] += f;
    st[6] += g;
    st[7] += h;
}

// Byte i of the padded message of length len: data, 0x80, zeros, 64-bit big-endian bit length.
__device__ __forceinline__ uint32_t padded_byte(const uint8_t *msg, int64_t len, int64_t padded_len, int64_t i) {
    if (i < len) {
        return msg[i];
    }
    if (i == len) {
        return 0x80u;
    }
    if (i >= padded_len - 8) {
        const uint64_t bits = static_cast<uint64_t>(len) * 8u;
        return static_cast<uint32_t>((bits >> (8 * (padded_len - 1 - i))) & 0xffu);
    }
    return 0u;
}

// One lane per string: key = big-endian signed int64 of SHA-256(bytes)[0:8]
// (kv_cache_manager/py_connector/sglang/connector.py:397-401).
__global__ __launch_bounds__(64) void sha256_first8_kernel(const uint8_t *__restrict__ bytes,
                                                           const int64_t *__restrict__ offsets, int32_t N,
                                                           int64_t *__restrict__ out) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= N) {
        return;
    }
    const uint8_t *msg = bytes + offsets[i];
    const int64_t len = offsets[i + 1] - offsets[i];
    const int64_t padded_len = ((len + 8) / 64 + 1) * 64;
    uint32_t st[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
    for (int64_t base = 0; base < padded_len; base += 64) {
        uint32_t w[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int64_t p = base + 4 * j;
            w[j] = (padded_byte(msg, len, padded_len, p) << 24) | (padded_byte(msg, len, padded_len, p + 1) << 16) |
                   (padded_byte(msg, len, padded_len, p + 2) << 8) | padded_byte(msg, len, padded_len, p + 3);
        }
        sha256_compress(st, w);
    }
    out[i] = static_cast<int64_t>((static_cast<uint64_t>(st[0]) << 32) | st[1]);
}

// ------------------------------------------------------------------------------------------- iov CRC-32

// kv_cache_manager/client/src/internal/sdk/sdk_buffer_check_util.cu:10-19.
__device__ __forceinline__ uint32_t crc32_byte(uint32_t crc, uint8_t data) {
    crc ^= data;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t mask = 0u - (crc & 1u);
        crc = (crc >> 1) ^ (0xEDB88320u & mask);
    }
    return crc;
}

// One lane per iov, head bytes then tail bytes through one running CRC (sdk_buffer_check_util.cu:21-44).
__global__ __launch_bounds__(256) void iov_crc32_kernel(const kvcm_iov_device *__restrict__ iovs, int32_t n,
                                                        uint32_t *__restrict__ out, size_t cal_bytes) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    const uint8_t *p = static_cast<const uint8_t *>(iovs[i].base);
    const size_t size = iovs[i].size;
    if (!p || size < cal_bytes) {
        // cal_bytes comes from the first iov only: an iov without an address, or shorter than that, is not read at
        // all and gets the value 0 (the reference reads out of bounds here). 0 is also a possible CRC, so callers
        // that cannot rule such iovs out check them on the host first, as the C++ and Python layers above do.
        out[i] = 0;
        return;
    }
    uint32_t crc = 0xFFFFFFFFu;
    for (size_t k = 0; k < cal_bytes; ++k) {
        crc = crc32_byte(crc, p[k]);
    }
    for (size_t k = size - cal_bytes; k < size; ++k) {
        crc = crc32_byte(crc, p[k]);
    }
    out[i] = ~crc;
}

// Non-zero makes every launch take the loader path that a workgroup spanning >= 4 GiB of tokens would take. A
// compile-time matter: the shipped library is built with 0 and has no switch; the parity tests build this file a second
// time, with KVCM_TEST_FORCE_GENERAL_LOADER=1, into a library of their own.
#ifndef KVCM_TEST_FORCE_GENERAL_LOADER
#define KVCM_TEST_FORCE_GENERAL_LOADER 0
#endif
constexpr int32_t kForceGeneralLoader = KVCM_TEST_FORCE_GENERAL_LOADER;

// How keys reach memory, by block size, token width and number of requests in the launch (hash_tokens_kernel<.., KS>).
// Chosen from timings on tokens that are not in the memory-side cache. 16-token blocks, us for requests of 4096 tokens,
// direct / spread / burst:
//   8-byte tokens   64: 61 / 58 / 60      1024: 61 / 59 / 63     4096: 65 / 60 / 64      8192: 76 / 64 / 70
//                   10 240: 83 / 76 / 73  12 288: 92 / 85 / 83   16 384: 112 / 111 / 107   32 768: 227 / 219 / 209
//   4-byte tokens   4096: 56 / 58 / 63    8192: 58 / 58 / 64     10 240: 64 / 62 / 66    12 288: 72 / 66 / 67
//                   16 384: 85 / 81 / 78  32 768: 159 / 151 / 151
// 8-byte tokens: direct below 2048 requests (there the spread form gains 2 to 4 % on tokens from HBM and loses as much
// on resident ones, and costs requests of 1024 tokens 6 %), spread from 2048, burst from 10 240.
// 4-byte tokens: direct below 12 288, burst from there -- and the burst form of 4-byte tokens is the one with raw tiles
// (RAW = true; the 4-byte figures of these tables are those of the 64-token tiles of pre-added terms it replaced:
// 16 384 requests 78 -> 62-66 us) (the spread form would gain 3 % between 10 240 and 16 384
// requests: not worth one more kernel).
// Other block sizes, direct / burst:
//   block size 1, 8-byte tokens   64: 146 / 129   2048: 158 / 136   8192: 241 / 161   16 384: 300 / 202   32 768: 641 / 415
//                 4-byte tokens   512: 115 / 119  1024: 119 / 120 (resident: 116 / 92)   8192: 184 / 141   16 384: 249 / 175
//   block size 8, 8-byte tokens   1024: 72 / 69 (resident: 61 / 64)   2048: 74 / 70   8192: 98 / 77   16 384: 137 / 112
//                 4-byte tokens   8192: 69 / 71   12 288: 82 / 75   16 384: 100 / 83
//   block size 32, 8-byte tokens  4096: 60 / 61   8192: 69 / 65   12 288: 93 / 76   16 384: 115 / 99
//                  4-byte tokens  8192: 57 / 57   12 288: 69 / 62   16 384: 84 / 70
//   block size 64, 8-byte tokens  4096: 58 / 60   8192: 67 / 63   12 288: 85 / 75   16 384: 109 / 93
//                  4-byte tokens  8192: 55 / 57   12 288: 64 / 60   16 384: 77 / 72
//   block size 128 (requests of 16 384 tokens: a group is 8192), 8-byte tokens  4096: 210 / 208   8192: 242 / 222
//                  16 384: 419 / 356;  4-byte tokens  8192: 198 / 197   16 384: 264 / 204
#ifndef KVCM_HASH_SPREAD_FROM_8
#define KVCM_HASH_SPREAD_FROM_8 2048
#endif
// requests from which a launch takes the burst form; INT32_MAX = never
constexpr int32_t burst_from(int32_t block_size, bool tokens_8_byte) {
    switch (block_size) {
        case 1: return tokens_8_byte ? 1 : 1024;
        case 8: return tokens_8_byte ? 2048 : 12288;
        case 16: return tokens_8_byte ? 10240 : 12288;
        case 32: return tokens_8_byte ? 8192 : 12288;
        case 64: return tokens_8_byte ? 8192 : 12288;
        case 128: return tokens_8_byte ? 8192 : 12288;
        default: return INT32_MAX;
    }
}
#ifndef KVCM_HASH_BURST_SCALE  // for experiments: 0 = burst wherever it exists, a large number = never
#define KVCM_HASH_BURST_SCALE 1
#endif

template <typename TokT>
int32_t launch_hash(const TokT *d_tokens, const int64_t *d_token_offsets, int32_t R, int32_t block_size, int64_t seed,
                    int64_t *d_keys, const int64_t *d_key_offsets, hipStream_t stream) {
    if (R < 0 || block_size <= 0) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (R == 0) {
        return KVCM_OK;
    }
    if (!d_tokens || !d_token_offsets || !d_keys) {
        return KVCM_ERR_INVALID_ARG;
    }
    const dim3 grid(static_cast<uint32_t>((static_cast<int64_t>(R) + kReqs - 1) / kReqs));
    const int32_t force_global = kForceGeneralLoader;
#define KVCM_LAUNCH_HASH(CHUNK, BS)                                                                                  \
    hipLaunchKernelGGL((hash_tokens_kernel<TokT, CHUNK, BS>), grid, dim3(kThreads), 0, stream, d_tokens,            \
                       d_token_offsets, R, block_size, static_cast<uint64_t>(seed), d_keys, d_key_offsets, force_global)
    constexpr bool k8 = sizeof(TokT) == 8;
    const bool burst = R >= static_cast<int64_t>(burst_from(block_size, k8)) * KVCM_HASH_BURST_SCALE;
    const bool spread = block_size == 16 && k8 && !burst && R >= KVCM_HASH_SPREAD_FROM_8;
#define KVCM_LAUNCH_HASH_STAGED(CHUNK, BS, KS)                                                                       \
    hipLaunchKernelGGL((hash_tokens_kernel<TokT, CHUNK, BS, KS>), grid, dim3(kThreads), 0, stream, d_tokens,        \
                       d_token_offsets, R, block_size, static_cast<uint64_t>(seed), d_keys, d_key_offsets, force_global)
    // 4-byte tokens from as many requests as take the burst form: tiles of 128 raw tokens (512-byte pieces of the
    // token stream per request and load instruction instead of 256-byte ones). Cold timings, 16-token blocks, requests
    // of 4096 tokens, 64-token tiles of pre-added terms / raw tiles: 64 requests 56.8 / 57.3 us, 8192 58.1 / 60.2,
    // 12 288 66.6 / 62.2, 16 384 77.3 / 66.4, 32 768 149 / 127.
    const bool raw = !k8 && burst && (block_size == 8 || block_size == 16 || block_size == 32 || block_size == 64 ||
                                      block_size == 128);
#define KVCM_LAUNCH_HASH_RAW(BS)                                                                                      \
    hipLaunchKernelGGL((hash_tokens_kernel<TokT, 8, BS, kKeysBurst, true>), grid, dim3(kThreads), 0, stream, d_tokens, \
                       d_token_offsets, R, block_size, static_cast<uint64_t>(seed), d_keys, d_key_offsets, force_global)
    if (raw) {
        if constexpr (!k8) {
            switch (block_size) {
                case 8: KVCM_LAUNCH_HASH_RAW(8); break;
                case 16: KVCM_LAUNCH_HASH_RAW(16); break;
                case 32: KVCM_LAUNCH_HASH_RAW(32); break;
                case 64: KVCM_LAUNCH_HASH_RAW(64); break;
                default: KVCM_LAUNCH_HASH_RAW(128); break;
            }
        }
    } else if (spread) {
        if constexpr (k8) {
            KVCM_LAUNCH_HASH_STAGED(8, 16, kKeysSpread);
        }
    } else if (block_size == 16) {  // the engines' usual block sizes get kernels of their own
        if (k8 && burst) {  // 4-byte tokens take the burst form with raw tiles, above
            if constexpr (k8) {
                KVCM_LAUNCH_HASH_STAGED(8, 16, kKeysBurst);
            }
        } else {
            KVCM_LAUNCH_HASH(8, 16);
        }
    } else if (block_size == 8) {
        if (k8 && burst) {  // 4-byte tokens take the burst form with raw tiles, above
            if constexpr (k8) {
                KVCM_LAUNCH_HASH_STAGED(8, 8, kKeysBurst);
            }
        } else {
            KVCM_LAUNCH_HASH(8, 8);
        }
    } else if (block_size == 32) {
        if (k8 && burst) {  // 4-byte tokens take the burst form with raw tiles, above
            if constexpr (k8) {
                KVCM_LAUNCH_HASH_STAGED(8, 32, kKeysBurst);
            }
        } else {
            KVCM_LAUNCH_HASH(8, 32);
        }
    } else if (block_size == 64) {
        if (k8 && burst) {  // 4-byte tokens take the burst form with raw tiles, above
            if constexpr (k8) {
                KVCM_LAUNCH_HASH_STAGED(8, 64, kKeysBurst);
            }
        } else {
            KVCM_LAUNCH_HASH(8, 64);
        }
    } else if (block_size == 128) {
        if (k8 && burst) {  // 4-byte tokens take the burst form with raw tiles, above
            if constexpr (k8) {
                KVCM_LAUNCH_HASH_STAGED(8, 128, kKeysBurst);
            }
        } else {
            KVCM_LAUNCH_HASH(8, 128);
        }
    } else if (block_size == 1) {  // the prefix chain over digests: a key after every step
        if (burst) {
            KVCM_LAUNCH_HASH_STAGED(1, 1, kKeysBurst);
        } else {
            KVCM_LAUNCH_HASH(1, 1);
        }
    } else if (block_size % 8 == 0) {
        KVCM_LAUNCH_HASH(8, 0);
    } else {
        KVCM_LAUNCH_HASH(1, 0);
    }
#undef KVCM_LAUNCH_HASH_RAW
#undef KVCM_LAUNCH_HASH_STAGED
#undef KVCM_LAUNCH_HASH
    return launch_status();
}

}  // namespace
}  // namespace kvcm

extern "C" {

int32_t kvcm_hip_hash_tokens(const int64_t *d_tokens, const int64_t *d_token_offsets, int32_t R, int32_t block_size,
                             int64_t seed, int64_t *d_keys, const int64_t *d_key_offsets, kvcm_stream_t stream) {
    return kvcm::launch_hash<int64_t>(d_tokens, d_token_offsets, R, block_size, seed, d_keys, d_key_offsets,
                                      static_cast<hipStream_t>(stream));
}

int32_t kvcm_hip_hash_tokens_i32(const int32_t *d_tokens, const int64_t *d_token_offsets, int32_t R,
                                 int32_t block_size, int64_t seed, int64_t *d_keys, const int64_t *d_key_offsets,
                                 kvcm_stream_t stream) {
    return kvcm::launch_hash<int32_t>(d_tokens, d_token_offsets, R, block_size, seed, d_keys, d_key_offsets,
                                      static_cast<hipStream_t>(stream));
}

int32_t kvcm_hip_prefix_chain(const int64_t *d_digests, const int64_t *d_offsets, int32_t R, int64_t *d_keys,
                              kvcm_stream_t stream) {
    // ApplyPrefixHash (trace_util.cc:47-56) is the token fold with one element per key: block_size 1,
    // seed 0, keys laid out like the digests.
    return kvcm::launch_hash<int64_t>(d_digests, d_offsets, R, 1, 0, d_keys, d_offsets,
                                      static_cast<hipStream_t>(stream));
}

int32_t kvcm_hip_sha256_first8_be(const uint8_t *d_bytes, const int64_t *d_offsets, int32_t N, int64_t *d_out,
                                  kvcm_stream_t stream) {
    if (N < 0) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (N == 0) {
        return KVCM_OK;
    }
    if (!d_bytes || !d_offsets || !d_out) {
        return KVCM_ERR_INVALID_ARG;
    }
    hipLaunchKernelGGL(kvcm::sha256_first8_kernel, dim3((N + 63) / 64), dim3(64), 0, static_cast<hipStream_t>(stream),
                       d_bytes, d_offsets, N, d_out);
    return kvcm::launch_status();
}

int32_t kvcm_hip_iov_crc32(const kvcm_iov_device *d_iovs, int32_t n, uint32_t *d_crc, size_t cal_bytes,
                           kvcm_stream_t stream) {
    if (n < 0) {
        return KVCM_ERR_INVALID_ARG;
    }
    if (n == 0) {
        return KVCM_OK;
    }
    if (!d_iovs || !d_crc) {
        return KVCM_ERR_INVALID_ARG;
    }
    hipLaunchKernelGGL(kvcm::iov_crc32_kernel, dim3((n + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                       d_iovs, n, d_crc, cal_bytes);
    return kvcm::launch_status();
}

}  // extern "C"
