/*
 * kvcm_oracle.c -- CPU restatement (plain C) of the reference's save/load hot path.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP path and the CPU baseline of bench.py.
 * The product never links, loads or calls this file.
 *
 * What pins each function (tests/test_oracle_*.py):
 *   kvcm_ref_hash_step / hash_array / gen_key_vector / hash_tokens / prefix_chain
 *       - the reference header kv_cache_manager/manager/hash_util.h compiled as it lies
 *         (oracle/_ref, built by oracle/Makefile) on random and extreme inputs;
 *       - golden vectors written by that build (tests/golden/hash_golden.json), which travel;
 *       - closed form H(0, v) = v + C; sign cases (negative state => arithmetic shift matters);
 *         a second restatement on Python big integers; prefix and truncation invariants.
 *   kvcm_ref_sha256 / sha256_first8_be
 *       - hashlib.sha256 (FIPS 180-4) on the standard vectors and random strings of every length
 *         across the padding boundaries.
 *   kvcm_ref_iov_crc32 / blocks_hash_from_crcs
 *       - the reference's own known answers (sdk_buffer_check_util_test.cc:13-74) and zlib.crc32 on
 *         head||tail; the fold is checked against oracle/_ref's HashIntArray<uint32_t>.
 *   kvcm_ref_gather_ex / scatter_ex / batch_* / generate_blocks_idx
 *       - pure permutation copies: checked against NumPy fancy indexing written from the reference's
 *         index algebra, against the expected-value loops of the reference's own kernel test
 *         (py_connector/test/kernel/test_batch_gather_scatter.py:91-114,201-216), ramp-valued pools
 *         whose values name their own slot, scatter(gather) = identity, and canary guard bands.
 *   The trailer (per-block scale) interleave has no reference counterpart: brute force only.
 *   kvcm_ref_first_occurrence / mask_to_indices
 *       - brute force on small inputs, np.unique(return_index, return_inverse) on large ones, extreme signed keys;
 *         the reference's parsing loop (py_connector/vllm/v1_connector.py:835-850) restated in Python, both branches.
 *         first_occurrence has no reference counterpart (the manager filters per request, cache_manager.cc:589-635).
 *   kvcm_ref_file_put / file_get
 *       - the reference's own unit test at its own values (client/src/internal/sdk/test/local_file_sdk_test.cc:35-95);
 *         the byte layout checked directly (blkid * size offsets, zero holes, a file never shrinks, spill into the
 *         next block allowed, iovs past the end refused).
 *   kvcm_ref_copy_iovs
 *       - brute-force layout checks: ignored iovs take no room (hf3fs_usrbio_client.cc:484-486), order kept, canary
 *         bytes after the last piece.
 */
#define _GNU_SOURCE
#include "kvcm_oracle.h"

#include <fcntl.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#define KVCM_GOLDEN 0x9e3779b97f4a7c15ULL

/* ------------------------------------------------------------------ hashing */

/* hash_util.h:10: hash ^= hasher(value) + C + (hash << 12) + (hash >> 32), on int64_t.
 * Restated on uint64_t so that the wrap-around is defined; the right shift is arithmetic. */
static inline uint64_t hash_step_u64(uint64_t h, uint64_t v) {
    uint64_t sar = h >> 32;
    if (h >> 63) {
        sar |= 0xFFFFFFFF00000000ULL;
    }
    return h ^ (v + KVCM_GOLDEN + (h << 12) + sar);
}

int64_t kvcm_ref_hash_step(int64_t hash, int64_t value) {
    return (int64_t)hash_step_u64((uint64_t)hash, (uint64_t)value);
}

int64_t kvcm_ref_hash_array(int64_t hash, const int64_t *begin, const int64_t *end) {
    uint64_t h = (uint64_t)hash;
    while (begin != end) {
        h = hash_step_u64(h, (uint64_t)*begin);
        begin++;
    }
    return (int64_t)h;
}

/* cache_manager.cc:76-87: total_blocks = size / block_size; the state carries across blocks. */
int64_t kvcm_ref_gen_key_vector(const int64_t *tokens, int64_t n, int64_t block_size, int64_t seed,
                                int64_t *keys) {
    if (block_size <= 0 || n < 0) {
        return 0;
    }
    int64_t total_blocks = n / block_size;
    int64_t hash = seed;
    for (int64_t index = 0; index < total_blocks; index++) {
        const int64_t *pos = tokens + index * block_size;
        hash = kvcm_ref_hash_array(hash, pos, pos + block_size);
        keys[index] = hash;
    }
    return total_blocks;
}

static int64_t key_base(const int64_t *token_offsets, const int64_t *key_offsets, int32_t r,
                        int32_t block_size) {
    if (key_offsets) {
        return key_offsets[r];
    }
    return (int64_t)r * ((token_offsets[1] - token_offsets[0]) / block_size);
}

int32_t kvcm_ref_hash_tokens(const int64_t *tokens, const int64_t *token_offsets, int32_t R,
                             int32_t block_size, int64_t seed, int64_t *keys,
                             const int64_t *key_offsets) {
    if (R < 0 || block_size <= 0 || (R > 0 && (!tokens || !token_offsets || !keys))) {
        return -1;
    }
    for (int32_t r = 0; r < R; r++) {
        int64_t n = token_offsets[r + 1] - token_offsets[r];
        kvcm_ref_gen_key_vector(tokens + token_offsets[r], n, block_size, seed,
                                keys + key_base(token_offsets, key_offsets, r, block_size));
    }
    return 0;
}

int32_t kvcm_ref_hash_tokens_i32(const int32_t *tokens, const int64_t *token_offsets, int32_t R,
                                 int32_t block_size, int64_t seed, int64_t *keys,
                                 const int64_t *key_offsets) {
    if (R < 0 || block_size <= 0 || (R > 0 && (!tokens || !token_offsets || !keys))) {
        return -1;
    }
    for (int32_t r = 0; r < R; r++) {
        const int32_t *t = tokens + token_offsets[r];
        int64_t n = token_offsets[r + 1] - token_offsets[r];
        int64_t *out = keys + key_base(token_offsets, key_offsets, r, block_size);
        uint64_t h = (uint64_t)seed;
        for (int64_t b = 0; b < n / block_size; b++) {
            for (int64_t i = 0; i < block_size; i++) {
                h = hash_step_u64(h, (uint64_t)(int64_t)t[b * block_size + i]);
            }
            out[b] = (int64_t)h;
        }
    }
    return 0;
}

struct hash_job {
    const int64_t *tokens;
    const int64_t *token_offsets;
    const int64_t *key_offsets;
    int64_t *keys;
    int32_t R, block_size, first, step;
    int64_t seed;
};

static void *hash_worker(void *arg) {
    struct hash_job *j = (struct hash_job *)arg;
    for (int32_t r = j->first; r < j->R; r += j->step) {
        int64_t n = j->token_offsets[r + 1] - j->token_offsets[r];
        kvcm_ref_gen_key_vector(j->tokens + j->token_offsets[r], n, j->block_size, j->seed,
                                j->keys + key_base(j->token_offsets, j->key_offsets, r, j->block_size));
    }
    return NULL;
}

int32_t kvcm_ref_hash_tokens_mt(const int64_t *tokens, const int64_t *token_offsets, int32_t R,
                                int32_t block_size, int64_t seed, int64_t *keys,
                                const int64_t *key_offsets, int32_t threads) {
    if (R < 0 || block_size <= 0 || (R > 0 && (!tokens || !token_offsets || !keys))) {
        return -1;
    }
    if (threads < 1) {
        threads = 1;
    }
    if (threads > 256) {
        threads = 256;
    }
    pthread_t tid[256];
    struct hash_job jobs[256];
    for (int32_t t = 0; t < threads; t++) {
        struct hash_job j = {tokens, token_offsets, key_offsets, keys, R, block_size, t, threads, seed};
        jobs[t] = j;
    }
    for (int32_t t = 1; t < threads; t++) {
        pthread_create(&tid[t], NULL, hash_worker, &jobs[t]);
    }
    hash_worker(&jobs[0]);
    for (int32_t t = 1; t < threads; t++) {
        pthread_join(tid[t], NULL);
    }
    return 0;
}

/* trace_util.cc:47-56: one step per element, every intermediate state is a key. */
int32_t kvcm_ref_prefix_chain(const int64_t *digests, const int64_t *offsets, int32_t R, int64_t *keys) {
    if (R < 0 || (R > 0 && (!digests || !offsets || !keys))) {
        return -1;
    }
    for (int32_t r = 0; r < R; r++) {
        int64_t hash = 0;
        for (int64_t i = offsets[r]; i < offsets[r + 1]; i++) {
            hash = kvcm_ref_hash_step(hash, digests[i]);
            keys[i] = hash;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ SHA-256 (FIPS 180-4) */

static const uint32_t sha_k[64] = {
    0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5,
    0xd807aa98, 0x12835b01, 0x243185be, 0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174,
    0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa, 0x5cb0a9dc, 0x76f988da,
    0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967,
    0x27b70a85, 0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85,
    0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3, 0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070,
    0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f, 0x682e6ff3,
    0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};

static inline uint32_t rotr32(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }

static void sha256_compress(uint32_t st[8], const uint8_t blk[64]) {
    uint32_t w[64];
    for (int i = 0; i < 16; i++) {
        w[i] = ((uint32_t)blk[4 * i] << 24) | ((uint32_t)blk[4 * i + 1] << 16) |
               ((uint32_t)blk[4 * i + 2] << 8) | (uint32_t)blk[4 * i + 3];
    }
    for (int i = 16; i < 64; i++) {
        uint32_t s0 = rotr32(w[i - 15], 7) ^ rotr32(w[i - 15], 18) ^ (w[i - 15] >> 3);
        uint32_t s1 = rotr32(w[i - 2], 17) ^ rotr32(w[i - 2], 19) ^ (w[i - 2] >> 10);
        w[i] = w[i - 16] + s0 + w[i - 7] + s1;
    }
    uint32_t a = st[0], b = st[1], c = st[2], d = st[3], e = st[4], f = st[5], g = st[6], h = st[7];
    for (int i = 0; i < 64; i++) {
        uint32_t S1 = rotr32(e, 6) ^ rotr32(e, 11) ^ rotr32(e, 25);
        uint32_t ch = (e & f) ^ (~e & g);
        uint32_t t1 = h + S1 + ch + sha_k[i] + w[i];
        uint32_t S0 = rotr32(a, 2) ^ rotr32(a, 13) ^ rotr32(a, 22);
        uint32_t mj = (a & b) ^ (a & c) ^ (b & c);
        uint32_t t2 = S0 + mj;
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

void kvcm_ref_sha256(const uint8_t *msg, size_t len, uint8_t digest[32]) {
    uint32_t st[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a,
                      0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
    size_t full = len / 64;
    for (size_t i = 0; i < full; i++) {
        sha256_compress(st, msg + 64 * i);
    }
    uint8_t tail[128];
    size_t rem = len - 64 * full;
    memset(tail, 0, sizeof tail);
    if (rem) {
        memcpy(tail, msg + 64 * full, rem);
    }
    tail[rem] = 0x80;
    size_t tail_len = (rem < 56) ? 64 : 128;
    uint64_t bits = (uint64_t)len * 8;
    for (int i = 0; i < 8; i++) {
        tail[tail_len - 1 - i] = (uint8_t)(bits >> (8 * i));
    }
    sha256_compress(st, tail);
    if (tail_len == 128) {
        sha256_compress(st, tail + 64);
    }
    for (int i = 0; i < 8; i++) {
        digest[4 * i] = (uint8_t)(st[i] >> 24);
        digest[4 * i + 1] = (uint8_t)(st[i] >> 16);
        digest[4 * i + 2] = (uint8_t)(st[i] >> 8);
        digest[4 * i + 3] = (uint8_t)st[i];
    }
}

/* sglang/connector.py:397-401: int.from_bytes(digest[:8], "big", signed=True). */
int32_t kvcm_ref_sha256_first8_be(const uint8_t *bytes, const int64_t *offsets, int32_t N, int64_t *out) {
    if (N < 0 || (N > 0 && (!offsets || !out))) {
        return -1;
    }
    for (int32_t i = 0; i < N; i++) {
        uint8_t dg[32];
        kvcm_ref_sha256(bytes + offsets[i], (size_t)(offsets[i + 1] - offsets[i]), dg);
        uint64_t v = 0;
        for (int k = 0; k < 8; k++) {
            v = (v << 8) | dg[k];
        }
        out[i] = (int64_t)v;
    }
    return 0;
}

/* ------------------------------------------------------------------ gather / scatter */

static int copy_desc_ok(const kvcm_ref_copy_desc *d) {
    if (!d || d->B < 0 || d->P <= 0 || d->T <= 0 || d->run_tokens <= 0 || d->row_bytes <= 0) {
        return 0;
    }
    if (d->T % d->run_tokens != 0 || d->ptrs_per_entry <= 0 || d->trailer_bytes < 0) {
        return 0;
    }
    if (d->B > 0 && (!d->ptr_table || !d->staging || !d->run_start)) {
        return 0;
    }
    if (d->trailer_bytes > 0 && (!d->trailer_ptr_table || !d->trailer_idx)) {
        return 0;
    }
    return 1;
}

/* One work block, both directions. gather: batch_gather_scatter_helper.py:57-97
 * (block_offset = dst_block_idx * P * T * D; layer_offset = block_offset + p * T * D;
 *  src = base_p + global_token_idx * D + dim); scatter swaps source and destination (:163-205).
 * Legacy layout and the out-of-range skip: gather_scatter_helper.py:29-47,80-97. */
static void copy_one_block(const kvcm_ref_copy_desc *d, int32_t b, int scatter) {
    const int32_t runs = d->T / d->run_tokens;
    const int64_t run_bytes = (int64_t)d->run_tokens * d->row_bytes;
    const int64_t slot = d->staging_idx ? d->staging_idx[b] : b;
    uint8_t *stage_block = (uint8_t *)d->staging + slot * d->staging_block_stride_bytes;
    for (int32_t p = 0; p < d->P; p++) {
        uint8_t *pool = (uint8_t *)d->ptr_table[p / d->ptrs_per_entry] +
                        (int64_t)(p % d->ptrs_per_entry) * d->entry_stride_bytes;
        uint8_t *tile = stage_block + (int64_t)p * d->staging_tile_stride_bytes;
        for (int32_t r = 0; r < runs; r++) {
            int64_t s = d->run_start[(int64_t)b * runs + r];
            if (d->slot_limit > 0 && s >= d->slot_limit) {
                continue;
            }
            if (s < 0) {
                /* No reference counterpart (a negative index is out of bounds there): the library's contract
                 * skips such runs, e.g. the -1 entries kvcm_hip_generate_blocks_idx writes past the block list. */
                continue;
            }
            uint8_t *row = pool + s * d->row_bytes;
            uint8_t *st = tile + (int64_t)r * run_bytes;
            if (scatter) {
                memcpy(row, st, (size_t)run_bytes);
            } else {
                memcpy(st, row, (size_t)run_bytes);
            }
        }
        if (d->trailer_bytes > 0 && d->trailer_idx[b] >= 0) { /* a negative trailer index skips the trailer */
            uint8_t *tr = (uint8_t *)d->trailer_ptr_table[p] + (int64_t)d->trailer_idx[b] * d->trailer_bytes;
            uint8_t *st = tile + (int64_t)d->T * d->row_bytes;
            if (scatter) {
                memcpy(tr, st, (size_t)d->trailer_bytes);
            } else {
                memcpy(st, tr, (size_t)d->trailer_bytes);
            }
        }
    }
}

int32_t kvcm_ref_gather_ex(const kvcm_ref_copy_desc *d) {
    if (!copy_desc_ok(d)) {
        return -1;
    }
    for (int32_t b = 0; b < d->B; b++) {
        copy_one_block(d, b, 0);
    }
    return 0;
}

int32_t kvcm_ref_scatter_ex(const kvcm_ref_copy_desc *d) {
    if (!copy_desc_ok(d)) {
        return -1;
    }
    for (int32_t b = 0; b < d->B; b++) {
        copy_one_block(d, b, 1);
    }
    return 0;
}

struct copy_job {
    const kvcm_ref_copy_desc *d;
    int32_t first, last, scatter;
};

static void *copy_worker(void *arg) {
    struct copy_job *j = (struct copy_job *)arg;
    for (int32_t b = j->first; b < j->last; b++) {
        copy_one_block(j->d, b, j->scatter);
    }
    return NULL;
}

static int32_t copy_mt(const kvcm_ref_copy_desc *d, int32_t threads, int scatter) {
    if (!copy_desc_ok(d)) {
        return -1;
    }
    if (threads < 1) {
        threads = 1;
    }
    if (threads > 256) {
        threads = 256;
    }
    pthread_t tid[256];
    struct copy_job jobs[256];
    for (int32_t t = 0; t < threads; t++) {
        jobs[t].d = d;
        jobs[t].first = (int32_t)((int64_t)d->B * t / threads);
        jobs[t].last = (int32_t)((int64_t)d->B * (t + 1) / threads);
        jobs[t].scatter = scatter;
    }
    for (int32_t t = 1; t < threads; t++) {
        pthread_create(&tid[t], NULL, copy_worker, &jobs[t]);
    }
    copy_worker(&jobs[0]);
    for (int32_t t = 1; t < threads; t++) {
        pthread_join(tid[t], NULL);
    }
    return 0;
}

int32_t kvcm_ref_gather_ex_mt(const kvcm_ref_copy_desc *d, int32_t threads) { return copy_mt(d, threads, 0); }
int32_t kvcm_ref_scatter_ex_mt(const kvcm_ref_copy_desc *d, int32_t threads) { return copy_mt(d, threads, 1); }

static kvcm_ref_copy_desc plain_desc(const void *const *ptr_table, int32_t P, void *staging,
                                     int64_t stride, const int32_t *token_idx, const int32_t *staging_idx,
                                     int32_t B, int32_t T, int64_t row_bytes) {
    kvcm_ref_copy_desc d;
    memset(&d, 0, sizeof d);
    d.ptr_table = ptr_table;
    d.P = P;
    d.ptrs_per_entry = 1;
    d.staging = staging;
    d.staging_block_stride_bytes = stride;
    d.staging_tile_stride_bytes = (int64_t)T * row_bytes;
    d.run_start = token_idx;
    d.staging_idx = staging_idx;
    d.B = B;
    d.T = T;
    d.run_tokens = 1;
    d.row_bytes = row_bytes;
    return d;
}

int32_t kvcm_ref_batch_gather(const void *const *ptr_table, int32_t P, void *staging,
                              int64_t staging_block_stride_bytes, const int32_t *token_idx,
                              const int32_t *staging_idx, int32_t B, int32_t T, int64_t row_bytes) {
    kvcm_ref_copy_desc d =
        plain_desc(ptr_table, P, staging, staging_block_stride_bytes, token_idx, staging_idx, B, T, row_bytes);
    return kvcm_ref_gather_ex(&d);
}

int32_t kvcm_ref_batch_scatter(const void *const *ptr_table, int32_t P, const void *staging,
                               int64_t staging_block_stride_bytes, const int32_t *token_idx,
                               const int32_t *staging_idx, int32_t B, int32_t T, int64_t row_bytes) {
    kvcm_ref_copy_desc d = plain_desc(ptr_table, P, (void *)staging, staging_block_stride_bytes, token_idx,
                                      staging_idx, B, T, row_bytes);
    return kvcm_ref_scatter_ex(&d);
}

/* v1_connector.py:308-320. */
int32_t kvcm_ref_generate_blocks_idx(const int32_t *manager_block_idxes, int32_t B,
                                     const int32_t *local_block_ids, int32_t n_local, int32_t T_mgr,
                                     int32_t T_eng, int32_t *out) {
    int32_t bad = 0;
    for (int32_t b = 0; b < B; b++) {
        for (int32_t i = 0; i < T_mgr; i++) {
            int64_t now_token_idx = (int64_t)manager_block_idxes[b] * T_mgr + i;
            int64_t blk = now_token_idx / T_eng;
            if (blk >= n_local || blk < 0) {
                out[(int64_t)b * T_mgr + i] = -1;
                bad = 1;
                continue;
            }
            int64_t token_offset = now_token_idx % T_eng;
            out[(int64_t)b * T_mgr + i] = (int32_t)((int64_t)local_block_ids[blk] * T_eng + token_offset);
        }
    }
    return bad;
}

/* ------------------------------------------------------------------ buffer check */

/* sdk_buffer_check_util.cu:10-19. */
static inline uint32_t crc32_byte(uint32_t crc, uint8_t data) {
    crc ^= data;
    for (int i = 0; i < 8; ++i) {
        uint32_t mask = 0u - (crc & 1u);
        crc = (crc >> 1) ^ (0xEDB88320u & mask);
    }
    return crc;
}

/* sdk_buffer_check_util.cu:21-44: head bytes then tail bytes through one running CRC. */
int32_t kvcm_ref_iov_crc32(const kvcm_ref_iov *iovs, int32_t n, uint32_t *crc_out, size_t cal_bytes) {
    if (n < 0 || (n > 0 && (!iovs || !crc_out))) {
        return -1;
    }
    for (int32_t k = 0; k < n; k++) {
        const uint8_t *p = (const uint8_t *)iovs[k].base;
        uint32_t crc = 0xFFFFFFFFu;
        for (size_t i = 0; i < cal_bytes; i++) {
            crc = crc32_byte(crc, p[i]);
        }
        for (size_t i = iovs[k].size - cal_bytes; i < iovs[k].size; i++) {
            crc = crc32_byte(crc, p[i]);
        }
        crc_out[k] = ~crc;
    }
    return 0;
}

/* sdk_buffer_check_util.cc:56-60 with HashIntArray<uint32_t> (common/hash_util.h:17-25):
 * std::hash<uint32_t> is the identity, so each CRC enters the chain zero-extended. */
int32_t kvcm_ref_blocks_hash_from_crcs(const uint32_t *crcs, int64_t n_crcs, int32_t iovs_per_block,
                                       int64_t *out_hashes) {
    if (iovs_per_block <= 0 || n_crcs < 0) {
        return -1;
    }
    int64_t nb = 0;
    for (int64_t off = 0; off + iovs_per_block <= n_crcs; off += iovs_per_block) {
        uint64_t h = 0;
        for (int32_t i = 0; i < iovs_per_block; i++) {
            h = hash_step_u64(h, (uint64_t)crcs[off + i]);
        }
        out_hashes[nb++] = (int64_t)h;
    }
    return 0;
}

/* ------------------------------------------------------------------ which blocks to save */

struct key_pos {
    int64_t key;
    int32_t pos;
};

static int key_pos_less(const void *a, const void *b) {
    const struct key_pos *x = (const struct key_pos *)a, *y = (const struct key_pos *)b;
    if (x->key != y->key) {
        return x->key < y->key ? -1 : 1;
    }
    return x->pos < y->pos ? -1 : (x->pos > y->pos);
}

/* first_idx[i] = smallest j with keys[j] == keys[i]. No reference counterpart (the manager filters shared blocks
 * request by request against its index, cache_manager.cc:589-635); stated by sorting (key, position) pairs. */
int32_t kvcm_ref_first_occurrence(const int64_t *keys, int64_t n, int32_t *first_idx, uint8_t *is_repeat) {
    if (n < 0 || (n > 0 && (!keys || !first_idx))) {
        return -1;
    }
    struct key_pos *kp = (struct key_pos *)malloc(sizeof(struct key_pos) * (size_t)(n ? n : 1));
    for (int64_t i = 0; i < n; i++) {
        kp[i].key = keys[i];
        kp[i].pos = (int32_t)i;
    }
    qsort(kp, (size_t)n, sizeof(struct key_pos), key_pos_less);
    int32_t head = 0;
    for (int64_t i = 0; i < n; i++) {
        if (i == 0 || kp[i].key != kp[i - 1].key) {
            head = kp[i].pos;
        }
        first_idx[kp[i].pos] = head;
    }
    free(kp);
    for (int64_t i = 0; is_repeat && i < n; i++) {
        is_repeat[i] = first_idx[i] != (int32_t)i;
    }
    return 0;
}

/* v1_connector.py:835-850, bool_masks branch: the indices whose mask entry is false, in order.
 * mask2 (optional) is OR-ed in. Returns the number of indices written. */
int64_t kvcm_ref_mask_to_indices(const uint8_t *mask, const uint8_t *mask2, int64_t n, int32_t *indices) {
    int64_t count = 0;
    for (int64_t idx = 0; idx < n; idx++) {
        int is_saved = mask[idx] != 0 || (mask2 && mask2[idx] != 0);
        if (!is_saved) {
            indices[count++] = (int32_t)idx;
        }
    }
    return count;
}

/* ------------------------------------------------------------------ block files (host iovs only) */

/* local_file_sdk.cc:262-364 (DoPut) after Alloc (:136-159): the file is created when missing, grown with fallocate
 * to (max blkid + 1) * bsz, mapped, and every iov is memcpy'd to blkid * bsz + running offset; ignored or null
 * iovs only advance the offset. Returns 0, -1 (the reference's invalid-parameter cases) or -4 (file I/O).
 * The parent directory must exist (the tests make it). Like the reference, a failure half-way leaves the bytes
 * already copied in the file. */
int32_t kvcm_ref_file_put(const char *path, int64_t bsz, const uint64_t *blkids, const uint64_t *sizes,
                          const int32_t *iov_counts, const kvcm_ref_fiov *iovs, int32_t n_blocks) {
    if (n_blocks <= 0) {
        return -1;
    }
    uint64_t max_blkid = 0, required_size = 0;
    for (int32_t i = 0; i < n_blocks; i++) {
        if ((uint64_t)bsz != sizes[i]) {
            return -1;
        }
        if (blkids[i] > max_blkid) {
            max_blkid = blkids[i];
        }
        if ((max_blkid + 1) * (uint64_t)bsz > required_size) {
            required_size = (max_blkid + 1) * (uint64_t)bsz;
        }
    }
    int fd = open(path, O_RDWR | O_CREAT, 0644);
    if (fd < 0) {
        return -4;
    }
    if (fallocate(fd, 0, 0, (off_t)required_size) != 0) {
        close(fd);
        return -4;
    }
    char *dst = (char *)mmap(NULL, required_size, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
    if (dst == MAP_FAILED) {
        close(fd);
        return -4;
    }
    int32_t rc = 0;
    int64_t first = 0;
    for (int32_t i = 0; i < n_blocks && rc == 0; i++) {
        uint64_t offset = blkids[i] * (uint64_t)bsz;
        for (int32_t k = 0; k < iov_counts[i]; k++) {
            const kvcm_ref_fiov *iov = &iovs[first + k];
            if (offset + iov->size > required_size) {
                rc = -1;
                break;
            }
            if (!iov->ignore && iov->base && iov->size > 0) {
                memcpy(dst + offset, iov->base, iov->size);
            }
            offset += iov->size;
        }
        first += iov_counts[i];
    }
    msync(dst, required_size, MS_SYNC);
    munmap(dst, required_size);
    close(fd);
    return rc;
}

/* local_file_sdk.cc:161-260 (DoGet): the file must exist; iovs beyond its end are refused. */
int32_t kvcm_ref_file_get(const char *path, int64_t bsz, const uint64_t *blkids, const uint64_t *sizes,
                          const int32_t *iov_counts, const kvcm_ref_fiov *iovs, int32_t n_blocks) {
    if (n_blocks <= 0) {
        return -1;
    }
    int fd = open(path, O_RDONLY);
    if (fd < 0) {
        return -4;
    }
    struct stat st;
    if (fstat(fd, &st) != 0) {
        close(fd);
        return -4;
    }
    size_t file_size = (size_t)st.st_size;
    char *src = (char *)mmap(NULL, file_size, PROT_READ, MAP_PRIVATE, fd, 0);
    if (src == MAP_FAILED) {
        close(fd);
        return -4;
    }
    int32_t rc = 0;
    int64_t first = 0;
    for (int32_t i = 0; i < n_blocks && rc == 0; i++) {
        if ((uint64_t)bsz != sizes[i]) {
            rc = -1;
            break;
        }
        uint64_t offset = blkids[i] * (uint64_t)bsz;
        for (int32_t k = 0; k < iov_counts[i]; k++) {
            const kvcm_ref_fiov *iov = &iovs[first + k];
            if (offset + iov->size > file_size) {
                rc = -1;
                break;
            }
            if (!iov->ignore && iov->base && iov->size > 0) {
                memcpy(iov->base, src + offset, iov->size);
            }
            offset += iov->size;
        }
        first += iov_counts[i];
    }
    munmap(src, file_size);
    close(fd);
    return rc;
}

/* hf3fs_usrbio_client.cc:478-505 (CopyIovs) on host iovs: pieces back to back in the I/O buffer; an ignored iov is
 * skipped WITHOUT advancing the offset (:484-486), a null base is not tested for there (the caller never passes one). */
int64_t kvcm_ref_copy_iovs(void *host_buffer, const kvcm_ref_fiov *iovs, int32_t n, int32_t load) {
    int64_t iov_offset = 0;
    char *iov_base = (char *)host_buffer;
    for (int32_t i = 0; i < n; i++) {
        const kvcm_ref_fiov *iov = &iovs[i];
        if (iov->ignore) {
            continue;
        }
        if (load) {
            memcpy(iov->base, iov_base + iov_offset, iov->size);
        } else {
            memcpy(iov_base + iov_offset, iov->base, iov->size);
        }
        iov_offset += (int64_t)iov->size;
    }
    return iov_offset;
}
