// sanitize_host.cpp -- the host code of this repository under AddressSanitizer + UndefinedBehaviorSanitizer and,
// in a second build, ThreadSanitizer, on a machine without a GPU (make -C tests/cpp sanitize).
//
// What is compiled in, with a plain host compiler: oracle/kvcm_oracle.c (the checker itself), the library's host-only
// translation units tair_kvcache_amd/csrc/kvcm_file.hip and kvcm_host.hip, the host walk over index lists
// (kvcm_host_idx.h) and the C++ layer include/kvcm_hip.hpp. The HIP runtime underneath is fake_hip.cpp: malloc'd
// "device" memory and streams that really are asynchronous. The three kernel entry points the C++ layer calls are
// stand-ins that do the oracle's work in stream order.
//
// Scenarios: the oracle's threaded forms; the index-list walk against brute force; block files with host iovs and
// with device iovs from 16 concurrent callers; a big get shared among helper threads; a store destroyed while a get
// or a put is still inside it; the blocking cell pool of the buffer check with more threads than cells.
#include <unistd.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "fake_hip.h"
#include "kvcm_hip.hpp"
#include "kvcm_host_idx.h"
#include "kvcm_oracle.h"

#define CHECK(cond)                                                                  \
    do {                                                                             \
        if (!(cond)) {                                                               \
            std::fprintf(stderr, "%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond); \
            std::exit(1);                                                            \
        }                                                                            \
    } while (0)

// ---- stand-ins of the kernel entry points that include/kvcm_hip.hpp calls: the oracle's work, in stream order
extern "C" int32_t kvcm_hip_hash_tokens(const int64_t *d_tokens, const int64_t *d_token_offsets, int32_t R,
                                        int32_t block_size, int64_t seed, int64_t *d_keys, const int64_t *d_key_offsets,
                                        kvcm_stream_t stream) {
    fake_hip_enqueue(stream, [=] {
        kvcm_ref_hash_tokens(d_tokens, d_token_offsets, R, block_size, seed, d_keys, d_key_offsets);
    });
    return KVCM_OK;
}
extern "C" int32_t kvcm_hip_iov_crc32(const kvcm_iov_device *d_iovs, int32_t n, uint32_t *d_crc, size_t cal_bytes,
                                      kvcm_stream_t stream) {
    fake_hip_enqueue(stream, [=] {
        kvcm_ref_iov_crc32(reinterpret_cast<const kvcm_ref_iov *>(d_iovs), n, d_crc, cal_bytes);
    });
    return KVCM_OK;
}
extern "C" int64_t kvcm_hip_first_occurrence_workspace_bytes(int64_t n) { return n * 8 + 4096; }
extern "C" int32_t kvcm_hip_first_occurrence(const int64_t *d_keys, int64_t n, void *, int64_t, int32_t *d_first_idx,
                                             uint8_t *d_is_repeat, kvcm_stream_t stream) {
    fake_hip_enqueue(stream, [=] { kvcm_ref_first_occurrence(d_keys, n, d_first_idx, d_is_repeat); });
    return KVCM_OK;
}

namespace {

std::string g_dir;

std::vector<uint8_t> pattern(size_t n, uint32_t seed) {
    std::vector<uint8_t> v(n);
    uint32_t x = seed * 2654435761u + 12345u;
    for (size_t i = 0; i < n; ++i) {
        x = x * 1664525u + 1013904223u;
        v[i] = static_cast<uint8_t>(x >> 24);
    }
    return v;
}

void oracle_threaded_forms() {
    std::mt19937_64 rng(1);
    const int32_t R = 37, bs = 16;
    std::vector<int64_t> toff(R + 1, 0), koff(R + 1, 0);
    for (int32_t r = 0; r < R; ++r) {
        const int64_t len = static_cast<int64_t>(rng() % 700);
        toff[r + 1] = toff[r] + len;
        koff[r + 1] = koff[r] + len / bs;
    }
    std::vector<int64_t> tok(static_cast<size_t>(toff[R]) + 1);
    for (auto &t : tok) {
        t = static_cast<int64_t>(rng());
    }
    std::vector<int64_t> k1(static_cast<size_t>(koff[R]) + 1, 7), k8 = k1;
    CHECK(kvcm_ref_hash_tokens(tok.data(), toff.data(), R, bs, -5, k1.data(), koff.data()) == 0);
    CHECK(kvcm_ref_hash_tokens_mt(tok.data(), toff.data(), R, bs, -5, k8.data(), koff.data(), 8) == 0);
    CHECK(k1 == k8);
    // extremes of the step: shifts of negative states, wrap-around of the sums
    CHECK(kvcm_ref_hash_step(0, 0) == static_cast<int64_t>(0x9e3779b97f4a7c15ULL));
    (void)kvcm_ref_hash_step(INT64_MIN, INT64_MAX);
    (void)kvcm_ref_hash_step(-1, INT64_MIN);

    const int32_t P = 6, T = 16, B = 40, slots = 64;
    const int64_t row = 96, n_slots = 2048;
    std::vector<std::vector<uint8_t>> pools;
    std::vector<const void *> table;
    for (int p = 0; p < P; ++p) {
        pools.push_back(pattern(static_cast<size_t>(n_slots * row), 100 + p));
        table.push_back(pools.back().data());
    }
    std::vector<int32_t> idx(B * T), sidx(B);
    for (auto &v : idx) {
        v = static_cast<int32_t>(rng() % n_slots);
    }
    idx[5] = -1;
    for (int32_t b = 0; b < B; ++b) {
        sidx[b] = (b * 7) % slots;
    }
    std::vector<uint8_t> st1(static_cast<size_t>(slots * P * T * row), 0xEE), st8 = st1;
    kvcm_ref_copy_desc d{};
    d.ptr_table = table.data(), d.P = P, d.ptrs_per_entry = 1, d.staging = st1.data();
    d.staging_block_stride_bytes = P * T * row, d.staging_tile_stride_bytes = T * row;
    d.run_start = idx.data(), d.staging_idx = sidx.data(), d.B = B, d.T = T, d.run_tokens = 1, d.row_bytes = row;
    CHECK(kvcm_ref_gather_ex(&d) == 0);
    d.staging = st8.data();
    CHECK(kvcm_ref_gather_ex_mt(&d, 8) == 0);
    CHECK(st1 == st8);
    uint8_t digest[32];
    kvcm_ref_sha256(reinterpret_cast<const uint8_t *>("abc"), 3, digest);
    CHECK(digest[0] == 0xba && digest[31] == 0xad);
    std::puts("ok oracle: threaded forms equal the serial ones");
}

void index_list_walk() {
    std::mt19937 rng(2);
    for (int it = 0; it < 2000; ++it) {
        const int32_t T = std::vector<int32_t>{1, 4, 16, 24, 64}[rng() % 5], B = 1 + rng() % 60;
        const int32_t want_r_choices[] = {1, 2, 4, 8, T};
        int32_t base_r = want_r_choices[rng() % 5];
        if (T % base_r != 0) {
            base_r = 1;
        }
        std::vector<int32_t> idx(static_cast<size_t>(B) * T);
        for (int32_t b = 0; b < B; ++b) {
            for (int32_t k = 0; k < T / base_r; ++k) {
                const int32_t start = static_cast<int32_t>(rng() % 100000) * 2 * T;  // runs never touch by accident
                for (int32_t j = 0; j < base_r; ++j) {
                    idx[static_cast<size_t>(b) * T + k * base_r + j] = start + j;
                }
            }
        }
        if (it % 7 == 0) {
            idx[rng() % idx.size()] = -1;
        }
        int32_t r = 0;
        CHECK(kvcm::walk_host_idx(idx.data(), nullptr, B, T, 0, 0, &r) == KVCM_OK);
        CHECK(r >= 1 && T % r == 0);
        // r describes the lists: every run of r is consecutive and non-negative, or starts a skipped row of its own
        for (int32_t b = 0; b < B; ++b) {
            for (int32_t j = 0; j < T; ++j) {
                const int32_t v = idx[static_cast<size_t>(b) * T + j], s = idx[static_cast<size_t>(b) * T + j / r * r];
                CHECK(r == 1 || (s >= 0 && v == s + j % r));
            }
        }
        if (it % 7 != 0) {
            CHECK(r == base_r || r % base_r == 0);
        }
        const int32_t runs = T / r, per = kvcm::kEmbedInts / (runs + 1);
        kvcm::EmbeddedIdx emb;
        for (int32_t b0 = 0; b0 < B; b0 += per) {
            const int32_t nb = std::min(per, B - b0);
            kvcm::fill_embedded(&emb, idx.data(), nullptr, b0, nb, T, r);
            CHECK(emb.v[0] == idx[static_cast<size_t>(b0) * T] && emb.v[nb * runs + nb - 1] == b0 + nb - 1);
        }
    }
    const int32_t edge[4] = {INT32_MAX - 1, INT32_MAX, 0, 1};  // no successor of INT32_MAX: the walk adds in 64 bits
    int32_t r = 0;
    CHECK(kvcm::walk_host_idx(edge, nullptr, 1, 4, 0, 0, &r) == KVCM_OK && r == 2);
    CHECK(kvcm::walk_host_idx(edge, nullptr, 1, 4, 100, 0, &r) == KVCM_ERR_OUT_OF_RANGE);
    const int32_t st[1] = {3};
    CHECK(kvcm::walk_host_idx(edge + 2, st, 1, 2, 0, 3, &r) == KVCM_ERR_OUT_OF_RANGE);
    std::puts("ok index lists: run discovery and range checks");
}

void blocks_hash() {
    std::mt19937 rng(3);
    std::vector<uint32_t> crcs(23);
    for (auto &c : crcs) {
        c = rng();
    }
    std::vector<int64_t> a(5, 1), b(5, 2);
    CHECK(kvcm_blocks_hash_from_crcs(crcs.data(), 23, 5, a.data()) == KVCM_OK);
    CHECK(kvcm_ref_blocks_hash_from_crcs(crcs.data(), 23, 5, b.data()) == 0);
    a[4] = b[4] = 0;  // 23 / 5 = 4 whole blocks
    CHECK(a == b);
    CHECK(kvcm_blocks_hash_from_crcs(crcs.data(), 23, 0, a.data()) == KVCM_ERR_INVALID_ARG);
    CHECK(std::string(kvcm_hip_error_string(KVCM_ERR_OUT_OF_RANGE)) == "index out of range");
    CHECK(kvcm_hip_version() >= 200);
    std::puts("ok host helpers");
}

// One caller's work on a store: writes `blocks` blocks of two iovs each (device or host memory) to its own file and to
// a file every caller shares (disjoint block ids), reads them back into fresh memory, compares.
void put_get_roundtrip(kvcm::LocalFileStore &store, int caller, int blocks, size_t bsz, bool device) {
    const uint8_t type = device ? KVCM_MEMORY_GPU : KVCM_MEMORY_CPU;
    const size_t a = bsz / 4, b = bsz - a;
    for (const std::string &path : {g_dir + "/own_" + std::to_string(caller), g_dir + "/shared"}) {
        std::vector<std::vector<uint8_t>> src, dst;
        std::vector<uint64_t> blkids;
        kvcm::BlockBuffers out, in;
        for (int i = 0; i < blocks; ++i) {
            src.push_back(pattern(bsz, static_cast<uint32_t>(caller * 1000 + i)));
            dst.emplace_back(bsz, 0);
        }
        for (int i = 0; i < blocks; ++i) {
            blkids.push_back(static_cast<uint64_t>(caller * blocks + (i * 5) % blocks));
            out.push_back({{{type, 0, src[i].data(), a}, {type, 0, src[i].data() + a, b}}});
            in.push_back({{{type, 0, dst[i].data(), a}, {type, 0, dst[i].data() + a, b}}});
        }
        CHECK(store.Put(path.c_str(), blkids, out) == KVCM_OK);
        CHECK(store.Get(path.c_str(), blkids, in) == KVCM_OK);
        for (int i = 0; i < blocks; ++i) {
            CHECK(src[i] == dst[i]);
        }
    }
}

void file_store_concurrent_callers() {
    for (bool device : {false, true}) {
        kvcm::LocalFileStore store(1 << 16, 24 * 1024 + 512, /*sync_on_put=*/false, /*io_threads=*/4);
        CHECK(store.Valid());
        std::vector<std::thread> th;
        for (int c = 0; c < 16; ++c) {
            th.emplace_back([&, c] { put_get_roundtrip(store, c, 6, 1 << 16, device); });
        }
        for (auto &t : th) {
            t.join();
        }
    }
    CHECK(fake_hip_live_allocations() == 0);  // every lane, stream, event and bounce buffer was given back
    std::puts("ok block files: 16 concurrent callers, host iovs and device iovs");
}

void big_get_shared_among_helpers() {
    const size_t bsz = 1 << 20;
    const int blocks = 24;  // consecutive block ids: one 24 MiB segment, 96 chunks of 256 KiB, four movers
    kvcm::LocalFileStore store(static_cast<int64_t>(bsz), 256 * 1024, false, 4);
    std::vector<uint8_t> src = pattern(bsz * blocks, 77), dst(bsz * blocks, 0);
    std::vector<uint64_t> blkids;
    kvcm::BlockBuffers out, in;
    for (int i = 0; i < blocks; ++i) {
        blkids.push_back(static_cast<uint64_t>(i));
        out.push_back({{{KVCM_MEMORY_GPU, 0, src.data() + i * bsz, bsz}}});
        in.push_back({{{KVCM_MEMORY_GPU, 0, dst.data() + i * bsz, bsz}}});
    }
    const std::string path = g_dir + "/big";
    CHECK(store.Put(path.c_str(), blkids, out) == KVCM_OK);
    CHECK(store.Get(path.c_str(), blkids, in) == KVCM_OK);
    CHECK(src == dst);
    // refused before a byte moves: wrong size parameter, an iov beyond the end of the file
    CHECK(store.Get(path.c_str(), {0}, {in[0]}, {bsz + 1}) == KVCM_ERR_INVALID_ARG);
    CHECK(store.Get(path.c_str(), {static_cast<uint64_t>(blocks)}, {in[0]}) == KVCM_ERR_INVALID_ARG);
    std::puts("ok block files: one big get shared among helper threads");
}

// kvcm_file_store_destroy while another thread is inside a get (or put) of the same store: the destroyer has to wait
// for the call, its helper jobs and its lanes. The stand-in runtime reports when the transfer has entered the library.
void destroy_while_a_transfer_runs() {
    const size_t bsz = 1 << 20;
    const int blocks = 8;
    std::vector<uint8_t> src = pattern(bsz * blocks, 5);
    std::vector<uint64_t> blkids, sizes(blocks, bsz);
    std::vector<int32_t> counts(blocks, 1);
    for (int i = 0; i < blocks; ++i) {
        blkids.push_back(static_cast<uint64_t>(i));
    }
    const std::string path = g_dir + "/destroy";
    {
        kvcm::LocalFileStore seed(static_cast<int64_t>(bsz), 64 * 1024, false, 4);
        kvcm::BlockBuffers out;
        for (int i = 0; i < blocks; ++i) {
            out.push_back({{{KVCM_MEMORY_GPU, 0, src.data() + i * bsz, bsz}}});
        }
        CHECK(seed.Put(path.c_str(), blkids, out) == KVCM_OK);
    }
    for (int round = 0; round < 24; ++round) {
        const bool put = round % 3 == 2;
        kvcm_file_store *store = nullptr;
        CHECK(kvcm_file_store_create(static_cast<int64_t>(bsz), 64 * 1024, 0, 1 + round % 4, &store) == KVCM_OK);
        std::vector<uint8_t> dst(bsz * blocks, 0);
        std::vector<kvcm_iov> iovs;
        for (int i = 0; i < blocks; ++i) {
            iovs.push_back({KVCM_MEMORY_GPU, 0, (put ? src.data() : dst.data()) + i * bsz, bsz});
        }
        std::mutex mu;
        std::condition_variable cv;
        bool inside = false;
        fake_hip_on_get_device([&] {
            std::lock_guard<std::mutex> lock(mu);
            inside = true;
            cv.notify_all();
        });
        std::atomic<int32_t> rc{-99};
        std::thread mover([&] {
            const std::string target = put ? path + "_w" + std::to_string(round) : path;
            rc = put ? kvcm_file_store_put(store, target.c_str(), blkids.data(), sizes.data(), counts.data(),
                                           iovs.data(), blocks)
                     : kvcm_file_store_get(store, target.c_str(), blkids.data(), sizes.data(), counts.data(),
                                           iovs.data(), blocks);
        });
        {
            std::unique_lock<std::mutex> lock(mu);
            cv.wait(lock, [&] { return inside; });
        }
        kvcm_file_store_destroy(store);  // the transfer is inside the library right now
        CHECK(rc.load() == KVCM_OK);     // ... and was over before destroy returned
        mover.join();
        fake_hip_on_get_device({});
        if (!put) {
            CHECK(dst == src);
        }
    }
    CHECK(fake_hip_live_allocations() == 0);
    std::puts("ok block files: a store destroyed while a get or put is inside it");
}

void copy_iovs_mixed() {
    std::vector<uint8_t> a = pattern(1000, 1), b = pattern(333, 2), c = pattern(4096, 3), buf(8192, 0), want(8192, 0);
    kvcm_iov iovs[4] = {{KVCM_MEMORY_CPU, 0, a.data(), a.size()},
                        {KVCM_MEMORY_GPU, 1, b.data(), b.size()},
                        {KVCM_MEMORY_GPU, 0, c.data(), c.size()},
                        {KVCM_MEMORY_CPU, 0, nullptr, 17}};
    CHECK(kvcm_copy_iovs(buf.data(), buf.size(), iovs, 4, 0, nullptr) == KVCM_OK);
    // the oracle follows the reference, which does not expect an iov without an address: it gets the first three
    CHECK(kvcm_ref_copy_iovs(want.data(), reinterpret_cast<const kvcm_ref_fiov *>(iovs), 3, 0) == 1000 + 4096);
    CHECK(buf == want);
    CHECK(kvcm_copy_iovs(buf.data(), 100, iovs, 4, 0, nullptr) == KVCM_ERR_INVALID_ARG);
    std::puts("ok CopyIovs");
}

void buffer_check_pool_blocks_and_wakes() {
    kvcm::SdkBufferCheckPool pool(2);
    CHECK(pool.Init(64));
    std::vector<std::vector<uint8_t>> data;
    kvcm::BlockBuffers bufs;
    for (int i = 0; i < 12; ++i) {
        data.push_back(pattern(512 + i, 40 + i));
    }
    for (int b = 0; b < 4; ++b) {
        kvcm::BlockBuffer bb;
        for (int k = 0; k < 3; ++k) {
            bb.iovs.push_back({KVCM_MEMORY_GPU, 0, data[b * 3 + k].data(), data[b * 3 + k].size()});
        }
        bufs.push_back(bb);
    }
    std::vector<kvcm_ref_iov> flat;
    for (auto &d : data) {
        flat.push_back({d.data(), d.size()});
    }
    std::vector<uint32_t> crc(12);
    std::vector<int64_t> want(4);
    CHECK(kvcm_ref_iov_crc32(flat.data(), 12, crc.data(), 4) == 0);
    CHECK(kvcm_ref_blocks_hash_from_crcs(crc.data(), 12, 3, want.data()) == 0);
    std::atomic<int> bad{0};
    std::vector<std::thread> th;
    for (int t = 0; t < 8; ++t) {  // four times as many threads as cells: GetCell blocks and is woken
        th.emplace_back([&] {
            for (int i = 0; i < 40; ++i) {
                if (pool.GetBlocksHash(bufs) != want) {
                    bad++;
                }
            }
        });
    }
    for (auto &t : th) {
        t.join();
    }
    CHECK(bad.load() == 0 && pool.FreeCells() == 2);
    std::vector<kvcm::TokenIdsVector> reqs = {{1, 2, 3, 4, 5, 6, 7, 8, 9}, {}, {-1, -2, -3, -4}};
    std::vector<kvcm::KeyVector> keys;
    CHECK(kvcm::GenKeyVectors(reqs, 4, &keys) == KVCM_OK && keys[0].size() == 2 && keys[1].empty() && keys[2].size() == 1);
    int64_t k0[2];
    CHECK(kvcm_ref_gen_key_vector(reqs[0].data(), 9, 4, 0, k0) == 2 && keys[0][0] == k0[0] && keys[0][1] == k0[1]);
    std::puts("ok buffer-check pool: 8 threads on 2 cells; GenKeyVectors");
}

}  // namespace

int main() {
    char tmpl[] = "/tmp/kvcm_sanitize_XXXXXX";
    CHECK(mkdtemp(tmpl) != nullptr);
    g_dir = tmpl;
    oracle_threaded_forms();
    index_list_walk();
    blocks_hash();
    file_store_concurrent_callers();
    big_get_shared_among_helpers();
    destroy_while_a_transfer_runs();
    copy_iovs_mixed();
    buffer_check_pool_blocks_and_wakes();
    CHECK(fake_hip_live_allocations() == 0);
    const std::string rm = "rm -rf " + g_dir;
    CHECK(std::system(rm.c_str()) == 0);
    std::puts("sanitize_host: all scenarios passed");
    return 0;
}
