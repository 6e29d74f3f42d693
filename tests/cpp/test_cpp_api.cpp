// C++ tests of the C-ABI and of include/kvcm_hip.hpp on the GPU, checked against the C oracle (the checker is
// linked here and only here). The CRC cases are the reference's own known answers
// (kv_cache_manager/client/src/internal/sdk/test/sdk_buffer_check_util_test.cc:13-74) run through this library.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <atomic>
#include <string>
#include <thread>
#include <vector>

#include "kvcm_hip.hpp"
#include "kvcm_oracle.h"

static int g_failed = 0, g_run = 0;
#define EXPECT(cond)                                                        \
    do {                                                                    \
        ++g_run;                                                            \
        if (!(cond)) {                                                      \
            ++g_failed;                                                     \
            std::printf("FAILED %s:%d  %s\n", __FILE__, __LINE__, #cond);   \
        }                                                                   \
    } while (0)

static std::vector<uint32_t> crc_of(const std::string &s, size_t min_cal) {
    char *buffer = nullptr;
    if (hipMalloc(reinterpret_cast<void **>(&buffer), s.size()) != hipSuccess) {
        return {0xBAD};
    }
    (void)hipMemcpy(buffer, s.data(), s.size(), hipMemcpyHostToDevice);
    std::vector<kvcm_iov_device> iovs_h{{buffer, s.size()}};
    auto crcs = kvcm::GetIovsCrc(iovs_h, min_cal);
    (void)hipFree(buffer);
    return crcs;
}

static void test_crc_known_answers() {
    EXPECT(crc_of("1234xxxxxxxx5678", 8) == std::vector<uint32_t>({0xDE28307C}));
    EXPECT(crc_of("1234xxxxxxxx5678", 4) == std::vector<uint32_t>({0x9AE0DAAF}));
    EXPECT(crc_of("1278", 4) == std::vector<uint32_t>({0xF639698C}));
    EXPECT(crc_of("1", 4).empty());
}

static void test_blocks_hash() {
    const size_t byte_size = 4 * 1024;
    char *buffer = nullptr;
    EXPECT(hipMalloc(reinterpret_cast<void **>(&buffer), byte_size) == hipSuccess);
    std::string s(byte_size, 'a');
    for (size_t i = 0; i < byte_size; ++i) {
        s[i] = static_cast<char>('a' + i % 23);
    }
    (void)hipMemcpy(buffer, s.data(), byte_size, hipMemcpyHostToDevice);
    std::vector<kvcm_iov_device> iovs;
    std::vector<kvcm_ref_iov> ref_iovs;
    for (int i = 0; i < 4; ++i) {
        iovs.push_back({buffer + 1024 * i, 1024});
        ref_iovs.push_back({s.data() + 1024 * i, 1024});
    }
    auto hashes = kvcm::GetBlocksHash(iovs, 2);
    uint32_t crcs[4];
    int64_t want[2];
    kvcm_ref_iov_crc32(ref_iovs.data(), 4, crcs, 4);
    kvcm_ref_blocks_hash_from_crcs(crcs, 4, 2, want);
    EXPECT(hashes.size() == 2 && hashes[0] == want[0] && hashes[1] == want[1]);
    (void)hipFree(buffer);
}

static void test_gen_key_vector() {
    // known answer: tokens 0..63, block size 16, as the reference header computes them
    kvcm::TokenIdsVector ramp(64);
    for (int i = 0; i < 64; ++i) {
        ramp[i] = i;
    }
    auto keys = kvcm::GenKeyVector(ramp, 16);
    EXPECT(keys == kvcm::KeyVector({6556265598806870907LL, 1204744731699469120LL, -7610010845176483469LL,
                                    2681637840371060507LL}));
    EXPECT(kvcm::GenKeyVector({1, 2, 3}, 4).empty());
    EXPECT(kvcm::GenKeyVector({}, 16).empty());
    EXPECT(kvcm::GenKeyVector({456}, 1) == kvcm::KeyVector({-7046029254386352675LL}));

    std::mt19937_64 rng(7);
    std::vector<kvcm::TokenIdsVector> reqs;
    for (int r = 0; r < 150; ++r) {
        kvcm::TokenIdsVector t(rng() % 700);
        for (auto &v : t) {
            v = static_cast<int64_t>(rng());
        }
        reqs.push_back(t);
    }
    for (int64_t bs : {16, 7, 64}) {
        std::vector<kvcm::KeyVector> got;
        EXPECT(kvcm::GenKeyVectors(reqs, bs, &got) == KVCM_OK);
        bool same = got.size() == reqs.size();
        for (size_t r = 0; same && r < reqs.size(); ++r) {
            kvcm::KeyVector want(reqs[r].size() / bs);
            kvcm_ref_gen_key_vector(reqs[r].data(), static_cast<int64_t>(reqs[r].size()), bs, 0, want.data());
            same = got[r] == want;
        }
        EXPECT(same);
    }
    // ApplyPrefixHash == the chain with one element per key
    kvcm::TokenIdsVector ids(reqs[3].begin(), reqs[3].end());
    std::vector<int64_t> want(ids.size()), off{0, static_cast<int64_t>(ids.size())};
    kvcm_ref_prefix_chain(ids.data(), off.data(), 1, want.data());
    EXPECT(kvcm::ApplyPrefixHash(ids) == want);
    std::vector<kvcm::KeyVector> none;
    EXPECT(kvcm::GenKeyVectors(reqs, 0, &none) == KVCM_ERR_INVALID_ARG);
}

static void test_gather_scatter_c_abi() {
    // 3 layers x K/V, T = 16, rows of 256 bytes, 40 pool blocks, 9 work blocks in scrambled staging slots
    const int P = 6, T = 16, B = 9, slots = 12, nblk = 40;
    const int64_t row = 256, tile = T * row, blk = P * tile;
    std::mt19937 rng(5);
    std::vector<std::vector<uint8_t>> pools(P, std::vector<uint8_t>(nblk * tile));
    for (auto &p : pools) {
        for (auto &b : p) {
            b = static_cast<uint8_t>(rng());
        }
    }
    std::vector<int32_t> idx(B * T), sidx(B);
    for (int b = 0; b < B; ++b) {
        sidx[b] = (b * 5 + 3) % slots;
        for (int t = 0; t < T; ++t) {
            idx[b * T + t] = static_cast<int32_t>(rng() % (nblk * T));
        }
    }
    std::vector<uint8_t> want(slots * blk, 0x6B), got(slots * blk, 0x6B);
    std::vector<const void *> table_h(P);
    for (int p = 0; p < P; ++p) {
        table_h[p] = pools[p].data();
    }
    EXPECT(kvcm_ref_batch_gather(table_h.data(), P, want.data(), blk, idx.data(), sidx.data(), B, T, row) == 0);

    std::vector<void *> d_pools(P);
    for (int p = 0; p < P; ++p) {
        EXPECT(hipMalloc(&d_pools[p], pools[p].size()) == hipSuccess);
        (void)hipMemcpy(d_pools[p], pools[p].data(), pools[p].size(), hipMemcpyHostToDevice);
    }
    void **d_table;
    int32_t *d_idx, *d_sidx;
    uint8_t *d_stage;
    EXPECT(hipMalloc(reinterpret_cast<void **>(&d_table), P * sizeof(void *)) == hipSuccess);
    EXPECT(hipMalloc(reinterpret_cast<void **>(&d_idx), idx.size() * 4) == hipSuccess);
    EXPECT(hipMalloc(reinterpret_cast<void **>(&d_sidx), sidx.size() * 4) == hipSuccess);
    EXPECT(hipMalloc(reinterpret_cast<void **>(&d_stage), got.size()) == hipSuccess);
    (void)hipMemcpy(d_table, d_pools.data(), P * sizeof(void *), hipMemcpyHostToDevice);
    (void)hipMemcpy(d_idx, idx.data(), idx.size() * 4, hipMemcpyHostToDevice);
    (void)hipMemcpy(d_sidx, sidx.data(), sidx.size() * 4, hipMemcpyHostToDevice);
    (void)hipMemcpy(d_stage, got.data(), got.size(), hipMemcpyHostToDevice);
    hipStream_t stream;
    EXPECT(hipStreamCreate(&stream) == hipSuccess);
    EXPECT(kvcm_hip_batch_gather(d_table, P, d_stage, blk, d_idx, d_sidx, B, T, row, 0, stream) == KVCM_OK);
    EXPECT(hipStreamSynchronize(stream) == hipSuccess);
    (void)hipMemcpy(got.data(), d_stage, got.size(), hipMemcpyDeviceToHost);
    EXPECT(got == want);
    // a capped grid (the reference's sm_count = 3) gives the same bytes
    (void)hipMemset(d_stage, 0x6B, got.size());
    EXPECT(kvcm_hip_batch_gather(d_table, P, d_stage, blk, d_idx, d_sidx, B, T, row, 3, stream) == KVCM_OK);
    EXPECT(hipStreamSynchronize(stream) == hipSuccess);
    (void)hipMemcpy(got.data(), d_stage, got.size(), hipMemcpyDeviceToHost);
    EXPECT(got == want);
    EXPECT(kvcm_hip_batch_gather(d_table, P, d_stage, blk - 1, d_idx, d_sidx, B, T, row, 0, stream) ==
           KVCM_ERR_INVALID_ARG);
    EXPECT(std::string(kvcm_hip_error_string(KVCM_ERR_TOO_LARGE)).size() > 0);
    for (auto p : d_pools) {
        (void)hipFree(p);
    }
    (void)hipFree(d_table);
    (void)hipFree(d_idx);
    (void)hipFree(d_sidx);
    (void)hipFree(d_stage);
    (void)hipStreamDestroy(stream);
}

// The reference's own GPU unit test of the local-file SDK restated on this library
// (kv_cache_manager/client/src/internal/sdk/test/local_file_sdk_test.cc:97-172): two device iovs of one 1024-byte
// block, a URI size that does not match refused, the bytes read back into fresh device memory.
static void test_local_file_put_get_with_gpu() {
    const char *test_data = "this is local file test";
    const char *test_data_2 = "and this is another local file test";
    const size_t len1 = std::strlen(test_data), len2 = std::strlen(test_data_2);
    std::string host_put = std::string(test_data) + test_data_2;
    char tmpl[] = "/tmp/kvcm_cpp_XXXXXX";
    const char *dir = mkdtemp(tmpl);
    EXPECT(dir != nullptr);
    const std::string path = std::string(dir ? dir : "/tmp") + "/local_file/test_gpu.txt";

    char *gpu_put = nullptr, *gpu_get = nullptr;
    EXPECT(hipMalloc(reinterpret_cast<void **>(&gpu_put), len1 + len2) == hipSuccess);
    EXPECT(hipMalloc(reinterpret_cast<void **>(&gpu_get), len1 + len2) == hipSuccess);
    EXPECT(hipMemcpy(gpu_put, host_put.data(), len1 + len2, hipMemcpyHostToDevice) == hipSuccess);
    EXPECT(hipMemset(gpu_get, 0, len1 + len2) == hipSuccess);

    kvcm::LocalFileStore sdk(1024);
    EXPECT(sdk.Valid());
    kvcm::BlockBuffer buf;
    buf.iovs.push_back(kvcm_iov{KVCM_MEMORY_GPU, 0, gpu_put, len1});
    buf.iovs.push_back(kvcm_iov{KVCM_MEMORY_GPU, 0, gpu_put + len1, len2});
    EXPECT(sdk.Put(path.c_str(), {0}, {buf}, {1023}) == KVCM_ERR_INVALID_ARG);
    EXPECT(sdk.Put(path.c_str(), {0}, {buf}) == KVCM_OK);

    // the file is what the reference's DoPut leaves (restated in the oracle, host iovs)
    const std::string ref_path = std::string(dir ? dir : "/tmp") + "/reference.bin";
    const uint64_t blkid = 0, size = 1024;
    const int32_t count = 2;
    kvcm_ref_fiov fiovs[2] = {{0, 0, const_cast<char *>(host_put.data()), len1},
                              {0, 0, const_cast<char *>(host_put.data()) + len1, len2}};
    EXPECT(kvcm_ref_file_put(ref_path.c_str(), 1024, &blkid, &size, &count, fiovs, 1) == 0);
    auto slurp = [](const std::string &p) {
        std::string out;
        if (FILE *f = std::fopen(p.c_str(), "rb")) {
            char chunk[4096];
            size_t got;
            while ((got = std::fread(chunk, 1, sizeof chunk, f)) > 0) {
                out.append(chunk, got);
            }
            std::fclose(f);
        }
        return out;
    };
    EXPECT(slurp(path).size() == 1024 && slurp(path) == slurp(ref_path));

    kvcm::BlockBuffer gbuf;
    gbuf.iovs.push_back(kvcm_iov{KVCM_MEMORY_GPU, 0, gpu_get, len1});
    gbuf.iovs.push_back(kvcm_iov{KVCM_MEMORY_GPU, 0, gpu_get + len1, len2});
    EXPECT(sdk.Get(path.c_str(), {0}, {gbuf}, {1023}) == KVCM_ERR_INVALID_ARG);
    EXPECT(sdk.Get(ref_path.c_str(), {0}, {gbuf}) == KVCM_OK);
    std::string host_get(len1 + len2, '\0');
    EXPECT(hipMemcpy(&host_get[0], gpu_get, len1 + len2, hipMemcpyDeviceToHost) == hipSuccess);
    EXPECT(host_get == host_put);
    EXPECT(sdk.Get((path + ".missing").c_str(), {0}, {gbuf}) == KVCM_ERR_IO);
    (void)hipFree(gpu_put);
    (void)hipFree(gpu_get);
}

static void test_first_occurrence() {
    std::mt19937_64 rng(99);
    std::vector<int64_t> base(700), keys(5000);
    for (auto &b : base) {
        b = static_cast<int64_t>(rng());
    }
    for (auto &k : keys) {
        k = base[rng() % base.size()];
    }
    keys[7] = INT64_MIN;
    keys[4999] = INT64_MIN;
    std::vector<int32_t> got, want(keys.size());
    EXPECT(kvcm::FirstOccurrence(keys, &got) == KVCM_OK);
    EXPECT(kvcm_ref_first_occurrence(keys.data(), static_cast<int64_t>(keys.size()), want.data(), nullptr) == 0);
    EXPECT(got == want);
    EXPECT(got[4999] == 7);
    std::vector<int32_t> none;
    EXPECT(kvcm::FirstOccurrence({}, &none) == KVCM_OK && none.empty());
}

// SdkBufferCheckPool as the reference's tests use it
// (kv_cache_manager/client/src/internal/sdk/test/sdk_buffer_check_util_test.cc:283-382): equal buffers give equal
// block hashes through a cell, cells are handed out and taken back, eight threads share four cells.
static kvcm::BlockBuffer four_iov_block(char fill, size_t byte_size = 4 * 1024) {
    char *buffer = nullptr;
    EXPECT(hipMalloc(reinterpret_cast<void **>(&buffer), byte_size) == hipSuccess);
    std::string init(byte_size, fill);
    (void)hipMemcpy(buffer, init.data(), byte_size, hipMemcpyHostToDevice);
    kvcm::BlockBuffer b;
    for (int i = 0; i < 4; ++i) {
        b.iovs.push_back(kvcm_iov{KVCM_MEMORY_GPU, 0, buffer + 1024 * i, 1024});
    }
    return b;
}

static void test_buffer_check_pool() {
    const size_t max_check_iov_num = 10;
    {
        kvcm::SdkBufferCheckPool pool;
        EXPECT(pool.Init(max_check_iov_num));
        kvcm::BlockBuffers blocks{four_iov_block('a'), four_iov_block('a'), four_iov_block('a')};
        auto handle = pool.GetCell();
        auto hashes = kvcm::GetBlocksHash(blocks, handle->d_iovs, handle->d_crcs, handle->h_iovs, max_check_iov_num,
                                          handle->stream);
        EXPECT(hashes.size() == 2);  // the third block's iovs would exceed max_check_iov_num: not checked
        EXPECT(hashes.size() == 2 && hashes[0] == hashes[1]);
        // the value: CRC of "aaaa" + "aaaa" per iov, chained over four iovs, from the oracle
        std::string a(1024, 'a');
        kvcm_ref_iov ref[4] = {{a.data(), 1024}, {a.data(), 1024}, {a.data(), 1024}, {a.data(), 1024}};
        uint32_t crcs[4];
        int64_t want[1];
        kvcm_ref_iov_crc32(ref, 4, crcs, 4);
        kvcm_ref_blocks_hash_from_crcs(crcs, 4, 4, want);
        EXPECT(!hashes.empty() && hashes[0] == want[0]);
        // an iov shorter than the bytes taken per end, or without an address: nothing is launched
        kvcm::BlockBuffers bad{four_iov_block('a')};
        bad[0].iovs[2].size = 3;
        EXPECT(kvcm::GetBlocksHash(bad, handle->d_iovs, handle->d_crcs, handle->h_iovs, max_check_iov_num,
                                   handle->stream).empty());
        bad[0].iovs[2].size = 1024;
        bad[0].iovs[1].base = nullptr;
        EXPECT(kvcm::GetBlocksHash(bad, handle->d_iovs, handle->d_crcs, handle->h_iovs, max_check_iov_num,
                                   handle->stream).empty());
    }
    {
        kvcm::SdkBufferCheckPool pool(2);
        EXPECT(pool.Init(max_check_iov_num));
        EXPECT(pool.FreeCells() == 2);
        {
            auto h1 = pool.GetCell();
            EXPECT(pool.FreeCells() == 1);
            auto h2 = pool.GetCell();
            EXPECT(pool.FreeCells() == 0);
            EXPECT(h1->d_iovs != h2->d_iovs && h1->stream != h2->stream);
        }
        EXPECT(pool.FreeCells() == 2);
    }
    {
        kvcm::SdkBufferCheckPool pool;
        EXPECT(pool.Init(max_check_iov_num));
        std::vector<kvcm::BlockBuffers> sets{{four_iov_block('a')}, {four_iov_block('a')}};
        const auto expect = pool.GetBlocksHash(sets[0]);
        EXPECT(expect.size() == 1);
        std::atomic<int> wrong{0};
        for (int round = 0; round < 20; ++round) {
            std::vector<std::thread> threads;
            for (int j = 0; j < 8; ++j) {
                threads.emplace_back([&, round] {
                    if (pool.GetBlocksHash(sets[round % 2]) != expect) {
                        wrong.fetch_add(1);
                    }
                });
            }
            for (auto &t : threads) {
                t.join();
            }
        }
        EXPECT(wrong.load() == 0);
        EXPECT(pool.FreeCells() == 4);
    }
}

int main() {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n == 0) {
        std::printf("no GPU\n");
        return 2;
    }
    test_crc_known_answers();
    test_blocks_hash();
    test_gen_key_vector();
    test_gather_scatter_c_abi();
    test_local_file_put_get_with_gpu();
    test_first_occurrence();
    test_buffer_check_pool();
    std::printf("%d checks, %d failed\n", g_run, g_failed);
    return g_failed == 0 ? 0 : 1;
}
