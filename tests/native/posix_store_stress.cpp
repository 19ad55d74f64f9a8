// Stress driver for the host-only posix store, built with ThreadSanitizer by test_host_tsan.py:
// six threads dump, look up and load disjoint blocks (4 shards x 2 tensors each) through one
// store; exits non-zero on a wrong byte, a failed call or (through TSan) a data race.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>
#include "ucm_hip.h"

int main(int argc, char** argv)
{
    const char* root = argv[1];
    const char* backends[1] = {root};
    ucm_posix_config_t c{};
    c.storage_backends = backends; c.n_backends = 1; c.device_id = 0;
    c.tensor_size = 4096; c.shard_size = 8192; c.block_size = 32768;
    c.data_trans_concurrency = 8; c.lookup_concurrency = 4; c.timeout_ms = 10000; c.data_dir_shard_bytes = 1;
    ucm_posix_store_t* st = nullptr;
    if (ucm_posix_store_create(&c, &st) != UCM_OK) { printf("create: %s\n", ucm_last_error()); return 1; }
    int bad = 0;
    auto work = [&](int tid) {
        for (int round = 0; round < 10; ++round) {
            const int nb = 8, spb = 4;
            std::vector<uint8_t> ids(16 * nb * spb);
            std::vector<uint64_t> idx(nb * spb);
            std::vector<std::vector<uint8_t>> bufs(nb * spb * 2, std::vector<uint8_t>(4096));
            std::vector<void*> addrs(nb * spb * 2);
            for (int b = 0; b < nb; ++b)
                for (int s = 0; s < spb; ++s) {
                    uint8_t* id = &ids[16 * (b * spb + s)];
                    std::memset(id, 0, 16); id[0] = (uint8_t)tid; id[1] = (uint8_t)round; id[2] = (uint8_t)b;
                    idx[b * spb + s] = s;
                    for (int t = 0; t < 2; ++t) {
                        auto& v = bufs[(b * spb + s) * 2 + t];
                        for (size_t i = 0; i < v.size(); ++i) v[i] = (uint8_t)(tid * 31 + round * 7 + b * 3 + s * 5 + t + i);
                        addrs[(b * spb + s) * 2 + t] = v.data();
                    }
                }
            int64_t task = 0;
            if (ucm_posix_store_dump(st, ids.data(), idx.data(), addrs.data(), nb * spb, &task) != UCM_OK) { ++bad; continue; }
            int32_t fin = 0; (void)ucm_posix_store_check(st, task, &fin);
            if (ucm_posix_store_wait(st, task) != UCM_OK) { ++bad; continue; }
            std::vector<uint8_t> one(16 * nb);
            for (int b = 0; b < nb; ++b) std::memcpy(&one[16 * b], &ids[16 * b * spb], 16);
            int64_t last = -2;
            if (ucm_posix_store_lookup_on_prefix(st, one.data(), nb, &last) != UCM_OK || last != nb - 1) ++bad;
            std::vector<std::vector<uint8_t>> out(nb * spb * 2, std::vector<uint8_t>(4096));
            for (size_t i = 0; i < out.size(); ++i) addrs[i] = out[i].data();
            if (ucm_posix_store_load(st, ids.data(), idx.data(), addrs.data(), nb * spb, &task) != UCM_OK) { ++bad; continue; }
            if (ucm_posix_store_wait(st, task) != UCM_OK) { ++bad; continue; }
            for (size_t i = 0; i < out.size(); ++i) if (out[i] != bufs[i]) ++bad;
        }
    };
    std::vector<std::thread> th;
    for (int i = 0; i < 6; ++i) th.emplace_back(work, i);
    for (auto& t : th) t.join();
    ucm_posix_store_destroy(st);
    printf("bad=%d\n", bad);
    return bad != 0;
}
