// Stress driver for the cache store's host runtime (staging-node table, dump / load worker
// threads, task table), built with ThreadSanitizer by test_host_tsan.py and run WITHOUT a GPU:
// the few HIP calls and the copy-stream entry points the store uses are replaced below by
// host-memory stand-ins ("device" addresses are ordinary host buffers, a copy is a memcpy).
// The backend behind the store is asynchronous on purpose: load() returns at once and a thread
// of its own fills the staging node a little later, wait() joins it.  Tasks that name a shard
// the backend does not hold fail while loads of their earlier shards are still in flight; the
// nodes of such a task must not be handed to another key before those loads have ended (TSan
// reports the overlapping writes otherwise).  Exits non-zero on a wrong byte, a wrong status or
// a data race.
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <thread>
#include <vector>

#include "ucm_hip.h"

// ---- stand-ins for the HIP runtime calls of cache_store.hip ----
extern "C" hipError_t hipHostMalloc(void** p, size_t n, unsigned int) { *p = std::malloc(n); return *p ? hipSuccess : hipErrorOutOfMemory; }
extern "C" hipError_t hipHostFree(void* p) { std::free(p); return hipSuccess; }
extern "C" hipError_t hipSetDevice(int) { return hipSuccess; }
extern "C" hipError_t hipGetLastError(void) { return hipSuccess; }
extern "C" const char* hipGetErrorString(hipError_t) { return "stub"; }

// ---- stand-ins for the copy streams (trans.hip) ----
struct ucm_trans_stream { int unused; };
extern "C" int ucm_trans_setup(int32_t) { return UCM_OK; }
extern "C" int ucm_trans_stream_create(int, ucm_trans_stream_t** out) { *out = new ucm_trans_stream{0}; return UCM_OK; }
extern "C" int ucm_trans_stream_destroy(ucm_trans_stream_t* s) { delete s; return UCM_OK; }
extern "C" int ucm_trans_stream_sync(ucm_trans_stream_t*) { return UCM_OK; }
extern "C" int ucm_trans_stream_wait_event(ucm_trans_stream_t*, void*) { return UCM_OK; }
extern "C" int ucm_trans_gather(ucm_trans_stream_t*, const void* const* src, int, void* dst, size_t size, size_t number, int)
{
    for (size_t i = 0; i < number; ++i) std::memcpy((char*)dst + i * size, src[i], size);
    return UCM_OK;
}
extern "C" int ucm_trans_scatter(ucm_trans_stream_t*, const void* src, void* const* dst, int, size_t size, size_t number, int)
{
    for (size_t i = 0; i < number; ++i) std::memcpy(dst[i], (const char*)src + i * size, size);
    return UCM_OK;
}
extern "C" int ucm_trans_batch(ucm_trans_stream_t*, const void* const* src, void* const* dst, int, size_t size,
                               size_t number, int)
{
    for (size_t i = 0; i < number; ++i) std::memcpy(dst[i], src[i], size);
    return UCM_OK;
}

namespace {

constexpr size_t kShard = 4096;

struct KeyT {
    uint8_t id[16];
    uint64_t shard;
    bool operator<(const KeyT& o) const
    {
        const int c = std::memcmp(id, o.id, 16);
        return c < 0 || (c == 0 && shard < o.shard);
    }
};

// The slow tier: an in-memory table filled by dump(), read by load(); both run on threads of
// their own and finish some hundred microseconds after the hook has returned.
struct SlowStore {
    std::mutex mu;
    std::map<KeyT, std::vector<uint8_t>> shards;
    std::map<int64_t, std::thread> running;
    int64_t next = 1;
};

int64_t be_move(void* ctx, const uint8_t* ids, const uint64_t* idx, void* const* host, size_t n, size_t size,
                bool load)
{
    SlowStore* s = (SlowStore*)ctx;
    std::vector<KeyT> keys(n);
    std::vector<void*> hp(host, host + n);
    for (size_t i = 0; i < n; ++i) {
        std::memcpy(keys[i].id, ids + 16 * i, 16);
        keys[i].shard = idx[i];
    }
    std::lock_guard<std::mutex> lock(s->mu);
    if (load)
        for (const KeyT& k : keys)
            if (!s->shards.count(k)) return UCM_ENOOBJ;
    const int64_t h = s->next++;
    s->running.emplace(h, std::thread([s, keys, hp, size, load] {
        std::this_thread::sleep_for(std::chrono::microseconds(300));
        for (size_t i = 0; i < keys.size(); ++i) {
            if (load) {
                std::vector<uint8_t> copy;
                {
                    std::lock_guard<std::mutex> l2(s->mu);
                    copy = s->shards[keys[i]];
                }
                std::memcpy(hp[i], copy.data(), size);
            } else {
                std::vector<uint8_t> copy((uint8_t*)hp[i], (uint8_t*)hp[i] + size);
                std::lock_guard<std::mutex> l2(s->mu);
                s->shards[keys[i]] = std::move(copy);
            }
        }
    }));
    return h;
}
int64_t be_dump(void* c, const uint8_t* ids, const uint64_t* idx, void* const* host, size_t n, size_t sz) { return be_move(c, ids, idx, host, n, sz, false); }
int64_t be_load(void* c, const uint8_t* ids, const uint64_t* idx, void* const* host, size_t n, size_t sz) { return be_move(c, ids, idx, host, n, sz, true); }
int be_wait(void* ctx, int64_t h)
{
    SlowStore* s = (SlowStore*)ctx;
    std::thread t;
    {
        std::lock_guard<std::mutex> lock(s->mu);
        auto it = s->running.find(h);
        if (it == s->running.end()) return UCM_ENOOBJ;
        t = std::move(it->second);
        s->running.erase(it);
    }
    t.join();
    return UCM_OK;
}
int be_lookup(void* ctx, const uint8_t* ids, size_t n, uint8_t* found)
{
    SlowStore* s = (SlowStore*)ctx;
    std::lock_guard<std::mutex> lock(s->mu);
    for (size_t i = 0; i < n; ++i) {
        KeyT k{};
        std::memcpy(k.id, ids + 16 * i, 16);
        k.shard = 0;
        found[i] = s->shards.count(k) ? 1 : 0;
    }
    return UCM_OK;
}

uint8_t pattern(int tid, int round, int blk, size_t i) { return (uint8_t)(tid * 37 + round * 11 + blk * 5 + i); }

}  // namespace

int main()
{
    SlowStore slow;
    ucm_cache_backend_t be{&slow, be_lookup, be_dump, be_load, be_wait};
    const size_t sizes[2] = {kShard / 2, kShard / 2};
    ucm_cache_store_t* st = nullptr;
    // 20 staging nodes for 4 threads x 6 shards per task: nodes are recycled all the time, and
    // now and then a task finds every node held ("all nodes in use"), a legal failure
    if (ucm_cache_store_create(0, sizes, 2, 20 * kShard, 64, 5000, &be, &st) != UCM_OK) {
        std::printf("create: %s\n", ucm_last_error());
        return 1;
    }
    std::atomic<int> bad{0}, good_loads{0};
    auto work = [&](int tid) {
        const int nb = 6;
        for (int round = 0; round < 25; ++round) {
            std::vector<uint8_t> ids(16 * nb, 0);
            std::vector<uint64_t> idx(nb, 0);
            std::vector<std::vector<uint8_t>> src(nb * 2, std::vector<uint8_t>(kShard / 2));
            std::vector<void*> addrs(nb * 2);
            for (int b = 0; b < nb; ++b) {
                ids[16 * b] = (uint8_t)tid; ids[16 * b + 1] = (uint8_t)round; ids[16 * b + 2] = (uint8_t)b;
                for (int t = 0; t < 2; ++t) {
                    auto& v = src[b * 2 + t];
                    for (size_t i = 0; i < v.size(); ++i) v[i] = pattern(tid, round, b * 2 + t, i);
                    addrs[b * 2 + t] = v.data();
                }
            }
            int64_t task = 0;
            if (ucm_cache_store_dump(st, ids.data(), idx.data(), addrs.data(), nb, nullptr, &task) != UCM_OK) { ++bad; continue; }
            const int drc = ucm_cache_store_wait(st, task);
            if (drc == UCM_ERROR) continue;  // every node held by the other threads
            if (drc != UCM_OK) { ++bad; continue; }
            // a task whose LAST shard exists nowhere: the loads of the shards before it are
            // already running in the backend when the task fails
            std::vector<uint8_t> ids2(ids);
            ids2[16 * (nb - 1) + 3] = 0xEE;
            std::vector<std::vector<uint8_t>> junk(nb * 2, std::vector<uint8_t>(kShard / 2));
            std::vector<void*> jaddrs(nb * 2);
            for (size_t i = 0; i < junk.size(); ++i) jaddrs[i] = junk[i].data();
            if (ucm_cache_store_load(st, ids2.data(), idx.data(), jaddrs.data(), nb, &task) != UCM_OK) { ++bad; continue; }
            if (ucm_cache_store_wait(st, task) != UCM_ERROR) ++bad;
            // and right behind it a good load that competes for the same nodes
            std::vector<std::vector<uint8_t>> out(nb * 2, std::vector<uint8_t>(kShard / 2));
            for (size_t i = 0; i < out.size(); ++i) addrs[i] = out[i].data();
            if (ucm_cache_store_load(st, ids.data(), idx.data(), addrs.data(), nb, &task) != UCM_OK) { ++bad; continue; }
            const int rc = ucm_cache_store_wait(st, task);
            if (rc == UCM_OK) {
                ++good_loads;
                for (size_t i = 0; i < out.size(); ++i) if (out[i] != src[i]) ++bad;
            } else if (rc != UCM_ERROR) {  // "all nodes in use" under contention is a legal failure
                ++bad;
            }
        }
    };
    std::vector<std::thread> th;
    for (int i = 0; i < 4; ++i) th.emplace_back(work, i);
    for (auto& t : th) t.join();
    // dumps still on their way to the backend are waited for by destroy, not cut short
    std::vector<uint8_t> last_a(kShard / 2, 1), last_b(kShard / 2, 2);  // "device" memory: outlives the store
    {
        std::vector<uint8_t> id(16, 0xAB);
        uint64_t ix = 0;
        void* ad[2] = {last_a.data(), last_b.data()};
        int64_t task = 0;
        if (ucm_cache_store_dump(st, id.data(), &ix, ad, 1, nullptr, &task) != UCM_OK) ++bad;
    }
    ucm_cache_store_destroy(st);
    {
        std::lock_guard<std::mutex> lock(slow.mu);
        if (!slow.running.empty()) { std::printf("destroy left %zu backend transfers unwaited\n", slow.running.size()); ++bad; }
    }
    std::printf("bad=%d good_loads=%d\n", bad.load(), good_loads.load());
    return bad.load() != 0 || good_loads.load() < 20;
}
