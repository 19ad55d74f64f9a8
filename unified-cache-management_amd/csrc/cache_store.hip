// Pinned-host staging cache between the paged KV cache in HBM and a slower store backend:
// the caller of the gather / scatter kernels.
//
// Follows the reference's CacheStore (ucm/store/cache/cc/): TransBuffer (trans_buffer.cc:
// a table of shard-sized pinned nodes keyed by (block id, shard index), reference counts, a
// ready flag, ring replacement of unreferenced nodes), DumpQueue (dump_queue.cc: device ->
// node, then hand the node to the backend), LoadQueue (load_queue.cc: backend -> node when it
// is not resident, then node -> device), TransManager / TaskWrapper (task ids, Check, Wait with
// a timeout, a failure set; ucm/store/detail/template/task_wrapper.h:40-110).
//
// Design for MI355X, one process per GPU:
//   * a task's shards move in ONE kernel launch over a pointer table with one entry per
//     (shard, tensor) — the kernel writes straight into pinned host memory at PCIe speed —
//     where the reference issues one cudaMemcpyAsync per tensor of every shard
//     (dump_queue.cc:145-161, load_queue.cc:178-194);
//   * the node table lives in process memory behind one mutex: the reference's
//     shared-memory table with per-bucket process-shared locks exists so that several worker
//     processes of one host can share a cache, which one process per GPU does not need;
//   * a dump is gated on the producer's event with hipStreamWaitEvent on the store's own
//     side stream (default priority), never by blocking the caller.
#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <deque>
#include <memory>
#include <mutex>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "common.h"
#include "host_queue.h"

namespace {

struct Key {
    uint8_t id[16];
    uint64_t shard;
    bool operator==(const Key& o) const { return shard == o.shard && std::memcmp(id, o.id, 16) == 0; }
};

struct KeyHash {
    size_t operator()(const Key& k) const
    {
        uint64_t a, b;
        std::memcpy(&a, k.id, 8);
        std::memcpy(&b, k.id + 8, 8);
        uint64_t h = a * 0x9e3779b97f4a7c15ull ^ (b + 0x9e3779b97f4a7c15ull + (a << 6) + (a >> 2));
        return (size_t)(h ^ (k.shard * 0xff51afd7ed558ccdull));
    }
};

// Pinned slab of shard-sized nodes + (block, shard) -> node table.  Semantics of
// TransBuffer::Get / Exist / Alloc (trans_buffer.cc:473-585): a hit returns the node and makes
// the caller its owner iff nobody else holds it; a miss takes the next node of a ring that
// nobody holds, forgets what it cached and hands it over not-ready.
class StagingBuffer {
public:
    ~StagingBuffer()
    {
        if (data_) (void)hipHostFree(data_);
    }
    int setup(size_t node_size, size_t capacity)
    {
        node_size_ = node_size;
        n_ = node_size ? capacity / node_size : 0;
        UCM_REQUIRE(n_ >= 1, "buffer capacity %zu holds no shard of %zu bytes", capacity, node_size);
        UCM_HIP_TRY(hipHostMalloc(&data_, n_ * node_size, hipHostMallocDefault));
        meta_.assign(n_, Node{});
        index_.reserve(n_ * 2);
        return UCM_OK;
    }
    size_t nodes() const { return n_; }
    // UCM_ENOSPACE-like failure when every node is held
    int get(const Key& k, size_t* pos, bool* owner)
    {
        std::lock_guard<std::mutex> lock(mu_);
        auto it = index_.find(k);
        if (it != index_.end()) {
            Node& nd = meta_[it->second];
            *owner = nd.ref == 0;
            ++nd.ref;
            *pos = it->second;
            return UCM_OK;
        }
        for (size_t tried = 0; tried < n_; ++tried) {
            const size_t i = head_;
            head_ = head_ + 1 == n_ ? 0 : head_ + 1;
            Node& nd = meta_[i];
            if (nd.ref > 0) continue;
            if (nd.used) index_.erase(nd.key);
            nd.key = k;
            nd.used = true;
            nd.ready = false;
            nd.ref = 1;
            index_.emplace(k, i);
            *pos = i;
            *owner = true;
            return UCM_OK;
        }
        return ucm::fail(UCM_ERROR, "all %zu staging nodes are in use", n_);
    }
    bool exist(const Key& k)
    {
        std::lock_guard<std::mutex> lock(mu_);
        return index_.find(k) != index_.end();
    }
    void* data(size_t pos) const { return (char*)data_ + pos * node_size_; }
    bool ready(size_t pos)
    {
        std::lock_guard<std::mutex> lock(mu_);
        return meta_[pos].ready;
    }
    void mark_ready(size_t pos)
    {
        std::lock_guard<std::mutex> lock(mu_);
        meta_[pos].ready = true;
    }
    void release(size_t pos)
    {
        std::lock_guard<std::mutex> lock(mu_);
        if (meta_[pos].ref > 0) --meta_[pos].ref;
    }
    // drops a node whose content never became valid, so that no later lookup finds it
    void discard(size_t pos)
    {
        std::lock_guard<std::mutex> lock(mu_);
        Node& nd = meta_[pos];
        if (nd.ref > 0) --nd.ref;
        if (nd.ref == 0 && nd.used && !nd.ready) {
            index_.erase(nd.key);
            nd.used = false;
        }
    }

private:
    struct Node {
        Key key{};
        size_t ref = 0;
        bool ready = false;
        bool used = false;
    };
    std::mutex mu_;
    std::unordered_map<Key, size_t, KeyHash> index_;
    std::vector<Node> meta_;
    size_t head_ = 0, n_ = 0, node_size_ = 0;
    void* data_ = nullptr;
};

struct Shard {
    Key key;
    std::vector<void*> addrs;  // one device address per tensor of the shard
};

struct Task {
    int64_t id = 0;
    bool load = false;
    std::vector<Shard> shards;
    void* prerequisite = nullptr;  // hipEvent_t the dump waits for
};

using TaskPtr = std::shared_ptr<Task>;
using WaiterPtr = std::shared_ptr<Waiter>;

struct LoadCtx {
    TaskPtr task;
    WaiterPtr waiter;
    std::vector<size_t> pos;        // staging node of every shard
    std::vector<int64_t> backend;   // backend load handle of every shard, 0 = none
};

struct DumpCtx {
    int64_t task = 0;
    int64_t backend = 0;
    std::vector<size_t> held;
};

}  // namespace

struct ucm_cache_store {
    int device = 0;
    std::vector<size_t> tensor_sizes;
    std::vector<size_t> tensor_offsets;
    size_t shard_size = 0;
    size_t timeout_ms = 30000;
    StagingBuffer buffer;
    ucm_cache_backend_t backend{};
    bool has_backend = false;

    std::mutex tasks_mu;
    std::unordered_map<int64_t, std::pair<TaskPtr, WaiterPtr>> tasks;
    std::mutex fail_mu;
    std::unordered_set<int64_t> failures;
    std::atomic<int64_t> next_id{1};

    BoundedQueue<std::pair<TaskPtr, WaiterPtr>> dump_waiting, load_waiting;
    BoundedQueue<LoadCtx> load_running;
    BoundedQueue<DumpCtx> dumping;
    std::atomic<bool> stop{false};
    std::atomic<bool> stop_backend{false};  // set after the dump dispatcher has been joined
    ucm_trans_stream_t* dump_stream = nullptr;
    ucm_trans_stream_t* load_stream = nullptr;
    std::thread dump_dispatcher, dump_backend, load_dispatcher, load_transfer;

    bool failed(int64_t id)
    {
        std::lock_guard<std::mutex> lock(fail_mu);
        return failures.count(id) != 0;
    }
    void fail(int64_t id)
    {
        std::lock_guard<std::mutex> lock(fail_mu);
        failures.insert(id);
    }
    void clear_failure(int64_t id)
    {
        std::lock_guard<std::mutex> lock(fail_mu);
        failures.erase(id);
    }
};

namespace {

// (shard, tensor) chunk i moves between dev[i] and host[i]; to_device = false: device -> host.
// Mixed tensor sizes: one kernel launch per distinct size over a pointer table.
int move_chunks(ucm_cache_store* st, ucm_trans_stream_t* stream, const std::vector<size_t>& pos,
                const std::vector<const Shard*>& shards, bool to_device)
{
    const size_t nt = st->tensor_sizes.size();
    std::vector<size_t> sizes(st->tensor_sizes);
    std::sort(sizes.begin(), sizes.end());
    sizes.erase(std::unique(sizes.begin(), sizes.end()), sizes.end());
    if (sizes.size() == 1) {
        // equal tensors (the usual KV layout): a shard's node is the flat side of a gather /
        // scatter, which the copy stream stages through device memory and moves over PCIe with
        // the copy engine, so that kernels of other streams keep running beside the transfer
        for (size_t s = 0; s < shards.size(); ++s) {
            void* node = st->buffer.data(pos[s]);
            const int rc = to_device
                               ? ucm_trans_scatter(stream, node, shards[s]->addrs.data(), 0, sizes[0], nt, 0)
                               : ucm_trans_gather(stream, (const void* const*)shards[s]->addrs.data(), 0, node,
                                                  sizes[0], nt, 0);
            if (rc != UCM_OK) return rc;
        }
        return UCM_OK;
    }
    std::vector<const void*> src;
    std::vector<void*> dst;
    for (size_t size : sizes) {
        src.clear();
        dst.clear();
        for (size_t s = 0; s < shards.size(); ++s) {
            char* node = (char*)st->buffer.data(pos[s]);
            for (size_t t = 0; t < nt; ++t) {
                if (st->tensor_sizes[t] != size) continue;
                void* dev = shards[s]->addrs[t];
                void* host = node + st->tensor_offsets[t];
                src.push_back(to_device ? host : dev);
                dst.push_back(to_device ? dev : host);
            }
        }
        if (src.empty()) continue;
        int rc = ucm_trans_batch(stream, src.data(), dst.data(), 0, size, src.size(), 0);
        if (rc != UCM_OK) return rc;
    }
    return UCM_OK;
}

int dump_one(ucm_cache_store* st, const TaskPtr& task)
{
    if (task->prerequisite) {
        int rc = ucm_trans_stream_wait_event(st->dump_stream, task->prerequisite);
        if (rc != UCM_OK) return rc;
    }
    DumpCtx ctx;
    ctx.task = task->id;
    std::vector<size_t> copy_pos;
    std::vector<const Shard*> copy_shards, owned;
    int rc = UCM_OK;
    for (const Shard& sh : task->shards) {
        size_t pos = 0;
        bool owner = false;
        rc = st->buffer.get(sh.key, &pos, &owner);
        if (rc != UCM_OK) break;
        if (!owner) {  // somebody else is already writing or reading this shard
            st->buffer.release(pos);
            continue;
        }
        if (!st->buffer.ready(pos)) {
            copy_pos.push_back(pos);
            copy_shards.push_back(&sh);
        }
        ctx.held.push_back(pos);
        owned.push_back(&sh);
    }
    if (rc == UCM_OK && !copy_pos.empty()) {
        rc = move_chunks(st, st->dump_stream, copy_pos, copy_shards, false);
        if (rc == UCM_OK) rc = ucm_trans_stream_sync(st->dump_stream);
    }
    if (rc != UCM_OK) {
        for (size_t p : ctx.held) st->buffer.discard(p);
        return rc;
    }
    for (size_t p : ctx.held) st->buffer.mark_ready(p);
    if (st->has_backend && st->backend.dump && !ctx.held.empty()) {
        std::vector<uint8_t> ids(owned.size() * 16);
        std::vector<uint64_t> idx(owned.size());
        std::vector<void*> host(owned.size());
        for (size_t i = 0; i < owned.size(); ++i) {
            std::memcpy(&ids[i * 16], owned[i]->key.id, 16);
            idx[i] = owned[i]->key.shard;
            host[i] = st->buffer.data(ctx.held[i]);
        }
        const int64_t h = st->backend.dump(st->backend.ctx, ids.data(), idx.data(), host.data(),
                                           owned.size(), st->shard_size);
        if (h < 0) {
            for (size_t p : ctx.held) st->buffer.release(p);
            return ucm::fail((int)h, "backend refused the dump of task %lld", (long long)task->id);
        }
        ctx.backend = h;
        st->dumping.push(std::move(ctx));  // nodes stay held until the backend has them
    } else {
        for (size_t p : ctx.held) st->buffer.release(p);
    }
    return UCM_OK;
}

void dump_dispatch_stage(ucm_cache_store* st)
{
    (void)hipSetDevice(st->device);
    std::pair<TaskPtr, WaiterPtr> pr;
    while (st->dump_waiting.pop(pr, st->stop)) {
        if (!st->failed(pr.first->id) && dump_one(st, pr.first) != UCM_OK) st->fail(pr.first->id);
        pr.second->done();
        pr = {};
    }
}

void dump_backend_stage(ucm_cache_store* st)
{
    DumpCtx ctx;
    while (st->dumping.pop(ctx, st->stop_backend)) {
        if (ctx.backend > 0 && st->backend.wait) (void)st->backend.wait(st->backend.ctx, ctx.backend);
        for (size_t p : ctx.held) st->buffer.release(p);
        ctx = {};
    }
}

void load_dispatch_stage(ucm_cache_store* st)
{
    std::pair<TaskPtr, WaiterPtr> pr;
    while (st->load_waiting.pop(pr, st->stop)) {
        const TaskPtr& task = pr.first;
        if (st->failed(task->id)) {
            pr.second->done();
            pr = {};
            continue;
        }
        LoadCtx ctx;
        ctx.task = task;
        ctx.waiter = pr.second;
        bool ok = true;
        for (const Shard& sh : task->shards) {
            size_t pos = 0;
            bool owner = false;
            if (st->buffer.get(sh.key, &pos, &owner) != UCM_OK) {
                ok = false;
                break;
            }
            int64_t h = 0;
            if (owner && !st->buffer.ready(pos)) {
                // not resident: the backend fills the node (load_queue.cc:96-110)
                if (st->has_backend && st->backend.load) {
                    void* host = st->buffer.data(pos);
                    h = st->backend.load(st->backend.ctx, sh.key.id, &sh.key.shard, &host, 1,
                                         st->shard_size);
                }
                if (h <= 0) {
                    st->buffer.discard(pos);
                    ok = false;
                    break;
                }
            }
            ctx.pos.push_back(pos);
            ctx.backend.push_back(h);
        }
        if (!ok) {
            for (size_t i = 0; i < ctx.pos.size(); ++i) {
                if (ctx.backend[i] > 0) {
                    // the backend may still be writing into the node: it goes back to the ring
                    // only after that load has ended, whatever its outcome
                    if (st->backend.wait) (void)st->backend.wait(st->backend.ctx, ctx.backend[i]);
                    st->buffer.discard(ctx.pos[i]);
                } else {
                    st->buffer.release(ctx.pos[i]);
                }
            }
            st->fail(task->id);
            pr.second->done();
        } else {
            st->load_running.push(std::move(ctx));
        }
        pr = {};
    }
}

void load_transfer_stage(ucm_cache_store* st)
{
    (void)hipSetDevice(st->device);
    LoadCtx ctx;
    while (st->load_running.pop(ctx, st->stop)) {
        const int64_t id = ctx.task->id;
        bool ok = !st->failed(id);
        const auto deadline = Clock::now() + std::chrono::milliseconds(st->timeout_ms);
        std::vector<char> waited(ctx.pos.size(), 0);
        for (size_t i = 0; ok && i < ctx.pos.size(); ++i) {
            if (ctx.backend[i] > 0) {
                ok = !st->backend.wait || st->backend.wait(st->backend.ctx, ctx.backend[i]) == UCM_OK;
                waited[i] = 1;
                if (ok) st->buffer.mark_ready(ctx.pos[i]);
            } else {
                // another task is filling this node (load_queue.cc:168-174)
                while (!st->buffer.ready(ctx.pos[i])) {
                    if (st->failed(id) || Clock::now() > deadline) {
                        ok = false;
                        break;
                    }
                    std::this_thread::yield();
                }
            }
        }
        if (ok) {
            std::vector<const Shard*> shards;
            for (const Shard& sh : ctx.task->shards) shards.push_back(&sh);
            ok = move_chunks(st, st->load_stream, ctx.pos, shards, true) == UCM_OK &&
                 ucm_trans_stream_sync(st->load_stream) == UCM_OK;
        }
        for (size_t i = 0; i < ctx.pos.size(); ++i) {
            // a load the loop above never reached (an earlier shard failed, the task was marked
            // failed or timed out) may still be writing into its node: wait before the node can
            // be handed to another key
            if (ctx.backend[i] > 0 && !waited[i] && st->backend.wait)
                (void)st->backend.wait(st->backend.ctx, ctx.backend[i]);
            if (!ok && ctx.backend[i] > 0 && !st->buffer.ready(ctx.pos[i])) st->buffer.discard(ctx.pos[i]);
            else st->buffer.release(ctx.pos[i]);
        }
        if (!ok) st->fail(id);
        ctx.waiter->done();
        ctx = {};
    }
}

int submit(ucm_cache_store* st, bool load, const uint8_t* block_ids, const uint64_t* shard_idx,
           void* const* addrs, size_t n, void* prerequisite, int64_t* task_out)
{
    ucm::clear_error();
    UCM_REQUIRE(st && task_out, "null store or task pointer");
    UCM_REQUIRE(n == 0 || (block_ids && shard_idx && addrs), "null shard description");
    const size_t nt = st->tensor_sizes.size();
    auto task = std::make_shared<Task>();
    task->id = st->next_id.fetch_add(1);
    task->load = load;
    task->prerequisite = prerequisite;
    task->shards.resize(n);
    for (size_t i = 0; i < n; ++i) {
        std::memcpy(task->shards[i].key.id, block_ids + i * 16, 16);
        task->shards[i].key.shard = shard_idx[i];
        task->shards[i].addrs.assign(addrs + i * nt, addrs + (i + 1) * nt);
        for (void* p : task->shards[i].addrs) UCM_REQUIRE(p, "null device address in shard %zu", i);
    }
    auto waiter = std::make_shared<Waiter>();
    {
        std::lock_guard<std::mutex> lock(st->tasks_mu);
        st->tasks.emplace(task->id, std::make_pair(task, waiter));
    }
    waiter->up();
    auto& q = load ? st->load_waiting : st->dump_waiting;
    if (!q.try_push(std::make_pair(task, waiter))) {
        // as the reference: the task exists, is marked failed and finishes at once
        // (dump_queue.cc:66-75, load_queue.cc:58-67)
        st->fail(task->id);
        waiter->done();
    }
    *task_out = task->id;
    return UCM_OK;
}

}  // namespace

extern "C" int ucm_cache_store_create(int32_t device_id, const size_t* tensor_sizes,
                                      size_t n_tensors, size_t buffer_bytes,
                                      size_t waiting_queue_depth, size_t timeout_ms,
                                      const ucm_cache_backend_t* backend, ucm_cache_store_t** out)
{
    ucm::clear_error();
    UCM_REQUIRE(out, "null output");
    UCM_REQUIRE(tensor_sizes && n_tensors > 0, "invalid tensor size");
    UCM_REQUIRE(waiting_queue_depth > 1, "invalid queue depth(%zu)", waiting_queue_depth);
    auto st = std::make_unique<ucm_cache_store>();
    st->device = device_id;
    st->timeout_ms = timeout_ms ? timeout_ms : 30000;
    size_t off = 0;
    for (size_t i = 0; i < n_tensors; ++i) {
        UCM_REQUIRE(tensor_sizes[i] > 0, "invalid tensor size");
        st->tensor_sizes.push_back(tensor_sizes[i]);
        st->tensor_offsets.push_back(off);
        off += tensor_sizes[i];
    }
    st->shard_size = off;
    if (backend) {
        st->backend = *backend;
        st->has_backend = true;
    }
    int rc = ucm_trans_setup(device_id);
    if (rc != UCM_OK) return rc;
    rc = st->buffer.setup(st->shard_size, buffer_bytes);
    if (rc != UCM_OK) return rc;
    rc = ucm_trans_stream_create(UCM_TRANS_SM, &st->dump_stream);
    if (rc != UCM_OK) return rc;
    rc = ucm_trans_stream_create(UCM_TRANS_SM, &st->load_stream);
    if (rc != UCM_OK) {
        (void)ucm_trans_stream_destroy(st->dump_stream);
        return rc;
    }
    st->dump_waiting.setup(waiting_queue_depth);
    st->load_waiting.setup(waiting_queue_depth);
    ucm_cache_store* p = st.get();
    st->dump_dispatcher = std::thread(dump_dispatch_stage, p);
    st->dump_backend = std::thread(dump_backend_stage, p);
    st->load_dispatcher = std::thread(load_dispatch_stage, p);
    st->load_transfer = std::thread(load_transfer_stage, p);
    *out = st.release();
    return UCM_OK;
}

extern "C" int ucm_cache_store_destroy(ucm_cache_store_t* st)
{
    ucm::clear_error();
    if (!st) return UCM_OK;
    st->stop.store(true);
    for (std::thread* t : {&st->dump_dispatcher, &st->load_dispatcher, &st->load_transfer})
        if (t->joinable()) t->join();
    // only now can no new backend dump appear: let the backend stage wait for the ones in flight
    // (their source is the pinned slab, freed below) and exit
    st->stop_backend.store(true);
    if (st->dump_backend.joinable()) st->dump_backend.join();
    (void)ucm_trans_stream_destroy(st->dump_stream);
    (void)ucm_trans_stream_destroy(st->load_stream);
    delete st;
    return UCM_OK;
}

extern "C" int ucm_cache_store_lookup(ucm_cache_store_t* st, const uint8_t* block_ids, size_t n,
                                      uint8_t* found)
{
    ucm::clear_error();
    UCM_REQUIRE(st && (n == 0 || (block_ids && found)), "null argument");
    std::vector<uint8_t> miss_ids;
    std::vector<size_t> miss_idx;
    for (size_t i = 0; i < n; ++i) {
        Key k{};
        std::memcpy(k.id, block_ids + i * 16, 16);
        k.shard = 0;  // a block is present when its first shard is (buffer_manager.h:88)
        found[i] = st->buffer.exist(k) ? 1 : 0;
        if (!found[i]) {
            miss_ids.insert(miss_ids.end(), block_ids + i * 16, block_ids + (i + 1) * 16);
            miss_idx.push_back(i);
        }
    }
    if (!miss_idx.empty() && st->has_backend && st->backend.lookup) {
        std::vector<uint8_t> res(miss_idx.size(), 0);
        const int rc = st->backend.lookup(st->backend.ctx, miss_ids.data(), miss_idx.size(), res.data());
        if (rc != UCM_OK) return ucm::fail(rc, "backend lookup failed");
        for (size_t i = 0; i < miss_idx.size(); ++i) found[miss_idx[i]] = res[i] ? 1 : 0;
    }
    return UCM_OK;
}

extern "C" int ucm_cache_store_lookup_on_prefix(ucm_cache_store_t* st, const uint8_t* block_ids,
                                                size_t n, int64_t* last_found)
{
    ucm::clear_error();
    UCM_REQUIRE(last_found, "null output");
    std::vector<uint8_t> found(n);
    const int rc = ucm_cache_store_lookup(st, block_ids, n, found.data());
    if (rc != UCM_OK) return rc;
    int64_t i = 0;
    while (i < (int64_t)n && found[i]) ++i;
    *last_found = i - 1;
    return UCM_OK;
}

extern "C" int ucm_cache_store_dump(ucm_cache_store_t* st, const uint8_t* block_ids,
                                    const uint64_t* shard_idx, void* const* device_addrs, size_t n,
                                    void* prerequisite_event, int64_t* task)
{
    return submit(st, false, block_ids, shard_idx, device_addrs, n, prerequisite_event, task);
}

extern "C" int ucm_cache_store_load(ucm_cache_store_t* st, const uint8_t* block_ids,
                                    const uint64_t* shard_idx, void* const* device_addrs, size_t n,
                                    int64_t* task)
{
    return submit(st, true, block_ids, shard_idx, device_addrs, n, nullptr, task);
}

extern "C" int ucm_cache_store_check(ucm_cache_store_t* st, int64_t task, int* finished)
{
    ucm::clear_error();
    UCM_REQUIRE(st && finished, "null argument");
    WaiterPtr w;
    {
        std::lock_guard<std::mutex> lock(st->tasks_mu);
        auto it = st->tasks.find(task);
        if (it == st->tasks.end()) return ucm::fail(UCM_ENOOBJ, "unknown task %lld", (long long)task);
        w = it->second.second;
    }
    *finished = w->check() ? 1 : 0;
    return UCM_OK;
}

extern "C" int ucm_cache_store_wait(ucm_cache_store_t* st, int64_t task)
{
    ucm::clear_error();
    UCM_REQUIRE(st, "null store");
    WaiterPtr w;
    {
        std::lock_guard<std::mutex> lock(st->tasks_mu);
        auto it = st->tasks.find(task);
        if (it == st->tasks.end()) return ucm::fail(UCM_ENOOBJ, "unknown task %lld", (long long)task);
        w = it->second.second;
        st->tasks.erase(it);
    }
    if (!w->wait_for(st->timeout_ms)) {
        // mark it failed so that the stages skip what is left of it, then let it drain
        st->fail(task);
        while (!w->wait_for(2000)) {}
        st->clear_failure(task);
        return ucm::fail(UCM_ETIMEOUT, "task %lld timed out", (long long)task);
    }
    if (st->failed(task)) {
        st->clear_failure(task);
        return ucm::fail(UCM_ERROR, "task %lld failed", (long long)task);
    }
    return UCM_OK;
}

extern "C" size_t ucm_cache_store_nodes(ucm_cache_store_t* st) { return st ? st->buffer.nodes() : 0; }
