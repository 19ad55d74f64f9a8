// File-per-block store on a POSIX file system, in the reference's on-disk format, so that
// blocks persisted by either implementation can be read by the other.
//
// Follows ucm/store/posix/cc/: SpaceLayout (space_layout.cc: where a block's file lives),
// PosixFile (posix_file.cc: permissions, pread / pwrite), TransQueue (trans_queue.cc: what a
// dump and a load do to a file), SpaceManager (space_manager.cc: lookup), HotnessTracker
// (hotness_tracker.cc) and ShardGarbageCollector (shard_gc.cc).  The format:
//   * one file per block, named by the 32 lowercase hex digits of its 16-byte id;
//   * directory = <backend>/<first data_dir_shard_bytes hex digits of the name>/, or
//     <backend>/data/ when data_dir_shard_bytes is 0; with several backends a block lives in
//     backend number std::hash<std::string_view>(id bytes) % n_backends;
//   * shard `index` of a block occupies bytes [index * shard_size, (index + 1) * shard_size) and
//     is the concatenation of its tensors, tensor_size bytes each;
//   * a file is written under the name <name>.tmp and renamed to <name> once the block's last
//     shard (index == block_size / shard_size - 1) has been written; only renamed files are
//     visible to lookup and load.
// This part of the library is host-only: addresses are host pointers (under the cache store,
// the pinned staging shards), and no HIP call is made.
#include <dirent.h>
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>
#include <utime.h>

#include <algorithm>
#include <cerrno>
#include <cstring>
#include <functional>
#include <memory>
#include <queue>
#include <random>
#include <string>
#include <string_view>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "common.h"
#include "host_queue.h"

namespace {

constexpr const char* kDataRoot = "data";
constexpr const char* kActivatedExt = ".tmp";
constexpr mode_t kFilePerm = S_IRUSR | S_IWUSR | S_IRGRP | S_IROTH;  // posix_file.cc:30
constexpr mode_t kDirPerm = S_IRWXU | S_IRWXG | S_IROTH;             // posix_file.cc:31

struct BlockId {
    uint8_t b[16];
    bool operator==(const BlockId& o) const { return std::memcmp(b, o.b, 16) == 0; }
};

struct BlockIdHash {  // ucm/store/detail/type/types.h:39-45
    size_t operator()(const BlockId& id) const noexcept
    {
        return std::hash<std::string_view>{}(std::string_view(reinterpret_cast<const char*>(id.b), 16));
    }
};

std::string file_name(const BlockId& id)
{
    static const char hex[] = "0123456789abcdef";
    std::string s(32, '0');
    for (int i = 0; i < 16; ++i) {
        s[2 * i] = hex[id.b[i] >> 4];
        s[2 * i + 1] = hex[id.b[i] & 15];
    }
    return s;
}

bool parse_name(const char* name, BlockId* id)
{
    if (std::strlen(name) != 32) return false;
    for (int i = 0; i < 16; ++i) {
        int v[2];
        for (int j = 0; j < 2; ++j) {
            const char c = name[2 * i + j];
            if (c >= '0' && c <= '9') v[j] = c - '0';
            else if (c >= 'a' && c <= 'f') v[j] = c - 'a' + 10;
            else return false;
        }
        id->b[i] = (uint8_t)(v[0] << 4 | v[1]);
    }
    return true;
}

struct IoUnit {
    int64_t task = 0;
    bool load = false;
    BlockId id{};
    uint64_t index = 0;
    std::vector<void*> addrs;
    std::shared_ptr<Waiter> waiter;
};

struct LookupJob {
    const BlockId* ids = nullptr;
    size_t begin = 0, n = 0, stride = 1;
    std::shared_ptr<std::atomic<int64_t>> first_fail;
    std::shared_ptr<Waiter> waiter;
};

// Shards of one block being written by this process: the rename happens when the shard with
// the last index has been written AND no other write of the block is still queued or running,
// so that a shard written late cannot land in a stray .tmp file after the rename.
struct Pending {
    int inflight = 0;
    bool commit = false;
    bool ok = true;
};

}  // namespace

struct ucm_posix_store {
    std::vector<std::string> backends;  // each ends with '/'
    std::vector<std::string> roots;     // relative shard directories
    size_t shard_digits = 3;
    int device_id = -1;
    size_t tensor_size = 0, shard_size = 0, block_size = 0;
    size_t tensors_per_shard = 0, shards_per_block = 0;
    bool io_direct = false;
    size_t timeout_ms = 30000;
    bool transfer = false, hotness = false;

    std::atomic<bool> stop{false};
    BoundedQueue<IoUnit> load_q, dump_q;
    std::vector<std::thread> io_workers;
    BoundedQueue<LookupJob> lookup_q;
    std::vector<std::thread> lookup_workers;
    size_t lookup_concurrency = 16;

    std::mutex tasks_mu;
    std::unordered_map<int64_t, std::shared_ptr<Waiter>> tasks;
    std::unordered_set<int64_t> failures;
    int64_t next_id = 1;

    std::mutex pending_mu;
    std::unordered_map<BlockId, Pending, BlockIdHash> pending;

    // hotness tracker: found blocks get their mtime refreshed by one background thread
    std::mutex touch_mu;
    std::vector<BlockId> touch_list;
    std::thread touch_worker;

    // garbage collector
    bool gc = false;
    size_t max_files = 0;
    double gc_recycle_percent = 0.1, gc_trigger_ratio = 0.7, gc_sample_ratio = 0.1;
    size_t gc_max_per_shard = 50000, gc_interval_s = 30;
    std::mutex gc_mu;
    std::condition_variable gc_cv;
    std::thread gc_worker;
    std::atomic<uint64_t> gc_removed{0};

    std::string path_of(const BlockId& id, bool activated) const
    {
        const std::string& be =
            backends.size() == 1 ? backends.front() : backends[BlockIdHash{}(id) % backends.size()];
        const std::string name = file_name(id);
        std::string p = be;
        p += shard_digits ? name.substr(0, shard_digits) : std::string(kDataRoot);
        p += '/';
        p += name;
        if (activated) p += kActivatedExt;
        return p;
    }
    bool failed(int64_t id)
    {
        std::lock_guard<std::mutex> lock(tasks_mu);
        return failures.count(id) != 0;
    }
    void fail(int64_t id)
    {
        std::lock_guard<std::mutex> lock(tasks_mu);
        failures.insert(id);
    }
};

namespace {

// SpaceLayout::CommitFile (space_layout.cc:101-111)
int commit_file(const ucm_posix_store* st, const BlockId& id, bool success)
{
    const std::string activated = st->path_of(id, true);
    int rc = UCM_OK;
    if (success) {
        if (::rename(activated.c_str(), st->path_of(id, false).c_str()) != 0)
            rc = errno == ENOENT ? UCM_ENOOBJ : UCM_EOSERROR;
    }
    if (!success || rc != UCM_OK) ::remove(activated.c_str());
    return rc;
}

bool block_present(const ucm_posix_store* st, const BlockId& id)
{
    // SpaceManager::Lookup (space_manager.cc:96-108): exists, readable and writable
    return ::access(st->path_of(id, false).c_str(), F_OK | R_OK | W_OK) == 0;
}

// TransQueue::H2S / S2H (trans_queue.cc:127-169)
bool move_shard(const ucm_posix_store* st, const IoUnit& u)
{
    const std::string path = st->path_of(u.id, !u.load);
    int flags = u.load ? O_RDONLY : (O_CREAT | O_WRONLY);
    if (st->io_direct) flags |= O_DIRECT;
    const int fd = ::open(path.c_str(), flags, kFilePerm);
    if (fd < 0) return false;
    off64_t off = (off64_t)(st->shard_size * u.index);
    bool ok = true;
    for (void* addr : u.addrs) {
        const ssize_t n = u.load ? ::pread64(fd, addr, st->tensor_size, off)
                                 : ::pwrite64(fd, addr, st->tensor_size, off);
        if (n != (ssize_t)st->tensor_size) {
            ok = false;
            break;
        }
        off += (off64_t)st->tensor_size;
    }
    ::close(fd);
    return ok;
}

void io_worker(ucm_posix_store* st, BoundedQueue<IoUnit>* q)
{
    IoUnit u;
    while (q->pop(u, st->stop)) {
        bool ok = true;
        const bool skip = st->failed(u.task);  // an earlier shard of the task failed
        if (!skip) ok = move_shard(st, u);
        if (!u.load) {
            bool do_commit = false, commit_ok = false;
            {
                std::lock_guard<std::mutex> lock(st->pending_mu);
                Pending& p = st->pending[u.id];
                if (skip || !ok) p.ok = false;
                if (u.index + 1 == st->shards_per_block) p.commit = true;
                if (--p.inflight == 0) {
                    do_commit = p.commit;
                    commit_ok = p.ok;
                    st->pending.erase(u.id);
                }
            }
            if (do_commit) (void)commit_file(st, u.id, commit_ok);
        }
        if (!ok) st->fail(u.task);
        u.waiter->done();
        u = {};
    }
}

// SpaceManager::OnLookupPrefix (space_manager.cc:110-130): worker `begin` of `stride` checks
// blocks begin, begin + stride, ... and stops at the first miss anybody has seen so far
void lookup_worker(ucm_posix_store* st)
{
    LookupJob j;
    while (st->lookup_q.pop(j, st->stop)) {
        for (size_t i = j.begin; i < j.n; i += j.stride) {
            if (j.first_fail->load() < (int64_t)i) break;
            if (!block_present(st, j.ids[i])) {
                int64_t cur = j.first_fail->load();
                while ((int64_t)i < cur && !j.first_fail->compare_exchange_weak(cur, (int64_t)i)) {
                }
                break;
            }
            if (st->hotness) {
                std::lock_guard<std::mutex> lock(st->touch_mu);
                st->touch_list.push_back(j.ids[i]);
            }
        }
        j.waiter->done();
        j = {};
    }
}

void touch_worker(ucm_posix_store* st)  // HotnessTracker::UtimeWorkerLoop
{
    std::vector<BlockId> todo;
    while (!st->stop.load()) {
        {
            std::lock_guard<std::mutex> lock(st->touch_mu);
            todo.swap(st->touch_list);
        }
        if (todo.empty()) {
            std::this_thread::sleep_for(std::chrono::microseconds(200));
            continue;
        }
        for (const BlockId& id : todo) (void)::utime(st->path_of(id, false).c_str(), nullptr);
        todo.clear();
    }
}

int64_t prefix_lookup(ucm_posix_store* st, const BlockId* ids, size_t n)
{
    if (n == 0) return -1;
    auto first_fail = std::make_shared<std::atomic<int64_t>>((int64_t)n);
    auto waiter = std::make_shared<Waiter>();
    const size_t workers = std::min(n, st->lookup_concurrency);
    waiter->pending = (int)workers;
    for (size_t b = 0; b < workers; ++b) st->lookup_q.push(LookupJob{ids, b, n, workers, first_fail, waiter});
    if (!waiter->wait_for(st->timeout_ms)) {
        // the jobs still hold `ids`: they must finish before the caller's array may go away
        while (!waiter->wait_for(1000)) {
        }
        return -2;
    }
    return first_fail->load() - 1;
}

// ---- garbage collection (space_layout.cc:185-257, shard_gc.cc) ----
size_t count_files(const ucm_posix_store* st, const std::string& root)
{
    DIR* dir = ::opendir((st->backends.front() + root).c_str());
    if (!dir) return 0;
    size_t n = 0;
    while (dirent* e = ::readdir(dir)) {
        if (e->d_name[0] == '.' || std::strstr(e->d_name, kActivatedExt)) continue;
        ++n;
    }
    ::closedir(dir);
    return n;
}

// the oldest recycle_percent of the files of one shard directory, at most max_count
std::vector<BlockId> oldest_files(const ucm_posix_store* st, const std::string& root, double recycle_percent,
                                  size_t max_count)
{
    const std::string dir_path = st->backends.front() + root;
    DIR* dir = ::opendir(dir_path.c_str());
    if (!dir) return {};
    using Entry = std::pair<time_t, BlockId>;
    auto newer_first = [](const Entry& a, const Entry& b) { return a.first < b.first; };
    std::priority_queue<Entry, std::vector<Entry>, decltype(newer_first)> heap(newer_first);  // max-heap by mtime
    size_t total = 0;
    while (dirent* e = ::readdir(dir)) {
        if (e->d_name[0] == '.' || std::strstr(e->d_name, kActivatedExt)) continue;
        struct stat sb;
        if (::stat((dir_path + "/" + e->d_name).c_str(), &sb) != 0 || !S_ISREG(sb.st_mode)) continue;
        BlockId id;
        if (!parse_name(e->d_name, &id)) continue;
        ++total;
        heap.emplace(sb.st_mtime, id);
        if (heap.size() > max_count) heap.pop();  // keep the max_count oldest
    }
    ::closedir(dir);
    size_t want = std::min((size_t)(total * recycle_percent), max_count);
    if (total == 0 || want == 0) return {};
    while (heap.size() > want) heap.pop();
    std::vector<BlockId> out;
    out.reserve(heap.size());
    while (!heap.empty()) {
        out.push_back(heap.top().second);
        heap.pop();
    }
    return out;
}

std::vector<std::string> sample_roots(const ucm_posix_store* st, double ratio)
{
    if (ratio >= 1.0) return st->roots;
    std::vector<std::string> r = st->roots;
    const size_t n = std::max<size_t>(1, (size_t)(r.size() * ratio));
    std::mt19937 gen(std::random_device{}());
    std::shuffle(r.begin(), r.end(), gen);
    r.resize(n);
    return r;
}

bool gc_should_trigger(const ucm_posix_store* st)
{
    const auto sample = sample_roots(st, st->gc_sample_ratio);
    size_t files = 0;
    for (const auto& r : sample) files += count_files(st, r);
    const size_t avg = files / sample.size();
    const size_t threshold = (size_t)(st->max_files / st->roots.size() * st->gc_trigger_ratio);
    return avg >= threshold;
}

// one pass over every shard directory; true when some directory hit the per-pass limit
bool gc_execute(ucm_posix_store* st)
{
    bool limited = false;
    for (const auto& r : st->roots) {
        const auto victims = oldest_files(st, r, st->gc_recycle_percent, st->gc_max_per_shard);
        for (const BlockId& id : victims) ::remove(st->path_of(id, false).c_str());
        st->gc_removed += victims.size();
        if (victims.size() >= st->gc_max_per_shard) limited = true;
        if (st->stop.load()) break;
    }
    return limited;
}

void gc_check(ucm_posix_store* st)  // one turn of ShardGarbageCollector::GCCheckLoop
{
    bool trigger = gc_should_trigger(st);
    while (!st->stop.load() && trigger) {
        if (gc_execute(st)) continue;
        trigger = gc_should_trigger(st);
    }
}

void gc_loop(ucm_posix_store* st)
{
    while (!st->stop.load()) {
        gc_check(st);
        std::unique_lock<std::mutex> lock(st->gc_mu);
        st->gc_cv.wait_for(lock, std::chrono::seconds(st->gc_interval_s), [st] { return st->stop.load(); });
    }
}

int add_backend(ucm_posix_store* st, std::string path)
{
    if (path.empty()) return ucm::fail(UCM_EPARAM, "empty storage backend path");
    if (path.back() != '/') path += '/';
    if (st->backends.empty()) {  // AddFirstStorageBackend: creates the shard directories
        for (const auto& r : st->roots) {
            const std::string dir = path + r;
            if (::mkdir(dir.c_str(), kDirPerm) != 0) {
                if (errno != EEXIST) return ucm::fail(UCM_EOSERROR, "mkdir(%s): %s", dir.c_str(), std::strerror(errno));
            } else {
                (void)::chmod(dir.c_str(), kDirPerm);
            }
        }
    } else {  // AddSecondaryStorageBackend: must already hold the directories
        if (std::find(st->backends.begin(), st->backends.end(), path) != st->backends.end()) return UCM_OK;
        for (const auto& r : st->roots) {
            const std::string dir = path + r;
            if (::access(dir.c_str(), R_OK | W_OK) != 0)
                return ucm::fail(errno == ENOENT ? UCM_ENOOBJ : UCM_EOSERROR, "access(%s): %s", dir.c_str(),
                                 std::strerror(errno));
        }
    }
    st->backends.push_back(std::move(path));
    return UCM_OK;
}

std::vector<std::string> hex_roots(size_t digits)
{
    if (digits == 0) return {kDataRoot};
    static const char hex[] = "0123456789abcdef";
    const size_t n = (size_t)1 << (digits * 4);
    std::vector<std::string> out;
    out.reserve(n);
    for (size_t i = 0; i < n; ++i) {
        std::string s(digits, '0');
        size_t t = i;
        for (size_t j = digits; j-- > 0;) {
            s[j] = hex[t & 15];
            t >>= 4;
        }
        out.push_back(std::move(s));
    }
    return out;
}

int submit(ucm_posix_store* st, bool load, const uint8_t* block_ids, const uint64_t* shard_idx,
           void* const* host_addrs, size_t n, int64_t* task)
{
    UCM_REQUIRE(st && task, "null store or task pointer");
    if (!st->transfer) return ucm::fail(UCM_ERROR, "transfer is not enable");
    UCM_REQUIRE(n == 0 || (block_ids && shard_idx && host_addrs), "null pointer");
    for (size_t i = 0; i < n; ++i) {
        UCM_REQUIRE(shard_idx[i] < st->shards_per_block, "shard index %llu outside the block (%zu shards)",
                    (unsigned long long)shard_idx[i], st->shards_per_block);
        for (size_t t = 0; t < st->tensors_per_shard; ++t)
            UCM_REQUIRE(host_addrs[i * st->tensors_per_shard + t], "null address in shard %zu", i);
    }
    auto waiter = std::make_shared<Waiter>();
    waiter->pending = (int)n;
    int64_t id;
    {
        std::lock_guard<std::mutex> lock(st->tasks_mu);
        id = st->next_id++;
        st->tasks.emplace(id, waiter);
    }
    if (!load) {
        std::lock_guard<std::mutex> lock(st->pending_mu);
        for (size_t i = 0; i < n; ++i) {
            BlockId b;
            std::memcpy(b.b, block_ids + 16 * i, 16);
            ++st->pending[b].inflight;
        }
    }
    for (size_t i = 0; i < n; ++i) {
        IoUnit u;
        u.task = id;
        u.load = load;
        std::memcpy(u.id.b, block_ids + 16 * i, 16);
        u.index = shard_idx[i];
        u.addrs.assign(host_addrs + i * st->tensors_per_shard, host_addrs + (i + 1) * st->tensors_per_shard);
        u.waiter = waiter;
        (load ? st->load_q : st->dump_q).push(std::move(u));
    }
    *task = id;
    return UCM_OK;
}

// ---- hooks that put the store beneath a cache store ----
int be_lookup(void* ctx, const uint8_t* ids, size_t n, uint8_t* found)
{
    return ucm_posix_store_lookup((ucm_posix_store_t*)ctx, ids, n, found);
}
int64_t be_move(ucm_posix_store* st, bool load, const uint8_t* ids, const uint64_t* idx, void* const* host,
                size_t n, size_t shard_size)
{
    if (shard_size != st->shard_size || st->tensor_size != st->shard_size)
        return ucm::fail(UCM_EPARAM, "beneath a cache store tensor_size and shard_size must both be %zu", shard_size);
    int64_t task = 0;
    const int rc = submit(st, load, ids, idx, host, n, &task);
    return rc == UCM_OK ? task : rc;
}
int64_t be_dump(void* ctx, const uint8_t* ids, const uint64_t* idx, void* const* host, size_t n, size_t shard_size)
{
    return be_move((ucm_posix_store*)ctx, false, ids, idx, host, n, shard_size);
}
int64_t be_load(void* ctx, const uint8_t* ids, const uint64_t* idx, void* const* host, size_t n, size_t shard_size)
{
    return be_move((ucm_posix_store*)ctx, true, ids, idx, host, n, shard_size);
}
// The cache store hands the waited-for staging nodes to other keys as soon as this returns, so
// here "the workers still hold the buffers" is not an answer: keep waiting.
int be_wait(void* ctx, int64_t handle)
{
    int rc;
    while ((rc = ucm_posix_store_wait((ucm_posix_store_t*)ctx, handle)) == UCM_ERETRY) {
    }
    return rc;
}

}  // namespace

extern "C" int ucm_posix_store_create(const ucm_posix_config_t* c, ucm_posix_store_t** out)
{
    ucm::clear_error();
    UCM_REQUIRE(c && out, "null config or output pointer");
    // PosixStore::CheckConfig (posix_store.cc:131-193)
    UCM_REQUIRE(c->storage_backends && c->n_backends > 0, "invalid storage backends");
    UCM_REQUIRE(c->device_id >= -1, "invalid device(%d)", c->device_id);
    UCM_REQUIRE(c->lookup_concurrency > 0, "invalid lookup concurrency(0)");
    const size_t lookup_conc = c->lookup_concurrency;
    UCM_REQUIRE(c->data_dir_shard_bytes <= 5, "invalid shard bytes(%zu)", c->data_dir_shard_bytes);
    const bool transfer = c->device_id >= 0;
    if (transfer) {
        UCM_REQUIRE(c->tensor_size != 0 && c->shard_size >= c->tensor_size && c->block_size >= c->shard_size &&
                        c->shard_size % c->tensor_size == 0 && c->block_size % c->shard_size == 0,
                    "invalid size(%zu,%zu,%zu)", c->tensor_size, c->shard_size, c->block_size);
        UCM_REQUIRE(c->data_trans_concurrency > 0, "invalid psync concurrency(0)");
    }
    const bool gc = c->gc_enable && c->capacity_bytes > 0;
    if (gc) {
        UCM_REQUIRE(c->gc_recycle_percent > 0 && c->gc_recycle_percent <= 1.0, "invalid gc recycle percent(%f)",
                    c->gc_recycle_percent);
        UCM_REQUIRE(c->gc_trigger_threshold_ratio > 0 && c->gc_trigger_threshold_ratio <= 1.0,
                    "invalid gc trigger threshold ratio(%f)", c->gc_trigger_threshold_ratio);
        UCM_REQUIRE(c->gc_max_recycle_count_per_shard > 0, "invalid gc max recycle count per shard(0)");
        UCM_REQUIRE(c->gc_shard_sample_ratio > 0 && c->gc_shard_sample_ratio <= 1.0,
                    "invalid gc shard sample ratio(%f)", c->gc_shard_sample_ratio);
        UCM_REQUIRE(c->gc_check_interval_sec > 0, "invalid gc check interval(0)");
        UCM_REQUIRE(c->block_size > 0, "garbage collection needs block_size");
    }
    std::unique_ptr<ucm_posix_store> st(new ucm_posix_store);
    st->device_id = c->device_id;
    st->tensor_size = c->tensor_size;
    st->shard_size = c->shard_size;
    st->block_size = c->block_size;
    st->tensors_per_shard = transfer ? c->shard_size / c->tensor_size : 0;
    st->shards_per_block = transfer ? c->block_size / c->shard_size : 0;
    st->io_direct = c->io_direct != 0;
    st->timeout_ms = c->timeout_ms ? c->timeout_ms : 30000;
    st->shard_digits = c->data_dir_shard_bytes;
    st->transfer = transfer;
    st->hotness = c->device_id == -1;
    st->lookup_concurrency = lookup_conc;
    st->roots = hex_roots(st->shard_digits);
    for (size_t i = 0; i < c->n_backends; ++i) {
        UCM_REQUIRE(c->storage_backends[i], "null storage backend path");
        const int rc = add_backend(st.get(), c->storage_backends[i]);
        if (rc != UCM_OK) return rc;
    }
    if (gc) {
        // ShardGarbageCollector::ValidateAndInitCapacity (shard_gc.cc:31-53)
        st->max_files = c->capacity_bytes / c->block_size;
        st->gc_recycle_percent = c->gc_recycle_percent;
        st->gc_trigger_ratio = c->gc_trigger_threshold_ratio;
        st->gc_sample_ratio = c->gc_shard_sample_ratio;
        st->gc_max_per_shard = c->gc_max_recycle_count_per_shard;
        st->gc_interval_s = c->gc_check_interval_sec;
        const size_t per_shard = (size_t)(st->max_files / st->roots.size() * st->gc_trigger_ratio);
        UCM_REQUIRE((size_t)(per_shard * st->gc_recycle_percent) > 0,
                    "capacity (%zu bytes) is too small, GC cannot recycle any files", c->capacity_bytes);
        st->gc = true;
    }
    ucm_posix_store* p = st.get();
    if (transfer) {
        const size_t workers = c->data_trans_concurrency;
        p->load_q.setup((size_t)-1);
        p->dump_q.setup((size_t)-1);
        for (size_t i = 0; i < workers; ++i) {
            p->io_workers.emplace_back(io_worker, p, &p->load_q);
            p->io_workers.emplace_back(io_worker, p, &p->dump_q);
        }
    }
    p->lookup_q.setup((size_t)-1);
    for (size_t i = 0; i < lookup_conc; ++i) p->lookup_workers.emplace_back(lookup_worker, p);
    if (p->hotness) p->touch_worker = std::thread(touch_worker, p);
    if (p->gc) p->gc_worker = std::thread(gc_loop, p);
    *out = st.release();
    return UCM_OK;
}

extern "C" int ucm_posix_store_destroy(ucm_posix_store_t* st)
{
    ucm::clear_error();
    if (!st) return UCM_OK;
    {
        std::lock_guard<std::mutex> lock(st->gc_mu);
        st->stop.store(true);
    }
    st->gc_cv.notify_all();
    for (auto& t : st->io_workers) t.join();      // queues are drained before the workers leave
    for (auto& t : st->lookup_workers) t.join();
    if (st->touch_worker.joinable()) st->touch_worker.join();
    if (st->gc_worker.joinable()) st->gc_worker.join();
    delete st;
    return UCM_OK;
}

extern "C" int64_t ucm_posix_store_data_file_path(ucm_posix_store_t* st, const uint8_t* block_id,
                                                  int32_t activated, char* buf, size_t cap)
{
    ucm::clear_error();
    UCM_REQUIRE(st && block_id, "null pointer");
    BlockId id;
    std::memcpy(id.b, block_id, 16);
    const std::string p = st->path_of(id, activated != 0);
    if (buf && cap) {
        const size_t n = std::min(cap - 1, p.size());
        std::memcpy(buf, p.data(), n);
        buf[n] = 0;
    }
    return (int64_t)p.size();
}

extern "C" int ucm_posix_store_commit(ucm_posix_store_t* st, const uint8_t* block_id, int32_t success)
{
    ucm::clear_error();
    UCM_REQUIRE(st && block_id, "null pointer");
    BlockId id;
    std::memcpy(id.b, block_id, 16);
    const int rc = commit_file(st, id, success != 0);
    if (rc != UCM_OK) return ucm::fail(rc, "commit of %s failed", file_name(id).c_str());
    return UCM_OK;
}

extern "C" int ucm_posix_store_lookup_on_prefix(ucm_posix_store_t* st, const uint8_t* block_ids, size_t n,
                                                int64_t* last_found)
{
    ucm::clear_error();
    UCM_REQUIRE(st && last_found && (n == 0 || block_ids), "null pointer");
    static_assert(sizeof(BlockId) == 16, "block ids are read in place");
    const int64_t r = prefix_lookup(st, reinterpret_cast<const BlockId*>(block_ids), n);
    if (r == -2) return ucm::fail(UCM_ETIMEOUT, "failed to lookup some blocks");
    *last_found = r;
    return UCM_OK;
}

extern "C" int ucm_posix_store_lookup(ucm_posix_store_t* st, const uint8_t* block_ids, size_t n, uint8_t* found)
{
    // SpaceManager::Lookup (space_manager.cc:56-64): true for the leading run that is present
    int64_t last = -1;
    UCM_REQUIRE(n == 0 || found, "null pointer");
    const int rc = ucm_posix_store_lookup_on_prefix(st, block_ids, n, &last);
    if (rc != UCM_OK) return rc;
    for (size_t i = 0; i < n; ++i) found[i] = (int64_t)i <= last ? 1 : 0;
    return UCM_OK;
}

extern "C" int ucm_posix_store_dump(ucm_posix_store_t* st, const uint8_t* block_ids, const uint64_t* shard_idx,
                                    void* const* host_addrs, size_t n, int64_t* task)
{
    ucm::clear_error();
    return submit(st, false, block_ids, shard_idx, host_addrs, n, task);
}

extern "C" int ucm_posix_store_load(ucm_posix_store_t* st, const uint8_t* block_ids, const uint64_t* shard_idx,
                                    void* const* host_addrs, size_t n, int64_t* task)
{
    ucm::clear_error();
    return submit(st, true, block_ids, shard_idx, host_addrs, n, task);
}

extern "C" int ucm_posix_store_check(ucm_posix_store_t* st, int64_t task, int32_t* finished)
{
    ucm::clear_error();
    UCM_REQUIRE(st && finished, "null pointer");
    std::shared_ptr<Waiter> w;
    {
        std::lock_guard<std::mutex> lock(st->tasks_mu);
        auto it = st->tasks.find(task);
        if (it == st->tasks.end()) return ucm::fail(UCM_ENOOBJ, "no task %lld", (long long)task);
        w = it->second;
    }
    *finished = w->check() ? 1 : 0;
    return UCM_OK;
}

extern "C" int ucm_posix_store_wait(ucm_posix_store_t* st, int64_t task)
{
    ucm::clear_error();
    UCM_REQUIRE(st, "null store");
    std::shared_ptr<Waiter> w;
    {
        std::lock_guard<std::mutex> lock(st->tasks_mu);
        auto it = st->tasks.find(task);
        if (it == st->tasks.end()) return ucm::fail(UCM_ENOOBJ, "no task %lld", (long long)task);
        w = it->second;
    }
    const bool done = w->wait_for(st->timeout_ms);
    if (!done) {
        {
            std::lock_guard<std::mutex> lock(st->tasks_mu);
            st->failures.insert(task);  // shards still queued are skipped
        }
        // the caller's buffers are free to reuse once this returns, so the units that are queued
        // (now skipped) or in the middle of their read / write must have drained first.  That drain
        // is bounded too (a worker stuck in a read or write on a dead mount never returns): after
        // four more time-outs the task stays registered and the caller is told that its buffers are
        // still in use.
        bool drained = false;
        for (int i = 0; i < 4 && !drained; ++i) drained = w->wait_for(st->timeout_ms ? st->timeout_ms : 1000);
        if (!drained)
            return ucm::fail(UCM_ERETRY,
                             "task %lld timed out and its file workers have not returned after %zu ms more: the "
                             "buffers of this task must not be reused or freed; wait on the task again",
                             (long long)task, 4 * st->timeout_ms);
    }
    bool failed;
    {
        std::lock_guard<std::mutex> lock(st->tasks_mu);
        failed = st->failures.count(task) != 0;
        st->tasks.erase(task);
        st->failures.erase(task);
    }
    if (!done) return ucm::fail(UCM_ETIMEOUT, "task %lld timed out after %zu ms", (long long)task, st->timeout_ms);
    if (failed) return ucm::fail(UCM_ERROR, "task %lld failed", (long long)task);
    return UCM_OK;
}

extern "C" int ucm_posix_store_gc_once(ucm_posix_store_t* st, uint64_t* removed)
{
    ucm::clear_error();
    UCM_REQUIRE(st, "null store");
    if (!st->gc) return ucm::fail(UCM_EUNSUPPORTED, "garbage collection is not configured");
    const uint64_t before = st->gc_removed.load();
    gc_check(st);
    if (removed) *removed = st->gc_removed.load() - before;
    return UCM_OK;
}

extern "C" int ucm_posix_store_backend(ucm_posix_store_t* st, ucm_cache_backend_t* out)
{
    ucm::clear_error();
    UCM_REQUIRE(st && out, "null pointer");
    out->ctx = st;
    out->lookup = be_lookup;
    out->dump = be_dump;
    out->load = be_load;
    out->wait = be_wait;
    return UCM_OK;
}
