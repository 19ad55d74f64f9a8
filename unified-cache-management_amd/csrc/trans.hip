// KV block gather / scatter between the paged HBM cache and flat (pinned host or device)
// buffers, on side HIP streams.
//
// Mirrors the surface of the reference's UC::Trans::{Device,Stream,Buffer}
// (ucm/shared/trans/stream.h:32-54, device.h:32-39, buffer.h:32-47).  Two stream kinds:
//   CE  one hipMemcpyAsync per chunk (ucm/shared/trans/cuda/cuda_stream.cc:63-80,110-127);
//   SM  one kernel moves every chunk (ucm/shared/trans/cuda/cuda_sm_kernel.cu:52-114), here
//       shaped for MI355X: one workgroup per 4 KiB segment, one 128-bit non-temporal load and
//       store per lane and no loop, instead of the reference's fixed 32x256 grid-stride threads.
//       Many short workgroups let the dispatcher interleave reads and writes across all HBM
//       channels; on this part that moves 25-30 % more bytes per second than a persistent
//       grid-stride copy.  A copy with a HOST end is the exception.  Kernel stores into pinned
//       host memory fill the PCIe link (55 GB/s) but hold up every other kernel on the GPU while
//       they run: a decode step of 32 us beside such a dump takes 47 us with 8 copy workgroups
//       (28 GB/s), 72 us with 16 (44 GB/s) and stalls for milliseconds from 32 workgroups on —
//       bounding the grid, as the reference does (cuda_sm_kernel.cu:29-32), does not help here.
//       So gather / scatter / paged copies whose flat side is host memory go in two stages per
//       piece of up to kStageBytes: the kernel compacts between the paged cache and a device
//       staging buffer at HBM speed, and one copy-engine transfer moves the piece over PCIe
//       (54-56 GB/s with the decode step running beside it at 35-37 us, no stalls).  Batch copies
//       (two pointer tables) with a host end keep the direct kernel on kHostCopyGroups
//       workgroups.
#include "common.h"

#include <cstring>
#include <mutex>
#include <new>
#include <vector>

namespace {

constexpr int kThreads = 256;
constexpr size_t kSeg = (size_t)kThreads * 16;  // 4 KiB per workgroup
constexpr int kSlots = 4;
constexpr size_t kHostCopyGroups = 16;          // workgroups of a batch copy with a host end
// Device staging of host-ended copies, per stream.  A piece costs its kernel (40 us at this size) and
// two dependent launches before the link is busy again: 64 MiB pieces reach 54.5 GB/s to the host,
// 256 MiB pieces 55.8 GB/s (a flat copy-engine transfer: 57.0 GB/s).  Two staging buffers with the
// transfers (or the kernels) on a second stream, joined by events, were slower than either: 37 and
// 44 GB/s - every cross-stream dependency costs more than the kernel it would hide.
constexpr size_t kStageBytes = (size_t)256 << 20;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Copies `bytes` (<= kSeg) from src to dst with the whole workgroup.  16-byte vectors when both
// ends are 16-byte aligned, bytes otherwise.
__device__ __forceinline__ void wg_copy(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                        size_t bytes)
{
    if ((((uintptr_t)src | (uintptr_t)dst) & 15) == 0) {
        const size_t nvec = bytes >> 4;
        const u32x4* s = reinterpret_cast<const u32x4*>(src);
        u32x4* d = reinterpret_cast<u32x4*>(dst);
        if (threadIdx.x < nvec)
            __builtin_nontemporal_store(__builtin_nontemporal_load(s + threadIdx.x), d + threadIdx.x);
        const size_t tail = (nvec << 4) + threadIdx.x;
        if (tail < bytes) dst[tail] = src[tail];
    } else {
        for (size_t i = threadIdx.x; i < bytes; i += kThreads) dst[i] = src[i];
    }
}

// mode 0: gather  dst_flat + i*size <- src_tab[i]
// mode 1: scatter dst_tab[i]        <- src_flat + i*size
// mode 2: batch   dst_tab[i]        <- src_tab[i]
template <int MODE>
__global__ __launch_bounds__(kThreads) void table_copy_kernel(const uint64_t* __restrict__ src_tab,
                                                              const uint64_t* __restrict__ dst_tab,
                                                              const uint8_t* src_flat,
                                                              uint8_t* dst_flat, size_t size,
                                                              size_t number, size_t segs_per_chunk)
{
    // one segment per workgroup, or a bounded grid striding over the segments
    const size_t groups = (size_t)gridDim.y * gridDim.x;
    for (size_t seg = (size_t)blockIdx.y * gridDim.x + blockIdx.x; seg < number * segs_per_chunk; seg += groups) {
        const size_t i = seg / segs_per_chunk;
        const size_t off = (seg - i * segs_per_chunk) * kSeg;
        const size_t bytes = (size - off < kSeg) ? size - off : kSeg;
        const uint8_t* s = (MODE == 1) ? src_flat + i * size : (const uint8_t*)src_tab[i];
        uint8_t* d = (MODE == 0) ? dst_flat + i * size : (uint8_t*)dst_tab[i];
        wg_copy(s + off, d + off, bytes);
    }
}

// Table-free paged copy.  meta: [n_cols] base, [n_cols] col_bytes, [n_cols] col offset in a
// flat row, then segs_per_row entries (col << 40 | offset-in-col), then block ids (int32).
__global__ __launch_bounds__(kThreads) void paged_copy_kernel(const uint64_t* __restrict__ meta,
                                                              int n_cols, size_t segs_per_row,
                                                              size_t row_bytes, size_t n_blocks,
                                                              uint8_t* flat, int to_cache,
                                                              size_t first_block)
{
    const uint64_t* base = meta;
    const uint64_t* cbytes = meta + n_cols;
    const uint64_t* coff = meta + 2 * n_cols;
    const uint64_t* segmap = meta + 3 * n_cols;
    const int32_t* ids = reinterpret_cast<const int32_t*>(segmap + segs_per_row);
    const size_t groups = (size_t)gridDim.y * gridDim.x;
    for (size_t seg = (size_t)blockIdx.y * gridDim.x + blockIdx.x; seg < n_blocks * segs_per_row; seg += groups) {
        const size_t i = seg / segs_per_row;
        const uint64_t e = segmap[seg - i * segs_per_row];
        const int c = (int)(e >> 40);
        const size_t off = (size_t)(e & ((1ull << 40) - 1));
        const size_t csz = cbytes[c];
        const size_t bytes = (csz - off < kSeg) ? csz - off : kSeg;
        uint8_t* cache_p = (uint8_t*)(base[c] + (uint64_t)ids[first_block + i] * csz) + off;
        uint8_t* flat_p = flat + i * row_bytes + coff[c] + off;
        if (to_cache) wg_copy(flat_p, cache_p, bytes);
        else wg_copy(cache_p, flat_p, bytes);
    }
}

struct Slot {
    void* host = nullptr;  // pinned staging for tables
    void* dev = nullptr;
    size_t cap = 0;
    hipEvent_t done = nullptr;
    bool busy = false;
};

}  // namespace

struct ucm_trans_stream {
    int kind = UCM_TRANS_CE;
    int device = 0;
    hipStream_t stream = nullptr;
    Slot slots[kSlots];
    int next = 0;
    int num_cus = 256;
    void* stage = nullptr;  // device staging buffer of host-ended copies
    size_t stage_cap = 0;
    std::mutex mu;
};

namespace {

// Returns a staging slot with room for `bytes`, waiting for its previous user if needed.
int acquire_slot(ucm_trans_stream* s, size_t bytes, Slot** out)
{
    Slot& sl = s->slots[s->next];
    s->next = (s->next + 1) % kSlots;
    if (sl.busy) {
        UCM_HIP_TRY(hipEventSynchronize(sl.done));
        sl.busy = false;
    }
    if (sl.cap < bytes) {
        if (sl.host) (void)hipHostFree(sl.host);
        if (sl.dev) (void)hipFree(sl.dev);
        sl.host = sl.dev = nullptr;
        sl.cap = 0;
        size_t cap = 1 << 16;
        while (cap < bytes) cap <<= 1;
        UCM_HIP_TRY(hipHostMalloc(&sl.host, cap, hipHostMallocDefault));
        UCM_HIP_TRY(hipMalloc(&sl.dev, cap));
        sl.cap = cap;
    }
    if (!sl.done) UCM_HIP_TRY(hipEventCreateWithFlags(&sl.done, hipEventDisableTiming));
    *out = &sl;
    return UCM_OK;
}

int release_slot(ucm_trans_stream* s, Slot* sl)
{
    UCM_HIP_TRY(hipEventRecord(sl->done, s->stream));
    sl->busy = true;
    return UCM_OK;
}

// True when p lies in host memory the device can address (pinned or registered).
bool is_host_memory(const void* p)
{
    if (!p) return false;
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return attr.type == hipMemoryTypeHost;
}

// One workgroup per segment, folded over x and y (x <= 2^20) so that any count fits a grid;
// at most kHostCopyGroups workgroups when an end of the copy is host memory.
dim3 grid_for(size_t total_segs, bool host_end = false)
{
    if (host_end && total_segs > kHostCopyGroups) total_segs = kHostCopyGroups;
    const size_t gx = total_segs < (1u << 20) ? (total_segs ? total_segs : 1) : (1u << 20);
    const size_t gy = (total_segs + gx - 1) / gx;
    return dim3((unsigned)gx, (unsigned)(gy ? gy : 1));
}

// Staging buffer with room for `want` bytes (at most kStageBytes are asked for); grows by
// replacing the buffer once the stream has drained.
int ensure_stage(ucm_trans_stream* s, size_t want)
{
    if (s->stage_cap >= want) return UCM_OK;
    if (s->stage) {
        UCM_HIP_TRY(hipStreamSynchronize(s->stream));
        (void)hipFree(s->stage);
        s->stage = nullptr;
        s->stage_cap = 0;
    }
    size_t cap = (size_t)1 << 20;
    while (cap < want) cap <<= 1;
    UCM_HIP_TRY(hipMalloc(&s->stage, cap));
    s->stage_cap = cap;
    return UCM_OK;
}

int finish(ucm_trans_stream* s, int sync)
{
    if (sync) UCM_HIP_TRY(hipStreamSynchronize(s->stream));
    return UCM_OK;
}

// mode as in table_copy_kernel
int table_copy(ucm_trans_stream* s, int mode, const void* const* src_tab,
               const void* const* dst_tab, const void* src_flat, void* dst_flat,
               int table_on_device, size_t size, size_t number, int sync)
{
    ucm::clear_error();
    UCM_REQUIRE(s, "null stream");
    if (number == 0 || size == 0) return finish(s, sync);
    UCM_REQUIRE(mode == 1 || src_tab, "null source table");
    UCM_REQUIRE(mode == 0 || dst_tab, "null destination table");
    UCM_REQUIRE(mode != 1 || src_flat, "null source buffer");
    UCM_REQUIRE(mode != 0 || dst_flat, "null destination buffer");
    std::lock_guard<std::mutex> lock(s->mu);

    if (s->kind == UCM_TRANS_CE) {
        if (table_on_device)
            return ucm::fail(UCM_EPARAM, "a copy-engine stream needs host pointer tables");
        for (size_t i = 0; i < number; ++i) {
            const void* sp = (mode == 1) ? (const char*)src_flat + i * size : src_tab[i];
            void* dp = (mode == 0) ? (char*)dst_flat + i * size : (void*)dst_tab[i];
            UCM_HIP_TRY(hipMemcpyAsync(dp, sp, size, hipMemcpyDefault, s->stream));
        }
        return finish(s, sync);
    }

    const uint64_t* d_src = (const uint64_t*)src_tab;
    const uint64_t* d_dst = (const uint64_t*)dst_tab;
    Slot* sl = nullptr;
    if (!table_on_device) {
        const size_t ntab = (mode == 2) ? 2 : 1;
        const size_t bytes = ntab * number * sizeof(uint64_t);
        int rc = acquire_slot(s, bytes, &sl);
        if (rc != UCM_OK) return rc;
        uint64_t* h = (uint64_t*)sl->host;
        if (mode != 1) std::memcpy(h, src_tab, number * 8);
        if (mode == 1) std::memcpy(h, dst_tab, number * 8);
        if (mode == 2) std::memcpy(h + number, dst_tab, number * 8);
        UCM_HIP_TRY(hipMemcpyAsync(sl->dev, sl->host, bytes, hipMemcpyHostToDevice, s->stream));
        d_src = (mode != 1) ? (const uint64_t*)sl->dev : nullptr;
        d_dst = (mode == 1) ? (const uint64_t*)sl->dev
                            : (mode == 2 ? (const uint64_t*)sl->dev + number : nullptr);
    }
    const size_t segs = (size + kSeg - 1) / kSeg;
    // host tables can be inspected; a device-resident table says nothing about what it points to
    bool host_end = mode != 2 && is_host_memory(mode == 1 ? src_flat : dst_flat);
    if (host_end && size <= kStageBytes) {
        // two stages per piece of whole chunks: kernel <-> device staging, copy engine <-> host
        const size_t per_piece = kStageBytes / size;
        const size_t first_piece = number < per_piece ? number : per_piece;
        int rc = ensure_stage(s, first_piece * size);
        if (rc != UCM_OK) return rc;
        for (size_t first = 0; first < number; first += per_piece) {
            const size_t n = number - first < per_piece ? number - first : per_piece;
            const dim3 pgrid = grid_for(n * segs);
            if (mode == 0) {
                hipLaunchKernelGGL(table_copy_kernel<0>, pgrid, dim3(kThreads), 0, s->stream, d_src + first, d_dst,
                                   (const uint8_t*)nullptr, (uint8_t*)s->stage, size, n, segs);
                UCM_HIP_TRY(hipMemcpyAsync((char*)dst_flat + first * size, s->stage, n * size,
                                           hipMemcpyDeviceToHost, s->stream));
            } else {
                UCM_HIP_TRY(hipMemcpyAsync(s->stage, (const char*)src_flat + first * size, n * size,
                                           hipMemcpyHostToDevice, s->stream));
                hipLaunchKernelGGL(table_copy_kernel<1>, pgrid, dim3(kThreads), 0, s->stream, d_src, d_dst + first,
                                   (const uint8_t*)s->stage, (uint8_t*)nullptr, size, n, segs);
            }
        }
        rc = ucm::launch_status("table_copy_kernel");
        if (rc != UCM_OK) return rc;
        if (sl) {
            rc = release_slot(s, sl);
            if (rc != UCM_OK) return rc;
        }
        return finish(s, sync);
    }
    if (!host_end && mode == 2 && !table_on_device) host_end = is_host_memory(src_tab[0]) || is_host_memory(dst_tab[0]);
    const dim3 grid = grid_for(number * segs, host_end);
    if (mode == 0)
        hipLaunchKernelGGL(table_copy_kernel<0>, grid, dim3(kThreads), 0, s->stream, d_src, d_dst,
                           (const uint8_t*)nullptr, (uint8_t*)dst_flat, size, number, segs);
    else if (mode == 1)
        hipLaunchKernelGGL(table_copy_kernel<1>, grid, dim3(kThreads), 0, s->stream, d_src, d_dst,
                           (const uint8_t*)src_flat, (uint8_t*)nullptr, size, number, segs);
    else
        hipLaunchKernelGGL(table_copy_kernel<2>, grid, dim3(kThreads), 0, s->stream, d_src, d_dst,
                           (const uint8_t*)nullptr, (uint8_t*)nullptr, size, number, segs);
    int rc = ucm::launch_status("table_copy_kernel");
    if (rc != UCM_OK) return rc;
    if (sl) {
        rc = release_slot(s, sl);
        if (rc != UCM_OK) return rc;
    }
    return finish(s, sync);
}

struct CallbackBox {
    void (*cb)(int, void*);
    void* user;
};

void callback_trampoline(hipStream_t, hipError_t status, void* data)
{
    CallbackBox* box = static_cast<CallbackBox*>(data);
    box->cb(status == hipSuccess ? 1 : 0, box->user);
    delete box;
}

}  // namespace

extern "C" int ucm_trans_setup(int32_t device_id)
{
    ucm::clear_error();
    int n = 0;
    UCM_HIP_TRY(hipGetDeviceCount(&n));
    UCM_REQUIRE(device_id >= 0 && device_id < n, "device id %d outside [0, %d)", device_id, n);
    UCM_HIP_TRY(hipSetDevice(device_id));
    return UCM_OK;
}

extern "C" int ucm_trans_stream_create(int kind, ucm_trans_stream_t** out)
{
    ucm::clear_error();
    UCM_REQUIRE(out, "null out pointer");
    UCM_REQUIRE(kind == UCM_TRANS_CE || kind == UCM_TRANS_SM, "unknown stream kind %d", kind);
    ucm_trans_stream* s = new (std::nothrow) ucm_trans_stream();
    if (!s) return ucm::fail(UCM_EOOM, "out of host memory");
    s->kind = kind;
    hipError_t e = hipGetDevice(&s->device);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking);
    if (e == hipSuccess) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, s->device) == hipSuccess && prop.multiProcessorCount > 0)
            s->num_cus = prop.multiProcessorCount;
    }
    if (e != hipSuccess) {
        delete s;
        return ucm::hip_fail(e, "stream creation");
    }
    *out = s;
    return UCM_OK;
}

extern "C" int ucm_trans_stream_destroy(ucm_trans_stream_t* s)
{
    ucm::clear_error();
    if (!s) return UCM_OK;
    (void)hipStreamSynchronize(s->stream);
    for (Slot& sl : s->slots) {
        if (sl.done) (void)hipEventDestroy(sl.done);
        if (sl.host) (void)hipHostFree(sl.host);
        if (sl.dev) (void)hipFree(sl.dev);
    }
    if (s->stage) (void)hipFree(s->stage);
    (void)hipStreamDestroy(s->stream);
    delete s;
    return UCM_OK;
}

extern "C" void* ucm_trans_stream_handle(ucm_trans_stream_t* s) { return s ? (void*)s->stream : nullptr; }

extern "C" int ucm_trans_stream_sync(ucm_trans_stream_t* s)
{
    ucm::clear_error();
    UCM_REQUIRE(s, "null stream");
    UCM_HIP_TRY(hipStreamSynchronize(s->stream));
    return UCM_OK;
}

extern "C" int ucm_trans_stream_wait_event(ucm_trans_stream_t* s, void* event)
{
    ucm::clear_error();
    UCM_REQUIRE(s, "null stream");
    if (!event) return UCM_OK;
    UCM_HIP_TRY(hipStreamWaitEvent(s->stream, (hipEvent_t)event, 0));
    return UCM_OK;
}

extern "C" int ucm_trans_stream_append_callback(ucm_trans_stream_t* s,
                                                void (*cb)(int ok, void* user), void* user)
{
    ucm::clear_error();
    UCM_REQUIRE(s && cb, "null stream or callback");
    CallbackBox* box = new (std::nothrow) CallbackBox{cb, user};
    if (!box) return ucm::fail(UCM_EOOM, "out of memory for appending callback");
    hipError_t e = hipStreamAddCallback(s->stream, callback_trampoline, box, 0);
    if (e != hipSuccess) {
        delete box;
        return ucm::hip_fail(e, "hipStreamAddCallback");
    }
    return UCM_OK;
}

extern "C" int ucm_trans_d2h(ucm_trans_stream_t* s, const void* device, void* host, size_t size,
                             int sync)
{
    ucm::clear_error();
    UCM_REQUIRE(s && device && host, "null argument");
    UCM_HIP_TRY(hipMemcpyAsync(host, device, size, hipMemcpyDeviceToHost, s->stream));
    return finish(s, sync);
}

extern "C" int ucm_trans_h2d(ucm_trans_stream_t* s, const void* host, void* device, size_t size,
                             int sync)
{
    ucm::clear_error();
    UCM_REQUIRE(s && device && host, "null argument");
    UCM_HIP_TRY(hipMemcpyAsync(device, host, size, hipMemcpyHostToDevice, s->stream));
    return finish(s, sync);
}

extern "C" int ucm_trans_gather(ucm_trans_stream_t* s, const void* const* src, int table_on_device,
                                void* dst, size_t size, size_t number, int sync)
{
    return table_copy(s, 0, src, nullptr, nullptr, dst, table_on_device, size, number, sync);
}

extern "C" int ucm_trans_scatter(ucm_trans_stream_t* s, const void* src, void* const* dst,
                                 int table_on_device, size_t size, size_t number, int sync)
{
    return table_copy(s, 1, nullptr, (const void* const*)dst, src, nullptr, table_on_device, size,
                      number, sync);
}

extern "C" int ucm_trans_batch(ucm_trans_stream_t* s, const void* const* src, void* const* dst,
                               int table_on_device, size_t size, size_t number, int sync)
{
    return table_copy(s, 2, src, (const void* const*)dst, nullptr, nullptr, table_on_device, size,
                      number, sync);
}

extern "C" int ucm_trans_paged_copy(ucm_trans_stream_t* s, const uint64_t* base,
                                    const uint64_t* col_bytes, int32_t n_cols,
                                    const int32_t* block_ids, int64_t n_blocks,
                                    int64_t n_cache_blocks, void* flat, int to_cache, int sync)
{
    ucm::clear_error();
    UCM_REQUIRE(n_cols > 0 && n_blocks >= 0 && n_cache_blocks >= 0, "bad sizes");
    UCM_REQUIRE(base && col_bytes && flat && (block_ids || n_blocks == 0), "null argument");
    // an id outside the cache would become a wild device address inside the kernel
    for (int64_t i = 0; i < n_blocks; ++i)
        UCM_REQUIRE(block_ids[i] >= 0 && (n_cache_blocks == 0 || block_ids[i] < n_cache_blocks),
                    "block_ids[%lld] = %d outside the cache's %lld blocks", (long long)i, block_ids[i],
                    (long long)n_cache_blocks);
    UCM_REQUIRE(s, "null stream");
    UCM_REQUIRE(s->kind == UCM_TRANS_SM, "paged copy needs an SM stream");
    if (n_blocks == 0) return finish(s, sync);
    std::lock_guard<std::mutex> lock(s->mu);

    size_t row_bytes = 0, segs_per_row = 0;
    for (int c = 0; c < n_cols; ++c) {
        UCM_REQUIRE(col_bytes[c] > 0 && col_bytes[c] < (1ull << 40), "column %d size out of range", c);
        row_bytes += col_bytes[c];
        segs_per_row += (col_bytes[c] + kSeg - 1) / kSeg;
    }
    const size_t meta_words = 3 * (size_t)n_cols + segs_per_row;
    const size_t bytes = meta_words * 8 + (size_t)n_blocks * 4;
    Slot* sl = nullptr;
    int rc = acquire_slot(s, bytes, &sl);
    if (rc != UCM_OK) return rc;
    uint64_t* h = (uint64_t*)sl->host;
    size_t off = 0, si = 0;
    for (int c = 0; c < n_cols; ++c) {
        h[c] = base[c];
        h[n_cols + c] = col_bytes[c];
        h[2 * n_cols + c] = off;
        off += col_bytes[c];
        for (size_t o = 0; o < col_bytes[c]; o += kSeg) h[3 * n_cols + si++] = ((uint64_t)c << 40) | o;
    }
    std::memcpy(h + meta_words, block_ids, (size_t)n_blocks * 4);
    UCM_HIP_TRY(hipMemcpyAsync(sl->dev, sl->host, bytes, hipMemcpyHostToDevice, s->stream));
    const bool host_end = is_host_memory(flat);
    if (host_end && row_bytes <= kStageBytes) {
        // two stages per piece of whole blocks, as in table_copy()
        const size_t per_piece = kStageBytes / row_bytes;
        const size_t first_piece = (size_t)n_blocks < per_piece ? (size_t)n_blocks : per_piece;
        rc = ensure_stage(s, first_piece * row_bytes);
        if (rc != UCM_OK) return rc;
        for (size_t first = 0; first < (size_t)n_blocks; first += per_piece) {
            const size_t n = (size_t)n_blocks - first < per_piece ? (size_t)n_blocks - first : per_piece;
            const dim3 pgrid = grid_for(n * segs_per_row);
            char* hp = (char*)flat + first * row_bytes;
            if (to_cache) UCM_HIP_TRY(hipMemcpyAsync(s->stage, hp, n * row_bytes, hipMemcpyHostToDevice, s->stream));
            hipLaunchKernelGGL(paged_copy_kernel, pgrid, dim3(kThreads), 0, s->stream, (const uint64_t*)sl->dev,
                               (int)n_cols, segs_per_row, row_bytes, n, (uint8_t*)s->stage, to_cache, first);
            if (!to_cache) UCM_HIP_TRY(hipMemcpyAsync(hp, s->stage, n * row_bytes, hipMemcpyDeviceToHost, s->stream));
        }
    } else {
        const dim3 grid = grid_for((size_t)n_blocks * segs_per_row, host_end);
        hipLaunchKernelGGL(paged_copy_kernel, grid, dim3(kThreads), 0, s->stream,
                           (const uint64_t*)sl->dev, (int)n_cols, segs_per_row, row_bytes,
                           (size_t)n_blocks, (uint8_t*)flat, to_cache, (size_t)0);
    }
    rc = ucm::launch_status("paged_copy_kernel");
    if (rc != UCM_OK) return rc;
    rc = release_slot(s, sl);
    if (rc != UCM_OK) return rc;
    return finish(s, sync);
}

extern "C" int ucm_trans_host_alloc(size_t size, void** out)
{
    ucm::clear_error();
    UCM_REQUIRE(out && size > 0, "bad argument");
    UCM_HIP_TRY(hipHostMalloc(out, size, hipHostMallocDefault));
    return UCM_OK;
}

extern "C" int ucm_trans_host_free(void* p)
{
    ucm::clear_error();
    if (!p) return UCM_OK;
    UCM_HIP_TRY(hipHostFree(p));
    return UCM_OK;
}

extern "C" int ucm_trans_device_alloc(size_t size, void** out)
{
    ucm::clear_error();
    UCM_REQUIRE(out && size > 0, "bad argument");
    UCM_HIP_TRY(hipMalloc(out, size));
    return UCM_OK;
}

extern "C" int ucm_trans_device_free(void* p)
{
    ucm::clear_error();
    if (!p) return UCM_OK;
    UCM_HIP_TRY(hipFree(p));
    return UCM_OK;
}

extern "C" int ucm_trans_host_register(void* host, size_t size, void** device_alias)
{
    ucm::clear_error();
    UCM_REQUIRE(host && size > 0, "bad argument");
    UCM_HIP_TRY(hipHostRegister(host, size, hipHostRegisterDefault));
    if (device_alias) UCM_HIP_TRY(hipHostGetDevicePointer(device_alias, host, 0));
    return UCM_OK;
}

extern "C" int ucm_trans_host_unregister(void* host)
{
    ucm::clear_error();
    UCM_REQUIRE(host, "null pointer");
    UCM_HIP_TRY(hipHostUnregister(host));
    return UCM_OK;
}
