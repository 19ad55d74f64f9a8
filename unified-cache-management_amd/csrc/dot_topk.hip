// Float retrieval for gfx950: per request, dot products of one query with a list of candidate
// rows of a [n_items, dim] fp32 matrix, then the top-k candidates in descending score order.
//
// GPU counterpart of the reference's ESA retrieval backend
// (ucm/sparse/esa/retrieval/cpy/retrieval_backend.cpp:207-227: for every allowed index a
// sequential fp32 dot product, std::partial_sort by descending score, the first
// min(n_allowed, topk) pairs returned).  Two kernels:
//   * dot_score_kernel — HBM-bound gather: one wave per candidate row, 16-byte loads, the query
//     in LDS, a shuffle reduction; writes one fp32 score per candidate (candidates that are -1
//     or outside the matrix get a key below every number);
//   * topk_sort_kernel — one workgroup per request: 8-bit radix search for the k-th largest
//     order-preserving key, winners compacted into LDS (ties at the threshold in list order),
//     bitonic sort of (key, position) pairs.  Equal scores come out in list order; the
//     reference leaves ties unspecified.
// Scores differ from the reference's in the last bits (the partial sums are added in a
// different order); the tolerance is stated where the results are compared.
#include "common.h"

namespace {

constexpr int kDotThreads = 256;
constexpr int kRowsPerWave = 4;
constexpr int kSortThreads = 1024;
constexpr int kMaxTopk = 4096;  // winners sorted in LDS: 8 bytes each (32 KiB)

typedef float f32x4 __attribute__((ext_vector_type(4)));

// Order-preserving key of a score: larger score <-> larger key.  0 is reserved for "no
// candidate", 1 for NaN (below every number, above nothing else).
__device__ __forceinline__ uint32_t score_key(float s)
{
    if (s != s) return 1u;
    const uint32_t u = __float_as_uint(s);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct DotArgs {
    const float* data;
    int64_t n_items;
    int dim;
    const float* q;        // [B][dim]
    const int32_t* idx;    // [B][max_n], -1 = no candidate
    int max_n;
    float* scores;         // [B][max_n]
    uint32_t* keys;        // [B][max_n]
};

__global__ __launch_bounds__(kDotThreads) void dot_score_kernel(DotArgs a)
{
    extern __shared__ float qs[];  // the request's query
    const int b = blockIdx.y;
    const float* q = a.q + (int64_t)b * a.dim;
    for (int i = threadIdx.x; i < a.dim; i += kDotThreads) qs[i] = q[i];
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int first = (blockIdx.x * (kDotThreads / 64) + wave) * kRowsPerWave;
    const bool vec = (a.dim & 3) == 0;
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int j = first + r;
        if (j >= a.max_n) break;
        const int item = a.idx[(int64_t)b * a.max_n + j];
        const bool ok = item >= 0 && item < a.n_items;
        float acc = 0.0f;
        if (ok) {
            const float* row = a.data + (int64_t)item * a.dim;
            if (vec) {
                for (int c = lane * 4; c < a.dim; c += 256) {
                    const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(row + c));
                    const f32x4 y = *reinterpret_cast<const f32x4*>(qs + c);
                    acc = __builtin_fmaf(x.x, y.x, acc);
                    acc = __builtin_fmaf(x.y, y.y, acc);
                    acc = __builtin_fmaf(x.z, y.z, acc);
                    acc = __builtin_fmaf(x.w, y.w, acc);
                }
            } else {
                for (int c = lane; c < a.dim; c += 64) acc = __builtin_fmaf(row[c], qs[c], acc);
            }
        }
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) acc += __shfl_xor(acc, s);
        if (lane == 0) {
            a.scores[(int64_t)b * a.max_n + j] = ok ? acc : 0.0f;
            a.keys[(int64_t)b * a.max_n + j] = ok ? score_key(acc) : 0u;
        }
    }
}

struct SortArgs {
    const uint32_t* keys;   // [B][max_n]
    const float* scores;    // [B][max_n]
    const int32_t* idx;     // [B][max_n]
    int max_n, topk, cap;   // cap = power of two >= topk: LDS elements
    int32_t* out_idx;       // [B][topk]
    float* out_score;       // [B][topk]
};

// Exclusive prefix sum of one int per thread over the 1024-thread workgroup.
__device__ __forceinline__ int scan1024(int v, int* wsum, int* total)
{
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    int inc = v;
#pragma unroll
    for (int s = 1; s < 64; s <<= 1) {
        const int o = __shfl_up(inc, s);
        if (lane >= s) inc += o;
    }
    __syncthreads();
    if (lane == 63) wsum[w] = inc;
    __syncthreads();
    int base = 0, tot = 0;
    for (int i = 0; i < kSortThreads / 64; ++i) {
        const int x = wsum[i];
        if (i < w) base += x;
        tot += x;
    }
    *total = tot;
    return base + inc - v;
}

__global__ __launch_bounds__(kSortThreads) void topk_sort_kernel(SortArgs a)
{
    extern __shared__ unsigned long long win[];  // [cap] (key << 32) | ~position
    __shared__ int hist[256];
    __shared__ int wsum[kSortThreads / 64];
    __shared__ int s_digit, s_need, s_count;
    const int b = blockIdx.x;
    const uint32_t* keys = a.keys + (int64_t)b * a.max_n;
    const int tid = threadIdx.x;

    // candidates present
    int mine = 0;
    for (int i = tid; i < a.max_n; i += kSortThreads) mine += keys[i] != 0u;
    int n_valid;
    (void)scan1024(mine, wsum, &n_valid);
    const int kk = n_valid < a.topk ? n_valid : a.topk;

    // ---- radix search, 8 bits a pass, for the kk-th largest key among the candidates ----
    uint32_t prefix = 0, mask = 0;
    int need = kk;
    for (int shift = 24; shift >= 0 && kk > 0; shift -= 8) {
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        for (int i = tid; i < a.max_n; i += kSortThreads) {
            const uint32_t k = keys[i];
            if (k != 0u && (k & mask) == prefix) atomicAdd(&hist[(k >> shift) & 255], 1);
        }
        __syncthreads();
        if (tid == 0) {
            int d = 255, acc = 0;
            for (; d > 0; --d) {
                if (acc + hist[d] >= need) break;
                acc += hist[d];
            }
            s_digit = d;
            s_need = need - acc;  // still to take among keys with this digit
        }
        __syncthreads();
        prefix |= (uint32_t)s_digit << shift;
        mask |= 255u << shift;
        need = s_need;
        __syncthreads();
    }
    const uint32_t thr = prefix;  // the kk-th largest key; `need` of the keys equal to it are taken

    // ---- winners into LDS: every key above the threshold, the first `need` equal to it ----
    for (int i = tid; i < a.cap; i += kSortThreads) win[i] = 0ull;
    if (tid == 0) s_count = 0;
    __syncthreads();
    int eq_before = 0;  // keys equal to the threshold in earlier chunks
    for (int base = 0; base < a.max_n && kk > 0; base += kSortThreads) {
        const int i = base + tid;
        const uint32_t k = i < a.max_n ? keys[i] : 0u;
        const bool gt = k > thr && k != 0u;
        const bool eq = k == thr && k != 0u;
        int eq_total;
        const int eq_rank = eq_before + scan1024(eq ? 1 : 0, wsum, &eq_total);
        if (gt || (eq && eq_rank < need)) {
            const int slot = atomicAdd(&s_count, 1);
            win[slot] = ((unsigned long long)k << 32) | (uint32_t)(~(uint32_t)i);
        }
        eq_before += eq_total;
    }
    __syncthreads();

    // ---- bitonic sort, descending: larger key first, then smaller position ----
    for (int size = 2; size <= a.cap; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int t = tid; t < a.cap / 2; t += kSortThreads) {
                const int lo = 2 * t - (t & (stride - 1));
                const int hi = lo + stride;
                const bool desc = (lo & size) == 0;
                const unsigned long long x = win[lo], y = win[hi];
                if ((x < y) == desc) {
                    win[lo] = y;
                    win[hi] = x;
                }
            }
            __syncthreads();
        }
    }

    for (int t = tid; t < a.topk; t += kSortThreads) {
        int32_t oi = -1;
        float os = 0.0f;
        if (t < kk) {
            const int pos = (int)(~(uint32_t)(win[t] & 0xffffffffull));
            oi = a.idx[(int64_t)b * a.max_n + pos];
            os = a.scores[(int64_t)b * a.max_n + pos];
        }
        a.out_idx[(int64_t)b * a.topk + t] = oi;
        a.out_score[(int64_t)b * a.topk + t] = os;
    }
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

extern "C" size_t ucm_dot_topk_workspace_bytes(int32_t B, int32_t max_n)
{
    if (B <= 0 || max_n <= 0) return 256;
    return 2 * align256((size_t)B * max_n * 4);
}

extern "C" int ucm_dot_topk(const float* data, int64_t n_items, int32_t dim, const float* query,
                            const int32_t* indexes, int32_t B, int32_t max_n, int32_t topk,
                            int32_t* out_idx, float* out_score, void* workspace,
                            size_t workspace_bytes, ucm_stream_t stream)
{
    ucm::clear_error();
    UCM_REQUIRE(B >= 0 && B <= 65535, "batch %d out of range [0, 65535]", B);
    if (B == 0) return UCM_OK;
    UCM_REQUIRE(data && query && indexes && out_idx && out_score, "null pointer");
    UCM_REQUIRE(n_items > 0 && dim > 0 && max_n > 0, "non-positive shape");
    UCM_REQUIRE(topk > 0, "topk %d must be positive", topk);
    if (topk > kMaxTopk) return ucm::fail(UCM_EUNSUPPORTED, "topk %d above %d", topk, kMaxTopk);
    UCM_REQUIRE((size_t)dim * 4 <= 64 * 1024, "dim %d above 16384", dim);
    UCM_REQUIRE(workspace && workspace_bytes >= ucm_dot_topk_workspace_bytes(B, max_n),
                "workspace too small");
    UCM_REQUIRE((((uintptr_t)data | (uintptr_t)workspace) & 15) == 0, "data must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    DotArgs d{};
    d.data = data; d.n_items = n_items; d.dim = dim; d.q = query; d.idx = indexes; d.max_n = max_n;
    d.scores = (float*)workspace;
    d.keys = (uint32_t*)((char*)workspace + align256((size_t)B * max_n * 4));
    const int rows_per_wg = (kDotThreads / 64) * kRowsPerWave;
    hipLaunchKernelGGL(dot_score_kernel, dim3((unsigned)ucm::ceil_div(max_n, rows_per_wg), (unsigned)B),
                       dim3(kDotThreads), (size_t)dim * 4, st, d);
    int rc = ucm::launch_status("dot_score_kernel");
    if (rc != UCM_OK) return rc;
    SortArgs s{};
    s.keys = d.keys; s.scores = d.scores; s.idx = indexes; s.max_n = max_n; s.topk = topk;
    int cap = 2;
    while (cap < topk) cap <<= 1;
    s.cap = cap;
    s.out_idx = out_idx; s.out_score = out_score;
    hipLaunchKernelGGL(topk_sort_kernel, dim3((unsigned)B), dim3(kSortThreads), (size_t)cap * 8, st, s);
    return ucm::launch_status("topk_sort_kernel");
}
