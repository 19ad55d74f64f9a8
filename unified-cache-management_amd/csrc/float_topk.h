// Selection shared by the float retrieval paths: the k best of a row of fp32 scores in
// descending order.  One 1024-thread workgroup per row: four 8-bit radix passes over
// order-preserving 32-bit keys find the k-th largest, winners are compacted into LDS (ties at
// the threshold in list order) and a bitonic sort orders (key, position) pairs, so equal
// scores come out in list order.  Included by the translation units that launch it.
#pragma once

#include "common.h"

namespace {

constexpr int kSortThreads = 1024;
constexpr int kMaxTopk = 4096;  // winners sorted in LDS: 8 bytes each (32 KiB)

// Order-preserving key of a score: larger score <-> larger key.  0 is reserved for "no
// candidate", 1 for NaN (below every number, above nothing else).
__device__ __forceinline__ uint32_t score_key(float s)
{
    if (s != s) return 1u;
    const uint32_t u = __float_as_uint(s);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
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
        // digits in descending order, one per thread: the chosen digit is where the running
        // count first reaches `need`
        const int cnt = tid < 256 ? hist[255 - tid] : 0;
        int all;
        const int before = scan1024(cnt, wsum, &all);
        if (tid < 256 && before < need && before + cnt >= need) {
            s_digit = 255 - tid;
            s_need = need - before;  // still to take among keys with this digit
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

// Short rows (max_n <= 1024, e.g. the blocks of one request): every candidate counts the
// candidates that come before it in the output order (larger key, or equal key and earlier
// position) and writes itself at that rank.  No search and no sort: n broadcast reads from LDS
// per thread.  Same output as topk_sort_kernel.
__global__ __launch_bounds__(kSortThreads) void topk_rank_kernel(SortArgs a)
{
    __shared__ __align__(16) uint32_t k_lds[kSortThreads];
    const int b = blockIdx.x, tid = threadIdx.x;
    const uint32_t* keys = a.keys + (int64_t)b * a.max_n;
    const uint32_t mine = tid < a.max_n ? keys[tid] : 0u;
    k_lds[tid] = mine;
    for (int t = tid; t < a.topk; t += kSortThreads) {  // slots no candidate reaches
        a.out_idx[(int64_t)b * a.topk + t] = -1;
        a.out_score[(int64_t)b * a.topk + t] = 0.0f;
    }
    __syncthreads();  // also orders the fill above before the winners' writes below
    if (mine == 0u) return;
    int rank = 0;
    const int n4 = a.max_n & ~3;
    for (int j = 0; j < n4; j += 4) {
        const uint4 o = *reinterpret_cast<const uint4*>(k_lds + j);
        rank += (o.x > mine || (o.x == mine && j < tid)) + (o.y > mine || (o.y == mine && j + 1 < tid)) +
                (o.z > mine || (o.z == mine && j + 2 < tid)) + (o.w > mine || (o.w == mine && j + 3 < tid));
    }
    for (int j = n4; j < a.max_n; ++j) {
        const uint32_t o = k_lds[j];
        rank += (o > mine || (o == mine && j < tid));
    }
    if (rank < a.topk) {
        a.out_idx[(int64_t)b * a.topk + rank] = a.idx[(int64_t)b * a.max_n + tid];
        a.out_score[(int64_t)b * a.topk + rank] = a.scores[(int64_t)b * a.max_n + tid];
    }
}

// cap = power of two >= topk
inline int launch_topk_sort(const SortArgs& in, int rows, hipStream_t st)
{
    if (in.max_n <= kSortThreads) {
        hipLaunchKernelGGL(topk_rank_kernel, dim3((unsigned)rows), dim3(kSortThreads), 0, st, in);
        return ucm::launch_status("topk_rank_kernel");
    }
    SortArgs s = in;
    int cap = 2;
    while (cap < s.topk) cap <<= 1;
    s.cap = cap;
    hipLaunchKernelGGL(topk_sort_kernel, dim3((unsigned)rows), dim3(kSortThreads), (size_t)cap * 8, st, s);
    return ucm::launch_status("topk_sort_kernel");
}

}  // namespace
