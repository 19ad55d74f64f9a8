// Selection shared by the float retrieval paths: the k best of a row of fp32 scores in
// descending order.  One 1024-thread workgroup per row: four 8-bit radix passes over
// order-preserving 32-bit keys find the k-th largest, winners are compacted into LDS (ties at
// the threshold in list order) and ordered as (key, position) pairs by segment-wise bitonic
// networks followed by pairwise merges, so equal scores come out in list order.  Included by the translation units that launch it.
#pragma once

#include "common.h"

namespace {

constexpr int kSortThreads = 1024;
constexpr int kMaxTopk = 4096;  // winners sorted in LDS: 8 bytes each (32 KiB)
constexpr int kBuckets = 1024;   // equal-width key buckets of the ordering fast path (one per thread)
constexpr int kBucketMax = 48;   // entries a bucket may hold on that path
constexpr int kRegKeys = 8;     // keys a thread keeps in registers: rows of up to 8192 candidates

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

// REG: the row has at most kRegKeys * 1024 candidates and every thread keeps its keys in
// registers for all phases (one round trip to memory instead of one per phase and chunk).
template <bool REG>
__global__ __launch_bounds__(kSortThreads) void topk_sort_kernel(SortArgs a)
{
    extern __shared__ unsigned long long win[];  // [cap] (key << 32) | ~position
    __shared__ int hist[256];
    __shared__ int wsum[kSortThreads / 64];
    __shared__ int s_digit, s_need;
    __shared__ int bcount[kBuckets], bfill[kBuckets], bbase[kBuckets];
    const int b = blockIdx.x;
    const uint32_t* keys = a.keys + (int64_t)b * a.max_n;
    const int tid = threadIdx.x, lane = tid & 63;

    // REG: thread t holds list positions t * kRegKeys .. + kRegKeys - 1 (consecutive, so that one
    // prefix sum over per-thread counts orders the whole list)
    uint32_t kreg[REG ? kRegKeys : 1];
    if constexpr (REG) {
        static_assert(kRegKeys == 8, "two 16-byte loads per thread");
        const bool vec = (reinterpret_cast<uintptr_t>(keys) & 15) == 0;  // uniform
        if (vec && (tid + 1) * kRegKeys <= a.max_n) {
            const uint4 lo = *reinterpret_cast<const uint4*>(keys + tid * kRegKeys);
            const uint4 hi = *reinterpret_cast<const uint4*>(keys + tid * kRegKeys + 4);
            kreg[0] = lo.x; kreg[1] = lo.y; kreg[2] = lo.z; kreg[3] = lo.w;
            kreg[4] = hi.x; kreg[5] = hi.y; kreg[6] = hi.z; kreg[7] = hi.w;
        } else {
#pragma unroll
            for (int e = 0; e < kRegKeys; ++e) {
                const int i = tid * kRegKeys + e;
                kreg[e] = i < a.max_n ? keys[i] : 0u;
            }
        }
    }
    // f(chunk, key) over the thread's keys; uniform control flow.  Without REG chunk e covers
    // list positions e * 1024 + tid.
    auto for_chunks = [&](auto&& f) {
        if constexpr (REG) {
#pragma unroll
            for (int e = 0; e < kRegKeys; ++e) f(e, kreg[e]);
        } else {
            for (int e = 0; e * kSortThreads < a.max_n; ++e) {
                const int i = e * kSortThreads + tid;
                f(e, i < a.max_n ? keys[i] : 0u);
            }
        }
    };

    // candidates present
    int mine = 0;
    for_chunks([&](int, uint32_t k) { mine += k != 0u; });
    int n_valid;
    (void)scan1024(mine, wsum, &n_valid);
    const int kk = n_valid < a.topk ? n_valid : a.topk;

    // ---- radix search, 8 bits a pass, for the kk-th largest key among the candidates ----
    uint32_t prefix = 0, mask = 0;
    int need = kk;
    for (int shift = 24; shift >= 0 && kk > 0; shift -= 8) {
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        for_chunks([&](int, uint32_t k) {
            const bool in = k != 0u && (k & mask) == prefix;
            const int d = (k >> shift) & 255;
            // scores of one magnitude share their leading digits: when a whole wave holds one
            // digit its first lane adds the count (64 lanes adding to one LDS word serialise)
            const unsigned long long act = __ballot(in);
            if (act != 0ull) {
                const int first = __ffsll((long long)act) - 1;
                const int d0 = __shfl(d, first);
                if (__ballot(in && d == d0) == act) {
                    if (lane == first) atomicAdd(&hist[d0], __popcll(act));
                } else if (in) {
                    atomicAdd(&hist[d], 1);
                }
            }
        });
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

    // ---- winners into LDS: every key above the threshold, then the first `need` equal to it.
    //      Slots come from a prefix sum over the list (both counts packed into one scan), not
    //      from a shared counter: thousands of increments of one LDS word would serialise ----
    for (int i = tid; i < a.cap; i += kSortThreads) win[i] = 0ull;
    __syncthreads();
    const int n_gt = kk - need;  // keys above the threshold
    int gt_before = 0, eq_before = 0;
    if (kk > 0) {
        if constexpr (REG) {
            int my_gt = 0, my_eq = 0;
#pragma unroll
            for (int e = 0; e < kRegKeys; ++e) {
                my_gt += kreg[e] > thr && kreg[e] != 0u;
                my_eq += kreg[e] == thr && kreg[e] != 0u;
            }
            int total;
            const int before = scan1024(my_gt | (my_eq << 16), wsum, &total);
            int gt_at = before & 0xffff, eq_at = before >> 16;
#pragma unroll
            for (int e = 0; e < kRegKeys; ++e) {
                const uint32_t k = kreg[e];
                const int i = tid * kRegKeys + e;
                int slot = -1;
                if (k > thr && k != 0u) slot = gt_at++;
                else if (k == thr && k != 0u) {
                    if (eq_at < need) slot = n_gt + eq_at;
                    ++eq_at;
                }
                if (slot >= 0) win[slot] = ((unsigned long long)k << 32) | (uint32_t)(~(uint32_t)i);
            }
        } else {
            for_chunks([&](int e, uint32_t k) {
                const int i = e * kSortThreads + tid;
                const bool gt = k > thr && k != 0u;
                const bool eq = k == thr && k != 0u;
                int total;
                const int before = scan1024((gt ? 1 : 0) | (eq ? 1 << 16 : 0), wsum, &total);
                const int eq_rank = eq_before + (before >> 16);
                int slot = -1;
                if (gt) slot = gt_before + (before & 0xffff);
                else if (eq && eq_rank < need) slot = n_gt + eq_rank;
                if (slot >= 0) win[slot] = ((unsigned long long)k << 32) | (uint32_t)(~(uint32_t)i);
                gt_before += total & 0xffff;
                eq_before += total >> 16;
            });
        }
    }
    __syncthreads();

    // ---- order the winners, descending: larger key first, then smaller position ----
    // Fast path: the winners' keys lie in [thr, kmax]; 1024 equal-width buckets over that range
    // (descending), a prefix sum over the bucket counts, every winner dropped into its bucket,
    // then ranked among the few entries that share it.  Six barriers and a handful of LDS accesses
    // per entry.  A bucket of more than kBucketMax entries (many equal or tightly clustered scores)
    // sends the row down the general path below.
    constexpr int kPer = kMaxTopk / kSortThreads;  // entries per thread at the largest cap
    uint32_t kmax_part = 0u;
    unsigned long long x[kPer];
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
        const int i = tid + e * kSortThreads;
        x[e] = i < kk ? win[i] : 0ull;
        const uint32_t k = (uint32_t)(x[e] >> 32);
        kmax_part = k > kmax_part ? k : kmax_part;
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const uint32_t other = (uint32_t)__shfl_xor((int)kmax_part, o);
        kmax_part = other > kmax_part ? other : kmax_part;
    }
    if (tid < kBuckets) {
        bcount[tid] = 0;
        bfill[tid] = 0;
    }
    if (lane == 0) wsum[tid >> 6] = (int)kmax_part;
    __syncthreads();
    uint32_t kmax = 0u;
    for (int w = 0; w < kSortThreads / 64; ++w) kmax = (uint32_t)wsum[w] > kmax ? (uint32_t)wsum[w] : kmax;
    const uint32_t range = kmax > thr ? kmax - thr : 0u;
    const int bits = range ? 32 - __builtin_clz(range) : 0;
    const int bshift = bits > 10 ? bits - 10 : 0;
    int bucket[kPer];
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
        const int i = tid + e * kSortThreads;
        bucket[e] = -1;
        if (i < kk) {
            bucket[e] = (kBuckets - 1) - (int)(((uint32_t)(x[e] >> 32) - thr) >> bshift);
            atomicAdd(&bcount[bucket[e]], 1);
        }
    }
    __syncthreads();
    const int my_count = tid < kBuckets ? bcount[tid] : 0;
    int all_winners;
    const int my_base = scan1024(my_count, wsum, &all_winners);
    const bool crowded = __syncthreads_or(my_count > kBucketMax);
    if (!crowded) {
        if (tid < kBuckets) bbase[tid] = my_base;
        __syncthreads();
#pragma unroll
        for (int e = 0; e < kPer; ++e)
            if (bucket[e] >= 0) win[bbase[bucket[e]] + atomicAdd(&bfill[bucket[e]], 1)] = x[e];
        __syncthreads();
        int dst[kPer];
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
            dst[e] = -1;
            if (bucket[e] >= 0) {
                const int first = bbase[bucket[e]], n = bcount[bucket[e]];
                int ahead = 0;  // entries of the bucket that go before this one
                for (int j = 0; j < n; ++j) ahead += win[first + j] > x[e];
                dst[e] = first + ahead;
            }
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < kPer; ++e)
            if (dst[e] >= 0) win[dst[e]] = x[e];
        __syncthreads();
    } else {
        // General path:
        // (a) bitonic networks over aligned segments of 256 entries, every segment descending;
        // (b) sorted runs merged pairwise: an entry's place in the merged run is its place in its
        //     own run plus the number of entries of the sibling run that go before it (binary
        //     search; the left run wins ties, which only the empty slots have).  For 4096 entries
        //     that is 36 + 2 * 4 barriers where one network over everything takes 78.
        const int seg = a.cap < 256 ? a.cap : 256;
        for (int size = 2; size <= seg; size <<= 1) {
            for (int stride = size >> 1; stride > 0; stride >>= 1) {
                for (int t = tid; t < a.cap / 2; t += kSortThreads) {
                    const int lo = 2 * t - (t & (stride - 1));
                    const int hi = lo + stride;
                    const bool desc = size == seg || (lo & size) == 0;
                    const unsigned long long p = win[lo], q = win[hi];
                    if ((p < q) == desc) {
                        win[lo] = q;
                        win[hi] = p;
                    }
                }
                __syncthreads();
            }
        }
        for (int run = seg; run < a.cap; run <<= 1) {
            int dst[kPer];
            const int sh = __builtin_ctz(run);
#pragma unroll
            for (int e = 0; e < kPer; ++e) {
                const int i = tid + e * kSortThreads;
                dst[e] = -1;
                if (i < a.cap) {
                    x[e] = win[i];
                    const int r = i >> sh, at = i & (run - 1);
                    const unsigned long long* sib = win + (r ^ 1) * run;
                    const bool left = (r & 1) == 0;
                    int lo = 0, hi = run;  // entries of the sibling run that go before x[e]
                    while (lo < hi) {
                        const int mid = (lo + hi) >> 1;
                        const unsigned long long o = sib[mid];
                        if (o > x[e] || (!left && o == x[e])) lo = mid + 1;
                        else hi = mid;
                    }
                    dst[e] = (r >> 1) * 2 * run + at + lo;
                }
            }
            __syncthreads();
#pragma unroll
            for (int e = 0; e < kPer; ++e)
                if (dst[e] >= 0) win[dst[e]] = x[e];
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
// position — one comparison of (key, ~position) pairs) and writes itself at that rank.  No
// search and no sort.  The 1024 threads share the work: P = 1024 / n (rounded down to a power
// of two, at most 64) neighbouring lanes split one candidate's comparisons and add their counts
// with shuffles.  Same output as topk_sort_kernel.
__global__ __launch_bounds__(kSortThreads) void topk_rank_kernel(SortArgs a)
{
    __shared__ __align__(16) unsigned long long c_lds[kSortThreads];
    const int b = blockIdx.x, tid = threadIdx.x;
    const uint32_t* keys = a.keys + (int64_t)b * a.max_n;
    {
        const uint32_t k = tid < a.max_n ? keys[tid] : 0u;
        c_lds[tid] = k ? ((unsigned long long)k << 32) | (uint32_t)(~(uint32_t)tid) : 0ull;
    }
    for (int t = tid; t < a.topk; t += kSortThreads) {  // slots no candidate reaches
        a.out_idx[(int64_t)b * a.topk + t] = -1;
        a.out_score[(int64_t)b * a.topk + t] = 0.0f;
    }
    __syncthreads();  // also orders the fill above before the winners' writes below
    int shift = 0;    // P = 1 << shift lanes per candidate
    while (shift < 6 && (a.max_n << (shift + 1)) <= kSortThreads) ++shift;
    const int cand = tid >> shift, part = tid & ((1 << shift) - 1);
    const int span = (((a.max_n + (1 << shift) - 1) >> shift) + 1) & ~1;  // even: 16-byte reads
    const unsigned long long mine = cand < a.max_n ? c_lds[cand] : 0ull;
    int rank = 0;
    const int j0 = part * span;
    int j1 = j0 + span;
    j1 = j1 < a.max_n ? j1 : a.max_n;
    for (int j = j0; j + 1 < j1; j += 2) {
        const ulonglong2 o = *reinterpret_cast<const ulonglong2*>(c_lds + j);
        rank += (o.x > mine) + (o.y > mine);
    }
    if (j0 < j1 && ((j1 - j0) & 1)) rank += c_lds[j1 - 1] > mine;
    for (int o = 1; o < (1 << shift); o <<= 1) rank += __shfl_xor(rank, o);
    if (part == 0 && mine != 0ull && rank < a.topk) {
        a.out_idx[(int64_t)b * a.topk + rank] = a.idx[(int64_t)b * a.max_n + cand];
        a.out_score[(int64_t)b * a.topk + rank] = a.scores[(int64_t)b * a.max_n + cand];
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
    if (s.max_n <= kRegKeys * kSortThreads)
        hipLaunchKernelGGL(topk_sort_kernel<true>, dim3((unsigned)rows), dim3(kSortThreads), (size_t)cap * 8, st, s);
    else
        hipLaunchKernelGGL(topk_sort_kernel<false>, dim3((unsigned)rows), dim3(kSortThreads), (size_t)cap * 8, st, s);
    return ucm::launch_status("topk_sort_kernel");
}

}  // namespace
