// KVStar block retrieval for gfx950: attention-probability mass per KV block, then top-k.
//
// GPU counterpart of the reference's CPU kernel
// (ucm/sparse/kvstar/retrieve/core/domain/retrieve_task/simd_compute_kernel.cpp:816-985, the
// scalar form; its NEON / AVX forms compute the same quantities in other summation orders):
//   1. optional channel pruning of the queries: q'[x, H, j] = q[x, H, pruned_index[H / g, j]];
//   2. scores[x, H, s] = q'[x, H, :] . k[s, H / g, :] over the S = n_blocks * M block
//      representatives, fp16 inputs, fp32 accumulation;
//   3. softmax over s for every (x, H) (left unnormalised when the sum of exponentials is
//      <= 1e-9, as the reference does);
//   4. block score[n] = sum over x, H and the M representatives of block n;
//   5. the topk blocks by descending score.
// Kernels: qk_score_kernel (one thread per (s, kv head), the head's query rows broadcast from
// LDS, K read once: the HBM-bound part), row_stats_kernel (max and sum of exponentials per
// (x, H) row), block_mass_kernel (probabilities summed over rows in a fixed order, then over a
// block's representatives: deterministic, no atomics) and the shared top-k selection.
// Sums are taken in a different order than the reference's loops; the tolerance is stated
// where the results are compared.  Equal scores come out in ascending block order (the
// reference's heap pops them in descending block order).
#include <hip/hip_fp16.h>

#include "common.h"
#include "float_topk.h"

namespace {

constexpr int kQkThreads = 256;  // the matrix-core kernel stages 32 query rows with 8 threads each
constexpr int kStatThreads = 1024;
constexpr int kRowTile = 16;  // query rows of one KV head scored per pass over a K vector

struct QkArgs {
    const __half* q;        // [X, Hq, d_orig]
    const __half* k;        // [S, Hkv, d]
    const int64_t* pruned;  // [Hkv, d] or null
    int X, Hq, Hkv, g, d_orig, d;
    int64_t S;
    float* scores;          // [X * Hq, S]
};

// grid = (ceil(S / 256), Hkv, ceil(X * g / kRowTile)); LDS: kRowTile rows of d floats
__global__ __launch_bounds__(kQkThreads) void qk_score_kernel(QkArgs a)
{
    extern __shared__ __align__(16) float qs[];  // [kRowTile][d]
    __shared__ int orow[kRowTile];               // score row x * Hq + H of each query row, -1 = none
    const int h = blockIdx.y;
    const int row0 = blockIdx.z * kRowTile;  // first (x, gg) pair of this pass
    const int rows = a.X * a.g;
    if (threadIdx.x < kRowTile) {
        const int rr = row0 + threadIdx.x;
        orow[threadIdx.x] = rr < rows ? (rr / a.g) * a.Hq + h * a.g + rr % a.g : -1;
    }
    // stage the pass's query rows of KV head h: row r = x * g + gg  <->  q head H = h * g + gg
    for (int i = threadIdx.x; i < kRowTile * a.d; i += kQkThreads) {
        const int r = row0 + i / a.d, j = i % a.d;
        float v = 0.0f;
        if (r < rows) {
            const int x = r / a.g, H = h * a.g + r % a.g;
            int64_t src = a.pruned ? a.pruned[(int64_t)h * a.d + j] : j;
            src = src < 0 ? 0 : (src >= a.d_orig ? a.d_orig - 1 : src);  // stay inside the row
            v = __half2float(a.q[((int64_t)x * a.Hq + H) * a.d_orig + src]);
        }
        qs[i] = v;
    }
    __syncthreads();
    const int64_t s = (int64_t)blockIdx.x * kQkThreads + threadIdx.x;
    if (s >= a.S) return;
    const __half* kv = a.k + (s * a.Hkv + h) * a.d;
    float acc[kRowTile];
#pragma unroll
    for (int r = 0; r < kRowTile; ++r) acc[r] = 0.0f;
    if ((a.d & 7) == 0) {  // 16-byte pieces of the K vector
        for (int j = 0; j < a.d; j += 8) {
            const uint4 raw = *reinterpret_cast<const uint4*>(kv + j);
            __half hv[8];
            __builtin_memcpy(hv, &raw, 16);
            float kf[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) kf[i] = __half2float(hv[i]);
#pragma unroll
            for (int r = 0; r < kRowTile; ++r) {  // 16-byte LDS reads, the same address in all lanes
                const float4 qa = *reinterpret_cast<const float4*>(qs + r * a.d + j);
                const float4 qb = *reinterpret_cast<const float4*>(qs + r * a.d + j + 4);
                float t = acc[r];
                t = __builtin_fmaf(qa.x, kf[0], t);
                t = __builtin_fmaf(qa.y, kf[1], t);
                t = __builtin_fmaf(qa.z, kf[2], t);
                t = __builtin_fmaf(qa.w, kf[3], t);
                t = __builtin_fmaf(qb.x, kf[4], t);
                t = __builtin_fmaf(qb.y, kf[5], t);
                t = __builtin_fmaf(qb.z, kf[6], t);
                t = __builtin_fmaf(qb.w, kf[7], t);
                acc[r] = t;
            }
        }
    } else {
        for (int j = 0; j < a.d; ++j) {
            const float kf = __half2float(kv[j]);
#pragma unroll
            for (int r = 0; r < kRowTile; ++r) acc[r] = __builtin_fmaf(qs[r * a.d + j], kf, acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < kRowTile; ++r) {
        const int o = orow[r];
        if (o >= 0) a.scores[(int64_t)o * a.S + s] = acc[r];
    }
}

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// q.k on the matrix cores for head dims that are multiples of 16: one workgroup per (128
// representatives, KV head, 32 query rows); the query tile (channel-pruned) is gathered once
// into LDS, then each wave takes 32 representatives: d / 16 v_mfma_f32_32x32x16_f16 with the
// query tile as the A operand (lane: row lane % 32, eight channels of the k-step, one 16-byte
// LDS read) and the representatives as the B operand (one 16-byte global load per lane and
// k-step).  Accumulator v of a lane is
// score[row 8 (v / 4) + 4 (lane / 32) + v % 4][representative lane % 32]: lanes 0..31 store 32
// consecutive floats of one score row.  grid = (ceil(S / 128), Hkv, ceil(X g / 32));
// LDS = 32 rows of (d + 8) halves.
__global__ __launch_bounds__(kQkThreads) void qk_mfma_kernel(QkArgs a)
{
    extern __shared__ __align__(16) _Float16 qt[];  // [32][d + 8]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = blockIdx.y;
    const int rows = a.X * a.g;
    const int dp = a.d + 8;  // row pitch: 16 bytes of padding spread the rows over the banks
    const _Float16* q = reinterpret_cast<const _Float16*>(a.q);
    {
        // eight threads per query row, each taking every eighth channel: one division per thread
        const int rl = threadIdx.x >> 3;
        const int rr = blockIdx.z * 32 + rl;
        const bool ok = rr < rows;
        const _Float16* qrow = q + ((int64_t)(ok ? rr / a.g : 0) * a.Hq + h * a.g + (ok ? rr % a.g : 0)) * a.d_orig;
        for (int j = threadIdx.x & 7; j < a.d; j += 8) {
            int64_t src = a.pruned ? a.pruned[(int64_t)h * a.d + j] : j;
            src = src < 0 ? 0 : (src >= a.d_orig ? a.d_orig - 1 : src);  // stay inside the row
            qt[rl * dp + j] = ok ? qrow[src] : (_Float16)0;
        }
    }
    __syncthreads();
    const int64_t s0 = ((int64_t)blockIdx.x * (kQkThreads / 64) + wave) * 32;
    if (s0 >= a.S) return;  // wave-uniform, after the only barrier
    int64_t s = s0 + (lane & 31);
    const bool s_ok = s < a.S;
    if (!s_ok) s = a.S - 1;
    const int kb = (lane >> 5) * 8;  // channels kb .. kb + 7 of a k-step
    const __half* kv = a.k + (s * a.Hkv + h) * a.d + kb;
    const _Float16* qa_row = qt + (lane & 31) * dp + kb;
    f32x16 acc = {0};
    for (int c = 0; c < a.d; c += 16) {
        const f16x8 qa = *reinterpret_cast<const f16x8*>(qa_row + c);
        const f16x8 kk = *reinterpret_cast<const f16x8*>(kv + c);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa, kk, acc, 0, 0, 0);
    }
    // score row of query row lane % 32 (one division per lane, handed round by shuffles:
    // sixteen divisions per lane in the store loop cost more than the matrix products)
    const int r = blockIdx.z * 32 + (lane & 31);
    const int orow = r < rows ? (r / a.g) * a.Hq + h * a.g + r % a.g : -1;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int o = __shfl(orow, 8 * (v / 4) + 4 * (lane >> 5) + (v % 4));
        if (s_ok && o >= 0) a.scores[(int64_t)o * a.S + s] = acc[v];
    }
}

// Running (max, sum of exp(x - max)) pairs merge associatively; a side that has seen nothing
// carries max = -inf and sum = 0.
__device__ __forceinline__ void merge_stats(float& m, float& sum, float om, float osum)
{
    const float nm = fmaxf(m, om);
    if (nm == -INFINITY) return;
    sum = sum * expf(m - nm) + osum * expf(om - nm);
    m = nm;
}

// One workgroup per (x, H) row: max over s and sum of exp(score - max), in one pass over the
// row (eight loads in flight per thread, running pairs merged at the end).
__global__ __launch_bounds__(kStatThreads) void row_stats_kernel(const float* __restrict__ scores,
                                                                 int64_t S, float* __restrict__ stats)
{
    __shared__ float red_m[kStatThreads / 64], red_s[kStatThreads / 64];
    const float* row = scores + (int64_t)blockIdx.x * S;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    float m = -INFINITY, sum = 0.0f;
    for (int64_t base = threadIdx.x; base < S; base += 8 * kStatThreads) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int64_t s = base + (int64_t)i * kStatThreads;
            v[i] = s < S ? row[s] : -INFINITY;
        }
        float cm = v[0];
#pragma unroll
        for (int i = 1; i < 8; ++i) cm = fmaxf(cm, v[i]);
        if (cm == -INFINITY) continue;
        float cs = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) cs += expf(v[i] - cm);
        merge_stats(m, sum, cm, cs);
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) merge_stats(m, sum, __shfl_xor(m, o), __shfl_xor(sum, o));
    if (lane == 0) {
        red_m[w] = m;
        red_s[w] = sum;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float tm = red_m[0], ts = red_s[0];
        for (int i = 1; i < kStatThreads / 64; ++i) merge_stats(tm, ts, red_m[i], red_s[i]);
        stats[2 * blockIdx.x] = tm;
        // the reference normalises only when the sum exceeds 1e-9
        stats[2 * blockIdx.x + 1] = ts > 1e-9f ? 1.0f / ts : 1.0f;
    }
}

// One workgroup per block n: probabilities of its M representatives summed over all rows, in a
// fixed order (strided partial sums, xor-shuffle tree, then the waves in turn).
__global__ __launch_bounds__(kStatThreads) void block_mass_kernel(const float* __restrict__ scores,
                                                                  const float* __restrict__ stats,
                                                                  int rows, int64_t S, int M,
                                                                  float* __restrict__ mass,
                                                                  uint32_t* __restrict__ keys,
                                                                  int32_t* __restrict__ ident)
{
    __shared__ float red[kStatThreads / 64];
    const int64_t n = blockIdx.x;
    const float* base = scores + n * M;
    const int total = rows * M;
    float part = 0.0f;
    // element e = r * M + m; e advances by the workgroup size: (r, m) follow without a division
    const int dr = kStatThreads / M, dm = kStatThreads % M;
    int r = threadIdx.x / M, m = threadIdx.x % M;
#pragma unroll 4
    for (int e = threadIdx.x; e < total; e += kStatThreads) {
        part += expf(base[(int64_t)r * S + m] - stats[2 * r]) * stats[2 * r + 1];
        r += dr;
        m += dm;
        if (m >= M) {
            m -= M;
            ++r;
        }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) part += __shfl_xor(part, o);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = part;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.0f;
        for (int i = 0; i < kStatThreads / 64; ++i) t += red[i];
        mass[n] = t;
        keys[n] = score_key(t);
        ident[n] = (int32_t)n;
    }
}

size_t align256k(size_t v) { return (v + 255) & ~(size_t)255; }

struct KvstarWs {
    float* scores;
    float* stats;
    float* mass;
    uint32_t* keys;
    int32_t* ident;
    size_t bytes;
};

KvstarWs carve_kvstar(void* base, int64_t rows, int64_t S, int64_t n_blocks)
{
    KvstarWs w{};
    size_t off = 0;
    w.scores = (float*)((char*)base + off);
    off += align256k((size_t)rows * S * 4);
    w.stats = (float*)((char*)base + off);
    off += align256k((size_t)rows * 8);
    w.mass = (float*)((char*)base + off);
    off += align256k((size_t)n_blocks * 4);
    w.keys = (uint32_t*)((char*)base + off);
    off += align256k((size_t)n_blocks * 4);
    w.ident = (int32_t*)((char*)base + off);
    off += align256k((size_t)n_blocks * 4);
    w.bytes = off;
    return w;
}

}  // namespace

extern "C" size_t ucm_kvstar_topk_workspace_bytes(int32_t X, int32_t Hq, int64_t n_blocks, int32_t M)
{
    if (X <= 0 || Hq <= 0 || n_blocks <= 0 || M <= 0) return 256;
    return carve_kvstar(nullptr, (int64_t)X * Hq, n_blocks * M, n_blocks).bytes;
}

extern "C" int ucm_kvstar_topk(const void* query, int32_t X, int32_t Hq, int32_t d_orig,
                               const void* blk_repre, int64_t n_blocks, int32_t M, int32_t Hkv,
                               int32_t d, const int64_t* pruned_index, int32_t topk,
                               int32_t* out_idx, float* out_score, void* workspace,
                               size_t workspace_bytes, ucm_stream_t stream)
{
    ucm::clear_error();
    UCM_REQUIRE(query && blk_repre && out_idx && out_score, "null pointer");
    UCM_REQUIRE(X > 0 && Hq > 0 && Hkv > 0 && d > 0 && d_orig > 0 && n_blocks > 0 && M > 0,
                "non-positive shape");
    UCM_REQUIRE(Hq % Hkv == 0, "Num_q_heads must be a divisible by num_kv_heads.");
    UCM_REQUIRE(pruned_index || d == d_orig,
                "Dimension mismatch: No dPrunedIndex, but Q and K head dims differ.");
    UCM_REQUIRE(topk > 0, "topk %d must be positive", topk);
    if (topk > kMaxTopk) return ucm::fail(UCM_EUNSUPPORTED, "topk %d above %d", topk, kMaxTopk);
    UCM_REQUIRE((size_t)kRowTile * d * 4 <= 64 * 1024, "head dim %d above 1024", d);
    UCM_REQUIRE(n_blocks <= INT32_MAX && n_blocks * M <= INT32_MAX, "too many block representatives");
    const int64_t rows = (int64_t)X * Hq, S = n_blocks * M;
    UCM_REQUIRE(rows <= 65535 && rows * M <= INT32_MAX, "too many query rows");
    UCM_REQUIRE(workspace && workspace_bytes >= ucm_kvstar_topk_workspace_bytes(X, Hq, n_blocks, M),
                "workspace too small");
    UCM_REQUIRE((((uintptr_t)blk_repre | (uintptr_t)workspace) & 15) == 0, "block representatives must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const KvstarWs w = carve_kvstar(workspace, rows, S, n_blocks);
    QkArgs a{};
    a.q = (const __half*)query; a.k = (const __half*)blk_repre; a.pruned = pruned_index;
    a.X = X; a.Hq = Hq; a.Hkv = Hkv; a.g = Hq / Hkv; a.d_orig = d_orig; a.d = d; a.S = S;
    a.scores = w.scores;
    const dim3 grid((unsigned)ucm::ceil_div(S, kQkThreads), (unsigned)Hkv,
                    (unsigned)ucm::ceil_div((int64_t)X * a.g, kRowTile));
    UCM_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "too many heads or query rows");
    int rc;
    if (d % 16 == 0 && d <= 512) {
        const dim3 mgrid((unsigned)ucm::ceil_div(S, 32 * (kQkThreads / 64)), (unsigned)Hkv,
                         (unsigned)ucm::ceil_div((int64_t)X * a.g, 32));
        UCM_REQUIRE(mgrid.z <= 65535, "too many query rows");
        hipLaunchKernelGGL(qk_mfma_kernel, mgrid, dim3(kQkThreads), (size_t)32 * (d + 8) * 2, st, a);
        rc = ucm::launch_status("qk_mfma_kernel");
    } else {
        hipLaunchKernelGGL(qk_score_kernel, grid, dim3(kQkThreads), (size_t)kRowTile * d * 4, st, a);
        rc = ucm::launch_status("qk_score_kernel");
    }
    if (rc != UCM_OK) return rc;
    hipLaunchKernelGGL(row_stats_kernel, dim3((unsigned)rows), dim3(kStatThreads), 0, st, w.scores, S, w.stats);
    rc = ucm::launch_status("row_stats_kernel");
    if (rc != UCM_OK) return rc;
    hipLaunchKernelGGL(block_mass_kernel, dim3((unsigned)n_blocks), dim3(kStatThreads), 0, st, w.scores,
                       w.stats, (int)rows, S, (int)M, w.mass, w.keys, w.ident);
    rc = ucm::launch_status("block_mass_kernel");
    if (rc != UCM_OK) return rc;
    SortArgs s{};
    s.keys = w.keys; s.scores = w.mass; s.idx = w.ident; s.max_n = (int)n_blocks; s.topk = topk;
    s.out_idx = out_idx; s.out_score = out_score;
    return launch_topk_sort(s, 1, st);
}
