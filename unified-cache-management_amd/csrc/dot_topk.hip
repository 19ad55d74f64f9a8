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
#include "float_topk.h"

namespace {

constexpr int kDotThreads = 256;
constexpr int kRowsPerWave = 4;

typedef float f32x4 __attribute__((ext_vector_type(4)));

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
    // the wave's candidates first, then their rows chunk by chunk with all of the wave's rows in
    // flight together: two round trips to memory instead of two per row
    int item[kRowsPerWave];
    bool ok[kRowsPerWave];
    const float* row[kRowsPerWave];
    float acc[kRowsPerWave];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int j = first + r;
        item[r] = j < a.max_n ? a.idx[(int64_t)b * a.max_n + j] : -1;
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        ok[r] = item[r] >= 0 && item[r] < a.n_items;
        row[r] = a.data + (int64_t)(ok[r] ? item[r] : 0) * a.dim;  // row 0 stands in: always readable
        acc[r] = 0.0f;
    }
    if (vec) {
        for (int c = lane * 4; c < a.dim; c += 256) {
            f32x4 x[kRowsPerWave];
#pragma unroll
            for (int r = 0; r < kRowsPerWave; ++r)
                x[r] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(row[r] + c));
            const f32x4 y = *reinterpret_cast<const f32x4*>(qs + c);
#pragma unroll
            for (int r = 0; r < kRowsPerWave; ++r) {
                acc[r] = __builtin_fmaf(x[r].x, y.x, acc[r]);
                acc[r] = __builtin_fmaf(x[r].y, y.y, acc[r]);
                acc[r] = __builtin_fmaf(x[r].z, y.z, acc[r]);
                acc[r] = __builtin_fmaf(x[r].w, y.w, acc[r]);
            }
        }
    } else {
        for (int c = lane; c < a.dim; c += 64) {
#pragma unroll
            for (int r = 0; r < kRowsPerWave; ++r) acc[r] = __builtin_fmaf(row[r][c], qs[c], acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        float t = acc[r];
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) t += __shfl_xor(t, s);
        const int j = first + r;
        if (lane == 0 && j < a.max_n) {
            a.scores[(int64_t)b * a.max_n + j] = ok[r] ? t : 0.0f;
            a.keys[(int64_t)b * a.max_n + j] = ok[r] ? score_key(t) : 0u;
        }
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
    s.out_idx = out_idx; s.out_score = out_score;
    return launch_topk_sort(s, B, st);
}
