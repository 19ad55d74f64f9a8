/*
 * ucm_oracle.c — CPU restatement of the reference's sparse-retrieval / KV-transfer
 * arithmetic.  TEST INFRASTRUCTURE ONLY: it is the checker that the HIP library is
 * compared against (tests, the smoke check, and the CPU-baseline leg of the benchmark).
 * Nothing in the shipped library calls into this file.
 *
 * Each function names the reference lines it restates (paths relative to the reference
 * checkout).  Plain C, scalar loops; the *_mt entry uses pthreads with one thread per
 * request, which is the reference CPU backend's execution model
 * (ucm/sparse/gsa_on_device/csrc/cuda/hash_retrieval/cpy/hash_retrieval_backend.cpp:180-199,338).
 */
#define _GNU_SOURCE
#include <limits.h>
#include <math.h>
#include <pthread.h>
#include <sched.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_INF INT32_MAX

static inline int popc32(uint32_t v) { return __builtin_popcount(v); }

/* ------------------------------------------------------------------------------------
 * Encoder.  ucm/sparse/gsa_on_device/hash_encoder.py:359-370 (torch_hash_code):
 *   p = x @ W ; bit = p > 0 ; byte j = sum_i bit[8j+i] << i.
 * x [M,K] fp32 (callers widen bf16/fp16 exactly), W [K,N] fp32.
 * acc_f64 = 0: fp32 accumulation in ascending k; 1: fp64 accumulation.
 * margin (optional, [M,N]) = |p| / ||x_row||_2, used by tests for the tolerance rule.
 * ------------------------------------------------------------------------------------ */
void oracle_hash_encode(const float* x, int64_t M, int32_t K, const float* W, int32_t N,
                        int acc_f64, uint32_t* codes, float* margin)
{
    const int32_t Wd = N / 32;
    for (int64_t m = 0; m < M; ++m) {
        const float* xr = x + m * K;
        double nrm2 = 0.0;
        for (int32_t k = 0; k < K; ++k) nrm2 += (double)xr[k] * (double)xr[k];
        const double nrm = sqrt(nrm2);
        for (int32_t w = 0; w < Wd; ++w) codes[m * Wd + w] = 0u;
        for (int32_t n = 0; n < N; ++n) {
            double p;
            if (acc_f64) {
                double a = 0.0;
                for (int32_t k = 0; k < K; ++k) a += (double)xr[k] * (double)W[(int64_t)k * N + n];
                p = a;
            } else {
                float a = 0.0f;
                for (int32_t k = 0; k < K; ++k) a += xr[k] * W[(int64_t)k * N + n];
                p = (double)a;
            }
            if (p > 0.0) codes[m * Wd + (n >> 5)] |= 1u << (n & 31);
            if (margin) margin[m * N + n] = nrm > 0.0 ? (float)(fabs(p) / nrm) : 0.0f;
        }
    }
}

/*
 * Fused encode + paged store.  hash_encoder.py:263-356 (fused_hash_and_cache_kernel):
 * row (t,h) is encoded with W[min(h / heads_per_w, n_w-1)] and stored at
 * cache[slot/BS, slot%BS, h, :]; slots < 0 or >= NB*BS are skipped (:338-344).
 * x [T,H,K] fp32 contiguous, W [n_w,K,N]; cache strides in 32-bit words.
 */
void oracle_hash_encode_cache(const float* x, int64_t T, int32_t H, int32_t K, const float* W,
                              int32_t n_w, int32_t heads_per_w, int32_t N, const int64_t* slot,
                              uint32_t* cache, int64_t NB, int32_t BS, int64_t cs_block,
                              int64_t cs_token, int64_t cs_head)
{
    const int32_t Wd = N / 32;
    uint32_t* tmp = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)Wd);
    for (int64_t t = 0; t < T; ++t) {
        const int64_t s = slot[t];
        if (s < 0 || s >= NB * (int64_t)BS) continue;
        for (int32_t h = 0; h < H; ++h) {
            int32_t wi = heads_per_w > 0 ? h / heads_per_w : 0;
            if (wi > n_w - 1) wi = n_w - 1;
            oracle_hash_encode(x + (t * H + h) * (int64_t)K, 1, K, W + (int64_t)wi * K * N, N, 0,
                               tmp, NULL);
            uint32_t* dst = cache + (s / BS) * cs_block + (s % BS) * cs_token + h * cs_head;
            memcpy(dst, tmp, sizeof(uint32_t) * (size_t)Wd);
        }
    }
    free(tmp);
}

/*
 * Prefix-cache rehash.  gsa_on_device.py:574-588: the key blocks `block_ids` are gathered from
 * the paged KV cache (kv_cache[0][0][prefix_block_ids], reshaped to [-1, H, K]), the first
 * n_tokens rows are encoded and stored with the prefix slot mapping, which
 * rebuild_prefix_cache_info_for_req (:1142-1174) builds as
 *     slot(i) = block_ids[i / BS] * BS + i % BS.
 * k_cache [NBk,BS,H,K] fp32 contiguous.  A block id outside either cache drops its rows (the
 * reference would fault on the gather; the slot test of :338-344 covers the code cache side).
 */
void oracle_hash_encode_paged(const float* k_cache, int64_t NBk, int32_t BS, int32_t H, int32_t K,
                              const int32_t* block_ids, int64_t n_tokens, const float* W,
                              int32_t n_w, int32_t heads_per_w, int32_t N, uint32_t* cache,
                              int64_t NB, int64_t cs_block, int64_t cs_token, int64_t cs_head)
{
    for (int64_t i = 0; i < n_tokens; ++i) {
        const int64_t blk = block_ids[i / BS];
        if (blk < 0 || blk >= NBk || blk >= NB) continue;
        const int64_t slot = blk * BS + i % BS;
        const float* row = k_cache + (blk * BS + i % BS) * (int64_t)H * K;  /* the gathered row i */
        oracle_hash_encode_cache(row, 1, H, K, W, n_w, heads_per_w, N, &slot, cache, NB, BS,
                                 cs_block, cs_token, cs_head);
    }
}

/* Scatter of precomputed codes.  hash_encoder.py:136-195 (_reshape_and_cache_khash_kernel). */
void oracle_code_scatter(const uint32_t* codes, int64_t T, int32_t H, int32_t Wd,
                         const int64_t* slot, uint32_t* cache, int64_t NB, int32_t BS,
                         int64_t cs_block, int64_t cs_token, int64_t cs_head)
{
    for (int64_t t = 0; t < T; ++t) {
        const int64_t s = slot[t];
        if (s < 0 || s >= NB * (int64_t)BS) continue;
        for (int32_t h = 0; h < H; ++h)
            memcpy(cache + (s / BS) * cs_block + (s % BS) * cs_token + h * cs_head,
                   codes + (t * H + h) * (int64_t)Wd, sizeof(uint32_t) * (size_t)Wd);
    }
}

/* ------------------------------------------------------------------------------------
 * Scorer.
 * ------------------------------------------------------------------------------------ */

/* Group-summed Hamming distance of one cached token against the G query heads of KV head
 * h.  csrc/cuda/ham_dist/paged_ham_dist_mla.cu:172-178 (the KVGroup loop). */
static int32_t group_distance(const uint32_t* q_bh, int64_t q_stride_h, int32_t G,
                              const uint32_t* kcode, int32_t Wd)
{
    int32_t d = 0;
    for (int32_t g = 0; g < G; ++g)
        for (int32_t w = 0; w < Wd; ++w) d += popc32(q_bh[g * q_stride_h + w] ^ kcode[w]);
    return d;
}

/*
 * Per-token distances in the reference scorer's output shape.
 * paged_ham_dist_mla.cu:148-247: out[b,h,p] = distance; 0 if p < sink or
 * len-recent <= p < len; INF if p >= len (:194-197,213-214,243-244); with reduce_heads the
 * min over KV heads is written to out[b,0,p] (:203-211).
 * The cache is addressed [block, token, head] through explicit strides.
 * out int32 [B, (reduce ? 1 : Hkv), max_seq_len].
 */
void oracle_hamming_score(const uint32_t* q, int64_t q_stride_b, int64_t q_stride_h,
                          const uint32_t* kc, int64_t NB, int32_t BS, int32_t Hkv, int32_t Wd,
                          int64_t ks_block, int64_t ks_token, int64_t ks_head,
                          const int32_t* table, int32_t table_stride, int32_t max_blocks,
                          const int32_t* lens, int32_t B, int32_t Hq, int32_t max_seq_len,
                          int32_t sink, int32_t recent, int reduce_heads, int32_t* out)
{
    const int32_t G = Hq / Hkv;
    const int32_t Ho = reduce_heads ? 1 : Hkv;
    for (int32_t b = 0; b < B; ++b) {
        const int32_t len = lens[b];
        for (int32_t p = 0; p < max_seq_len; ++p) {
            const int32_t j = p / BS, t = p % BS;
            const int is_inf = p >= len;
            const int keep = (p < sink) || (p >= len - recent && p < len);
            int32_t red = ORACLE_INF;
            for (int32_t h = 0; h < Hkv; ++h) {
                int32_t v;
                if (is_inf) {
                    v = ORACLE_INF;
                } else if (keep) {
                    v = 0;
                } else {
                    const int64_t pb = table ? table[(int64_t)b * table_stride + j]
                                             : (int64_t)b * max_blocks + j;
                    if (pb < 0 || pb >= NB) {
                        v = ORACLE_INF;
                    } else {
                        v = group_distance(q + b * q_stride_b + (int64_t)h * G * q_stride_h,
                                           q_stride_h, G,
                                           kc + pb * ks_block + t * ks_token + h * ks_head, Wd);
                    }
                }
                if (reduce_heads) {
                    if (v < red) red = v;
                } else {
                    out[((int64_t)b * Ho + h) * max_seq_len + p] = v;
                }
            }
            if (reduce_heads) out[(int64_t)b * max_seq_len + p] = red;
        }
    }
}

/* flag bits, same values as the library's UCM_TOPK_* */
#define F_REDUCE_HEADS 1u
#define F_PHYSICAL 2u
#define F_SCORE_ORDER 4u
#define F_DISTANCE 8u

typedef struct {
    int32_t score;
    int32_t idx;
} cand_t;

/* (score desc, index asc): the deterministic order that fixes the reference's unspecified
 * ties (torch.topk in hamming_topk.py:49-51; std::partial_sort on .first only in
 * hash_retrieval_backend.cpp:396-400). */
static int cand_cmp(const void* a, const void* b)
{
    const cand_t* x = (const cand_t*)a;
    const cand_t* y = (const cand_t*)b;
    if (x->score != y->score) return x->score > y->score ? -1 : 1;
    return x->idx < y->idx ? -1 : (x->idx > y->idx ? 1 : 0);
}
static int idx_cmp(const void* a, const void* b)
{
    const cand_t* x = (const cand_t*)a;
    const cand_t* y = (const cand_t*)b;
    return x->idx < y->idx ? -1 : (x->idx > y->idx ? 1 : 0);
}

/*
 * Block scores of one request: s[h][j], j < nblk.
 * Block reduction = min distance over the block's valid tokens (hamming_topk.py:45-47)
 * restated as max similarity G*bits - d (the NPU op's form,
 * csrc/ascend/hamming_dist_top_k/op_kernel/hamming_dist_top_k_base.h:150-289).
 * Sink/recent positions have distance 0 (paged_ham_dist_mla.cu:194-197) so any block that
 * holds one scores G*bits.
 */
static void block_scores_one(const uint32_t* q_b, int64_t q_stride_h, const uint32_t* kc,
                             int64_t NB, int32_t BS, int32_t Hkv, int32_t Wd, int64_t ks_block,
                             int64_t ks_token, int64_t ks_head, const int32_t* table_b,
                             int64_t contiguous_base, int32_t len, int32_t G, int32_t sink,
                             int32_t recent, int32_t nblk, int32_t* s /* [Hkv][nblk] */)
{
    const int32_t full = G * 32 * Wd;
    for (int32_t j = 0; j < nblk; ++j) {
        const int64_t pb = table_b ? table_b[j] : contiguous_base + j;
        const int32_t p0 = j * BS;
        const int32_t p1 = (p0 + BS < len) ? p0 + BS : len; /* valid positions [p0,p1) */
        const int forced = (p0 < sink) || (p1 > len - recent);
        for (int32_t h = 0; h < Hkv; ++h) {
            int32_t best;
            if (pb < 0 || pb >= NB) {
                best = -1;
            } else if (forced) {
                best = full;
            } else {
                int32_t dmin = ORACLE_INF;
                for (int32_t p = p0; p < p1; ++p) {
                    const int32_t d =
                        group_distance(q_b + (int64_t)h * G * q_stride_h, q_stride_h, G,
                                       kc + pb * ks_block + (p - p0) * ks_token + h * ks_head, Wd);
                    if (d < dmin) dmin = d;
                }
                best = full - dmin;
            }
            s[(int64_t)h * nblk + j] = best;
        }
    }
}

static void topk_one(const uint32_t* q_b, int64_t q_stride_h, const uint32_t* kc, int64_t NB,
                     int32_t BS, int32_t Hkv, int32_t Wd, int64_t ks_block, int64_t ks_token,
                     int64_t ks_head, const int32_t* table_b, int64_t contiguous_base,
                     int32_t len, int32_t max_blocks, int32_t Hq, int32_t k, int32_t sink,
                     int32_t recent, uint32_t flags, int32_t* out_idx_b, int32_t* out_score_b)
{
    const int32_t G = Hq / Hkv;
    const int32_t full = G * 32 * Wd;
    const int32_t Ho = (flags & F_REDUCE_HEADS) ? 1 : Hkv;
    int32_t nblk = len > 0 ? (len + BS - 1) / BS : 0;
    if (nblk > max_blocks) nblk = max_blocks;
    for (int32_t i = 0; i < Ho * k; ++i) {
        out_idx_b[i] = -1;
        if (out_score_b) out_score_b[i] = 0;
    }
    if (nblk == 0) return;
    int32_t* s = (int32_t*)malloc(sizeof(int32_t) * (size_t)Hkv * (size_t)nblk);
    cand_t* c = (cand_t*)malloc(sizeof(cand_t) * (size_t)nblk);
    block_scores_one(q_b, q_stride_h, kc, NB, BS, Hkv, Wd, ks_block, ks_token, ks_head, table_b,
                     contiguous_base, len, G, sink, recent, nblk, s);
    for (int32_t ho = 0; ho < Ho; ++ho) {
        for (int32_t j = 0; j < nblk; ++j) {
            int32_t v;
            if (flags & F_REDUCE_HEADS) {
                v = s[j];
                for (int32_t h = 1; h < Hkv; ++h)
                    if (s[(int64_t)h * nblk + j] > v) v = s[(int64_t)h * nblk + j];
            } else {
                v = s[(int64_t)ho * nblk + j];
            }
            c[j].score = v;
            c[j].idx = j;
        }
        const int32_t kk = k < nblk ? k : nblk;
        qsort(c, (size_t)nblk, sizeof(cand_t), cand_cmp);
        if (!(flags & F_SCORE_ORDER)) qsort(c, (size_t)kk, sizeof(cand_t), idx_cmp);
        for (int32_t i = 0; i < kk; ++i) {
            const int32_t j = c[i].idx;
            out_idx_b[ho * k + i] =
                (flags & F_PHYSICAL) ? (table_b ? table_b[j] : (int32_t)(contiguous_base + j)) : j;
            if (out_score_b)
                out_score_b[ho * k + i] = (flags & F_DISTANCE) ? full - c[i].score : c[i].score;
        }
    }
    free(c);
    free(s);
}

typedef struct {
    const uint32_t* q;
    int64_t q_stride_b, q_stride_h;
    const uint32_t* kc;
    int64_t NB;
    int32_t BS, Hkv, Wd;
    int64_t ks_block, ks_token, ks_head;
    const int32_t* table;
    int32_t table_stride, max_blocks;
    const int32_t* lens;
    int32_t B, Hq, k, sink, recent;
    uint32_t flags;
    int32_t* out_idx;
    int32_t* out_score;
    int32_t b0, b1;
} topk_job_t;

static void* topk_range(void* arg)
{
    topk_job_t* a = (topk_job_t*)arg;
    const int32_t Ho = (a->flags & F_REDUCE_HEADS) ? 1 : a->Hkv;
    for (int32_t b = a->b0; b < a->b1; ++b)
        topk_one(a->q + b * a->q_stride_b, a->q_stride_h, a->kc, a->NB, a->BS, a->Hkv, a->Wd,
                 a->ks_block, a->ks_token, a->ks_head,
                 a->table ? a->table + (int64_t)b * a->table_stride : NULL,
                 (int64_t)b * a->max_blocks, a->lens[b], a->max_blocks, a->Hq, a->k, a->sink,
                 a->recent, a->flags, a->out_idx + (int64_t)b * Ho * a->k,
                 a->out_score ? a->out_score + (int64_t)b * Ho * a->k : NULL);
    return NULL;
}

/*
 * The same top-k with the work cut into (request, KV head) items that `nthreads` threads take
 * from a shared counter, each thread pinned to one of the cores this process may run on (the
 * reference's CPU backend pins its workers the same way, hash_retrieval_backend.cpp:188-199).
 * Timing variant for hosts with more cores than requests; per-head output only (no head reduce).
 */
typedef struct {
    topk_job_t job;
    volatile int32_t* next;
    int32_t core;
} topk_item_worker_t;

static void* topk_items(void* arg)
{
    topk_item_worker_t* w = (topk_item_worker_t*)arg;
    const topk_job_t* a = &w->job;
    if (w->core >= 0) {
        cpu_set_t set;
        CPU_ZERO(&set);
        CPU_SET(w->core, &set);
        (void)pthread_setaffinity_np(pthread_self(), sizeof(set), &set);
    }
    const int32_t G = a->Hq / a->Hkv;
    const int32_t total = a->B * a->Hkv;
    for (;;) {
        const int32_t i = __sync_fetch_and_add(w->next, 1);
        if (i >= total) break;
        const int32_t b = i / a->Hkv, h = i % a->Hkv;
        topk_one(a->q + b * a->q_stride_b + (int64_t)h * G * a->q_stride_h, a->q_stride_h,
                 a->kc + (int64_t)h * a->ks_head, a->NB, a->BS, 1, a->Wd, a->ks_block, a->ks_token,
                 a->ks_head, a->table ? a->table + (int64_t)b * a->table_stride : NULL,
                 (int64_t)b * a->max_blocks, a->lens[b], a->max_blocks, G, a->k, a->sink, a->recent,
                 a->flags & ~F_REDUCE_HEADS, a->out_idx + ((int64_t)b * a->Hkv + h) * a->k,
                 a->out_score ? a->out_score + ((int64_t)b * a->Hkv + h) * a->k : NULL);
    }
    return NULL;
}

void oracle_hamming_topk_items(const uint32_t* q, int64_t q_stride_b, int64_t q_stride_h,
                               const uint32_t* kc, int64_t NB, int32_t BS, int32_t Hkv, int32_t Wd,
                               int64_t ks_block, int64_t ks_token, int64_t ks_head,
                               const int32_t* table, int32_t table_stride, int32_t max_blocks,
                               const int32_t* lens, int32_t B, int32_t Hq, int32_t k, int32_t sink,
                               int32_t recent, uint32_t flags, int32_t* out_idx, int32_t* out_score,
                               int32_t nthreads)
{
    topk_job_t base = {q,  q_stride_b, q_stride_h, kc,     NB,        BS,    Hkv,
                       Wd, ks_block,   ks_token,   ks_head, table,     table_stride,
                       max_blocks, lens, B, Hq, k, sink, recent, flags, out_idx, out_score, 0, B};
    if (nthreads < 1) nthreads = 1;
    cpu_set_t allowed;
    int32_t cores[1024], ncores = 0;
    if (sched_getaffinity(0, sizeof(allowed), &allowed) == 0)
        for (int32_t c = 0; c < 1024 && c < CPU_SETSIZE; ++c)
            if (CPU_ISSET(c, &allowed)) cores[ncores++] = c;
    volatile int32_t next = 0;
    pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)nthreads);
    topk_item_worker_t* ws = (topk_item_worker_t*)malloc(sizeof(topk_item_worker_t) * (size_t)nthreads);
    for (int32_t i = 0; i < nthreads; ++i) {
        ws[i].job = base;
        ws[i].next = &next;
        ws[i].core = ncores ? cores[i % ncores] : -1;
        pthread_create(&th[i], NULL, topk_items, &ws[i]);
    }
    for (int32_t i = 0; i < nthreads; ++i) pthread_join(th[i], NULL);
    free(ws);
    free(th);
}

/*
 * Block top-k.  Follows hamming_topk.py:15-54 (block min, top-k, ascending sort, block
 * table gather), paged_ham_dist_mla.cu:148-247 (group sum, masking, sink/recent, head
 * reduce) and the ascending-index + table-map output of the NPU op
 * (hamming_dist_top_k_base.h:307-347).  nthreads > 1 splits requests over pthreads
 * (one request per thread at nthreads == B).
 * out_idx / out_score: int32 [B, (reduce ? 1 : Hkv), k]; unused slots -1 / 0.
 */
void oracle_hamming_topk(const uint32_t* q, int64_t q_stride_b, int64_t q_stride_h,
                         const uint32_t* kc, int64_t NB, int32_t BS, int32_t Hkv, int32_t Wd,
                         int64_t ks_block, int64_t ks_token, int64_t ks_head,
                         const int32_t* table, int32_t table_stride, int32_t max_blocks,
                         const int32_t* lens, int32_t B, int32_t Hq, int32_t k, int32_t sink,
                         int32_t recent, uint32_t flags, int32_t* out_idx, int32_t* out_score,
                         int32_t nthreads)
{
    topk_job_t base = {q,  q_stride_b, q_stride_h, kc,     NB,        BS,    Hkv,
                       Wd, ks_block,   ks_token,   ks_head, table,     table_stride,
                       max_blocks, lens, B, Hq, k, sink, recent, flags, out_idx, out_score, 0, B};
    if (nthreads <= 1 || B <= 1) {
        topk_range(&base);
        return;
    }
    if (nthreads > B) nthreads = B;
    pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)nthreads);
    topk_job_t* jobs = (topk_job_t*)malloc(sizeof(topk_job_t) * (size_t)nthreads);
    for (int32_t i = 0; i < nthreads; ++i) {
        jobs[i] = base;
        jobs[i].b0 = (int32_t)((int64_t)B * i / nthreads);
        jobs[i].b1 = (int32_t)((int64_t)B * (i + 1) / nthreads);
        pthread_create(&th[i], NULL, topk_range, &jobs[i]);
    }
    for (int32_t i = 0; i < nthreads; ++i) pthread_join(th[i], NULL);
    free(jobs);
    free(th);
}

/*
 * The CPU retrieval backend's form.  hash_retrieval_backend.cpp:321-407: for every row b
 * and every allowed block index (entries == -1 removed, :241-246) the score is the min
 * over ALL block_size tokens of popcount(q xor k) over dim bytes, starting from
 * UINT16_MAX (:357-388, no masking); the top min(k, n_allowed) smallest scores are
 * returned in ascending score order (:396-406).  Ties are broken here by position in the
 * allowed list (the reference leaves them unspecified).
 * data u8 [NB,BS,dim]; query u8 [B,dim]; indexes i32 [B,max_idx];
 * out_idx/out_score i32 [B,k], unused slots -1 / 0.  out_n[b] = number of results.
 */
void oracle_hash_retrieval(const uint8_t* data, int64_t NB, int32_t BS, int32_t dim,
                           const uint8_t* query, int32_t B, const int32_t* indexes,
                           int32_t max_idx, int32_t k, int32_t* out_idx, int32_t* out_score,
                           int32_t* out_n)
{
    (void)NB;
    cand_t* c = (cand_t*)malloc(sizeof(cand_t) * (size_t)(max_idx > 0 ? max_idx : 1));
    int32_t* blk = (int32_t*)malloc(sizeof(int32_t) * (size_t)(max_idx > 0 ? max_idx : 1));
    for (int32_t b = 0; b < B; ++b) {
        const uint8_t* qp = query + (int64_t)b * dim;
        int32_t n = 0;
        for (int32_t i = 0; i < max_idx; ++i) {
            const int32_t idx = indexes[(int64_t)b * max_idx + i];
            if (idx == -1) continue;
            const uint8_t* base = data + (int64_t)idx * BS * dim;
            int32_t score = 65535;
            for (int32_t t = 0; t < BS; ++t) {
                int32_t sum = 0;
                for (int32_t d = 0; d < dim; ++d)
                    sum += __builtin_popcount((unsigned)(qp[d] ^ base[(int64_t)t * dim + d]));
                if (sum < score) {
                    score = sum;
                    if (score == 0) break;
                }
            }
            /* cand_cmp sorts by score desc: store the negated distance, position as idx */
            c[n].score = -score;
            c[n].idx = n;
            blk[n] = idx;
            ++n;
        }
        const int32_t kk = k < n ? k : n;
        qsort(c, (size_t)n, sizeof(cand_t), cand_cmp);
        for (int32_t i = 0; i < k; ++i) {
            out_idx[(int64_t)b * k + i] = i < kk ? blk[c[i].idx] : -1;
            out_score[(int64_t)b * k + i] = i < kk ? -c[i].score : 0;
        }
        if (out_n) out_n[b] = kk;
    }
    free(blk);
    free(c);
}

/* hamming_topk.py:7-12 (update_seq_lens). */
void oracle_update_seq_lens(const int32_t* lens, int32_t B, int32_t topk_tok, int32_t BS,
                            int32_t* out)
{
    for (int32_t b = 0; b < B; ++b) {
        int32_t over = lens[b] - topk_tok;
        if (over < 0) over = 0;
        out[b] = lens[b] - ((over + BS - 1) / BS) * BS;
    }
}

/* ------------------------------------------------------------------------------------
 * Transfer.  ucm/shared/trans/cuda/cuda_stream.cc:63-80,110-127 and
 * ucm/shared/trans/simu/simu_stream.cc:81-90,125-134: chunk i of `size` bytes.
 * ------------------------------------------------------------------------------------ */
void oracle_gather(const void* const* src, void* dst, size_t size, size_t number)
{
    for (size_t i = 0; i < number; ++i) memcpy((char*)dst + i * size, src[i], size);
}
void oracle_scatter(const void* src, void* const* dst, size_t size, size_t number)
{
    for (size_t i = 0; i < number; ++i) memcpy(dst[i], (const char*)src + i * size, size);
}
void oracle_batch(const void* const* src, void* const* dst, size_t size, size_t number)
{
    for (size_t i = 0; i < number; ++i) memcpy(dst[i], src[i], size);
}

/* ucm/integration/vllm/ucm_connector.py:135-148 (extract_block_addrs, block-first):
 * out[blk, col] = base[col] + block_id[blk] * col_bytes[col]. */
void oracle_block_addrs(const uint64_t* base, const uint64_t* col_bytes, int32_t n_cols,
                        const int32_t* block_ids, int64_t n_blocks, uint64_t* out)
{
    for (int64_t i = 0; i < n_blocks; ++i)
        for (int32_t c = 0; c < n_cols; ++c)
            out[i * n_cols + c] = base[c] + (uint64_t)block_ids[i] * col_bytes[c];
}

/* Paged copy with per-column sizes: the flat buffer holds (block, col) row-major, column
 * offsets accumulate (ucm/store/cache/cc/dump_queue.cc:145-161, load_queue.cc:178-194). */
void oracle_paged_copy(const uint64_t* base, const uint64_t* col_bytes, int32_t n_cols,
                       const int32_t* block_ids, int64_t n_blocks, void* flat, int to_cache)
{
    size_t off = 0;
    for (int64_t i = 0; i < n_blocks; ++i)
        for (int32_t c = 0; c < n_cols; ++c) {
            void* p = (void*)(uintptr_t)(base[c] + (uint64_t)block_ids[i] * col_bytes[c]);
            if (to_cache)
                memcpy(p, (char*)flat + off, (size_t)col_bytes[c]);
            else
                memcpy((char*)flat + off, p, (size_t)col_bytes[c]);
            off += (size_t)col_bytes[c];
        }
}

/* ------------------------------------------------------------------------------------
 * Float retrieval (ESA).  retrieval_backend.cpp:207-227: per request, every allowed index is
 * scored with a sequential fp32 dot product (no fused multiply-add: the reference module is
 * built for baseline x86-64), the pairs are partially sorted by descending score and the
 * first min(n_allowed, topk) returned.  Entries -1 of `indexes` are dropped when the request
 * is submitted (:96-104).  Ties: the reference's partial_sort leaves them open; here equal
 * scores keep list order.  out rows are padded with -1 / 0.
 * ------------------------------------------------------------------------------------ */
__attribute__((optimize("fp-contract=off"))) static float seq_dot(const float* q, const float* x,
                                                                  int32_t dim)
{
    float score = 0.0f;
    for (int32_t d = 0; d < dim; ++d) {
        const float p = q[d] * x[d];
        score = score + p;
    }
    return score;
}

typedef struct {
    float score;
    int32_t pos;
} dot_pair;

static int dot_pair_cmp(const void* a, const void* b)
{
    const dot_pair* x = (const dot_pair*)a;
    const dot_pair* y = (const dot_pair*)b;
    if (x->score > y->score) return -1;
    if (x->score < y->score) return 1;
    return (x->pos > y->pos) - (x->pos < y->pos);
}

void oracle_dot_topk(const float* data, int64_t n_items, int32_t dim, const float* query,
                     const int32_t* indexes, int32_t B, int32_t max_n, int32_t topk,
                     int32_t* out_idx, float* out_score)
{
    dot_pair* pairs = (dot_pair*)malloc(sizeof(dot_pair) * (size_t)(max_n > 0 ? max_n : 1));
    for (int32_t b = 0; b < B; ++b) {
        int32_t n = 0;
        for (int32_t j = 0; j < max_n; ++j) {
            const int32_t item = indexes[(int64_t)b * max_n + j];
            if (item < 0 || item >= n_items) continue;
            pairs[n].score = seq_dot(query + (int64_t)b * dim, data + (int64_t)item * dim, dim);
            pairs[n].pos = j;
            ++n;
        }
        qsort(pairs, (size_t)n, sizeof(dot_pair), dot_pair_cmp);
        for (int32_t t = 0; t < topk; ++t) {
            const int has = t < n;
            out_idx[(int64_t)b * topk + t] = has ? indexes[(int64_t)b * max_n + pairs[t].pos] : -1;
            out_score[(int64_t)b * topk + t] = has ? pairs[t].score : 0.0f;
        }
    }
    free(pairs);
}

/* ------------------------------------------------------------------------------------
 * KVStar block retrieval.  kvstar/retrieve/core/domain/retrieve_task/simd_compute_kernel.cpp
 * :816-985 (scalar_impl::execute_impl), statement by statement: channel pruning of the queries
 * (:846-872), sequential fp32 q.k over all S = n_blocks * M representatives (:885-911), softmax
 * per (token, q head) with the "sum_exp > 1e-9" guard (:913-942), block sums accumulated row by
 * row (:944-952), a size-topk min-heap of (score, block) pairs with strict-greater replacement,
 * emptied back to front (:954-977).  fp16 -> fp32 as fp16_to_float (:780-812).
 * all_scores (optional) receives the n_blocks block scores.
 * Pinned by mathematics only (tests/test_oracle_kvstar.py: a float64 library formulation,
 * closed forms, invariants, the heap's tie order, all 65,536 fp16 patterns): the reference's
 * translation unit needs its logger (spdlog, fmt), which this image lacks, so it cannot be
 * compiled for golden vectors, and the reference holds no test vectors for this kernel.
 * ------------------------------------------------------------------------------------ */
static float half_bits_to_float(uint16_t h)
{
    const uint32_t s = ((uint32_t)h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    uint32_t bits;
    if (e == 0) {
        if (m == 0) {
            bits = s;
        } else {  /* subnormal: normalise */
            uint32_t mm = m, ee = 113;
            while (!(mm & 0x400u)) {
                mm <<= 1;
                --ee;
            }
            bits = s | (ee << 23) | ((mm & 0x3FFu) << 13);
        }
    } else if (e == 0x1Fu) {
        bits = s | 0x7F800000u | (m << 13);
    } else {
        bits = s | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &bits, sizeof(f));
    return f;
}

void oracle_half_to_float(const uint16_t* h, int64_t n, float* out)
{
    for (int64_t i = 0; i < n; ++i) out[i] = half_bits_to_float(h[i]);
}

typedef struct {
    float score;
    int64_t idx;
} kv_pair;

static int kv_pair_less(kv_pair a, kv_pair b)  /* std::pair ordering */
{
    return a.score < b.score || (a.score == b.score && a.idx < b.idx);
}

static void heap_sift_down(kv_pair* h, int64_t n, int64_t i)
{
    for (;;) {
        int64_t l = 2 * i + 1, r = l + 1, m = i;
        if (l < n && kv_pair_less(h[l], h[m])) m = l;
        if (r < n && kv_pair_less(h[r], h[m])) m = r;
        if (m == i) return;
        kv_pair t = h[i];
        h[i] = h[m];
        h[m] = t;
        i = m;
    }
}

__attribute__((optimize("fp-contract=off")))
void oracle_kvstar_topk(const uint16_t* q, int32_t X, int32_t Hq, int32_t d_orig, const uint16_t* k,
                        int64_t n_blocks, int32_t M, int32_t Hkv, int32_t d, const int64_t* pruned,
                        int32_t topk, int64_t* out_idx, float* out_score, int32_t* out_count,
                        float* all_scores)
{
    const int32_t g = Hq / Hkv;
    const int64_t S = n_blocks * M, rows = (int64_t)X * Hq;
    float* sc = (float*)malloc(sizeof(float) * (size_t)(rows * S));
    float* qrow = (float*)malloc(sizeof(float) * (size_t)d);
    for (int64_t x = 0; x < X; ++x)
        for (int32_t h = 0; h < Hkv; ++h)
            for (int32_t gg = 0; gg < g; ++gg) {
                const int32_t H = h * g + gg;
                for (int32_t j = 0; j < d; ++j) {
                    const int64_t src = pruned ? pruned[(int64_t)h * d + j] : j;
                    qrow[j] = half_bits_to_float(q[(x * Hq + H) * (int64_t)d_orig + src]);
                }
                for (int64_t s = 0; s < S; ++s) {
                    const uint16_t* kv = k + (s * Hkv + h) * (int64_t)d;
                    float score = 0.0f;
                    for (int32_t j = 0; j < d; ++j) {
                        const float p = qrow[j] * half_bits_to_float(kv[j]);
                        score = score + p;
                    }
                    sc[(x * Hq + H) * S + s] = score;
                }
            }
    for (int64_t i = 0; i < rows; ++i) {
        float* cur = sc + i * S;
        float mx = cur[0];
        for (int64_t s = 1; s < S; ++s)
            if (cur[s] > mx) mx = cur[s];
        float sum = 0.0f;
        for (int64_t s = 0; s < S; ++s) {
            cur[s] = expf(cur[s] - mx);
            sum = sum + cur[s];
        }
        if (sum > 1e-9)
            for (int64_t s = 0; s < S; ++s) cur[s] = cur[s] / sum;
    }
    float* fin = (float*)calloc((size_t)n_blocks, sizeof(float));
    for (int64_t i = 0; i < rows; ++i)
        for (int64_t s = 0; s < S; ++s) fin[s / M] = fin[s / M] + sc[i * S + s];
    if (all_scores) memcpy(all_scores, fin, sizeof(float) * (size_t)n_blocks);
    kv_pair* heap = (kv_pair*)malloc(sizeof(kv_pair) * (size_t)(topk > 0 ? topk : 1));
    int64_t hn = 0;
    for (int64_t n = 0; n < n_blocks; ++n) {
        const kv_pair p = {fin[n], n};
        if (hn < topk) {  /* push */
            int64_t i = hn++;
            heap[i] = p;
            while (i > 0 && kv_pair_less(heap[i], heap[(i - 1) / 2])) {
                kv_pair t = heap[i];
                heap[i] = heap[(i - 1) / 2];
                heap[(i - 1) / 2] = t;
                i = (i - 1) / 2;
            }
        } else if (hn > 0 && fin[n] > heap[0].score) {  /* replace the minimum */
            heap[0] = p;
            heap_sift_down(heap, hn, 0);
        }
    }
    *out_count = (int32_t)hn;
    for (int64_t pos = hn - 1; pos >= 0; --pos) {  /* smallest pair goes last */
        out_idx[pos] = heap[0].idx;
        out_score[pos] = heap[0].score;
        heap[0] = heap[hn - 1];
        --hn;
        heap_sift_down(heap, hn, 0);
    }
    free(heap);
    free(fin);
    free(qrow);
    free(sc);
}
