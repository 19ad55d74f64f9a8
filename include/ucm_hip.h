/*
 * ucm_hip.h — C ABI of the MI355X (gfx950) sparse-retrieval and KV-transfer library.
 *
 * Every entry point takes plain pointers and sizes, returns an int status and never
 * throws.  Device pointers are ordinary HIP device addresses; `stream` arguments are a
 * `hipStream_t` passed as `void*` (NULL = the null stream).  Unless a function says
 * "sync" it only enqueues work on the given stream.
 *
 * Status codes follow the reference's UC::Status convention
 * (ucm/shared/infra/status/status.h:40-53): 0 = OK, -1 = generic error,
 * -50000-i = typed errors.  ucm_last_error() returns the message of the last failure
 * on the calling thread.
 */
#ifndef UCM_HIP_H
#define UCM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define UCM_OK            0
#define UCM_ERROR        (-1)
#define UCM_EPARAM       (-50000)
#define UCM_EOOM         (-50001)
#define UCM_EOSERROR     (-50002)
#define UCM_ERETRY       (-50004)
#define UCM_ENOOBJ       (-50005)
#define UCM_EUNSUPPORTED (-50008)
#define UCM_ETIMEOUT     (-50010)

/* element types of encoder inputs */
#define UCM_DT_BF16 0
#define UCM_DT_F16  1
#define UCM_DT_F32  2

typedef void* ucm_stream_t;

/* Library version (major*10000 + minor*100 + patch). */
int ucm_version(void);
/* Message of the last failing call on this thread ("" if none). */
const char* ucm_last_error(void);

/* ------------------------------------------------------------------------------------
 * 1. Hash encoder: codes = pack_lsb_first( x · W > 0 )
 * ------------------------------------------------------------------------------------ */

/*
 * Replaces HashEncoder.compute_hash (ucm/sparse/gsa_on_device/hash_encoder.py:450-507)
 * and its Triton kernel (hash_encoder.py:37-134).
 *
 * x        [T, H, K] of x_dtype, K contiguous; strides in elements.
 * w        [n_w, K, N_bits] row-major of w_dtype.  Head h uses matrix
 *          min(h / heads_per_w, n_w - 1); n_w = 1 shares one matrix (the reference's case).
 * out      uint32 [T, H, N_bits/32]; strides in 32-bit words.  Hash bit n of a row is bit
 *          n%32 of word n/32, i.e. byte n/8, bit n%8 (LSB first), little endian — the byte
 *          order torch_hash_code produces (hash_encoder.py:359-370).
 * A projection that is 0, -0 or NaN gives bit 0.  Requires K % 16 == 0, N_bits % 32 == 0.
 */
int ucm_hash_encode(const void* x, int x_dtype, int64_t T, int32_t H, int32_t K,
                    int64_t x_stride_t, int64_t x_stride_h,
                    const void* w, int w_dtype, int32_t n_w, int32_t heads_per_w,
                    int32_t N_bits,
                    uint32_t* out, int64_t out_stride_t, int64_t out_stride_h,
                    ucm_stream_t stream);

/*
 * Replaces HashEncoder.compute_hash_and_cache (hash_encoder.py:548-662) and
 * fused_hash_and_cache_kernel (hash_encoder.py:263-356): encode x[t,h,:] and store the
 * code at cache[slot/BS, slot%BS, h, :].  Rows whose slot is < 0 or >= NB*BS are
 * skipped (hash_encoder.py:338-344).
 *
 * slot_mapping  [T] int32 (slot_is_i64 = 0) or int64 (slot_is_i64 = 1), device memory.
 * cache         uint32 words; strides (block, token, head) in 32-bit words, the N_bits/32
 *               words of a code are contiguous.
 */
int ucm_hash_encode_cache(const void* x, int x_dtype, int64_t T, int32_t H, int32_t K,
                          int64_t x_stride_t, int64_t x_stride_h,
                          const void* w, int w_dtype, int32_t n_w, int32_t heads_per_w,
                          int32_t N_bits,
                          const void* slot_mapping, int slot_is_i64,
                          uint32_t* cache, int64_t NB, int32_t BS,
                          int64_t cs_block, int64_t cs_token, int64_t cs_head,
                          ucm_stream_t stream);

/*
 * Tuning and test hook, no counterpart in the reference.  Inputs of at least `rows` rows (tokens x
 * heads) with 64 or 128 input dimensions and 64 or 128 hash bits take the streaming kernel
 * (persistent waves, projection matrix in registers, rows loaded straight into LDS); smaller ones
 * take the tiled kernel.  Both give identical codes.  rows <= 0 restores the default (2^20).  The
 * setting belongs to the calling thread: encodes issued by other threads are not affected.
 */
int ucm_hash_encode_set_stream_threshold(int64_t rows);

/*
 * Measurement aid, no counterpart in the reference.  While a non-null address is set, every launch
 * of the persistent kernel for 512 input dimensions (encode_wide_kernel) issued by the calling thread
 * has its first workgroup write two 64-bit numbers there when it ends: the shader cycles and the
 * ticks of the constant 100 MHz counter between its first and its last instruction.  Their ratio is
 * the clock the workgroup ran at (cycles / ticks * 0.1 GHz); the part's clock under a matrix-heavy
 * load is well below its data-sheet maximum, and a launch time can only be judged beside it.  The
 * address must be 8-byte aligned device memory of at least 16 bytes that outlives the launches; pass
 * null to switch the probe off (the default).  Other kernels ignore it.
 */
int ucm_hash_encode_set_clock_probe(void* two_u64_in_device_memory);

/*
 * The streaming kernel's time-out contract, no counterpart in the reference.  With 2, 4 or 8 heads
 * of 128-bit codes side by side in a cache row the streaming kernel's waves exchange their codes
 * through LDS and wait for one another with a bounded number of polls; a wave that reaches the bound
 * goes on without waiting, so that a launch always ends.  The codes that launch wrote are then
 * undefined.  The wave reports it in a word of pinned host memory, and from then on EVERY encode entry
 * point (ucm_hash_encode, ucm_hash_encode_cache, ucm_hash_encode_paged and the decode-step calls that
 * encode) returns UCM_ERROR on that device, with a ucm_last_error() text that says so, before it
 * launches anything - a host-side read, no device synchronisation.  The failed launch itself has
 * returned UCM_OK (it ran later, asynchronously): a caller that must know before it uses the codes
 * synchronises the stream and calls ucm_hash_encode_stream_timeouts().  After rebuilding the codes
 * the caller acknowledges with ucm_hash_encode_clear_stream_timeouts().
 *
 * ucm_hash_encode_stream_timeouts: how many waits have reached the bound on the current device since
 * the library was loaded (0 in a healthy process; synchronises with the device), or a negative status.
 * ucm_hash_encode_clear_stream_timeouts: clears the current device's latch (not the count).
 * ucm_hash_encode_debug_trip_stream_latch: sets the current device's latch from the host, as a timed-out
 * wave would - for tests of the error path; no kernel is involved.
 */
int64_t ucm_hash_encode_stream_timeouts(void);
int ucm_hash_encode_clear_stream_timeouts(void);
int ucm_hash_encode_debug_trip_stream_latch(void);

/*
 * Re-encodes keys that already sit in the paged KV cache (prefix-cache hit): replaces the
 * gather `kv_cache[0][0][prefix_block_ids]` followed by compute_hash_and_cache with the
 * prefix slot mapping (ucm/sparse/gsa_on_device/gsa_on_device.py:574-588; the slot rule is
 * rebuild_prefix_cache_info_for_req, :1142-1174: slot(i) = block_ids[i / BS] * BS + i % BS).
 * The keys are read in place — no gathered copy — and token i % BS of key block
 * block_ids[i / BS] gets its code at the same block and token of the code cache.
 *
 * k_cache    [NBk, BS, H, K] of x_dtype; strides (block, token, head) in elements, the K
 *            values of a row are contiguous.
 * block_ids  [n_blocks] int32, device memory; n_tokens <= n_blocks * BS tokens are encoded
 *            (the last block may be partial).  Ids outside [0, min(NBk, NB)) are skipped.
 * cache      uint32 code cache [NB, BS, H, N_bits/32]; strides in 32-bit words.
 */
int ucm_hash_encode_paged(const void* k_cache, int x_dtype, int64_t NBk, int32_t BS, int32_t H,
                          int32_t K, int64_t ks_block, int64_t ks_token, int64_t ks_head,
                          const int32_t* block_ids, int64_t n_blocks, int64_t n_tokens,
                          const void* w, int w_dtype, int32_t n_w, int32_t heads_per_w,
                          int32_t N_bits,
                          uint32_t* cache, int64_t NB,
                          int64_t cs_block, int64_t cs_token, int64_t cs_head,
                          ucm_stream_t stream);

/*
 * Replaces reshape_and_cache_khash_triton (hash_encoder.py:136-261): scatter already
 * computed codes [T, H, Wd] into the paged code cache by slot.
 */
int ucm_code_scatter(const uint32_t* codes, int64_t T, int32_t H, int32_t Wd,
                     int64_t in_stride_t, int64_t in_stride_h,
                     const void* slot_mapping, int slot_is_i64,
                     uint32_t* cache, int64_t NB, int32_t BS,
                     int64_t cs_block, int64_t cs_token, int64_t cs_head,
                     ucm_stream_t stream);

/* ------------------------------------------------------------------------------------
 * 2. Hamming scorer + deterministic block top-k
 * ------------------------------------------------------------------------------------ */

/* flags of ucm_hamming_topk */
#define UCM_TOPK_REDUCE_HEADS    1u  /* one list per request: block score = max over KV heads
                                        (= the min over heads of paged_ham_dist_mla.cu:203-211) */
#define UCM_TOPK_RETURN_PHYSICAL 2u  /* out_idx holds block_table[b, j] instead of logical j
                                        (hamming_topk.py:54) */
#define UCM_TOPK_SCORE_ORDER     4u  /* order the k results by (score desc, index asc) instead
                                        of ascending index (hash_retrieval_backend.cpp:396-406) */
#define UCM_TOPK_DISTANCE        8u  /* out_score holds Hamming distance G*bits - s */

/* Bytes of device workspace ucm_hamming_topk needs for these sizes. */
size_t ucm_hamming_topk_workspace_bytes(int32_t B, int32_t Hkv, int32_t max_blocks);

/*
 * Replaces hamming.hamming_score + the torch min/topk/sort/gather chain of
 * cuda_hamming_topk (ucm/sparse/gsa_on_device/hamming_topk.py:15-54,
 * csrc/cuda/ham_dist/paged_ham_dist_mla.cu:111-248,332-443), with the per-KV-head,
 * similarity-score output contract of npu_hamming_dist_top_k
 * (csrc/ascend/torch_binding.cpp:39-57).
 *
 * q_codes     uint32 [B, Hq, Wd], strides in words (Wd contiguous).
 * k_cache     uint32 paged codes, logical shape [NB, BS, Hkv, Wd]; strides (block, token,
 *             head) in words, Wd contiguous.  Token-major [NB,BS,Hkv,Wd] and head-major
 *             [NB,Hkv,BS,Wd] caches are both expressed through the strides.
 * block_table int32 [B, table_stride], logical block j of request b is block_table[b, j].
 *             NULL = request b owns blocks b*max_blocks ... (contiguous cache).
 * seq_lens    int32 [B] valid tokens per request.
 * G = Hq / Hkv query heads are summed per KV head:
 *   s[b,h,j] = max over valid tokens t of block j of
 *              sum_g ( 32*Wd - popcount(q[b,h*G+g] xor k[table[b,j], t, h]) )      (int32)
 * A block holding a position < sink_tok or >= len - recent_tok gets s = G*32*Wd
 * (paged_ham_dist_mla.cu:194-197).  A table entry outside [0, NB) scores -1.
 * Per (b, h) [or per b with UCM_TOPK_REDUCE_HEADS] the min(k, nblk) blocks with the
 * largest s are selected, ties to the lower logical index, and written in ascending
 * logical index order; unused output slots get index -1 and score 0.
 *
 * out_idx, out_score  int32 [B, Hkv or 1, k]; out_score may be NULL.
 * workspace   device memory of at least ucm_hamming_topk_workspace_bytes(...) bytes,
 *             16-byte aligned; contents need no initialisation.
 */
int ucm_hamming_topk(const uint32_t* q_codes, int64_t q_stride_b, int64_t q_stride_h,
                     const uint32_t* k_cache, int64_t NB, int32_t BS, int32_t Hkv, int32_t Wd,
                     int64_t ks_block, int64_t ks_token, int64_t ks_head,
                     const int32_t* block_table, int32_t table_stride, int32_t max_blocks,
                     const int32_t* seq_lens,
                     int32_t B, int32_t Hq, int32_t k,
                     int32_t sink_tok, int32_t recent_tok, uint32_t flags,
                     int32_t* out_idx, int32_t* out_score,
                     void* workspace, size_t workspace_bytes,
                     ucm_stream_t stream);

/*
 * ucm_hamming_topk for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Arguments and results are those of ucm_hamming_topk without the workspace: block
 * scores and bit planes live in a fixed array of UCM_TOPK_STATIC_SCRATCH_BYTES that every GPU the
 * library runs on holds until the process ends.  Shapes whose
 * ucm_hamming_topk_workspace_bytes(B, Hkv, max_blocks) exceeds that size are rejected with
 * UCM_EPARAM.  The call allocates nothing; the array's address on the current device is looked
 * up on the first call on that device (make that call outside a graph capture).  All calls on
 * one GPU share the array: calls that overlap in time on one GPU (two streams, two threads)
 * race; calls on one stream are ordered and safe.
 */
#define UCM_TOPK_STATIC_SCRATCH_BYTES (4u << 20)
int ucm_hamming_topk_static(const uint32_t* q_codes, int64_t q_stride_b, int64_t q_stride_h,
                            const uint32_t* k_cache, int64_t NB, int32_t BS, int32_t Hkv, int32_t Wd,
                            int64_t ks_block, int64_t ks_token, int64_t ks_head,
                            const int32_t* block_table, int32_t table_stride, int32_t max_blocks,
                            const int32_t* seq_lens,
                            int32_t B, int32_t Hq, int32_t k,
                            int32_t sink_tok, int32_t recent_tok, uint32_t flags,
                            int32_t* out_idx, int32_t* out_score,
                            ucm_stream_t stream);

/*
 * Replaces kvlib::HammingScoreContiCUDA (csrc/cuda/ham_dist/operator.h:10-13,
 * paged_ham_dist_mla.cu:332-443) for callers that want its per-token output:
 * out[b, h, p] for p < max_seq_len is the group-summed Hamming distance of position p,
 * 0 for sink/recent positions and "infinity" for p >= seq_lens[b].
 * out_is_f16 = 1 writes IEEE half exactly as the reference (inf = 0x7C00);
 * out_is_f16 = 0 writes int32 with infinity = INT32_MAX.
 * reduce_heads = 1 writes the min over KV heads, shape [B, 1, max_seq_len].
 * workspace   optional device memory of at least ucm_hamming_score_workspace_bytes(...)
 *             bytes, 16-byte aligned, contents need no initialisation.  It holds the bit
 *             planes of the query counts, which the kernel for one KV head and more than 8
 *             query heads (the latent-attention layout) reads; with NULL that case runs on
 *             the slower general kernel, with the same results.  18-word codes in 64-token
 *             blocks with up to 128 query heads (and 8-word codes with 16 to 128) never need
 *             it: their kernel builds its weights itself.
 */
size_t ucm_hamming_score_workspace_bytes(int32_t B, int32_t Hq, int32_t Wd);
int ucm_hamming_score(const uint32_t* q_codes, int64_t q_stride_b, int64_t q_stride_h,
                      const uint32_t* k_cache, int64_t NB, int32_t BS, int32_t Hkv, int32_t Wd,
                      int64_t ks_block, int64_t ks_token, int64_t ks_head,
                      const int32_t* block_table, int32_t table_stride, int32_t max_blocks,
                      const int32_t* seq_lens,
                      int32_t B, int32_t Hq, int32_t max_seq_len,
                      int32_t sink_tok, int32_t recent_tok, int reduce_heads,
                      void* out, int out_is_f16,
                      void* workspace, size_t workspace_bytes,
                      ucm_stream_t stream);

/*
 * Measurement hook, no counterpart in the reference.  When both events (hipEvent_t) are
 * non-NULL, every following ucm_hamming_topk call on this thread launches its block-score
 * kernel with `before` / `after` as that dispatch's own start and stop events
 * (hipExtLaunchKernel), so hipEventElapsedTime(before, after) is the kernel's execution time.
 * Pass NULLs to switch it off.
 */
int ucm_hamming_topk_set_profile_events(void* before, void* after);

/*
 * Measurement aid, no counterpart in the reference.  While a non-null address is set, every launch of
 * the scorer for 64-token blocks of latent-attention codes (block_score_strip / token_score_strip: one
 * KV head, 18-word codes with up to 128 query heads, 8-word codes with 16 to 128) issued by the
 * calling thread through ucm_hamming_topk, ucm_hamming_score or a decode-step call has the last wave
 * of its first workgroup write two 64-bit numbers there when it ends: the shader cycles and the ticks
 * of the constant 100 MHz counter of its life.  cycles / ticks * 0.1 is the clock in GHz that the wave
 * ran at; the kernel's instruction counts can only be priced at that clock.  The address must be
 * 8-byte aligned device memory of at least 16 bytes that outlives the launches; pass null to switch
 * the probe off (the default).  Other kernels ignore it.
 */
int ucm_hamming_topk_set_clock_probe(void* two_u64_in_device_memory);

/*
 * Test hook, no counterpart in the reference.  Writes the names of the kernels that the last
 * ucm_hamming_topk / ucm_hamming_topk_static / ucm_sparse_decode_step* / ucm_gsa_decode_step /
 * ucm_hamming_score call on the calling thread launched, e.g.
 * "block_score_one<1,8,1,4,1>+select_wave_kernel<4>" or
 * "plane_kernel+block_score_lanes<4,0,8>+select_wave_kernel<4>" (family, then its template
 * arguments), cut to cap - 1 characters.  Returns the full length.  Several kernel families give
 * the same results at very different speeds; this lets a test pin which one a shape takes.
 */
int64_t ucm_hamming_last_dispatch(char* buf, size_t cap);

/*
 * One decode step of the GQA retrieval path in a single call: store the hash codes of the
 * step's new keys in the paged code cache, hash the step's queries, then score and select.
 * Replaces the call sequence of GSAOnDevice.attention_begin at decode
 * (ucm/sparse/gsa_on_device/gsa_on_device.py:564-572 cache_k_hash_gqa_cuda, :773-786
 * update_decode_topk_gqa_cuda): three launches issued back to back from native code.
 *
 * new_keys  [T, Hkv, K] (strides in elements), slot_mapping [T]: as ucm_hash_encode_cache;
 *           T = 0 skips the cache update.
 * queries   [B, Hq, K]  (strides in elements); query head h is projected with matrix
 *           min(h / (Hq/Hkv), n_w - 1) when n_w > 1 — the matrix of its KV head.
 * w         [n_w, K, N_bits]; n_w is 1 (shared) or Hkv.
 * q_codes   uint32 [B, Hq, N_bits/32] contiguous scratch that receives the query codes.
 * Remaining arguments as in ucm_hamming_topk (Wd = N_bits / 32).
 */
int ucm_sparse_decode_step(const void* new_keys, int64_t T, int64_t k_stride_t, int64_t k_stride_h,
                           const void* slot_mapping, int slot_is_i64,
                           const void* queries, int64_t q_stride_b, int64_t q_stride_h,
                           int x_dtype, int32_t K,
                           const void* w, int w_dtype, int32_t n_w, int32_t N_bits,
                           uint32_t* k_cache, int64_t NB, int32_t BS, int32_t Hkv,
                           int64_t ks_block, int64_t ks_token, int64_t ks_head,
                           const int32_t* block_table, int32_t table_stride, int32_t max_blocks,
                           const int32_t* seq_lens, int32_t B, int32_t Hq, int32_t k,
                           int32_t sink_tok, int32_t recent_tok, uint32_t flags,
                           uint32_t* q_codes, int32_t* out_idx, int32_t* out_score,
                           void* workspace, size_t workspace_bytes, ucm_stream_t stream);

/*
 * The same single call for the latent-attention (MLA) layout: one KV head whose code is the
 * nope part's hash followed by the rope part's hash (GSAOnDevice with is_mla,
 * ucm/sparse/gsa_on_device/gsa_on_device.py:426-455 cache_k_hash_mla_cuda — hash_code followed by
 * vLLM's concat_and_cache_mla — and :667-709 update_decode_topk_mla_cuda).  Each part has its own
 * projection matrix; both parts of the step's new keys go to the paged code cache, both parts
 * of the (already head-reduced, :376-393) queries to q_codes, then score and select.
 *
 * new_nope [T, K_nope], new_rope [T, K_rope] (row strides in elements), slot_mapping [T];
 * T = 0 skips the cache update.  q_nope [B, Hq, K_nope], q_rope [B, Hq, K_rope].
 * w_nope [K_nope, N_nope_bits], w_rope [K_rope, N_rope_bits].
 * k_cache  uint32 [NB, BS, Wd] with Wd = (N_nope_bits + N_rope_bits) / 32, strides in words.
 * q_codes  uint32 [B, Hq, Wd] contiguous scratch.  Remaining arguments as in ucm_hamming_topk
 * with Hkv = 1.
 */
int ucm_sparse_decode_step_mla(const void* new_nope, int64_t nope_stride_t,
                               const void* new_rope, int64_t rope_stride_t, int64_t T,
                               const void* slot_mapping, int slot_is_i64,
                               const void* q_nope, int64_t qn_stride_b, int64_t qn_stride_h,
                               const void* q_rope, int64_t qr_stride_b, int64_t qr_stride_h,
                               int x_dtype, int32_t K_nope, int32_t K_rope,
                               const void* w_nope, const void* w_rope, int w_dtype,
                               int32_t N_nope_bits, int32_t N_rope_bits,
                               uint32_t* k_cache, int64_t NB, int32_t BS,
                               int64_t ks_block, int64_t ks_token,
                               const int32_t* block_table, int32_t table_stride, int32_t max_blocks,
                               const int32_t* seq_lens, int32_t B, int32_t Hq, int32_t k,
                               int32_t sink_tok, int32_t recent_tok, uint32_t flags,
                               uint32_t* q_codes, int32_t* out_idx, int32_t* out_score,
                               void* workspace, size_t workspace_bytes, ucm_stream_t stream);

/*
 * The per-layer decode work of the reference's GQA plugin in one call, with the outputs in the
 * form its attention backend reads: replaces GSAOnDevice.attention_begin at decode
 * (ucm/sparse/gsa_on_device/gsa_on_device.py:564-572 cache_k_hash_gqa_cuda, :396-412 hash_code,
 * :773-811 update_decode_topk_gqa_cuda) and cuda_hamming_topk / update_seq_lens
 * (hamming_topk.py:7-54) — a dozen framework launches there, three kernel launches here.
 *
 *   1. the codes of the step's new keys go to the paged code cache (as ucm_hash_encode_cache);
 *   2. the queries of every KV head's group are averaged (fp32 sum, times 1/G, rounded to the
 *      input type — what `query.view(B, Hkv, G, D).mean(2)` gives, gsa_on_device.py:400-406) and
 *      hashed: q_codes uint32 [B, Hkv, N_bits/32], contiguous scratch;
 *   3. blocks are scored against their KV head's code, the best head counts
 *      (UCM_TOPK_REDUCE_HEADS, hamming_topk.py:33), blocks holding a position < sink_tok or
 *      >= len - recent_tok are always kept, and the topk_tok / BS best blocks are selected;
 *   4. new_block_table[b, 0 .. max_blocks) = the selected physical ids in logical order, 0 in
 *      every other entry (gsa_on_device.py:789-791); new_seq_lens[b] = len - ceil(max(len -
 *      topk_tok, 0) / BS) * BS (hamming_topk.py:7-12).  A request with len < seq_len_threshold
 *      (threshold > 0) keeps its own table row and length.
 *
 * Arguments as in ucm_sparse_decode_step; new_block_table int32 [B, new_table_stride] with
 * new_table_stride >= max_blocks <= 4096, new_seq_lens int32 [B].  Requires topk_tok % BS == 0,
 * recent_tok > 0 and topk_tok > sink_tok + recent_tok (hamming_topk.py:30-31); bf16 / fp16 inputs
 * of 64, 128, 256 or 512 dimensions.  Allocates nothing.
 */
int ucm_gsa_decode_step(const void* new_keys, int64_t T, int64_t k_stride_t, int64_t k_stride_h,
                        const void* slot_mapping, int slot_is_i64,
                        const void* queries, int64_t q_stride_b, int64_t q_stride_h,
                        int x_dtype, int32_t K,
                        const void* w, int w_dtype, int32_t n_w, int32_t N_bits,
                        uint32_t* k_cache, int64_t NB, int32_t BS, int32_t Hkv,
                        int64_t ks_block, int64_t ks_token, int64_t ks_head,
                        const int32_t* block_table, int32_t table_stride, int32_t max_blocks,
                        const int32_t* seq_lens, int32_t B, int32_t Hq, int32_t topk_tok,
                        int32_t sink_tok, int32_t recent_tok, int32_t seq_len_threshold,
                        uint32_t* q_codes, int32_t* new_block_table, int32_t new_table_stride,
                        int32_t* new_seq_lens, void* workspace, size_t workspace_bytes,
                        ucm_stream_t stream);

/*
 * The same for the latent-attention (MLA) plugin: replaces GSAOnDevice.attention_begin at decode with
 * is_mla (ucm/sparse/gsa_on_device/gsa_on_device.py:426-455 cache_k_hash_mla_cuda, :376-393 the head
 * reduction of hash_code, :667-709 update_decode_topk_mla_cuda) - two compute_hash + concat_and_cache_mla
 * launches for the keys, two means, two compute_hash and a cat for the queries, the scorer, min, topk,
 * sort, gather, zeros_like and a slice assignment there; three kernel launches here.
 *
 *   1. both parts of the step's new latent keys are hashed and written side by side into the paged
 *      code cache (nope words first);
 *   2. the Hq query heads are reduced to Hq / reduction_head_num rows - row i is the mean of heads
 *      i, i + Hq / R, i + 2 Hq / R, ... (`view(T, R, Hq / R, D).mean(1)`: fp32 sum, times 1 / R,
 *      rounded to the input type) - and both parts hashed: q_codes uint32 [B, Hq / R, Wd];
 *   3. every block is scored with the sum over those rows, blocks holding a position < sink_tok or
 *      >= len - recent_tok are always kept, the topk_tok / BS best are selected;
 *   4. new_block_table / new_seq_lens / seq_len_threshold as in ucm_gsa_decode_step.
 *
 * Arguments as in ucm_sparse_decode_step_mla and ucm_gsa_decode_step; reduction_head_num >= 1 divides
 * Hq.  Allocates nothing.
 */
int ucm_gsa_decode_step_mla(const void* new_nope, int64_t nope_stride_t,
                            const void* new_rope, int64_t rope_stride_t, int64_t T,
                            const void* slot_mapping, int slot_is_i64,
                            const void* q_nope, int64_t qn_stride_b, int64_t qn_stride_h,
                            const void* q_rope, int64_t qr_stride_b, int64_t qr_stride_h,
                            int x_dtype, int32_t K_nope, int32_t K_rope,
                            const void* w_nope, const void* w_rope, int w_dtype,
                            int32_t N_nope_bits, int32_t N_rope_bits,
                            uint32_t* k_cache, int64_t NB, int32_t BS,
                            int64_t ks_block, int64_t ks_token,
                            const int32_t* block_table, int32_t table_stride, int32_t max_blocks,
                            const int32_t* seq_lens, int32_t B, int32_t Hq,
                            int32_t reduction_head_num, int32_t topk_tok,
                            int32_t sink_tok, int32_t recent_tok, int32_t seq_len_threshold,
                            uint32_t* q_codes, int32_t* new_block_table, int32_t new_table_stride,
                            int32_t* new_seq_lens, void* workspace, size_t workspace_bytes,
                            ucm_stream_t stream);

/* Replaces update_seq_lens (hamming_topk.py:7-12):
 * out[b] = len[b] - ceil(max(len[b] - topk_tok, 0) / BS) * BS. */
int ucm_update_seq_lens(const int32_t* seq_lens, int32_t B, int32_t topk_tok, int32_t BS,
                        int32_t* out, ucm_stream_t stream);

/* ------------------------------------------------------------------------------------
 * 3. KV block gather / scatter ("trans")
 * ------------------------------------------------------------------------------------ */

typedef struct ucm_trans_stream ucm_trans_stream_t;

/* Replaces UC::Trans::Device::Setup (ucm/shared/trans/cuda/cuda_device.cc:32-73):
 * make device_id current for the calling thread.  A negative or absent id fails. */
int ucm_trans_setup(int32_t device_id);

/* Stream kinds: copy-engine (Device::MakeStream, cuda_stream.cc:28-33) and
 * compute-unit kernel copies (Device::MakeSMStream, cuda_sm_stream.cc:29-55). */
#define UCM_TRANS_CE 0
#define UCM_TRANS_SM 1
int ucm_trans_stream_create(int kind, ucm_trans_stream_t** out);
int ucm_trans_stream_destroy(ucm_trans_stream_t* s);
/* the underlying hipStream_t */
void* ucm_trans_stream_handle(ucm_trans_stream_t* s);
/* Stream::Synchronized (cuda_stream.cc:151-156) */
int ucm_trans_stream_sync(ucm_trans_stream_t* s);
/* Stream::WaitEvent (cuda_stream.cc:158-164); event is a hipEvent_t, NULL is a no-op */
int ucm_trans_stream_wait_event(ucm_trans_stream_t* s, void* event);
/* Stream::AppendCallback (cuda_stream.cc:131-149): cb(ok, user) runs on a runtime thread
 * once all work enqueued so far has finished. */
int ucm_trans_stream_append_callback(ucm_trans_stream_t* s, void (*cb)(int ok, void* user),
                                     void* user);

/* Single copies, Stream::DeviceToHost[Async] / HostToDevice[Async] (cuda_stream.cc:35-40,
 * 56-61,82-87,103-108).  `sync` != 0 waits for completion. */
int ucm_trans_d2h(ucm_trans_stream_t* s, const void* device, void* host, size_t size, int sync);
int ucm_trans_h2d(ucm_trans_stream_t* s, const void* host, void* device, size_t size, int sync);

/*
 * Pointer-table copies of `number` chunks of `size` bytes
 * (cuda_stream.cc:63-80,110-127; cuda_sm_kernel.cu:52-114).
 *   gather : dst + i*size  <- src[i]
 *   scatter: dst[i]        <- src + i*size
 *   batch  : dst[i]        <- src[i]
 * table_on_device = 0: the pointer arrays are host arrays (read before the call returns);
 * table_on_device = 1: they already live in device-readable memory
 * (the SM-stream convention, ucm/shared/test/case/trans/trans_test.cc:84-89).
 * On an SM stream one kernel moves all chunks; the flat side may be device memory or
 * pinned/registered host memory.  On a CE stream one hipMemcpyAsync is issued per chunk.
 * Unlike the reference's kernel (cuda_sm_kernel.cu:56) a tail shorter than the copy unit
 * is copied, not dropped.
 */
int ucm_trans_gather(ucm_trans_stream_t* s, const void* const* src, int table_on_device,
                     void* dst, size_t size, size_t number, int sync);
int ucm_trans_scatter(ucm_trans_stream_t* s, const void* src, void* const* dst,
                      int table_on_device, size_t size, size_t number, int sync);
int ucm_trans_batch(ucm_trans_stream_t* s, const void* const* src, void* const* dst,
                    int table_on_device, size_t size, size_t number, int sync);

/*
 * Table-free form for a paged KV cache whose address rule is
 *   addr(block, col) = base[col] + block_id * col_bytes[col]
 * (KVCacheLayout.extract_block_addrs, ucm/integration/vllm/ucm_connector.py:91-148).
 * The flat buffer is laid out (block, col) row-major, column c of a block at the running
 * sum of col_bytes (dump_queue.cc:145-161).  base / col_bytes are host arrays of n_cols
 * entries; block_ids is a host array of n_blocks entries.  to_cache = 0 gathers cache ->
 * flat, 1 scatters flat -> cache.  SM streams only.  Ids that are negative, or not below
 * n_cache_blocks (the number of blocks every column holds; 0 = unknown, only the sign is
 * checked), are refused with UCM_EPARAM before anything is launched.
 */
int ucm_trans_paged_copy(ucm_trans_stream_t* s, const uint64_t* base, const uint64_t* col_bytes,
                         int32_t n_cols, const int32_t* block_ids, int64_t n_blocks,
                         int64_t n_cache_blocks, void* flat, int to_cache, int sync);

/* Buffer::MakeHostBuffer / MakeDeviceBuffer / RegisterHostBuffer
 * (ucm/shared/trans/buffer.h:32-47, cuda/cuda_buffer.cc:29-56). */
int ucm_trans_host_alloc(size_t size, void** out);
int ucm_trans_host_free(void* p);
int ucm_trans_device_alloc(size_t size, void** out);
int ucm_trans_device_free(void* p);
int ucm_trans_host_register(void* host, size_t size, void** device_alias);
int ucm_trans_host_unregister(void* host);

/* ------------------------------------------------------------------------------------
 * 3b. Float retrieval (ESA): dot-product top-k over a candidate list
 * ------------------------------------------------------------------------------------ */

/*
 * GPU form of the reference's ESA retrieval backend
 * (ucm/sparse/esa/retrieval/cpy/retrieval_backend.cpp:207-227; submit :83-113): for request b,
 * every candidate indexes[b, j] != -1 is scored with dot(query[b, :], data[candidate, :]) and
 * the min(n_candidates, topk) best are returned in descending score order.
 *
 * data      fp32 [n_items, dim] (block representatives), device memory, 16-byte aligned.
 * query     fp32 [B, dim], indexes int32 [B, max_n]; entries -1 or outside [0, n_items) are
 *           no candidates.  topk <= 4096, dim <= 16384.
 * out_idx   int32 [B, topk], out_score fp32 [B, topk]; positions past a request's candidate
 *           count hold -1 / 0.  Equal scores keep list order (the reference leaves ties open).
 * Scores are fp32 sums taken in a different order than the reference's sequential loop: they
 * agree to ~1e-6 relative to sum |q_d x_d|.
 */
size_t ucm_dot_topk_workspace_bytes(int32_t B, int32_t max_n);
int ucm_dot_topk(const float* data, int64_t n_items, int32_t dim, const float* query,
                 const int32_t* indexes, int32_t B, int32_t max_n, int32_t topk,
                 int32_t* out_idx, float* out_score, void* workspace, size_t workspace_bytes,
                 ucm_stream_t stream);

/*
 * GPU form of KVStar's block retrieval
 * (ucm/sparse/kvstar/retrieve/core/domain/retrieve_task/simd_compute_kernel.cpp:816-985;
 * submitted through AsyncRetrieveByCPU, py_intf/py_intf.cpp:13-52): attention-probability mass
 * per KV block for a group of query tokens, then the topk blocks.
 *
 * query         fp16 [X, Hq, d_orig] contiguous (the last X query tokens of the request).
 * blk_repre     fp16 [n_blocks, M, Hkv, d] contiguous: M representative keys per block.
 * pruned_index  int64 [Hkv, d] or NULL: channel j of KV head h's keys corresponds to channel
 *               pruned_index[h, j] of the queries; NULL requires d == d_orig.
 * For every (x, H): p = softmax over all n_blocks * M representatives of q[x, H] . k[s, H/g]
 * (left unnormalised when the sum of exponentials is <= 1e-9, as the reference does);
 * score[n] = sum of p over x, H and the M representatives of block n.
 * out_idx / out_score  [topk]: blocks by descending score, -1 / 0 past n_blocks; equal scores
 *               in ascending block order.  topk <= 4096, d <= 1024, X * Hq <= 65535.
 */
size_t ucm_kvstar_topk_workspace_bytes(int32_t X, int32_t Hq, int64_t n_blocks, int32_t M);
int ucm_kvstar_topk(const void* query, int32_t X, int32_t Hq, int32_t d_orig,
                    const void* blk_repre, int64_t n_blocks, int32_t M, int32_t Hkv, int32_t d,
                    const int64_t* pruned_index, int32_t topk,
                    int32_t* out_idx, float* out_score, void* workspace, size_t workspace_bytes,
                    ucm_stream_t stream);

/* ------------------------------------------------------------------------------------
 * 4. Cache store: pinned-host staging cache in front of a slower store backend — the caller
 *    of the gather / scatter path (ucm/store/cache/cc/).
 * ------------------------------------------------------------------------------------ */

typedef struct ucm_cache_store ucm_cache_store_t;

/*
 * The slower tier behind the staging cache: the part of the reference's StoreV1 interface
 * (ucm/store/ucmstore_v1.h) that CacheStore calls on its `store_backend`
 * (dump_queue.cc:129, load_queue.cc:103, buffer_manager.h:103).  All hooks may be NULL; with a
 * NULL table the pinned buffer is the only tier.  `block_ids` are n x 16 bytes, `host` holds n
 * pointers to shards of `shard_size` bytes in pinned memory that stays valid until wait()
 * returns.  dump/load return a positive handle, or a negative status.
 */
typedef struct ucm_cache_backend {
    void* ctx;
    int (*lookup)(void* ctx, const uint8_t* block_ids, size_t n, uint8_t* found);
    int64_t (*dump)(void* ctx, const uint8_t* block_ids, const uint64_t* shard_idx,
                    void* const* host, size_t n, size_t shard_size);
    int64_t (*load)(void* ctx, const uint8_t* block_ids, const uint64_t* shard_idx,
                    void* const* host, size_t n, size_t shard_size);
    int (*wait)(void* ctx, int64_t handle);
} ucm_cache_backend_t;

/*
 * CacheStore::Setup (cache_store.cc:37-57) with the fields of its Config
 * (global_config.h:33-48): a shard is the concatenation of `n_tensors` pieces of
 * `tensor_sizes[i]` bytes (tensor_size_list), `buffer_bytes` of pinned memory hold
 * buffer_bytes / shard_size shards (cache_buffer_capacity_gb), `waiting_queue_depth` bounds
 * the submitted-but-not-started tasks of each direction, `timeout_ms` is Wait's limit
 * (0 = 30000).  Starts the dump and load worker threads.
 */
int ucm_cache_store_create(int32_t device_id, const size_t* tensor_sizes, size_t n_tensors,
                           size_t buffer_bytes, size_t waiting_queue_depth, size_t timeout_ms,
                           const ucm_cache_backend_t* backend, ucm_cache_store_t** out);
int ucm_cache_store_destroy(ucm_cache_store_t* store);
/* staging nodes the buffer holds */
size_t ucm_cache_store_nodes(ucm_cache_store_t* store);

/* CacheStore::Lookup / LookupOnPrefix (cache_store.cc:59-70, buffer_manager.h:66-127):
 * found[i] = block i is in the staging cache (its shard 0) or in the backend;
 * *last_found = index of the last block of the leading run that is present, -1 if none. */
int ucm_cache_store_lookup(ucm_cache_store_t* store, const uint8_t* block_ids, size_t n,
                           uint8_t* found);
int ucm_cache_store_lookup_on_prefix(ucm_cache_store_t* store, const uint8_t* block_ids, size_t n,
                                     int64_t* last_found);

/*
 * CacheStore::Dump / Load (cache_store.cc:72-89; DumpQueue::DumpOneTask dump_queue.cc:92-143,
 * LoadQueue::DispatchOneTask / TransferOneTask load_queue.cc:77-160).  A task is n shards;
 * shard i is (block_ids[16 i .. 16 i + 15], shard_idx[i]) and lives on the device as n_tensors
 * pieces at device_addrs[i * n_tensors + t].  Both calls only enqueue and return a task id.
 * Dump: waits for `prerequisite_event` (hipEvent_t, may be NULL) on the store's stream, copies
 * every shard that no other task is already staging into its pinned node with one kernel
 * launch, then hands the nodes to the backend.  Load: shards that are not resident are first
 * fetched from the backend into their node; the task fails if one is in neither tier.
 */
int ucm_cache_store_dump(ucm_cache_store_t* store, const uint8_t* block_ids,
                         const uint64_t* shard_idx, void* const* device_addrs, size_t n,
                         void* prerequisite_event, int64_t* task);
int ucm_cache_store_load(ucm_cache_store_t* store, const uint8_t* block_ids,
                         const uint64_t* shard_idx, void* const* device_addrs, size_t n,
                         int64_t* task);
/* CacheStore::Check / Wait (cache_store.cc:90-101; task_wrapper.h:62-107): Check reports
 * whether the task has finished (either way); Wait blocks up to timeout_ms, forgets the task
 * and returns UCM_OK, UCM_ERROR (the task failed), UCM_ETIMEOUT or UCM_ENOOBJ (unknown id). */
int ucm_cache_store_check(ucm_cache_store_t* store, int64_t task, int* finished);
int ucm_cache_store_wait(ucm_cache_store_t* store, int64_t task);

/* ======================================================================================
 * 5. Posix store: one file per block in the reference's on-disk format
 *    (ucm/store/posix/cc/).  Host-only: addresses are host pointers and no GPU is needed.
 *
 *    File of a block = <backend>/<dir>/<32 lowercase hex digits of the 16-byte id>, where
 *    <dir> is the first data_dir_shard_bytes digits of the name, or "data" when that is 0
 *    (space_layout.cc:88-99); with several backends the block lives in backend
 *    std::hash<std::string_view>(id) % n (space_layout.cc:164-170).  Shard `index` is the byte
 *    range [index * shard_size, (index + 1) * shard_size): its tensors, tensor_size bytes each,
 *    one after the other (trans_queue.cc:127-169).  A file is written as <name>.tmp and
 *    renamed when the block's last shard has been written (trans_queue.cc:117-119,
 *    space_layout.cc:101-111).
 * ====================================================================================== */
typedef struct ucm_posix_store ucm_posix_store_t;

/* Fields of the reference's Config (posix/cc/global_config.h:33-56) under the names of its
 * dictionary keys (posix_store.cc:104-129).  capacity_bytes stands for posix_capacity_gb. */
typedef struct ucm_posix_config {
    const char* const* storage_backends; /* existing directories; the first one gets the shard
                                            directories created, the others must hold them */
    size_t n_backends;
    int32_t device_id;             /* >= 0: dump / load enabled; -1: lookup only, and blocks
                                      found by a lookup get their mtime refreshed */
    int32_t io_direct;             /* O_DIRECT: addresses, sizes and offsets 4096-aligned */
    size_t tensor_size, shard_size, block_size;
    size_t data_trans_concurrency; /* threads per direction (posix_data_trans_concurrency) */
    size_t lookup_concurrency;     /* posix_lookup_concurrency */
    size_t timeout_ms;             /* 0 = 30000 */
    size_t data_dir_shard_bytes;   /* 0..5 hex digits of directory sharding */
    int32_t gc_enable;             /* posix_gc_enable; active only with capacity_bytes > 0 */
    int32_t reserved;
    size_t capacity_bytes;
    double gc_recycle_percent;            /* share of a directory's files removed per pass */
    double gc_trigger_threshold_ratio;    /* of capacity / block_size / directories */
    double gc_shard_sample_ratio;         /* directories counted to decide */
    size_t gc_max_recycle_count_per_shard;
    size_t gc_check_interval_sec;
} ucm_posix_config_t;

/* PosixStore::Setup (posix_store.cc:37-56) incl. CheckConfig (:131-193): UCM_EPARAM for the
 * configurations the reference rejects. */
int ucm_posix_store_create(const ucm_posix_config_t* config, ucm_posix_store_t** out);
int ucm_posix_store_destroy(ucm_posix_store_t* store);
/* SpaceLayout::DataFilePath (space_layout.cc:88-99): the path of the block's file, with the
 * ".tmp" suffix when `activated`.  Returns the path length (the text is cut to cap - 1). */
int64_t ucm_posix_store_data_file_path(ucm_posix_store_t* store, const uint8_t* block_id,
                                       int32_t activated, char* buf, size_t cap);
/* SpaceLayout::CommitFile (space_layout.cc:101-111): rename <name>.tmp to <name>
 * (success != 0) or remove it.  UCM_ENOOBJ when there is no such .tmp file. */
int ucm_posix_store_commit(ucm_posix_store_t* store, const uint8_t* block_id, int32_t success);
/* SpaceManager::LookupOnPrefix / Lookup (space_manager.cc:56-95): *last_found = index of the
 * last block of the leading run whose files exist (readable and writable), -1 if none;
 * found[i] = i <= *last_found (blocks after the first miss are reported absent). */
int ucm_posix_store_lookup_on_prefix(ucm_posix_store_t* store, const uint8_t* block_ids, size_t n,
                                     int64_t* last_found);
int ucm_posix_store_lookup(ucm_posix_store_t* store, const uint8_t* block_ids, size_t n,
                           uint8_t* found);
/* PosixStore::Dump / Load (posix_store.cc:75-93; TransQueue trans_queue.cc:66-169): shard i is
 * (block_ids[16 i ..], shard_idx[i]) with shard_size / tensor_size host addresses at
 * host_addrs[i * tensors_per_shard + t].  Both only enqueue and return a task id. */
int ucm_posix_store_dump(ucm_posix_store_t* store, const uint8_t* block_ids,
                         const uint64_t* shard_idx, void* const* host_addrs, size_t n,
                         int64_t* task);
int ucm_posix_store_load(ucm_posix_store_t* store, const uint8_t* block_ids,
                         const uint64_t* shard_idx, void* const* host_addrs, size_t n,
                         int64_t* task);
/* PosixStore::Check / Wait (posix_store.cc:94-103): as ucm_cache_store_check / _wait.  A wait that
 * times out does not return while a file worker may still read or write the task's buffers: it waits
 * up to four more time-outs for them to come back (queued units are skipped).  Normally it then
 * returns UCM_ETIMEOUT and forgets the task; if the workers are still stuck (a dead mount) it
 * returns UCM_ERETRY, keeps the task, and the buffers must not be reused or freed until a later wait
 * on the same task has returned something else. */
int ucm_posix_store_check(ucm_posix_store_t* store, int64_t task, int32_t* finished);
int ucm_posix_store_wait(ucm_posix_store_t* store, int64_t task);
/* One turn of the collector's loop now (ShardGarbageCollector::GCCheckLoop, shard_gc.cc:85-108):
 * sample directories, and while the average file count is at or above the threshold remove
 * each directory's oldest files by mtime.  *removed = files removed by this call. */
int ucm_posix_store_gc_once(ucm_posix_store_t* store, uint64_t* removed);
/* Fills the hooks that put this store beneath a cache store (the reference's "Cache|Posix"
 * pipeline, ucm/store/pipeline/connector.py:180-188; there as here the posix store is then
 * configured with tensor_size = shard_size).  `store` must outlive the cache store. */
int ucm_posix_store_backend(ucm_posix_store_t* store, ucm_cache_backend_t* out);

#ifdef __cplusplus
}
#endif
#endif /* UCM_HIP_H */
