// torch.ops.ucm_amd.*: the operators of the C ABI registered with PyTorch's dispatcher, so that
// callers that go through torch.ops (graph capture frameworks, torch.compile custom-op plumbing,
// C++ callers holding at::Tensor) reach the same kernels as the ctypes mirror.  This file contains
// no kernel and no arithmetic: every operator checks shapes, takes raw pointers, strides and the
// current stream out of its tensors and forwards them to libucm_hip.so.
//
// Counterparts in the reference: TORCH_LIBRARY registration of the NPU operator
// (ucm/sparse/gsa_on_device/csrc/ascend/torch_binding.cpp:39-79) and the pybind module of the CUDA
// scorer (ucm/sparse/gsa_on_device/csrc/cuda/ham_dist/cpy/hamming.cpp:4-6).
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <tuple>

#include "ucm_hip.h"

namespace {

int dtype_code(const at::Tensor& t)
{
    switch (t.scalar_type()) {
        case at::kBFloat16: return UCM_DT_BF16;
        case at::kHalf: return UCM_DT_F16;
        case at::kFloat: return UCM_DT_F32;
        default: TORCH_CHECK(false, "ucm_amd: unsupported element type ", t.scalar_type());
    }
}

void check_status(int rc, const char* what)
{
    TORCH_CHECK(rc == UCM_OK, "ucm_amd::", what, " failed (", rc, "): ", ucm_last_error());
}

ucm_stream_t current_stream(const at::Tensor& t)
{
    return (ucm_stream_t)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

void check_i32(const at::Tensor& t, const char* name)
{
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt, "ucm_amd: ", name, " must be an int32 tensor on the GPU");
}

// x [T, H, K]; w [K, N] or [n_w, K, N]; slot_mapping int32/int64 [T]; cache int32 [NB, BS, H, N / 32]
void hash_encode_cache(const at::Tensor& x, const at::Tensor& w, const at::Tensor& slot_mapping, at::Tensor cache)
{
    TORCH_CHECK(x.is_cuda() && x.dim() == 3 && x.stride(2) == 1, "ucm_amd: x must be [T, H, K] with contiguous rows");
    TORCH_CHECK(w.is_cuda() && (w.dim() == 2 || w.dim() == 3) && w.is_contiguous(), "ucm_amd: w must be [K, N] or [n_w, K, N]");
    check_i32(cache, "cache");
    TORCH_CHECK(cache.dim() == 4 && cache.stride(3) == 1, "ucm_amd: cache must be int32 [NB, BS, H, N / 32]");
    const int64_t T = x.size(0), H = x.size(1), K = x.size(2);
    const int64_t n_w = w.dim() == 3 ? w.size(0) : 1, N = w.size(-1);
    TORCH_CHECK(w.size(-2) == K && N % 32 == 0 && cache.size(2) == H && cache.size(3) == N / 32, "ucm_amd: shapes disagree");
    TORCH_CHECK(n_w == 1 || H % n_w == 0, "ucm_amd: heads must divide over the projections");
    TORCH_CHECK(slot_mapping.is_cuda() && slot_mapping.is_contiguous() && slot_mapping.numel() == T &&
                    (slot_mapping.scalar_type() == at::kInt || slot_mapping.scalar_type() == at::kLong),
                "ucm_amd: slot_mapping must be a contiguous int32 / int64 [T] tensor");
    check_status(ucm_hash_encode_cache(x.data_ptr(), dtype_code(x), T, (int32_t)H, (int32_t)K, x.stride(0), x.stride(1),
                                       w.data_ptr(), dtype_code(w), (int32_t)n_w, n_w > 1 ? (int32_t)(H / n_w) : 0,
                                       (int32_t)N, slot_mapping.data_ptr(), slot_mapping.scalar_type() == at::kLong,
                                       (uint32_t*)cache.data_ptr(), cache.size(0), (int32_t)cache.size(1),
                                       cache.stride(0), cache.stride(1), cache.stride(2), current_stream(x)),
                 "hash_encode_cache");
}

// q_codes int32 [B, Hq, Wd]; k_cache int32 [NB, BS, Hkv, Wd]; block_table int32 [B, max_blocks];
// seq_lens int32 [B]; flags = UCM_TOPK_* of ucm_hip.h.  Returns (indices, scores) int32 [B, Hkv | 1, k].
std::tuple<at::Tensor, at::Tensor> hamming_topk(const at::Tensor& q_codes, const at::Tensor& k_cache,
                                                const at::Tensor& block_table, const at::Tensor& seq_lens, int64_t k,
                                                int64_t sink_tok, int64_t recent_tok, int64_t flags)
{
    check_i32(q_codes, "q_codes");
    check_i32(k_cache, "k_cache");
    check_i32(block_table, "block_table");
    check_i32(seq_lens, "seq_lens");
    TORCH_CHECK(q_codes.dim() == 3 && q_codes.stride(2) == 1 && k_cache.dim() == 4 && k_cache.stride(3) == 1,
                "ucm_amd: q_codes [B, Hq, Wd] and k_cache [NB, BS, Hkv, Wd] with contiguous codes");
    TORCH_CHECK(block_table.dim() == 2 && block_table.stride(1) == 1 && seq_lens.is_contiguous(), "ucm_amd: table / lengths layout");
    const int64_t B = q_codes.size(0), Hq = q_codes.size(1), Wd = q_codes.size(2);
    const int64_t NB = k_cache.size(0), BS = k_cache.size(1), Hkv = k_cache.size(2);
    TORCH_CHECK(k_cache.size(3) == Wd && block_table.size(0) == B && seq_lens.numel() == B, "ucm_amd: shapes disagree");
    const int64_t max_blocks = block_table.size(1);
    const int64_t Ho = (flags & UCM_TOPK_REDUCE_HEADS) ? 1 : Hkv;
    at::Tensor idx = at::empty({B, Ho, k}, q_codes.options());
    at::Tensor score = at::empty({B, Ho, k}, q_codes.options());
    const size_t ws_bytes = ucm_hamming_topk_workspace_bytes((int32_t)B, (int32_t)Hkv, (int32_t)max_blocks);
    at::Tensor ws = at::empty({(int64_t)ws_bytes}, q_codes.options().dtype(at::kByte));
    check_status(ucm_hamming_topk((const uint32_t*)q_codes.data_ptr(), q_codes.stride(0), q_codes.stride(1),
                                  (const uint32_t*)k_cache.data_ptr(), NB, (int32_t)BS, (int32_t)Hkv, (int32_t)Wd,
                                  k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
                                  (const int32_t*)block_table.data_ptr(), (int32_t)block_table.stride(0),
                                  (int32_t)max_blocks, (const int32_t*)seq_lens.data_ptr(), (int32_t)B, (int32_t)Hq,
                                  (int32_t)k, (int32_t)sink_tok, (int32_t)recent_tok, (uint32_t)flags,
                                  (int32_t*)idx.data_ptr(), (int32_t*)score.data_ptr(), ws.data_ptr(), ws_bytes,
                                  current_stream(q_codes)),
                 "hamming_topk");
    return {idx, score};
}

// The GQA plugin's decode hook (ucm_gsa_decode_step): new_keys [T, Hkv, K] (T may be 0), slot_mapping
// [T], queries [B, Hq, K], w [K, N] or [Hkv, K, N], k_cache int32 [NB, BS, Hkv, N / 32] (updated in
// place).  Returns (new_block_table int32 [B, max_blocks], new_seq_lens int32 [B]).
std::tuple<at::Tensor, at::Tensor> gsa_decode_step(const at::Tensor& new_keys, const at::Tensor& slot_mapping,
                                                   const at::Tensor& queries, const at::Tensor& w, at::Tensor k_cache,
                                                   const at::Tensor& block_table, const at::Tensor& seq_lens,
                                                   int64_t topk_tok, int64_t sink_tok, int64_t recent_tok,
                                                   int64_t seq_len_threshold)
{
    check_i32(k_cache, "k_cache");
    check_i32(block_table, "block_table");
    check_i32(seq_lens, "seq_lens");
    TORCH_CHECK(queries.is_cuda() && queries.dim() == 3 && queries.stride(2) == 1, "ucm_amd: queries must be [B, Hq, K]");
    TORCH_CHECK(w.is_cuda() && (w.dim() == 2 || w.dim() == 3) && w.is_contiguous(), "ucm_amd: w must be [K, N] or [Hkv, K, N]");
    TORCH_CHECK(k_cache.dim() == 4 && k_cache.stride(3) == 1 && block_table.dim() == 2 && block_table.stride(1) == 1 &&
                    seq_lens.is_contiguous(),
                "ucm_amd: cache / table / lengths layout");
    const int64_t B = queries.size(0), Hq = queries.size(1), K = queries.size(2);
    const int64_t NB = k_cache.size(0), BS = k_cache.size(1), Hkv = k_cache.size(2), Wd = k_cache.size(3);
    const int64_t n_w = w.dim() == 3 ? w.size(0) : 1, N = w.size(-1);
    const int64_t T = new_keys.numel() ? new_keys.size(0) : 0;
    TORCH_CHECK(N == 32 * Wd && w.size(-2) == K && block_table.size(0) == B && seq_lens.numel() == B, "ucm_amd: shapes disagree");
    if (T) {
        TORCH_CHECK(new_keys.is_cuda() && new_keys.dim() == 3 && new_keys.size(1) == Hkv && new_keys.size(2) == K &&
                        new_keys.stride(2) == 1 && new_keys.scalar_type() == queries.scalar_type(),
                    "ucm_amd: new_keys must be [T, Hkv, K] of the queries' type");
        TORCH_CHECK(slot_mapping.is_cuda() && slot_mapping.is_contiguous() && slot_mapping.numel() == T &&
                        (slot_mapping.scalar_type() == at::kInt || slot_mapping.scalar_type() == at::kLong),
                    "ucm_amd: slot_mapping must be a contiguous int32 / int64 [T] tensor");
    }
    const int64_t max_blocks = block_table.size(1);
    at::Tensor q_codes = at::empty({B, Hkv, Wd}, k_cache.options());
    at::Tensor new_table = at::empty({B, max_blocks}, block_table.options());
    at::Tensor new_lens = at::empty({B}, seq_lens.options());
    const size_t ws_bytes = ucm_hamming_topk_workspace_bytes((int32_t)B, (int32_t)Hkv, (int32_t)max_blocks);
    at::Tensor ws = at::empty({(int64_t)ws_bytes}, k_cache.options().dtype(at::kByte));
    check_status(ucm_gsa_decode_step(T ? new_keys.data_ptr() : nullptr, T, T ? new_keys.stride(0) : 0, T ? new_keys.stride(1) : 0,
                                     T ? slot_mapping.data_ptr() : nullptr, T && slot_mapping.scalar_type() == at::kLong,
                                     queries.data_ptr(), queries.stride(0), queries.stride(1), dtype_code(queries),
                                     (int32_t)K, w.data_ptr(), dtype_code(w), (int32_t)n_w, (int32_t)N,
                                     (uint32_t*)k_cache.data_ptr(), NB, (int32_t)BS, (int32_t)Hkv, k_cache.stride(0),
                                     k_cache.stride(1), k_cache.stride(2), (const int32_t*)block_table.data_ptr(),
                                     (int32_t)block_table.stride(0), (int32_t)max_blocks,
                                     (const int32_t*)seq_lens.data_ptr(), (int32_t)B, (int32_t)Hq, (int32_t)topk_tok,
                                     (int32_t)sink_tok, (int32_t)recent_tok, (int32_t)seq_len_threshold,
                                     (uint32_t*)q_codes.data_ptr(), (int32_t*)new_table.data_ptr(), (int32_t)max_blocks,
                                     (int32_t*)new_lens.data_ptr(), ws.data_ptr(), ws_bytes, current_stream(queries)),
                 "gsa_decode_step");
    return {new_table, new_lens};
}

}  // namespace

TORCH_LIBRARY(ucm_amd, m)
{
    m.def("hash_encode_cache(Tensor x, Tensor w, Tensor slot_mapping, Tensor(a!) cache) -> ()");
    m.def("hamming_topk(Tensor q_codes, Tensor k_cache, Tensor block_table, Tensor seq_lens, int k, int sink_tok, "
          "int recent_tok, int flags) -> (Tensor, Tensor)");
    m.def("gsa_decode_step(Tensor new_keys, Tensor slot_mapping, Tensor queries, Tensor w, Tensor(a!) k_cache, "
          "Tensor block_table, Tensor seq_lens, int topk_tok, int sink_tok, int recent_tok, int seq_len_threshold) "
          "-> (Tensor, Tensor)");
}

// "CUDA" is the dispatch key of GPU tensors in the ROCm build as well
TORCH_LIBRARY_IMPL(ucm_amd, CUDA, m)
{
    m.impl("hash_encode_cache", &hash_encode_cache);
    m.impl("hamming_topk", &hamming_topk);
    m.impl("gsa_decode_step", &gsa_decode_step);
}
