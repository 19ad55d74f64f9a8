// Shared host-side helpers of the HIP library: status codes, per-thread error text,
// HIP error translation.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "ucm_hip.h"

namespace ucm {

// Stores a printf-formatted message for ucm_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

inline int hip_fail(hipError_t e, const char* what)
{
    // hipGetLastError() resets the sticky error so that a later, unrelated call does not
    // report this failure again.
    (void)hipGetLastError();
    return fail(e == hipErrorOutOfMemory ? UCM_EOOM : UCM_ERROR, "%s: %s", what,
                hipGetErrorString(e));
}

#define UCM_HIP_TRY(expr)                                          \
    do {                                                           \
        hipError_t e__ = (expr);                                   \
        if (e__ != hipSuccess) return ::ucm::hip_fail(e__, #expr); \
    } while (0)

#define UCM_REQUIRE(cond, ...)                                        \
    do {                                                              \
        if (!(cond)) return ::ucm::fail(UCM_EPARAM, __VA_ARGS__);     \
    } while (0)

inline int launch_status(const char* kernel)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(UCM_ERROR, "launch of %s failed: %s", kernel, hipGetErrorString(e));
    return UCM_OK;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// hash_encode.hip: one (new keys -> paged cache, queries -> codes) pair of a decode step.
// Strides of keys and queries in elements, of the cache and of q_codes in 32-bit words.
struct PairSpec {
    const void* keys; int64_t T; int Hkv; int64_t k_stride_t, k_stride_h;
    const void* slot; int slot_is_i64;
    uint32_t* cache; int64_t NB; int BS; int64_t cs_block, cs_token, cs_head;
    const void* queries; int64_t B; int Hq; int64_t q_stride_b, q_stride_h;
    uint32_t* q_codes; int64_t qc_stride_b, qc_stride_h;
    int x_dtype; int K; const void* w; int w_dtype; int n_w; int N_bits;
    int q_group_mean = 0;  // hash the mean of every KV head's query group: q_codes is [B, Hkv, Wd]
    // latent attention's head reduction: query row i of the Hq / q_reduce that are hashed is the mean
    // of heads i, i + Hq / q_reduce, i + 2 * Hq / q_reduce, ... (q_codes is [B, Hq / q_reduce, Wd])
    int q_reduce = 0;
};
// one launch when both jobs are small
int encode_pair(const PairSpec& p, hipStream_t st);
// two pairs; one launch when all four jobs are small and the input widths are 512 and 64
int encode_two_pairs(const PairSpec& a, const PairSpec& b, hipStream_t st);

}  // namespace ucm
