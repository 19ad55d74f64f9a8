// Sign-hash encoder for gfx950: codes = pack_lsb_first(x . W > 0), optionally scattered into
// the paged code cache.
//
// Follows the reference's HashEncoder (ucm/sparse/gsa_on_device/hash_encoder.py:359-370 for
// the arithmetic and bit order, :263-356 for the fused cache write, :136-195 for the code
// scatter).  Design for MI355X:
//   * bf16 / fp16 inputs go through v_mfma_f32_32x32x16_{bf16,f16}; a wave owns 32 rows and
//     walks the hash columns 32 at a time; the projection matrix slice lives in LDS, transposed
//     so that an operand is one 16-byte LDS read;
//   * rows are fetched with fully coalesced loads (8 rows x one 128-byte line per instruction,
//     two row tiles in flight per wave) and redistributed to the MFMA operand layout through a
//     swizzled 4 KiB LDS patch per wave: loading straight in operand layout touches every
//     cache line from four instructions and costs about a third of the bandwidth;
//   * the MFMA runs transposed (projection matrix as A, input rows as B), so a lane's 16
//     accumulators are 16 hash bits of one row: the signs are packed in-lane, interleaved with
//     the next column tile's MFMAs, and one half-wave swap joins the two halves of a word;
//   * the row's words are written with one store, either to a dense [T,H,Wd] tensor or to
//     cache[slot/BS, slot%BS, h, :].
// Everything else (fp32 operands, odd shapes, unaligned rows) takes a plain FMA kernel.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <atomic>
#include <mutex>

#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerWave = 32;
constexpr int kMfmaThreads = 256;                                // encode_mfma_kernel workgroup
constexpr int kMfmaWaves = kMfmaThreads / 64;
constexpr int kRowsPerWg = kMfmaWaves * kRowsPerWave;            // 128 rows per workgroup tile
constexpr int kTilesPerWg = 4;                                   // row tiles a workgroup encodes
constexpr int kStageBytes = kRowsPerWave * 128;                  // per wave: one 128-byte line of 32 rows
constexpr int kPad = 8;  // elements of padding per LDS row (16 bytes)

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct EncArgs {
    const void* x;
    int64_t T;
    int H, K;
    int64_t x_stride_t, x_stride_h;
    // paged input (src_blocks != null): row t is token t % BS of block src_blocks[t / BS] of a
    // [NBsrc, BS, H, K] tensor with block stride xs_block; its code goes to the same block and
    // token of the code cache
    const int32_t* src_blocks;
    int64_t xs_block, NBsrc;
    const void* w;
    int n_w, heads_per_w, N;
    // dense output (host side only: normalize_output() folds it into the paged form)
    uint32_t* out;
    int64_t out_stride_t, out_stride_h;
    // paged output; slot == null means slot(t) = t
    const void* slot;
    int slot_is_i64;
    uint32_t* cache;
    int64_t NB;
    int BS;
    int64_t cs_block, cs_token, cs_head;
    int BN;        // hash columns per workgroup slice
    // group mean (small-row kernel only): row (t, h) is the mean of the gmean source rows
    // (t, h * gmean + g) at x_stride_g elements from one another, rounded to the input type as
    // a framework's mean over the group would be; 0 or 1 = plain rows
    int gmean;
    int64_t x_stride_g;
    int bs_shift;  // log2(BS) when BS is a power of two, else -1
    // log2 of N / 32, of H and of heads_per_w where these are powers of two, else -1: the small-row
    // kernels decode a tile index with shifts then (an integer division is some forty instructions,
    // and a tile runs five of them, one wave to a SIMD, in front of its first load)
    int nt_shift, h_shift, hpw_shift;
    // streaming kernel: a word in pinned host memory that a wave sets when one of its bounded waits
    // gives up; the host reads it without touching the device (see stream_latch_tripped())
    unsigned int* timeout_flag;
};

__device__ __forceinline__ int weight_index(const EncArgs& a, int h)
{
    int wi = a.heads_per_w > 0 ? h / a.heads_per_w : 0;
    return wi < a.n_w ? wi : a.n_w - 1;
}

// t -> (t / BS, t % BS) without a division when BS is a power of two.
__device__ __forceinline__ void split_token(const EncArgs& a, int64_t t, int64_t& blk, int64_t& tok)
{
    if (a.bs_shift >= 0) {
        blk = t >> a.bs_shift;
        tok = t & (a.BS - 1);
    } else if (t < 0x7fffffff) {
        blk = (uint32_t)t / (uint32_t)a.BS;
        tok = (uint32_t)t % (uint32_t)a.BS;
    } else {
        blk = t / a.BS;
        tok = t % a.BS;
    }
}

// Element offset of input row (t, h); for a paged input an unusable block id reads block 0
// (the row is dropped when it is stored).
__device__ __forceinline__ int64_t src_offset(const EncArgs& a, int64_t t, int h)
{
    if (!a.src_blocks) return t * a.x_stride_t + (int64_t)h * a.x_stride_h;
    int64_t bi, tok;
    split_token(a, t, bi, tok);
    int64_t blk = a.src_blocks[bi];
    if (blk < 0 || blk >= a.NBsrc) blk = 0;
    return blk * a.xs_block + tok * a.x_stride_t + (int64_t)h * a.x_stride_h;
}

// A dense [T, H, Wd] output is handled as a paged one with one token per block and the
// identity slot mapping (normalize_output() on the host), so the kernels know one layout.
//
// Raw slot of row t as read from memory: the row index itself when there is no slot array.
// Split from the address arithmetic so that a kernel can issue the read long before it needs
// the value; a 32-bit slot is widened only in slot_dst().
struct RawSlot {
    uint32_t lo, hi;
};
__device__ __forceinline__ RawSlot fetch_slot(const EncArgs& a, int64_t t)
{
    RawSlot s;
    if (a.src_blocks) {
        int64_t bi, tok;
        split_token(a, t, bi, tok);
        s.lo = (uint32_t)a.src_blocks[bi];
        s.hi = 0;
    } else if (!a.slot) {
        s.lo = (uint32_t)t;
        s.hi = (uint32_t)((uint64_t)t >> 32);
    } else if (a.slot_is_i64) {
        const uint2 v = ((const uint2*)a.slot)[t];
        s.lo = v.x;
        s.hi = v.y;
    } else {
        s.lo = ((const uint32_t*)a.slot)[t];
        s.hi = 0;
    }
    return s;
}

// Branch-free variant for a kernel that prefetches slots: two unconditional 4-byte reads whose
// results land in fixed registers (a value merged from several branches would have to be
// waited for at the merge).  Without a slot array the reads hit the input rows instead (valid
// memory: the caller guarantees rows of at least 16 bytes) and slot_value() ignores them.
__device__ __forceinline__ RawSlot fetch_slot_flat(const EncArgs& a, int64_t t)
{
    const char* p = a.slot ? (const char*)a.slot : (const char*)a.x;
    int sh = a.slot_is_i64 ? 3 : 2;
    int hi_off = a.slot_is_i64 ? 4 : 0;
    int64_t i = t;
    if (a.src_blocks) {  // the "slot array" of a paged input is its block list
        int64_t tok;
        split_token(a, t, i, tok);
        p = (const char*)a.src_blocks;
        sh = 2;
        hi_off = 0;
    }
    const char* q = p + (i << sh);
    RawSlot s;
    s.lo = *(const uint32_t*)q;
    s.hi = *(const uint32_t*)(q + hi_off);
    return s;
}

// Destination of the code words of head h of the row with slot s, or null when the row must
// be skipped (slot outside the cache).
__device__ __forceinline__ uint32_t* slot_dst(const EncArgs& a, int64_t s, int h)
{
    if (s < 0 || s >= a.NB * (int64_t)a.BS) return nullptr;
    int64_t blk, tok;
    if (a.bs_shift >= 0) {  // the usual case: no integer division
        blk = s >> a.bs_shift;
        tok = s & (a.BS - 1);
    } else if (s < 0x7fffffff) {
        blk = (uint32_t)s / (uint32_t)a.BS;
        tok = (uint32_t)s % (uint32_t)a.BS;
    } else {
        blk = s / a.BS;
        tok = s % a.BS;
    }
    return a.cache + blk * a.cs_block + tok * a.cs_token + (int64_t)h * a.cs_head;
}

// Slot value of row t from its raw words.
__device__ __forceinline__ int64_t slot_value(const EncArgs& a, RawSlot raw, int64_t t)
{
    if (a.src_blocks) {
        const int64_t blk = (int32_t)raw.lo;
        if (blk < 0 || blk >= a.NBsrc) return -1;
        int64_t bi, tok;
        split_token(a, t, bi, tok);
        return blk * a.BS + tok;
    }
    if (!a.slot) return t;
    return a.slot_is_i64 ? (int64_t)(((uint64_t)raw.hi << 32) | raw.lo) : (int64_t)(int32_t)raw.lo;
}

__device__ __forceinline__ uint32_t* row_dst(const EncArgs& a, int64_t t, int h)
{
    return slot_dst(a, slot_value(a, fetch_slot(a, t), t), h);
}

// The MFMA is issued with the projection matrix as its A operand and the input rows as B, so
// accumulator register v of lane l is hash column 8*(v/4) + 4*(l/32) + v%4 of input row l%32:
// a lane holds 16 of the 32 sign bits of ONE row's output word and packs them in-lane.
// Plain C++ on purpose: the wait states between an MFMA and the first read of its result, and
// between a compare and the use of its mask, are inserted by the compiler only for
// instructions it can see.
//
// The matrix-core kernels start every accumulator at the smallest negative normal number
// instead of zero.  A projection that is exactly zero (an all-zero row) then stays negative,
// any other projection keeps its sign (|p| would have to be below 1.2e-38 to lose it), and
// "projection > 0" becomes "sign bit clear": one funnel shift per accumulator instead of a
// compare, a select and an or.  NaN is the one value whose sign bit says nothing; a row with a
// NaN input has NaN in every accumulator, so one accumulator per row is tested and the row's
// bits are cleared, as `NaN > 0` is false.
constexpr float kAccStart = -1.17549435e-38f;

__device__ __forceinline__ f32x16 acc_start()
{
    f32x16 a;
#pragma unroll
    for (int i = 0; i < 16; ++i) a[i] = kAccStart;
    return a;
}

// Half of the row's word: bit 8g + j is "accumulator 4g + j is positive" (g, j in 0..3).  Two
// independent chains (g = 3,2 and g = 1,0) halve the dependent-instruction latency.
__device__ __forceinline__ uint32_t pack_half(const f32x16& acc)
{
    uint32_t hi = 0, lo = 0;  // collect the sign bits: x = (x << 1) | sign
#pragma unroll
    for (int g = 1; g >= 0; --g) {
        if (g == 0) {
            hi <<= 4;
            lo <<= 4;
        }
#pragma unroll
        for (int j = 3; j >= 0; --j) {
            hi = __builtin_amdgcn_alignbit(hi, __float_as_uint(acc[4 * (g + 2) + j]), 31);
            lo = __builtin_amdgcn_alignbit(lo, __float_as_uint(acc[4 * g + j]), 31);
        }
    }
    // positive = sign bit clear: flip the 16 collected bits
    const uint32_t neg = (hi << 16) | lo;
    const uint32_t word = neg ^ 0x0F0F0F0Fu;
    return acc[0] != acc[0] ? 0u : word;
}

// Lanes l and l+32 hold the two interleaved halves (nibbles 0,2,4,6 and 1,3,5,7) of row l%32's
// word; `w` must already be shifted left by 4 in the upper lanes.  Returns the full word in both.
__device__ __forceinline__ uint32_t join_halves(uint32_t w)
{
    const auto r = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return r[0] | r[1];
}

template <typename V>
struct Mfma;
template <>
struct Mfma<bf16x8> {
    typedef __bf16 elem;
    static __device__ __forceinline__ f32x16 run(bf16x8 a, bf16x8 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Mfma<f16x8> {
    typedef _Float16 elem;
    static __device__ __forceinline__ f32x16 run(f16x8 a, f16x8 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// V: 8-element vector type of the 16-bit input format.  KS = K / 16.  NQ: column tiles of 32
// handled per group (divides the slice's tile count; 4 gives one 16-byte store per row).  NG:
// groups per slice when known at compile time (the group loop is then unrolled, which keeps
// the compiler from draining all outstanding loads in front of it), 0 = run-time count.
// grid = (groups of kTilesPerWg row tiles, column slices, heads); a workgroup stages its W slice
// in LDS once and then encodes its run of row tiles (128 rows each, 32 per wave).  Two waves
// per SIMD: the register budget holds two row tiles in flight per wave next to the one being
// computed.  The pipelined path is straight-line code with the same loads on every path, so
// that the compiler can count outstanding loads exactly and never waits for a prefetch it has
// just issued.
template <typename V, int KS, int NQ, int NG>
__global__ __launch_bounds__(kMfmaThreads) __attribute__((amdgpu_waves_per_eu(2, 3))) void encode_mfma_kernel(EncArgs a)
{
    extern __shared__ uint16_t wt[];  // [BN][K + kPad], k contiguous; then the waves' staging
    constexpr int K = KS * 16;
    constexpr int KP = K + kPad;
    const int h = blockIdx.z;
    const int n0 = blockIdx.y * a.BN;
    const int bn = (a.N - n0 < a.BN) ? a.N - n0 : a.BN;  // columns in this slice
    const uint16_t* wsrc = (const uint16_t*)a.w + (int64_t)weight_index(a, h) * K * a.N;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 31, kb = lane >> 5;
    const uint16_t* xbase = (const uint16_t*)a.x + (int64_t)h * a.x_stride_h;
    const int64_t tiles = (a.T + kRowsPerWg - 1) / kRowsPerWg;
    const int64_t first = (int64_t)blockIdx.x * kTilesPerWg;  // this workgroup's run of tiles

    // Rows are fetched one 128-byte line at a time: a load instruction covers 8 rows x 128
    // contiguous bytes (lane l: row 8j + l/8, 16-byte chunk l%8), so every cache line is touched
    // by exactly one instruction.  Register 4L + j of a lane then holds a piece of line L that
    // belongs to another lane's MFMA column; to_operands() redistributes through LDS.
    // Rows past T re-read the last row (their results are discarded).  Addresses are a uniform
    // 64-bit base per wave plus a 32-bit lane offset (the host checks that 32 rows span less
    // than 2 GiB).  With a paged input the wave's 32 rows lie in one block (the host checks that
    // the block size is a multiple of 32) whose id is read once per tile.
    auto wave_row0 = [&](int64_t tile) -> int64_t {
        const int64_t row0 = tile * kRowsPerWg + wave * kRowsPerWave;
        return row0 < a.T ? row0 : a.T - 1;
    };
    auto wave_block = [&](int64_t tile) -> int {  // paged input only
        int64_t bi, tok;
        split_token(a, wave_row0(tile), bi, tok);
        return a.src_blocks[bi];
    };
    auto wave_base = [&](int64_t tile, int sblk) -> const char* {
        const int64_t row0 = wave_row0(tile);
        int64_t off = row0 * a.x_stride_t;
        if (a.src_blocks) {
            int64_t bi, tok;
            split_token(a, row0, bi, tok);
            const int64_t blk = (sblk < 0 || sblk >= a.NBsrc) ? 0 : sblk;
            off = blk * a.xs_block + tok * a.x_stride_t;
        }
        return reinterpret_cast<const char*>(xbase + off);
    };
    auto row_offset = [&](int64_t tile, int j) -> uint32_t {
        const int q = 8 * j + (lane >> 3);
        const int64_t left = a.T - 1 - wave_row0(tile);  // last valid row, relative to the wave's first
        const uint32_t qq = (int64_t)q > left ? (uint32_t)left : (uint32_t)q;
        return (qq * (uint32_t)a.x_stride_t + (lane & 7) * 8) * 2u;
    };
    // `real` = false issues the same number of loads against one cache line of the tensor's
    // first row: the prefetch ring then has one instruction sequence on every path, which lets
    // the compiler count outstanding loads exactly instead of waiting for all of them.
    auto load_tile = [&](int64_t tile, int sblk, V (&dstv)[KS], bool real) {
        // masks instead of branches: both cases must be the same instruction stream
        const uint32_t m = real ? ~0u : 0u;
        const int64_t tc = real ? tile : (int64_t)0;
        const char* tb = real ? wave_base(tc, sblk) : reinterpret_cast<const char*>(xbase);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t off = row_offset(tc, j) & m;
#pragma unroll
            for (int L = 0; L < KS / 4; ++L)
                dstv[4 * L + j] = __builtin_nontemporal_load(
                    reinterpret_cast<const V*>(tb + off + ((L * 128) & m)));
        }
    };
    // Per wave 4 KiB of LDS: [32 rows][8 chunks of 16 bytes], chunk c of row q stored at slot
    // c ^ swz(q), swz(q) = (q ^ (q >> 3)) & 7, so that the row-major writes and the column reads
    // (consecutive rows, one chunk each) spread over all banks whether the hardware serves 8 or
    // 16 lanes of a 128-bit access per cycle.  Only this wave touches the region and a wave's
    // LDS operations execute in order, so no workgroup barrier is needed.
    uint8_t* stage = reinterpret_cast<uint8_t*>(wt) + (size_t)a.BN * KP * 2 + wave * kStageBytes;
    const int wq = lane >> 3;  // row within a group of 8 written by this lane
    uint32_t w_off[4], r_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int q = 8 * j + wq;
        w_off[j] = q * 128 + (((lane & 7) ^ ((q ^ (q >> 3)) & 7)) << 4);
        r_off[j] = r * 128 + (((2 * j + kb) ^ ((r ^ (r >> 3)) & 7)) << 4);
    }
    auto stage_line = [&](const V (&src)[KS], V (&dstv)[KS], int L) {
#pragma unroll
        for (int j = 0; j < 4; ++j) *reinterpret_cast<V*>(stage + w_off[j]) = src[4 * L + j];
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) dstv[4 * L + s4] = *reinterpret_cast<const V*>(stage + r_off[s4]);
        __builtin_amdgcn_wave_barrier();
    };
    auto to_operands = [&](const V (&src)[KS], V (&dstv)[KS]) {
#pragma unroll
        for (int L = 0; L < KS / 4; ++L) stage_line(src, dstv, L);
    };
    // Wide rows: no register prefetch; fetch, stage and redistribute line by line.
    auto load_operands = [&](int64_t tile, V (&dstv)[KS]) {
        const char* tb = wave_base(tile, a.src_blocks ? wave_block(tile) : 0);
        uint32_t off[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) off[j] = row_offset(tile, j);
#pragma unroll
        for (int L = 0; L < KS / 4; ++L) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<V*>(stage + w_off[j]) = *reinterpret_cast<const V*>(tb + off[j] + L * 128);
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4) dstv[4 * L + s4] = *reinterpret_cast<const V*>(stage + r_off[s4]);
            __builtin_amdgcn_wave_barrier();
        }
    };
    constexpr bool kPrefetch = KS <= 8;  // two tiles of rows fit in registers
    V av[KS];                            // MFMA operands of the current tile
    V raw0[kPrefetch ? KS : 1];          // rows of the next two tiles as fetched
    V raw1[kPrefetch ? KS : 1];

    // W[k0..k0+8][n0+8j..+8] -> wt[8j+c][k0..k0+8]: each thread transposes 8x8 patches of 16-bit
    // elements in registers (byte permutes) and writes eight 16-byte LDS rows.
    auto patch_load = [&](int idx, u32x4 (&row)[8]) {
        const int kq = idx / (bn / 8), j = idx % (bn / 8);
        const uint16_t* src = wsrc + (int64_t)(kq * 8) * a.N + n0 + 8 * j;
#pragma unroll
        for (int i = 0; i < 8; ++i) row[i] = *reinterpret_cast<const u32x4*>(src + (int64_t)i * a.N);
    };
    auto patch_store = [&](int idx, const u32x4 (&row)[8]) {
        const int kq = idx / (bn / 8), j = idx % (bn / 8);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
            u32x4 o;
            o.x = __builtin_amdgcn_perm(row[1][c >> 1], row[0][c >> 1], sel);
            o.y = __builtin_amdgcn_perm(row[3][c >> 1], row[2][c >> 1], sel);
            o.z = __builtin_amdgcn_perm(row[5][c >> 1], row[4][c >> 1], sel);
            o.w = __builtin_amdgcn_perm(row[7][c >> 1], row[6][c >> 1], sel);
            *reinterpret_cast<u32x4*>(wt + (8 * j + c) * KP + kq * 8) = o;
        }
    };
    constexpr bool kPipelined = kPrefetch && NG > 0;
    // paged input: the block ids of the wave's rows in each of the workgroup's tiles, up front
    int sblk[kTilesPerWg] = {0, 0, 0, 0};
    if constexpr (kPipelined) {
        if (a.src_blocks) {
#pragma unroll
            for (int i = 0; i < kTilesPerWg; ++i)
                sblk[i] = wave_block(first + i < tiles ? first + i : tiles - 1);
        }
    }
    if constexpr (kPipelined) {
        // slice width known at compile time: no loop, no divergence (surplus threads redo a
        // patch); the first two tiles' rows go out right behind the first patch loads
        constexpr int kPatches = (K / 8) * (NQ * NG * 4);
        constexpr int kRounds = (kPatches + kMfmaThreads - 1) / kMfmaThreads;
#pragma unroll
        for (int it = 0; it < kRounds; ++it) {
            const int idx = (threadIdx.x + it * kMfmaThreads) % kPatches;
            u32x4 row[8];
            patch_load(idx, row);
            if (it == 0) {
                load_tile(first, sblk[0], raw0, first < tiles);
                load_tile(first + 1, sblk[1], raw1, first + 1 < tiles);
            }
            patch_store(idx, row);
        }
    } else {
        const int npatch = (K / 8) * (bn / 8);
        for (int idx = threadIdx.x; idx < npatch; idx += kMfmaThreads) {
            u32x4 row[8];
            patch_load(idx, row);
            patch_store(idx, row);
        }
    }
    __syncthreads();

    const int nt_count = bn / 32;
    const int word0 = n0 / 32;

    // 32 hash columns x 32 rows: K/16 MFMAs into one accumulator tile
    auto project = [&](int nt) {
        f32x16 acc = acc_start();
        const uint16_t* bp = wt + (nt * 32 + r) * KP + kb * 8;
#pragma unroll
        for (int k0 = 0; k0 < KS; k0 += 4) {
            V bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) bv[i] = *reinterpret_cast<const V*>(bp + (k0 + i) * 16);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc = Mfma<V>::run(bv[i], av[k0 + i], acc);
        }
        return acc;
    };
    // All column tiles of the wave's 32 rows of `tile`, from the operands in av.
    auto encode_rows = [&](int64_t tile, uint32_t* dst) {
        // NQ column tiles per group, straight-line: the sign packing of one tile is independent
        // of the next tile's MFMAs, so the two can overlap
        auto group = [&](int nt0) {
            uint32_t words[NQ];
            f32x16 cur = project(nt0);
#pragma unroll
            for (int q = 1; q < NQ; ++q) {
                const f32x16 nxt = project(nt0 + q);
                words[q - 1] = pack_half(cur);
                cur = nxt;
            }
            words[NQ - 1] = pack_half(cur);
#pragma unroll
            for (int q = 0; q < NQ; ++q) words[q] = join_halves(kb ? words[q] << 4 : words[q]);
            if (dst) {
                uint32_t* d = dst + word0 + nt0;
                if (NQ == 4 && (((uintptr_t)d) & 15) == 0) {
                    u32x4 v = {words[0], words[1 % NQ], words[2 % NQ], words[3 % NQ]};
                    *reinterpret_cast<u32x4*>(d) = v;
                } else {
#pragma unroll
                    for (int q = 0; q < NQ; ++q) d[q] = words[q];
                }
            }
        };
        if constexpr (NG > 0) {
#pragma unroll
            for (int g = 0; g < NG; ++g) group(g * NQ);
        } else {
            for (int nt0 = 0; nt0 < nt_count; nt0 += NQ) group(nt0);
        }
    };
    // Lanes 0..31 own one row each.  The row's slot is fetched together with the tile's rows,
    // two tiles ahead, so that its value never has to be waited for behind younger loads
    // (a wave's loads return in issue order).
    auto tile_slot = [&](int64_t tile) -> RawSlot {
        int64_t t = tile * kRowsPerWg + wave * kRowsPerWave + r;
        if (t >= a.T) t = a.T - 1;  // in-bounds read; the row itself is masked in slot_target()
        return fetch_slot_flat(a, t);
    };
    auto slot_target = [&](int64_t tile, RawSlot s) -> uint32_t* {
        const int64_t t = tile * kRowsPerWg + wave * kRowsPerWave + r;
        return (t < a.T && lane < 32) ? slot_dst(a, slot_value(a, s, t), h) : nullptr;
    };

    if constexpr (kPipelined) {
        // ring of two fetched tiles, fully unrolled; tiles past the end are dummy loads and
        // masked stores
        RawSlot slot0 = tile_slot(first < tiles ? first : tiles - 1);
        RawSlot slot1 = tile_slot(first + 1 < tiles ? first + 1 : tiles - 1);
#pragma unroll
        for (int i = 0; i < kTilesPerWg; i += 2) {
            const int64_t t0 = first + i, t1 = first + i + 1;
            to_operands(raw0, av);
            uint32_t* dst = t0 < tiles ? slot_target(t0, slot0) : nullptr;
            if (i + 2 < kTilesPerWg) {
                slot0 = tile_slot(t0 + 2 < tiles ? t0 + 2 : tiles - 1);
                load_tile(t0 + 2, sblk[(i + 2) % kTilesPerWg], raw0, t0 + 2 < tiles);
            }
            encode_rows(t0, dst);
            to_operands(raw1, av);
            dst = t1 < tiles ? slot_target(t1, slot1) : nullptr;
            if (i + 3 < kTilesPerWg) {
                slot1 = tile_slot(t1 + 2 < tiles ? t1 + 2 : tiles - 1);
                load_tile(t1 + 2, sblk[(i + 3) % kTilesPerWg], raw1, t1 + 2 < tiles);
            }
            encode_rows(t1, dst);
        }
    } else {
        for (int64_t tile = first; tile < first + kTilesPerWg && tile < tiles; ++tile) {
            const RawSlot sl = tile_slot(tile);
            load_operands(tile, av);
            encode_rows(tile, slot_target(tile, sl));
        }
    }
}

// ---------------------------------------------------------------------------------------
// Streaming kernel for cache-build sizes (millions of rows, K * N <= 128 * 128).
//
// A wave owns one head and keeps that head's whole projection matrix in registers, already in
// MFMA operand layout (N/32 * K/16 operands of 4 registers: 128 at 128 x 128), so the inner loop
// reads nothing but rows.  Rows never pass through registers on their way in: every lane issues
// 16-byte loads that the memory pipeline writes straight into LDS (lane l of an instruction
// lands at byte 16 * l of that instruction's 1 KiB window), two 32-row tiles ahead of the tile
// being computed.  The lane -> (row, 16-byte chunk) assignment of a load instruction is free as
// long as 8 consecutive lanes cover one 128-byte line, so lane l fetches chunk (l % 8) ^ swz(row):
// the rows arrive in LDS already swizzled for the conflict-free operand reads
// (one 16-byte read per lane and MFMA k-step).  The slot-mapping entries of a tile travel the
// same way (one 4-byte load per lane into the 256 bytes behind the tile).
//
// The loads are inline assembly on purpose: the wave waits with an explicit count for "all but
// the newest tile's loads", which the compiler cannot express for loads whose destination is
// LDS (it waits for every outstanding one before any LDS read).  Loads and stores of a wave
// complete in issue order, and a wait for "at most n outstanding" only errs on the side of
// waiting when more operations were issued behind the awaited one than n — so the count names
// only the loads this code issues itself (a fixed number per tile; the last tile of a wave is
// awaited with a full drain) and the compiler's own stores and reads merely make it wait a
// little more.
//
// grid = persistent workgroups of 8 waves; global wave g: head g % H, tile stream g / H of
// `nstreams` (tiles stream, stream + nstreams, ...).  LDS per wave: 2 x (tile + 256 bytes).
// ---------------------------------------------------------------------------------------
constexpr int kStreamWaves = 8;
constexpr int kStreamThreads = kStreamWaves * 64;

// One row group J (8 rows x 128 bytes) of a tile's line 0 or 1.  The instruction's immediate
// offset moves the memory address AND the LDS address, so the window base of a line-1 load
// (LDS bytes 4096 + 1024 J) is given 128 bytes low.
#define UCM_DMA(J, WIN, OFF)                                            \
    "s_add_u32 m0, %[lds], " #WIN "\n\ts_nop 0\n\t"                     \
    "global_load_lds_dwordx4 %[o" #J "], %[base] offset:" #OFF " nt\n\t"

// m0 (the LDS window of a load-to-LDS instruction) is put back as it was: the compiler treats
// it as reserved and does not expect inline assembly to change it.
template <int LN>
__device__ __forceinline__ void stream_issue_rows(uint32_t lds, uint64_t base, const uint32_t (&off)[4])
{
    uint32_t keep;
    if constexpr (LN == 2) {
        asm volatile("s_mov_b32 %[keep], m0\n\t"
                     UCM_DMA(0, 0, 0) UCM_DMA(1, 1024, 0) UCM_DMA(2, 2048, 0) UCM_DMA(3, 3072, 0)
                     UCM_DMA(0, 3968, 128) UCM_DMA(1, 4992, 128) UCM_DMA(2, 6016, 128) UCM_DMA(3, 7040, 128)
                     "s_mov_b32 m0, %[keep]\n\t"
                     : [keep] "=&s"(keep)
                     : [lds] "s"(lds), [base] "s"(base), [o0] "v"(off[0]), [o1] "v"(off[1]),
                       [o2] "v"(off[2]), [o3] "v"(off[3])
                     : "memory", "scc");
    } else {
        asm volatile("s_mov_b32 %[keep], m0\n\t"
                     UCM_DMA(0, 0, 0) UCM_DMA(1, 1024, 0) UCM_DMA(2, 2048, 0) UCM_DMA(3, 3072, 0)
                     "s_mov_b32 m0, %[keep]\n\t"
                     : [keep] "=&s"(keep)
                     : [lds] "s"(lds), [base] "s"(base), [o0] "v"(off[0]), [o1] "v"(off[1]),
                       [o2] "v"(off[2]), [o3] "v"(off[3])
                     : "memory", "scc");
    }
}

__device__ __forceinline__ void stream_issue_slots(uint32_t lds, uint64_t base, uint32_t off)
{
    uint32_t keep;
    asm volatile("s_mov_b32 %[keep], m0\n\ts_mov_b32 m0, %[lds]\n\ts_nop 0\n\t"
                 "global_load_lds_dword %[o], %[base]\n\ts_mov_b32 m0, %[keep]\n\t"
                 : [keep] "=&s"(keep)
                 : [lds] "s"(lds), [base] "s"(base), [o] "v"(off)
                 : "memory");
}

template <int N>
__device__ __forceinline__ void stream_wait_loads()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ void stream_wait_lds()
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
}

// SLOT: 0 = identity slots (dense output), 1 = int32 slot mapping, 2 = int64 slot mapping.
// ACCS: accumulator tiles in flight (the MFMAs of ACCS column tiles are interleaved, so that a
// wave's consecutive MFMAs do not depend on each other).
//
// Stores: one 16-byte code per row and head.  Their size is what they cost: beside a 2 GiB read
// stream (304 us alone) the same 6.25 % of bytes written back take the stream to 392-405 us as
// whole 128-byte lines, 408 us as 64-byte pieces, 425-436 us as 32-byte pieces and 450-472 us as
// 16-byte pieces of lines that other workgroups complete (no arithmetic in any of these; the
// stores' cache policy and their clustering in time change nothing).  With one store per row and
// head this kernel sits at the last figure (2.1 GB of keys: 455-470 us into the paged cache).
//
// HC > 0 (HC = 2, 4 or 8 heads of four-word codes side by side in a token's cache row; the HC
// waves of a stream sit in one workgroup): the waves hand their codes to one another through a
// ring of kRing tiles in LDS and take turns storing whole rows (128 bytes at eight heads),
// kCombDelay tiles after the codes were produced, so that the storing wave normally finds all
// heads there and nobody runs in step with anybody.
// Two counters per ring slot: pub (codes handed in) and done (tiles stored); plain LDS
// operations of one wave complete in order, so a counter update that follows the data in program
// order is seen after the data.  Every wait is bounded: a wave that does not see its counter
// move gives up waiting and goes on: the kernel still ends, the codes of that launch are undefined,
// and the host refuses further encodes on the device until the caller has acknowledged it.
// 2.1 GB of keys: 403-411 us against 455-470 us = 5.6 TB/s of algorithmic bytes.  What made earlier
// forms of this slower than the plain stores (476-545 us): counters as volatile / atomic C++
// accesses (each waits for the row loads in flight), spilled registers reloaded inside the loop
// (scratch reloads count as vector loads and wait behind the row loads: hence two accumulator
// tiles here, not four), and the storing wave in step with the slowest of the eight.
constexpr int kRing = 5;
constexpr int kCombDelay = 2;
constexpr int ring_slot_bytes(int hc) { return 512 * hc + 128; }  // 32 rows x hc heads x 16 bytes, then the rows' 32 slots
// the two counters per ring slot, padded so that the next stream's ring starts 16-byte aligned
// (the ring is read and written with 16-byte LDS operations)
constexpr int kRingCounterBytes = 48;
static_assert(2 * kRing * (int)sizeof(int) <= kRingCounterBytes && kRingCounterBytes % 16 == 0, "counter area");
constexpr int ring_stream_bytes(int hc) { return kRing * ring_slot_bytes(hc) + kRingCounterBytes; }
constexpr int ring_lds_bytes(int hc)  // rings and counters of the 8 / hc streams of a workgroup
{
    return hc ? (8 / hc) * ring_stream_bytes(hc) : 0;
}
constexpr int kSpinLimit = 1 << 22;  // some tenths of a second

// Counter reads and updates as single LDS instructions with a wait of their own: a volatile or
// atomic access in C++ makes the compiler wait for every outstanding memory operation, the row
// loads in flight included.  The read waits inside the same statement: a register that an LDS read
// fills later, behind the compiler's back, may have been given to another value by then.
__device__ __forceinline__ int lds_peek(const int* counter)
{
    int v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)"
                 : "=v"(v)
                 : "v"((uint32_t)(uintptr_t)(const __attribute__((address_space(3))) int*)counter)
                 : "memory");
    return v;
}
__device__ __forceinline__ void lds_bump(int* counter)
{
    const uint32_t one = 1;
    asm volatile("ds_add_u32 %0, %1" ::"v"((uint32_t)(uintptr_t)(__attribute__((address_space(3))) int*)counter), "v"(one)
                 : "memory");
}
// Waits that ran into their limit, since the library was loaded (ucm_hash_encode_stream_timeouts).
__device__ unsigned int g_stream_wait_timeouts = 0;

// gave_up: set once a wait of this wave has run into the limit; the wave then never waits again,
// so a kernel that has gone wrong ends after one limit per wave, not one per tile.  The codes of
// such a launch are undefined; `flag` (pinned host memory) tells the host, which refuses every
// later encode on the device until the caller has acknowledged it.
__device__ __forceinline__ void lds_wait_at_least(const int* counter, int want, bool& gave_up, unsigned int* flag)
{
    if (gave_up) return;
    int spins = 0;
    while (lds_peek(counter) < want) {
        if (++spins > kSpinLimit) {
            gave_up = true;
            if ((threadIdx.x & 63) == 0) {
                atomicAdd(&g_stream_wait_timeouts, 1u);
                if (flag) __hip_atomic_store(flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
            break;
        }
        __builtin_amdgcn_s_sleep(1);
    }
}

template <typename V, int KS, int NT, int SLOT, int ACCS, int HC>
__global__ __launch_bounds__(kStreamThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void encode_stream_kernel(
    EncArgs a, int64_t ntiles, int nstreams)
{
    constexpr bool COMB = HC > 0;
    constexpr int HCn = HC > 0 ? HC : 8;  // keeps the index arithmetic of the unused branch well-formed
    extern __shared__ __attribute__((aligned(1024))) uint8_t stream_lds[];
    constexpr int K = KS * 16;
    constexpr int LN = KS / 4;                      // 128-byte lines per row
    constexpr int kTileBytes = kRowsPerWave * K * 2;
    constexpr int kBufBytes = kTileBytes + 256;     // the tile's 32 slots behind its rows
    constexpr int kLoads = 4 * LN + (SLOT ? 1 : 0);  // load instructions per tile

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int gw = blockIdx.x * kStreamWaves + wave;
    const int h = gw % a.H;
    const int stream = gw / a.H;
    const int r = lane & 31, kb = lane >> 5;

    uint8_t* mybuf = stream_lds + (size_t)wave * 2 * kBufBytes;

    // ---- the head's projection matrix, in operand layout, for the kernel's lifetime ----
    // 32 hash columns at a time are transposed through the wave's own (still unused) LDS: a lane
    // fetches one 8 x 8 patch of W (eight 16-byte rows), transposes it in registers and writes the
    // eight columns as LDS rows of K values; then every lane reads its K/16 operands.
    V wreg[NT][KS];
    {
        constexpr int KP = K + kPad;
        constexpr int kPatches = (K / 8) * 4;  // per 32 columns
        uint16_t* wt = reinterpret_cast<uint16_t*>(mybuf);
        const uint16_t* wsrc = (const uint16_t*)a.w + (int64_t)weight_index(a, h) * K * a.N;
        const int idx = lane % kPatches;
        const int kq = idx >> 2, j = idx & 3;
        // all patches of the head are requested before the first one is used: one round trip
        u32x4 row[NT][8];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const uint16_t* src = wsrc + (int64_t)(kq * 8) * a.N + nt * 32 + 8 * j;
#pragma unroll
            for (int i = 0; i < 8; ++i) row[nt][i] = *reinterpret_cast<const u32x4*>(src + (int64_t)i * a.N);
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
                u32x4 o;
                o.x = __builtin_amdgcn_perm(row[nt][1][c >> 1], row[nt][0][c >> 1], sel);
                o.y = __builtin_amdgcn_perm(row[nt][3][c >> 1], row[nt][2][c >> 1], sel);
                o.z = __builtin_amdgcn_perm(row[nt][5][c >> 1], row[nt][4][c >> 1], sel);
                o.w = __builtin_amdgcn_perm(row[nt][7][c >> 1], row[nt][6][c >> 1], sel);
                *reinterpret_cast<u32x4*>(wt + (8 * j + c) * KP + kq * 8) = o;
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                wreg[nt][ks] = *reinterpret_cast<const V*>(wt + r * KP + ks * 16 + kb * 8);
            __builtin_amdgcn_wave_barrier();
        }
        stream_wait_lds();  // the staging area becomes the row buffers from here on
    }

    const uint32_t lds0 = __builtin_amdgcn_readfirstlane(
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)mybuf);
    const uint16_t* xbase = (const uint16_t*)a.x + (int64_t)h * a.x_stride_h;
    const int slot_sz = SLOT == 2 ? 8 : 4;
    const uint32_t row_bytes = (uint32_t)(a.x_stride_t * 2);

    // lane's share of a tile's loads: row 8 j + lane / 8 of the tile, chunk (lane % 8) ^ swz(row);
    // rows past the end of the input re-read its last row
    uint32_t off_full[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t q = 8 * j + (lane >> 3);
        off_full[j] = q * row_bytes + ((((uint32_t)lane & 7) ^ ((q ^ (q >> 3)) & 7)) << 4);
    }
    const uint32_t slot_e = SLOT == 2 ? (uint32_t)lane >> 1 : (uint32_t)lane & 31;
    const uint32_t slot_full = slot_e * slot_sz + (SLOT == 2 ? ((uint32_t)lane & 1) * 4 : 0);
    auto issue = [&](int64_t tile, int b) {
        const int64_t t0 = tile * kRowsPerWave;
        const int64_t left64 = a.T - 1 - t0;
        const uint64_t base = (uint64_t)(uintptr_t)(xbase + t0 * a.x_stride_t);
        const uint32_t lds = lds0 + b * kBufBytes;
        uint32_t so = slot_full;
        if (left64 >= 31) {
            stream_issue_rows<LN>(lds, base, off_full);
        } else {
            const uint32_t left = (uint32_t)left64;
            uint32_t off[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t q = 8 * j + (lane >> 3);
                const uint32_t qq = q > left ? left : q;
                off[j] = qq * row_bytes + ((((uint32_t)lane & 7) ^ ((q ^ (q >> 3)) & 7)) << 4);
            }
            stream_issue_rows<LN>(lds, base, off);
            const uint32_t ee = slot_e > left ? left : slot_e;
            so = ee * slot_sz + (SLOT == 2 ? ((uint32_t)lane & 1) * 4 : 0);
        }
        if constexpr (SLOT != 0)
            // 4 bytes per lane: the tile's 32 slots (int64: lane l = half l % 2 of slot l / 2)
            stream_issue_slots(lds + kTileBytes, (uint64_t)(uintptr_t)((const char*)a.slot + t0 * slot_sz), so);
    };

    // operand read offsets (conflict-free with the swizzle above)
    uint32_t r_off[4];
#pragma unroll
    for (int c2 = 0; c2 < 4; ++c2) r_off[c2] = r * 128 + (((2 * c2 + kb) ^ ((r ^ (r >> 3)) & 7)) << 4);

    // The host only sends shapes here whose block size is a power of two, whose code rows are
    // 16-byte aligned when they are four words, and whose cache spans less than 2^31 words:
    // one shift, two 32-bit multiplications, one store.
    uint32_t words_prev[NT];
    uint32_t* dst_prev = nullptr;
    int32_t slot_prev = -1;  // COMB: the previous tile's slot of this lane's row, -1 = no store
    int prev_idx = -1;       // COMB: the previous tile's number in this stream (0, 1, 2, ...)
    int done_seen = 0;       // COMB: `done` of the ring slot the previous tile goes to, read in step()
    bool gave_up = false;    // COMB: a wait of this wave has hit its limit
#pragma unroll
    for (int q = 0; q < NT; ++q) words_prev[q] = 0;
    const int64_t n_slots = a.NB << a.bs_shift;
    uint32_t* const cache_h = a.cache + (int64_t)h * a.cs_head;
    const uint32_t csb = (uint32_t)a.cs_block, cst = (uint32_t)a.cs_token;

    // this stream's ring and its counters (a workgroup holds 8 / HC streams)
    constexpr int kSlotBytes = ring_slot_bytes(HCn);
    constexpr int kStreamRing = ring_stream_bytes(HCn);
    static_assert(kStreamRing % 16 == 0, "every stream's ring starts 16-byte aligned");
    uint8_t* const ring = stream_lds + (size_t)kStreamWaves * 2 * kBufBytes + (COMB ? (wave / HCn) * kStreamRing : 0);
    int* const pub = reinterpret_cast<int*>(ring + kRing * kSlotBytes);
    int* const done = pub + kRing;
    if constexpr (COMB) {
        if ((wave % HCn) == 0 && lane < 2 * kRing) pub[lane] = 0;
        __syncthreads();
    }
    // the wave whose turn it is stores tile j of this stream as 32 whole cache rows
    auto store_tile = [&](int j) {
        const int s = j % kRing;
        lds_wait_at_least(pub + s, HCn * (j / kRing + 1), gave_up, a.timeout_flag);
        asm volatile("" ::: "memory");
        const uint8_t* slot_base = ring + s * kSlotBytes;
#pragma unroll
        for (int u = 0; u < HCn / 2; ++u) {
            const int piece = u * 64 + lane;  // row piece / HC of the tile, head piece % HC
            const int ph = piece % HCn, pr = piece / HCn;
            const u32x4 code = *reinterpret_cast<const u32x4*>(slot_base + ph * 512 + ((pr ^ (2 * ph)) << 4));
            const int32_t sv = *reinterpret_cast<const int32_t*>(slot_base + 512 * HCn + pr * 4);
            if (sv >= 0) {
                const uint32_t svl = (uint32_t)sv;
                uint32_t* dst = a.cache + ((svl >> a.bs_shift) * csb + (svl & (uint32_t)(a.BS - 1)) * cst) + ph * 4;
                *reinterpret_cast<u32x4*>(dst) = code;
            }
        }
        asm volatile("" ::: "memory");
        if (lane == 0) lds_bump(done + s);
    };

    auto store_prev = [&]() {
        if constexpr (COMB) {
            if (prev_idx < 0) return;
            const int s = prev_idx % kRing, gen = prev_idx / kRing;
            // the slot's previous tile has been stored: normally known from the read in step()
            if (gen > 0 && done_seen < gen) lds_wait_at_least(done + s, gen, gave_up, a.timeout_flag);
            asm volatile("" ::: "memory");
            uint8_t* slot_base = ring + s * kSlotBytes;
            if (lane < 32) {
                const u32x4 v = {words_prev[0], words_prev[1 % NT], words_prev[2 % NT], words_prev[3 % NT]};
                // head-major in the ring, rows swizzled with the head: the 32 lanes of this write and
                // (at eight heads) the 64 lanes of the storing wave's reads each cover all banks
                *reinterpret_cast<u32x4*>(slot_base + h * 512 + ((r ^ (2 * h)) << 4)) = v;
                if ((prev_idx % HCn) == h) *reinterpret_cast<int32_t*>(slot_base + 512 * HCn + r * 4) = slot_prev;
            }
            asm volatile("" ::: "memory");
            if (lane == 0) lds_bump(pub + s);
            const int j = prev_idx - kCombDelay;
            if (j >= 0 && (j % HCn) == h) store_tile(j);
            return;
        }
        if (dst_prev) {
            if constexpr (NT == 4) {
                u32x4 v = {words_prev[0], words_prev[1 % NT], words_prev[2 % NT], words_prev[3 % NT]};
                *reinterpret_cast<u32x4*>(dst_prev) = v;
            } else {
#pragma unroll
                for (int q = 0; q < NT; ++q) dst_prev[q] = words_prev[q];
            }
        }
    };

    // newer: the next tile's loads are in flight behind this tile's; more: a tile two ahead exists
    auto step = [&](int64_t tile, int local, int b, bool newer, bool more) {
        const uint8_t* buf = mybuf + b * kBufBytes;
        if (newer) stream_wait_loads<kLoads>();  // everything but the newest tile's loads has landed
        else stream_wait_loads<0>();
        V av[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            av[ks] = *reinterpret_cast<const V*>(buf + (ks >> 2) * 4096 + r_off[ks & 3]);
        const int64_t t = tile * kRowsPerWave + r;
        int64_t sv = t;
        if constexpr (SLOT == 2) sv = *reinterpret_cast<const int64_t*>(buf + kTileBytes + r * 8);
        if constexpr (SLOT == 1) sv = *reinterpret_cast<const int32_t*>(buf + kTileBytes + r * 4);
        // the buffer may be overwritten from here on (COMB: the counter read shares the wait)
        if constexpr (COMB) done_seen = lds_peek(done + (prev_idx < 0 ? 0 : prev_idx % kRing));
        else stream_wait_lds();
        store_prev();
        if (more) issue(tile + 2 * (int64_t)nstreams, b);

        const bool ok = t < a.T && lane < 32 && sv >= 0 && sv < n_slots;
        const uint32_t svl = (uint32_t)sv;  // below 2^31 when ok
        if constexpr (COMB) {
            slot_prev = ok ? (int32_t)svl : -1;
            prev_idx = local;
        } else {
            dst_prev = ok ? cache_h + ((svl >> a.bs_shift) * csb + (svl & (uint32_t)(a.BS - 1)) * cst) : nullptr;
        }

#pragma unroll
        for (int n0 = 0; n0 < NT; n0 += ACCS) {
            f32x16 acc[ACCS];
#pragma unroll
            for (int q = 0; q < ACCS; ++q) acc[q] = acc_start();
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int q = 0; q < ACCS; ++q) acc[q] = Mfma<V>::run(wreg[n0 + q][ks], av[ks], acc[q]);
#pragma unroll
            for (int q = 0; q < ACCS; ++q) {
                const uint32_t half = pack_half(acc[q]);
                words_prev[n0 + q] = join_halves(kb ? half << 4 : half);
            }
        }
    };

    // tiles stream, stream + nstreams, ... : n of them
    const int64_t n = stream < ntiles ? (ntiles - 1 - stream) / nstreams + 1 : 0;
    int64_t tile = stream;
    if (n > 0) issue(tile, 0);
    if (n > 1) issue(tile + nstreams, 1);
    for (int64_t i = 0; i < n; i += 2) {
        step(tile, (int)i, 0, i + 1 < n, i + 2 < n);
        tile += nstreams;
        if (i + 1 >= n) break;
        step(tile, (int)i + 1, 1, i + 2 < n, i + 3 < n);
        tile += nstreams;
    }
    if constexpr (COMB) done_seen = lds_peek(done + (prev_idx < 0 ? 0 : prev_idx % kRing));
    store_prev();
    if constexpr (COMB) {
        // the last kCombDelay tiles have been handed in but not stored yet
        for (int j = (int)n - kCombDelay < 0 ? 0 : (int)n - kCombDelay; j < (int)n; ++j)
            if ((j % HCn) == h) store_tile(j);
    }
    // no load may still be writing into this workgroup's LDS when the wave ends
    stream_wait_loads<0>();
}

// ---------------------------------------------------------------------------------------
// Wide streaming encoder: K = 512 input dimensions (the latent vector of latent attention), one
// head, 256 or 512 hash bits, from some hundred thousand rows (building the code cache of a long
// prompt or after a store hit).
//
// 512 x 256 bf16 are 256 KiB - half of a compute unit's register file - so the projection cannot
// belong to one wave as in the 128-wide kernel above.  A persistent workgroup of four waves, one
// per SIMD, owns a slice of 256 hash columns for the kernel's lifetime, each wave 64 of them: 2 x
// 32 k-steps x 4 registers = 256 registers of MFMA A operands per lane, the whole accumulation
// half of the wave's register file.  The matrix instructions are written out (inline assembly)
// because the compiler will not keep operands there on its own: given the builtin it holds them
// in the other half, spills and copies.  (512 hash bits are two such slices, i.e. two launches
// over the same rows.)  What the four waves share are the rows: a tile of 32 rows (32 KiB) is
// brought in once per workgroup, straight from memory into LDS - every wave issues the loads of
// eight rows, lane l of a load fetching 16-byte piece l ^ (row & 7) so that the operand reads hit
// all banks - and every wave reads all of it as its B operands, each 16-byte read feeding two
// matrix instructions (128 KiB of LDS reads per tile; eight waves of 32 columns read 256 KiB).
//
// A wave has its SIMD to itself, so nothing hides what it waits for: the stream of matrix
// instructions must never stop.  Operand reads run eight k-steps ahead in a ring of registers
// (sixteen measured the same).  No operand of a written-out matrix instruction is written by a
// vector instruction anywhere near it: the compiler inserts the wait states between the two only
// for matrix instructions it knows.  An earlier form gave the accumulators their start value
// with 16 v_mov each - which the compiler is free to move down to the first matrix instruction
// of the next tile - and with sixteen reads ahead that instruction, never the second of its
// pair, now and then produced wrong sums for a row or two of a tile (426 of 560,000 words, the
// same ones in every run); the same form with sixteen idle cycles in front of a tile's first
// matrix instruction is right.  (The LDS wait counter, the first suspect, is exact: waits
// counted against up to 48 reads in flight release when they should.)  Four tiles are in the
// ring.  One bare barrier per
// tile, in its middle: behind it the next tile is complete in LDS (its reads start with the
// second half of this tile's matrix instructions, so the stream runs on from tile to tile),
// everybody is done with the previous tile (its slot takes the tile three ahead, one load
// instruction per k-step), and the words of the tile before that are complete.  The signs of
// tile i - 1 are packed while tile i is multiplied, from a second set of accumulators, four
// instructions per k-step (a wave issues about seven vector instructions between two pairs of
// matrix instructions for free; 25 in one place cost 70 cycles of matrix time).  A sum starts
// from a constant register set given to the tile's first matrix instruction as its C operand:
// no accumulator is ever re-initialised.  A wave's 2 x 32 x 32 products leave it as two words per
// row; the eight words of a row meet in a small LDS buffer (three in turn), and one wave - they
// take turns - stores the tile's 32 code rows, 16 bytes per lane.
//
// Measured on the part (shader clock counter against the 100 MHz counter, inside the kernel):
// a launch over 2^20 rows takes 440,000 cycles, and the clock under this load settles at 1.27
// to 1.55 GHz (1.9 GHz in the first launches): 0.31 ms.  262,144 of the cycles are matrix
// instructions (8,192 per wave x 32).  Without the row loads the same kernel takes 375,000
// cycles, with loads that hit in L2 about the same: what the loads cost is their issue - an
// instruction that finds the load path busy holds its wave, 80 cycles per instruction on
// average - not the wait for their data (leaving the waits out changes nothing).  Spreading the
// loads over the whole tile instead (each wave alone in its k-step) shortens their lead and was
// slower (590,000 to 655,000 cycles).  Eight waves of 32 columns, two per SIMD, one reading while
// the other multiplies: 465,000 to 508,000 cycles, 0.33 ms.
// ---------------------------------------------------------------------------------------
constexpr int kWideWaves = 4;
constexpr int kWideThreads = kWideWaves * 64;
constexpr int kWideRing = 4;
constexpr int kWideK = 512;
constexpr int kWideTileBytes = kRowsPerWave * kWideK * 2;  // 32 KiB
// a ring slot holds a tile; before the first tile it holds one wave's staged 32 columns of W (32
// rows of K + kPad values)
constexpr int kWideSlotBytes = kRowsPerWave * (kWideK + kPad) * 2;
constexpr int kWideCodeBytes = kRowsPerWave * 32;  // 32 rows x 8 words
constexpr int kWideMapRing = 8;                    // slot-mapping entries (256 bytes) of eight tiles
constexpr int kWideAhead = 8;                      // operand reads ahead of the matrix instructions, in k-steps
constexpr size_t kWideLds = (size_t)kWideRing * kWideSlotBytes + 3 * kWideCodeBytes + kWideMapRing * 256;
static_assert(kWideSlotBytes % 16 == 0 && kWideTileBytes <= kWideSlotBytes, "ring slot layout");
static_assert(kWideLds <= 160 * 1024, "ring exceeds the LDS");
static_assert((kWideK / 16) % kWideAhead == 0, "a tile's k-steps are whole turns of the operand ring");

typedef u32x4 u32x4_a4 __attribute__((aligned(4)));

// v_mfma_f32_32x32x16 with the A operand in the accumulation registers
template <typename V>
__device__ __forceinline__ void wide_mfma(f32x16& acc, const u32x4& w, const u32x4& b)
{
    if constexpr (std::is_same<V, bf16x8>::value)
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "a"(w), "v"(b));
    else
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "a"(w), "v"(b));
}

// first matrix instruction of a tile: the sum starts from `start` (which stays as it is)
template <typename V>
__device__ __forceinline__ void wide_mfma_first(f32x16& acc, const u32x4& w, const u32x4& b, const f32x16& start)
{
    if constexpr (std::is_same<V, bf16x8>::value)
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(acc) : "a"(w), "v"(b), "v"(start));
    else
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(acc) : "a"(w), "v"(b), "v"(start));
}

template <typename V, int SLOT>
__global__ __launch_bounds__(kWideThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void encode_wide_kernel(
    EncArgs a, int64_t ntiles, int nstreams, int col, unsigned long long* clock_probe)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t wide_lds[];
    constexpr int K = kWideK, KS = K / 16;
    constexpr int kLoads = 8 + (SLOT ? 1 : 0);  // load instructions per wave and tile
    // measurement aid (null in normal use): the first workgroup reports its own lifetime in shader
    // cycles and in ticks of the constant 100 MHz counter - their ratio is the clock it ran at
    unsigned long long probe_c0 = 0, probe_r0 = 0;
    if (clock_probe) {
        probe_c0 = __builtin_readcyclecounter();
        probe_r0 = __builtin_amdgcn_s_memrealtime();
    }
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 31, kb = lane >> 5;
    const int stream = blockIdx.x;
    uint8_t* const codes = wide_lds + (size_t)kWideRing * kWideSlotBytes;
    constexpr uint32_t kMapOff = (uint32_t)(kWideRing * kWideSlotBytes + 3 * kWideCodeBytes);

    // ---- this wave's 2 x 32 columns of W as MFMA A operands, for the kernel's lifetime ----
    // 8 x 8 patches (eight 16-byte rows each) are transposed in registers and written as 32 LDS
    // rows of K values into the wave's own ring slot, then every lane reads its K / 16 operands:
    // 32 columns at a time.  The empty statements pin what was read to the accumulation registers.
    u32x4 wreg[2][KS];
    {
        constexpr int KP = K + kPad;
        uint16_t* wt = reinterpret_cast<uint16_t*>(wide_lds + (size_t)wave * kWideSlotBytes);
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const uint16_t* wsrc =
                (const uint16_t*)a.w + (int64_t)weight_index(a, 0) * K * a.N + col * 256 + wave * 64 + g * 32;
#pragma unroll
            for (int half = 0; half < 2; ++half) {  // 256 patches, four per lane, two at a time
                u32x4 row[2][8];
#pragma unroll
                for (int it = 0; it < 2; ++it) {
                    const int idx = (half * 2 + it) * 64 + lane;
                    const uint16_t* src = wsrc + (int64_t)((idx >> 2) * 8) * a.N + 8 * (idx & 3);
#pragma unroll
                    for (int i = 0; i < 8; ++i) row[it][i] = *reinterpret_cast<const u32x4*>(src + (int64_t)i * a.N);
                }
#pragma unroll
                for (int it = 0; it < 2; ++it) {
                    const int idx = (half * 2 + it) * 64 + lane;
                    const int kq = idx >> 2, j = idx & 3;
#pragma unroll
                    for (int c = 0; c < 8; ++c) {
                        const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
                        u32x4 o;
                        o.x = __builtin_amdgcn_perm(row[it][1][c >> 1], row[it][0][c >> 1], sel);
                        o.y = __builtin_amdgcn_perm(row[it][3][c >> 1], row[it][2][c >> 1], sel);
                        o.z = __builtin_amdgcn_perm(row[it][5][c >> 1], row[it][4][c >> 1], sel);
                        o.w = __builtin_amdgcn_perm(row[it][7][c >> 1], row[it][6][c >> 1], sel);
                        *reinterpret_cast<u32x4*>(wt + (8 * j + c) * KP + kq * 8) = o;
                    }
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                wreg[g][ks] = *reinterpret_cast<const u32x4*>(wt + r * KP + ks * 16 + kb * 8);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(wreg[g][ks]));
        }
        __syncthreads();  // the staging areas become the row ring
    }

    const uint32_t lds0 = __builtin_amdgcn_readfirstlane(
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)wide_lds);
    const uint32_t row_bytes = (uint32_t)(a.x_stride_t * 2);
    constexpr int slot_sz = SLOT == 2 ? 8 : 4;
    const uint32_t slot_e = SLOT == 2 ? (uint32_t)lane >> 1 : (uint32_t)lane & 31;
    // A wave's share of a tile's loads: rows 8 * wave + j (j = 0..7), lane l fetching piece l ^ j;
    // rows past the end of the input re-read its last row.  Every wave also fetches the tile's 32
    // slot-mapping entries (all four write the same values): every wave counts the same loads.
    // The load instructions of a tile are issued one at a time, between matrix instructions.
    uint32_t off_full[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) off_full[j] = (8 * (uint32_t)wave + j) * row_bytes + (((uint32_t)lane ^ j) << 4);
    const uint32_t slot_full = slot_e * slot_sz + (SLOT == 2 ? ((uint32_t)lane & 1) * 4 : 0);
    // part p of the loads of `tile` (ring position `local`): p = 0..7 a row, p = 8 the slot mapping
    auto issue_part = [&](int64_t tile, int local, int p) {
        const int64_t t0 = tile * kRowsPerWave;
        const int64_t left64 = a.T - 1 - t0;
        if (p < 8) {
            const uint64_t base = (uint64_t)(uintptr_t)((const uint16_t*)a.x + t0 * a.x_stride_t);
            const uint32_t lds = lds0 + (local % kWideRing) * kWideSlotBytes + wave * 8192 + p * 1024;
            uint32_t off = off_full[p];
            if (left64 < 31) {
                const uint32_t left = (uint32_t)left64;
                const uint32_t q = 8 * (uint32_t)wave + p;
                off = (q > left ? left : q) * row_bytes + (((uint32_t)lane ^ p) << 4);
            }
            uint32_t keep;
            asm volatile("s_mov_b32 %[keep], m0\n\ts_mov_b32 m0, %[lds]\n\ts_nop 0\n\t"
                         "global_load_lds_dwordx4 %[o], %[base] nt\n\ts_mov_b32 m0, %[keep]\n\t"
                         : [keep] "=&s"(keep)
                         : [lds] "s"(lds), [base] "s"(base), [o] "v"(off)
                         : "memory");
        } else if constexpr (SLOT != 0) {
            uint32_t so = slot_full;
            if (left64 < 31) {
                const uint32_t left = (uint32_t)left64;
                const uint32_t ee = slot_e > left ? left : slot_e;
                so = ee * slot_sz + (SLOT == 2 ? ((uint32_t)lane & 1) * 4 : 0);
            }
            stream_issue_slots(lds0 + kMapOff + (local % kWideMapRing) * 256,
                               (uint64_t)(uintptr_t)((const char*)a.slot + t0 * slot_sz), so);
        }
    };
    auto issue = [&](int64_t tile, int local) {
#pragma unroll
        for (int p = 0; p < 9; ++p) issue_part(tile, local, p);
    };

    const uint32_t r_base = (uint32_t)r * 1024;
    const uint32_t r_swz = (uint32_t)r & 7;
    const int64_t n_slots = a.NB << a.bs_shift;
    const uint32_t csb = (uint32_t)a.cs_block, cst = (uint32_t)a.cs_token;
    uint32_t* const cache_c = a.cache + col * 8;

    // Every wave picks up every tile's slot-mapping entries and reads its code rows; the wave whose
    // turn it is stores them (lane l: half l & 1 of row l >> 1).  No branch around the LDS reads (a
    // join would make the compiler wait for every operand read in flight), and what they return is
    // used a few k-steps later, when younger operand reads are counted behind them.
    int64_t held = -1, sv_raw = 0;
    u32x4 code_raw = {0, 0, 0, 0};
    auto pick_read = [&](int local) {
        const uint8_t* slot_base = wide_lds + kMapOff + (local % kWideMapRing) * 256;
        const int row = lane >> 1;
        if constexpr (SLOT == 2) sv_raw = *reinterpret_cast<const int64_t*>(slot_base + row * 8);
        if constexpr (SLOT == 1) sv_raw = *reinterpret_cast<const int32_t*>(slot_base + row * 4);
        asm volatile("" ::: "memory");  // the read stays here
    };
    auto pick_use = [&](int64_t tile) {
        const int64_t t = tile * kRowsPerWave + (lane >> 1);
        const int64_t sv = SLOT == 0 ? t : sv_raw;
        held = (tile >= 0 && t < a.T && sv >= 0 && sv < n_slots) ? sv : -1;
    };
    auto store_read = [&](int local) {
        const int row = lane >> 1, half = lane & 1;
        code_raw = *reinterpret_cast<const u32x4*>(codes + (local % 3) * kWideCodeBytes + row * 32 + half * 16);
        asm volatile("" ::: "memory");
    };
    auto store_use = [&](bool mine) {
        if (held >= 0 && mine) {
            const uint32_t svl = (uint32_t)held;
            uint32_t* dst = cache_c + ((svl >> a.bs_shift) * csb + (svl & (uint32_t)(a.BS - 1)) * cst) + (lane & 1) * 4;
            *reinterpret_cast<u32x4_a4*>(dst) = code_raw;
        }
    };
    auto hand_in = [&](uint32_t w0, uint32_t w1, int local) {
        w0 = join_halves(kb ? w0 << 4 : w0);
        w1 = join_halves(kb ? w1 << 4 : w1);
        if (lane < 32) *reinterpret_cast<uint2*>(codes + (local % 3) * kWideCodeBytes + r * 32 + wave * 8) = uint2{w0, w1};
    };

    // tiles stream, stream + nstreams, ... : n of them, tile j in ring slot j % 4
    const int64_t n = stream < ntiles ? (ntiles - 1 - stream) / nstreams + 1 : 0;
    const int64_t tile0 = stream;
    constexpr int kAhead = kWideAhead;
    u32x4 b[kAhead];
    f32x16 cstart = acc_start();  // what every sum starts from
    asm volatile("" : "+v"(cstart));
    auto read_b = [&](int j, int ks) {
        const uint8_t* buf = wide_lds + (size_t)(j % kWideRing) * kWideSlotBytes;
        b[ks % kAhead] = *reinterpret_cast<const u32x4*>(buf + r_base + ((((uint32_t)(2 * ks) + kb) ^ r_swz) << 4));
    };
    // Tile j: its products go into (n0, n1) while the signs of tile j - 1 leave (p0, p1).  One
    // barrier, in the middle of the tile: behind it tile j + 1 is complete in LDS (its operand
    // reads start with the second half of tile j's matrix instructions, so the stream of matrix
    // instructions runs on from tile to tile), everybody is done reading tile j - 1 (its ring
    // slot takes tile j + 3), and the words of tile j - 2 are complete.  Tiles -1, -2 (before the
    // first) and n (behind the last) are handled like any other - their words go nowhere, the
    // reads of tile n find whatever the ring slot holds - so that the body has no branches but
    // the one around the loads of tile j + 3 (STEADY: taken for granted).
    auto tile_body = [&](auto steady, int64_t j64, f32x16& n0, f32x16& n1, f32x16& p0, f32x16& p1) {
        constexpr bool STEADY = decltype(steady)::value;
        const int j = (int)j64;
        // The signs of tile j - 1 leave (p0, p1) four instructions per k-step: a wave can issue
        // about seven vector instructions between two pairs of matrix instructions without
        // keeping the matrix cores waiting, and its address arithmetic takes some of them.
        uint32_t hi0 = 0, lo0 = 0, hi1 = 0, lo1 = 0, w0 = 0, w1 = 0;
#pragma unroll
        for (int ks = 0; ks < KS / 2; ++ks) {
            if (ks == 0) {
                wide_mfma_first<V>(n0, wreg[0][ks], b[ks % kAhead], cstart);
                wide_mfma_first<V>(n1, wreg[1][ks], b[ks % kAhead], cstart);
            } else {
                wide_mfma<V>(n0, wreg[0][ks], b[ks % kAhead]);
                wide_mfma<V>(n1, wreg[1][ks], b[ks % kAhead]);
            }
            if (ks + kAhead < KS) read_b(j, ks + kAhead);
            if (ks >= 1 && ks <= 8) {
                // pack_half, one step of its two chains per k-step
                const int st = ks - 1, g = 1 - st / 4, jj = 3 - st % 4;
                __builtin_amdgcn_sched_barrier(0);
                if (st == 4) {
                    hi0 <<= 4;
                    lo0 <<= 4;
                    hi1 <<= 4;
                    lo1 <<= 4;
                }
                hi0 = __builtin_amdgcn_alignbit(hi0, __float_as_uint(p0[4 * (g + 2) + jj]), 31);
                lo0 = __builtin_amdgcn_alignbit(lo0, __float_as_uint(p0[4 * g + jj]), 31);
                hi1 = __builtin_amdgcn_alignbit(hi1, __float_as_uint(p1[4 * (g + 2) + jj]), 31);
                lo1 = __builtin_amdgcn_alignbit(lo1, __float_as_uint(p1[4 * g + jj]), 31);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (ks == 9) {
                __builtin_amdgcn_sched_barrier(0);
                w0 = ((hi0 << 16) | lo0) ^ 0x0F0F0F0Fu;
                w1 = ((hi1 << 16) | lo1) ^ 0x0F0F0F0Fu;
                w0 = p0[0] != p0[0] ? 0u : w0;  // a row with a NaN: no bit set
                w1 = p1[0] != p1[0] ? 0u : w1;
                __builtin_amdgcn_sched_barrier(0);
            }
            if (ks == 10) {
                __builtin_amdgcn_sched_barrier(0);
                hand_in(w0, w1, j + 2);  // tile j - 1's place in the ring of three
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // this wave's loads of tile j + 1 have landed (those of tile j + 2 may be in flight)
        if (STEADY || j64 + 2 < n) stream_wait_loads<kLoads>();
        else stream_wait_loads<0>();
        asm volatile("s_barrier" ::: "memory");
        const bool more = STEADY || j64 + 3 < n;
        const int64_t tile3 = tile0 + (j64 + 3) * nstreams;
        const bool mine = ((j + 2) % kWideWaves) == wave && j >= 2;  // tile j - 2 is this wave's to store
#pragma unroll
        for (int ks = KS / 2; ks < KS; ++ks) {
            wide_mfma<V>(n0, wreg[0][ks], b[ks % kAhead]);
            wide_mfma<V>(n1, wreg[1][ks], b[ks % kAhead]);
            if (ks + kAhead < KS) read_b(j, ks + kAhead);
            else read_b(j + 1, ks + kAhead - KS);
            const int part = ks - KS / 2;
            if (part < 9 && more) issue_part(tile3, j + 3, part);
            if (part == 10) store_read(j + 1);  // tile j - 2's place in the ring of three
            if (part == 11) pick_read(j + 7);   // tile j - 1's entries
            if (part == 14) store_use(mine);
            if (part == 15) pick_use(tile0 + (j64 - 1) * nstreams);
        }
    };

    f32x16 accA0 = acc_start(), accA1 = acc_start(), accB0 = acc_start(), accB1 = acc_start();
    if (n > 0) issue(tile0, 0);
    if (n > 1) issue(tile0 + nstreams, 1);
    if (n > 2) issue(tile0 + 2 * (int64_t)nstreams, 2);
    if (n > 0) {
        if (n > 2) stream_wait_loads<2 * kLoads>();
        else if (n > 1) stream_wait_loads<kLoads>();
        else stream_wait_loads<0>();
        asm volatile("s_barrier" ::: "memory");  // tile 0 is complete
#pragma unroll
        for (int ks = 0; ks < kAhead; ++ks) read_b(0, ks);
        int64_t j = 0;
        for (; j + 4 < n; j += 2) {
            tile_body(std::true_type{}, j, accA0, accA1, accB0, accB1);
            tile_body(std::true_type{}, j + 1, accB0, accB1, accA0, accA1);
        }
        for (; j < n; j += 2) {
            tile_body(std::false_type{}, j, accA0, accA1, accB0, accB1);
            if (j + 1 < n) tile_body(std::false_type{}, j + 1, accB0, accB1, accA0, accA1);
        }
        // the last tile's products: out of the matrix cores, packed, handed in; then the last two
        // tiles' rows are stored
        const int last = (int)(n - 1);
        // nothing reads an accumulator before the matrix cores are done with it (choosing between
        // the two sets is already such a read)
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(accA0), "+v"(accA1), "+v"(accB0), "+v"(accB1));
        const f32x16& l0 = (last & 1) ? accB0 : accA0;
        const f32x16& l1 = (last & 1) ? accB1 : accA1;
        hand_in(pack_half(l0), pack_half(l1), last);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        store_read(last + 2);
        store_use(last >= 1 && ((last - 1) % kWideWaves) == wave);
        pick_read(last);
        pick_use(tile0 + (int64_t)last * nstreams);
        store_read(last);
        store_use((last % kWideWaves) == wave);
    }
    // no load may still be writing into this workgroup's LDS when the wave ends
    stream_wait_loads<0>();
    if (clock_probe && blockIdx.x == 0 && threadIdx.x == 0) {
        clock_probe[0] = __builtin_readcyclecounter() - probe_c0;
        clock_probe[1] = __builtin_amdgcn_s_memrealtime() - probe_r0;
    }
}

// Latency path for a handful of rows (decode): one wave per (job, head, 32 hash columns,
// 32 rows).  No LDS and no persistent loop: the B operand is assembled straight from the
// row-major projection matrix with eight 2-byte loads per k-step, all issued up front, so the
// whole kernel is one round trip to L2 plus K/16 MFMAs.  Up to two independent jobs (e.g. the
// step's new keys and its queries) share one launch.
struct EncJobs {
    EncArgs job[2];
    int waves0;  // waves of job 0; waves >= waves0 belong to job 1
};

// With one projection for all heads and fewer than 32 tokens (a decode step's queries: 16 tokens x
// 64 heads), a tile of 32 consecutive tokens of ONE head is mostly empty and every head's waves
// fetch the same columns of W again.  The rows of a tile are then 32 consecutive (token, head)
// pairs instead: half the waves, full tiles.
__host__ __device__ __forceinline__ bool small_rows_are_pairs(const EncArgs& a)
{
    if (a.H <= 1 || !(a.n_w == 1 || a.heads_per_w <= 0 || a.heads_per_w >= a.H)) return false;
    const int64_t by_head = ((a.T + kRowsPerWave - 1) / kRowsPerWave) * a.H;
    const int64_t by_pair = (a.T * a.H + kRowsPerWave - 1) / kRowsPerWave;
    return by_pair < by_head;
}

// One tile of job `a`: tile index wv counts (row tile, head, 32-column tile), columns fastest
// (row tiles of (token, head) pairs: (row tile, 32-column tile)).  SPLIT = 1: one wave per tile.
// SPLIT = 4 (rows of 256 and 512 values): the four waves of a workgroup take a quarter of the
// row's k-steps each and the partial sums meet in LDS - everything a wave does before its first
// matrix instruction (32 + 32 loads of 16 bytes per lane, 128 permutes, the LDS transpose at
// K = 512) is one chain, and a quarter of it per wave is a quarter of the chain.
template <typename V, int KS, int SPLIT = 1>
__device__ __forceinline__ void encode_small_body(const EncArgs& a, int wv)
{
    static_assert(KS % SPLIT == 0, "the row's k-steps divide evenly over the waves of a tile");
    constexpr int K = KS * 16;        // the row's width: what separates two projection matrices
    constexpr int KSL = KS / SPLIT;   // k-steps of this wave's slice
    constexpr int KL = KSL * 16;
    const int slice = SPLIT > 1 ? (int)(threadIdx.x >> 6) : 0;
    const int k0 = slice * KL;
    const int ntiles = a.N / 32;
    int nt;
    if (a.nt_shift >= 0) {
        nt = wv & (ntiles - 1);
        wv >>= a.nt_shift;
    } else {
        nt = wv % ntiles;
        wv /= ntiles;
    }
    const int lane = threadIdx.x & 63;
    const int r = lane & 31, kb = lane >> 5;
    const bool pairs = small_rows_are_pairs(a);
    int h;          // the lane's head (the wave's, unless the rows are pairs)
    int64_t t;      // the lane's token
    bool row_ok;
    if (pairs) {
        const int64_t rows = a.T * a.H;
        int64_t p = (int64_t)wv * kRowsPerWave + r;
        row_ok = p < rows;
        if (!row_ok) p = rows - 1;
        if (a.h_shift >= 0) {
            t = p >> a.h_shift;
            h = (int)(p & (a.H - 1));
        } else {
            t = p / a.H;
            h = (int)(p - t * a.H);
        }
    } else {
        int row_tile;
        if (a.h_shift >= 0) {
            h = wv & (a.H - 1);
            row_tile = wv >> a.h_shift;
        } else {
            h = wv % a.H;
            row_tile = wv / a.H;
        }
        t = (int64_t)row_tile * kRowsPerWave + r;
        row_ok = t < a.T;
        if (!row_ok) t = a.T - 1;
    }
    // wave-uniform either way
    int wi = 0;
    if (!pairs && a.heads_per_w > 0) wi = a.hpw_shift >= 0 ? h >> a.hpw_shift : h / a.heads_per_w;
    wi = wi < a.n_w ? wi : a.n_w - 1;
    const uint16_t* wsrc = (const uint16_t*)a.w + ((int64_t)wi * K + k0) * a.N + nt * 32 + r;
    const uint16_t* xr = (const uint16_t*)a.x + src_offset(a, t, h) + k0 + kb * 8;
    // where the row's word goes (a read of the slot mapping): asked for with the operands and
    // looked at after the matrix product - behind it, it is a round trip to memory of its own
    const RawSlot raw = fetch_slot_flat(a, t);

    // A wave holds its slice's operands in registers (K = 512 split four ways: 32 + 32, with the
    // patches on their way 125 in all, so that four workgroups fit a compute unit: with two, the
    // 594 tiles of a latent-attention step ran as 512 and then 82, and the launch took twice a
    // tile's time).
    V av[KSL];
    uint16_t bw[KSL][8];
    if (a.gmean > 1) {
        // fp32 sum of the group's rows in order, times 1/G, rounded to the input type.  Groups of
        // 2, 4 and 8 rows are written out: a load inside a loop of run-time length is waited for
        // before the next is issued (K / 16 x G round trips to L2 one after the other: 13 us of a
        // 15 us launch at K = 512, G = 2); written out, up to 64 loads are in flight at once.
        const float inv = 1.0f / (float)a.gmean;
        auto mean_rows = [&](auto gc) __attribute__((always_inline)) {
            constexpr int G = decltype(gc)::value;
            constexpr int kInFlight = SPLIT > 1 ? 16 : 64;  // a split tile's waves keep within a third of the registers
            constexpr int CH = KSL * G > kInFlight ? kInFlight / G : KSL;  // k-steps whose loads go out together
#pragma unroll
            for (int ks0 = 0; ks0 < KSL; ks0 += CH) {
                V v[CH][G];
#pragma unroll
                for (int c = 0; c < CH; ++c)
#pragma unroll
                    for (int g = 0; g < G; ++g)
                        v[c][g] = *reinterpret_cast<const V*>(xr + (int64_t)g * a.x_stride_g + (ks0 + c) * 16);
#pragma unroll
                for (int c = 0; c < CH; ++c) {
                    float sum[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) sum[i] = 0.0f;
#pragma unroll
                    for (int g = 0; g < G; ++g)
#pragma unroll
                        for (int i = 0; i < 8; ++i) sum[i] += (float)v[c][g][i];
                    V m;
#pragma unroll
                    for (int i = 0; i < 8; ++i) m[i] = (typename Mfma<V>::elem)(sum[i] * inv);  // round to nearest even
                    av[ks0 + c] = m;
                }
            }
        };
        if (a.gmean == 2) mean_rows(std::integral_constant<int, 2>{});
        else if (a.gmean == 4) mean_rows(std::integral_constant<int, 4>{});
        else if (a.gmean == 8) mean_rows(std::integral_constant<int, 8>{});
        else {
#pragma unroll
            for (int ks = 0; ks < KSL; ++ks) {
                float sum[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) sum[i] = 0.0f;
                for (int g = 0; g < a.gmean; ++g) {
                    const V v = *reinterpret_cast<const V*>(xr + (int64_t)g * a.x_stride_g + ks * 16);
#pragma unroll
                    for (int i = 0; i < 8; ++i) sum[i] += (float)v[i];
                }
                V m;
#pragma unroll
                for (int i = 0; i < 8; ++i) m[i] = (typename Mfma<V>::elem)(sum[i] * inv);  // round to nearest even
                av[ks] = m;
            }
        }
    } else {
#pragma unroll
        for (int ks = 0; ks < KSL; ++ks) av[ks] = *reinterpret_cast<const V*>(xr + ks * 16);
    }
    // The wave's 32 columns of W in operand layout (8 consecutive k of one column per lane and
    // k-step).  16-byte aligned weights: lanes fetch 8 x 8 patches (eight 16-byte rows each),
    // transpose them in registers and pass them through LDS - K / 16 loads per lane; fetching the
    // operands directly takes eight 2-byte loads per k-step (K / 2 per lane: 256 at K = 512).
    constexpr int KP = KL + kPad;
    __shared__ __align__(16) uint16_t wt_all[SPLIT][32 * KP];
    uint16_t* wt = wt_all[slice];
    V bv[KSL];
    if ((reinterpret_cast<uintptr_t>(a.w) & 15) == 0) {
        constexpr int kPatches = (KL / 8) * 4;
        constexpr int kIters = (kPatches + 63) / 64;
        const uint16_t* wslice = (const uint16_t*)a.w + ((int64_t)wi * K + k0) * a.N + nt * 32;
        u32x4 row[kIters][8];
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            const int idx = (it * 64 + lane) % kPatches;  // lanes past the last patch repeat one
            const uint16_t* src = wslice + (int64_t)((idx >> 2) * 8) * a.N + 8 * (idx & 3);
#pragma unroll
            for (int i = 0; i < 8; ++i) row[it][i] = *reinterpret_cast<const u32x4*>(src + (int64_t)i * a.N);
        }
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            const int idx = (it * 64 + lane) % kPatches;
            const int kq = idx >> 2, j = idx & 3;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
                u32x4 o;
                o.x = __builtin_amdgcn_perm(row[it][1][c >> 1], row[it][0][c >> 1], sel);
                o.y = __builtin_amdgcn_perm(row[it][3][c >> 1], row[it][2][c >> 1], sel);
                o.z = __builtin_amdgcn_perm(row[it][5][c >> 1], row[it][4][c >> 1], sel);
                o.w = __builtin_amdgcn_perm(row[it][7][c >> 1], row[it][6][c >> 1], sel);
                *reinterpret_cast<u32x4*>(wt + (8 * j + c) * KP + kq * 8) = o;
            }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int ks = 0; ks < KSL; ++ks) bv[ks] = *reinterpret_cast<const V*>(wt + r * KP + ks * 16 + kb * 8);
    } else {
#pragma unroll
        for (int ks = 0; ks < KSL; ++ks) {
#pragma unroll
            for (int i = 0; i < 8; ++i) bw[ks][i] = wsrc[(int64_t)(ks * 16 + kb * 8 + i) * a.N];
            __builtin_memcpy(&bv[ks], bw[ks], 16);
        }
    }

    f32x16 acc = acc_start();
#pragma unroll
    for (int ks = 0; ks < KSL; ++ks) acc = Mfma<V>::run(bv[ks], av[ks], acc);

    if (SPLIT > 1) {
        // the slices' sums meet in wave 0 in slice order.  Every slice starts from the same small
        // negative number, which vanishes in any sum that is not exactly zero and keeps a row of
        // zeros negative; NaN passes through the additions.
        // A wave's partial sums go where its slice of W was: its own reads of that region are
        // behind it (LDS operations of a wave complete in order), and nobody else touches it
        // before the barrier.
        static_assert(sizeof(wt_all[0]) >= 16 * 64 * sizeof(float), "a slice of W makes room for one wave's sums");
        float* part = reinterpret_cast<float*>(wt);
        if (slice > 0) {
#pragma unroll
            for (int i = 0; i < 16; ++i) part[i * 64 + lane] = acc[i];
        }
        __syncthreads();
        if (slice > 0) return;
#pragma unroll
        for (int sl = 1; sl < SPLIT; ++sl) {
            const float* other = reinterpret_cast<const float*>(wt_all[sl]);
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] += other[i * 64 + lane];
        }
    }
    const uint32_t half = pack_half(acc);
    const uint32_t word = join_halves(kb ? half << 4 : half);
    if (row_ok && lane < 32) {
        uint32_t* dst = slot_dst(a, slot_value(a, raw, t), h);
        if (dst) dst[nt] = word;
    }
}

// Touches every 64-byte line of a kernel-argument struct at once.  The compiler fetches a field
// where the code first needs it, behind the branches of the row addressing - a dozen scalar reads
// one after the other in a kernel that lives for a few microseconds; with the lines already in the
// scalar cache those reads are short.  (Copying the struct through pinned registers instead makes
// its pointers lose their address space: every access becomes a flat one.)
template <class T>
__device__ __forceinline__ void warm_args(const T& args)
{
    const uint32_t* src = reinterpret_cast<const uint32_t*>(&args);
    uint32_t t = 0;
#pragma unroll
    for (unsigned i = 0; i < sizeof(T) / 4; i += 16) t |= src[i];
    t |= src[sizeof(T) / 4 - 1];
    asm volatile("" ::"s"(t));
}

// waves that share a tile: rows of 256 values and more are split four ways
constexpr int small_split(int KS) { return KS >= 16 ? 4 : 1; }

template <typename V, int KS>
__global__ __launch_bounds__(64 * small_split(KS)) __attribute__((amdgpu_waves_per_eu(small_split(KS) > 1 ? 3 : 1, 8))) void encode_small_kernel(EncJobs js)
{
    warm_args(js);
    const bool second = (int)blockIdx.x >= js.waves0;
    encode_small_body<V, KS, small_split(KS)>(second ? js.job[1] : js.job[0],
                                              second ? blockIdx.x - js.waves0 : blockIdx.x);
}

// Four jobs in one launch, two of input width 16 * KSA and two of 16 * KSB (the two parts of a
// latent-attention step: new keys and queries of the nope and of the rope encoder).
struct EncJobs4 {
    EncArgs job[4];
    int end[4];  // first wave index past job i
};

template <typename V, int KSA, int KSB>
__global__ __launch_bounds__(64 * small_split(KSA)) __attribute__((amdgpu_waves_per_eu(3, 8))) void encode_small_mixed_kernel(EncJobs4 js)
{
    static_assert(small_split(KSB) == 1, "the narrow jobs' tiles take one wave of the workgroup");
    warm_args(js);
    const int w = blockIdx.x;
    if (w < js.end[1]) {
        const int j = w >= js.end[0] ? 1 : 0;
        encode_small_body<V, KSA, small_split(KSA)>(js.job[j], j ? w - js.end[0] : w);
    } else {
        if (threadIdx.x >= 64) return;  // a narrow tile is one wave's work
        const int j = w >= js.end[2] ? 3 : 2;
        encode_small_body<V, KSB>(js.job[j], w - js.end[j - 1]);
    }
}

__device__ __forceinline__ float load_as_float(const void* p, int dtype, int64_t i)
{
    if (dtype == UCM_DT_F32) return ((const float*)p)[i];
    if (dtype == UCM_DT_F16) return __half2float(((const __half*)p)[i]);
    const uint32_t u = (uint32_t)((const uint16_t*)p)[i] << 16;
    return __uint_as_float(u);
}

// Plain FMA path: one thread per (row, head, output word); fp32 accumulation in ascending k.
__global__ __launch_bounds__(kThreads) void encode_fma_kernel(EncArgs a, int x_dtype, int w_dtype)
{
    const int Wd = a.N / 32;
    const int64_t total = a.T * a.H * Wd;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * kThreads) {
        const int w = (int)(i % Wd);
        const int h = (int)((i / Wd) % a.H);
        const int64_t t = i / ((int64_t)Wd * a.H);
        uint32_t* dst = row_dst(a, t, h);
        if (!dst) continue;
        const int64_t xo = src_offset(a, t, h);
        const int64_t wo = (int64_t)weight_index(a, h) * a.K * a.N + w * 32;
        float acc[32];
#pragma unroll
        for (int j = 0; j < 32; ++j) acc[j] = 0.0f;
        for (int k = 0; k < a.K; ++k) {
            const float xv = load_as_float(a.x, x_dtype, xo + k);
#pragma unroll
            for (int j = 0; j < 32; ++j)
                acc[j] = __builtin_fmaf(xv, load_as_float(a.w, w_dtype, wo + (int64_t)k * a.N + j), acc[j]);
        }
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 32; ++j) word |= (acc[j] > 0.0f ? 1u : 0u) << j;
        dst[w] = word;
    }
}

__global__ __launch_bounds__(kThreads) void code_scatter_kernel(const uint32_t* __restrict__ codes,
                                                                int64_t T, int H, int Wd,
                                                                int64_t in_stride_t,
                                                                int64_t in_stride_h, EncArgs a)
{
    const int64_t total = T * H * Wd;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * kThreads) {
        const int w = (int)(i % Wd);
        const int h = (int)((i / Wd) % H);
        const int64_t t = i / ((int64_t)Wd * H);
        uint32_t* dst = row_dst(a, t, h);
        if (dst) dst[w] = codes[t * in_stride_t + (int64_t)h * in_stride_h + w];
    }
}

// Widest slice of hash columns (a multiple of 32 that divides N) whose transposed LDS image
// stays within `cap` bytes; 0 when not even 32 columns fit.
int pick_slice(int N, int K, size_t cap)
{
    for (int bn = N; bn >= 32; bn -= 32)
        if (N % bn == 0 && (size_t)bn * (K + kPad) * 2 <= cap) return bn;
    return 0;
}

template <typename V, int KS, int NQ, int NG>
int launch_mfma_q(const EncArgs& a, size_t lds, const dim3& grid, hipStream_t st)
{
    // 0 = not tried, 1 = large LDS allocations allowed, -1 = refused by the runtime
    static int big_lds = 0;
    if (lds > 64 * 1024) {
        if (big_lds == 0) {
            const hipError_t e =
                hipFuncSetAttribute((const void*)encode_mfma_kernel<V, KS, NQ, NG>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) (void)hipGetLastError();
            big_lds = (e == hipSuccess) ? 1 : -1;
        }
        if (big_lds < 0) return UCM_EUNSUPPORTED;
    }
    hipLaunchKernelGGL((encode_mfma_kernel<V, KS, NQ, NG>), grid, dim3(kMfmaThreads), lds, st, a);
    return ucm::launch_status("encode_mfma_kernel");
}

template <typename V, int KS>
int launch_mfma(EncArgs a, hipStream_t st)
{
    constexpr int K = KS * 16;
    constexpr size_t kStage = (size_t)kMfmaWaves * kStageBytes;
    for (size_t cap : {(size_t)160 * 1024, (size_t)64 * 1024}) {
        a.BN = pick_slice(a.N, K, cap - kStage);
        if (a.BN == 0) return ucm::fail(UCM_EUNSUPPORTED, "no LDS slice fits K=%d", K);
        const size_t lds = (size_t)a.BN * (K + kPad) * 2 + kStage;
        const int64_t tiles = (a.T + kRowsPerWg - 1) / kRowsPerWg;
        const int slices = a.N / a.BN;
        const dim3 grid((unsigned)ucm::ceil_div(tiles, kTilesPerWg), (unsigned)slices, (unsigned)a.H);
        const int nt = a.BN / 32;
        const int rc = nt == 4       ? launch_mfma_q<V, KS, 4, 1>(a, lds, grid, st)
                       : nt == 8     ? launch_mfma_q<V, KS, 4, 2>(a, lds, grid, st)
                       : nt % 4 == 0 ? launch_mfma_q<V, KS, 4, 0>(a, lds, grid, st)
                       : nt == 2     ? launch_mfma_q<V, KS, 2, 1>(a, lds, grid, st)
                       : nt == 1     ? launch_mfma_q<V, KS, 1, 1>(a, lds, grid, st)
                       : nt % 2 == 0 ? launch_mfma_q<V, KS, 2, 0>(a, lds, grid, st)
                                     : launch_mfma_q<V, KS, 1, 0>(a, lds, grid, st);
        // a refused large-LDS opt-in falls back to the slice that fits the default 64 KiB
        if (rc != UCM_EUNSUPPORTED || lds <= 64 * 1024) return rc;
    }
    return ucm::fail(UCM_EUNSUPPORTED, "no LDS slice fits K=%d", K);
}

template <typename V>
int dispatch_mfma(const EncArgs& a, hipStream_t st)
{
    switch (a.K) {
        case 64: return launch_mfma<V, 4>(a, st);
        case 128: return launch_mfma<V, 8>(a, st);
        case 256: return launch_mfma<V, 16>(a, st);
        case 512: return launch_mfma<V, 32>(a, st);
        default: return ucm::fail(UCM_ERROR, "internal: K %d has no MFMA kernel", a.K);
    }
}

constexpr int64_t kSmallRows = 256;  // at most this many rows per head take the latency path

bool mfma_eligible(const EncArgs& a, int x_dtype, int w_dtype)
{
    const bool same16 = (x_dtype == w_dtype) && (x_dtype == UCM_DT_BF16 || x_dtype == UCM_DT_F16);
    const bool k_ok = a.K == 64 || a.K == 128 || a.K == 256 || a.K == 512;
    // 16-byte row pieces; a wave's 32 rows must span less than 2 GiB (32-bit lane offsets)
    const bool aligned = (((uintptr_t)a.x | (uintptr_t)a.w) & 15) == 0 && a.x_stride_t % 8 == 0 &&
                         a.x_stride_h % 8 == 0 && a.x_stride_t >= 0 &&
                         a.x_stride_t < ((int64_t)1 << 31) / (2 * kRowsPerWave);
    // paged input: a wave's 32 rows must lie in one block
    const bool paged_ok = !a.src_blocks || (a.BS % kRowsPerWave == 0 && a.xs_block % 8 == 0);
    return same16 && k_ok && aligned && paged_ok;
}

// ---- streaming kernel: eligibility and launch ----
// rows x heads from which the streaming kernel is used: below about a million rows its fixed
// cost (every wave stages a projection matrix of its own, 256 persistent workgroups) loses against
// the tiled kernel (65,536 rows: 14.8 against 12.4 us; 1M rows: 67.6 against 71.8 us; 4M rows: 225
// against 262 us)
constexpr int64_t kStreamMinRows = (int64_t)1 << 20;
// the wide (K = 512) kernel pays for itself earlier: it replaces a tiled kernel that re-reads the
// rows once per slice of the projection (256 bits: 16,384 rows 19 against 26 us, 262,144 rows 74
// against 164 us; 512 bits: 32,768 rows 36 against 34 us, 65,536 rows 52 against 65 us, 262,144 rows
// 155 against 301 us)
constexpr int64_t kWideMinRows256 = (int64_t)1 << 14;
constexpr int64_t kWideMinRows512 = (int64_t)1 << 16;
// 0 = the defaults above; set per calling thread (a test hook must not move other threads' encodes)
thread_local int64_t t_stream_min_rows = 0;
thread_local unsigned long long* t_clock_probe = nullptr;  // see ucm_hash_encode_set_clock_probe()

int stream_workgroups()
{
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = 256;
        }
        cus = n;
    }
    return cus;
}

bool stream_eligible(const EncArgs& a, int x_dtype, int w_dtype)
{
    if (!mfma_eligible(a, x_dtype, w_dtype) || a.src_blocks) return false;
    if (!((a.K == 128 && (a.N == 128 || a.N == 64)) || (a.K == 64 && (a.N == 128 || a.N == 64)))) return false;
    if (a.T * a.H < (t_stream_min_rows > 0 ? t_stream_min_rows : kStreamMinRows)) return false;
    if (a.slot && ((uintptr_t)a.slot & 3)) return false;
    // one shift per slot, one 16-byte store per four-word code (set_block_shift() has run)
    if (a.bs_shift < 0) return false;
    if (a.N == 128 && ((((uintptr_t)a.cache) & 15) || a.cs_block % 4 || a.cs_token % 4 || a.cs_head % 4)) return false;
    // 32-bit offsets into the cache: non-negative strides, the last slot below 2^31 words
    if (a.cs_block < 0 || a.cs_token < 0 || a.cs_head < 0) return false;
    if ((double)a.NB * (double)a.cs_block + (double)a.BS * (double)a.cs_token >= 2147483648.0) return false;
    if ((double)a.NB * (double)a.BS >= 2147483648.0) return false;
    // every head needs at least one wave, and the heads must share the waves evenly
    const int waves = stream_workgroups() * kStreamWaves;
    return a.H <= waves;
}

template <typename V, int KS, int NT, int SLOT, int ACCS, int HC>
int launch_stream_a(const EncArgs& a, hipStream_t st)
{
    constexpr size_t lds = (size_t)kStreamWaves * 2 * (kRowsPerWave * KS * 32 + 256) + ring_lds_bytes(HC);
    static_assert(lds <= 160 * 1024, "row buffers and ring exceed the LDS");
    static int opted = 0;  // 0 = not tried, 1 = allowed, -1 = refused by the runtime
    if (opted == 0) {
        const hipError_t e = hipFuncSetAttribute((const void*)encode_stream_kernel<V, KS, NT, SLOT, ACCS, HC>,
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) (void)hipGetLastError();
        opted = (e == hipSuccess) ? 1 : -1;
    }
    if (opted < 0) return UCM_EUNSUPPORTED;
    int wgs = stream_workgroups();
    // total waves a multiple of the head count: lower the workgroup count until it is
    while (wgs > 1 && (wgs * kStreamWaves) % a.H) --wgs;
    if ((wgs * kStreamWaves) % a.H) return UCM_EUNSUPPORTED;
    const int nstreams = wgs * kStreamWaves / a.H;
    const int64_t ntiles = ucm::ceil_div(a.T, kRowsPerWave);
    hipLaunchKernelGGL((encode_stream_kernel<V, KS, NT, SLOT, ACCS, HC>), dim3((unsigned)wgs), dim3(kStreamThreads),
                       lds, st, a, ntiles, nstreams);
    return ucm::launch_status("encode_stream_kernel");
}

// Whole cache rows from one wave: 2, 4 or 8 heads of four-word codes that lie side by side in a
// token row aligned to its own size.  Returns the head count, 0 when the shape does not qualify.
int stream_combine(const EncArgs& a)
{
    if (!(a.H == 2 || a.H == 4 || a.H == 8) || a.N != 128 || a.cs_head != 4) return 0;
    if (a.cs_token != 4 * a.H || a.cs_block % (4 * a.H) || (((uintptr_t)a.cache) & (16 * a.H - 1))) return 0;
    return a.H;
}

template <typename V, int KS, int NT, int SLOT>
int launch_stream_i(const EncArgs& a, hipStream_t st)
{
    if constexpr (NT == 4) {
        switch (stream_combine(a)) {
            case 8: return launch_stream_a<V, KS, NT, SLOT, 2, 8>(a, st);
            case 4: return launch_stream_a<V, KS, NT, SLOT, 2, 4>(a, st);
            case 2: return launch_stream_a<V, KS, NT, SLOT, 2, 2>(a, st);
            default: break;
        }
    }
    return launch_stream_a<V, KS, NT, SLOT, (NT == 4 ? 4 : 2), 0>(a, st);
}

template <typename V, int KS, int NT>
int launch_stream_s(const EncArgs& a, hipStream_t st)
{
    if (!a.slot) return launch_stream_i<V, KS, NT, 0>(a, st);
    return a.slot_is_i64 ? launch_stream_i<V, KS, NT, 2>(a, st) : launch_stream_i<V, KS, NT, 1>(a, st);
}

template <typename V>
int launch_stream(const EncArgs& a, hipStream_t st)
{
    if (a.K == 128) return a.N == 128 ? launch_stream_s<V, 8, 4>(a, st) : launch_stream_s<V, 8, 2>(a, st);
    return a.N == 128 ? launch_stream_s<V, 4, 4>(a, st) : launch_stream_s<V, 4, 2>(a, st);
}

// The wide kernel takes one head of 512 input dimensions, 256 or 512 hash bits, dense rows.
bool wide_eligible(const EncArgs& a, int x_dtype, int w_dtype)
{
    if (!mfma_eligible(a, x_dtype, w_dtype) || a.src_blocks || a.gmean > 1) return false;
    if (a.K != kWideK || !(a.N == 256 || a.N == 512) || a.H != 1) return false;
    if (a.T < (t_stream_min_rows > 0 ? t_stream_min_rows : (a.N == 256 ? kWideMinRows256 : kWideMinRows512))) return false;
    if (a.slot && ((uintptr_t)a.slot & 3)) return false;
    if (a.bs_shift < 0 || (((uintptr_t)a.cache) & 3)) return false;
    // 32-bit offsets into the cache: non-negative strides, the last slot below 2^31 words
    if (a.cs_block < 0 || a.cs_token < 0) return false;
    if ((double)a.NB * (double)a.cs_block + (double)a.BS * (double)a.cs_token >= 2147483648.0) return false;
    if ((double)a.NB * (double)a.BS >= 2147483648.0) return false;
    return true;
}

template <typename V, int SLOT>
int launch_wide_s(const EncArgs& a, hipStream_t st)
{
    static int opted = 0;  // 0 = not tried, 1 = allowed, -1 = refused by the runtime
    if (opted == 0) {
        const hipError_t e = hipFuncSetAttribute((const void*)encode_wide_kernel<V, SLOT>,
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kWideLds);
        if (e != hipSuccess) (void)hipGetLastError();
        opted = (e == hipSuccess) ? 1 : -1;
    }
    if (opted < 0) return UCM_EUNSUPPORTED;
    const int ncol = a.N / 256;
    int wgs = stream_workgroups();
    wgs -= wgs % 8;
    if (wgs <= 0) return UCM_EUNSUPPORTED;
    const int64_t ntiles = ucm::ceil_div(a.T, kRowsPerWave);
    // one workgroup per compute unit and slice of 256 hash columns; a second slice is a second pass
    // over the rows (two slices side by side, meeting in L2, measured the same)
    for (int c = 0; c < ncol; ++c)
        hipLaunchKernelGGL((encode_wide_kernel<V, SLOT>), dim3((unsigned)wgs), dim3(kWideThreads), kWideLds, st, a,
                           ntiles, wgs, c, t_clock_probe);
    return ucm::launch_status("encode_wide_kernel");
}

template <typename V>
int launch_wide(const EncArgs& a, hipStream_t st)
{
    if (!a.slot) return launch_wide_s<V, 0>(a, st);
    return a.slot_is_i64 ? launch_wide_s<V, 2>(a, st) : launch_wide_s<V, 1>(a, st);
}

int64_t small_waves(const EncArgs& a)
{
    if (small_rows_are_pairs(a)) return ucm::ceil_div(a.T * a.H, kRowsPerWave) * (a.N / 32);
    return ucm::ceil_div(a.T, kRowsPerWave) * a.H * (a.N / 32);
}

template <typename V>
int launch_small(const EncJobs& js, int64_t waves, int K, hipStream_t st)
{
    const dim3 grid((unsigned)waves);
    switch (K) {
        case 64: hipLaunchKernelGGL((encode_small_kernel<V, 4>), grid, dim3(64), 0, st, js); break;
        case 128: hipLaunchKernelGGL((encode_small_kernel<V, 8>), grid, dim3(64), 0, st, js); break;
        case 256: hipLaunchKernelGGL((encode_small_kernel<V, 16>), grid, dim3(64 * small_split(16)), 0, st, js); break;
        case 512: hipLaunchKernelGGL((encode_small_kernel<V, 32>), grid, dim3(64 * small_split(32)), 0, st, js); break;
        default: return ucm::fail(UCM_ERROR, "internal: K %d has no small-row kernel", K);
    }
    return ucm::launch_status("encode_small_kernel");
}

// Folds a dense output into the paged form: block = row, one token per block, identity slots.
void normalize_output(EncArgs& a)
{
    if (a.cache) return;
    a.cache = a.out;
    a.slot = nullptr;
    a.slot_is_i64 = 1;
    a.NB = a.T > 0 ? a.T : 1;
    a.BS = 1;
    a.cs_block = a.out_stride_t;
    a.cs_token = 0;
    a.cs_head = a.out_stride_h;
}

void set_block_shift(EncArgs& a)
{
    normalize_output(a);
    a.bs_shift = -1;
    if (a.BS > 0 && (a.BS & (a.BS - 1)) == 0) a.bs_shift = __builtin_ctz((unsigned)a.BS);
    auto log2_or_minus1 = [](int v) { return v > 0 && (v & (v - 1)) == 0 ? __builtin_ctz((unsigned)v) : -1; };
    a.nt_shift = log2_or_minus1(a.N / 32);
    a.h_shift = log2_or_minus1(a.H);
    a.hpw_shift = log2_or_minus1(a.heads_per_w);
}

int check_shape(const EncArgs& a, int x_dtype, int w_dtype)
{
    UCM_REQUIRE(a.x && a.w, "null input");
    UCM_REQUIRE(a.T >= 0 && a.H > 0 && a.K > 0 && a.N > 0, "bad shape");
    UCM_REQUIRE(a.H <= 65535, "more than 65535 heads");
    UCM_REQUIRE(a.N % 32 == 0, "hash_bits %d must be a multiple of 32", a.N);
    UCM_REQUIRE(a.n_w >= 1 && a.heads_per_w >= 0, "bad weight layout");
    UCM_REQUIRE(x_dtype >= 0 && x_dtype <= 2 && w_dtype >= 0 && w_dtype <= 2, "unknown dtype");
    return UCM_OK;
}

// LDS-tiled FMA path for what the matrix-core kernels do not take (fp32 inputs, K that is not
// 64/128/256/512, row layouts they reject): a workgroup computes 64 rows x TN hash columns of
// one head, K in chunks of 16 staged in LDS (x transposed, k-major), each thread an 8 x 4
// micro-tile (32 fp32 accumulators, 32 FMAs per three 16-byte LDS reads).  A row's word is
// assembled from the eight neighbouring lanes that hold its 32 columns.  DT: element type of x
// and W (both the same).  grid = (ceil(T / 64), N / TN, H).
template <int DT, int TN>
__global__ __launch_bounds__(kThreads) void encode_tiled_kernel(EncArgs a)
{
    constexpr int TM = 64, KC = 16;
    __shared__ __align__(16) float xs[KC][TM];
    __shared__ __align__(16) float wsm[KC][TN];
    const int h = blockIdx.z;
    const int n0 = blockIdx.y * TN;
    const int64_t t0 = (int64_t)blockIdx.x * TM;
    const int tid = threadIdx.x;
    constexpr int CG = TN / 4;            // column groups of 4 (threads along N)
    constexpr int RG = kThreads / CG;     // row groups
    constexpr int RPT = TM / RG;          // rows per thread
    const int tx = tid % CG, ty = tid / CG;
    const int64_t wbase = (int64_t)weight_index(a, h) * a.K * a.N + n0;

    // the row this thread stages (tid / 4) and its four k positions per chunk
    const int xr = tid >> 2, xk = (tid & 3) * 4;
    int64_t xt = t0 + xr;
    if (xt >= a.T) xt = a.T - 1;  // in-bounds read; the row is dropped at the store
    const int64_t xo = src_offset(a, xt, h);

    float acc[RPT][4];
#pragma unroll
    for (int r = 0; r < RPT; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[r][c] = 0.0f;

    for (int k0 = 0; k0 < a.K; k0 += KC) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + xk + i;
            xs[xk + i][xr] = k < a.K ? load_as_float(a.x, DT, xo + k) : 0.0f;
        }
#pragma unroll
        for (int e = tid; e < KC * TN; e += kThreads) {
            const int kk = e / TN, c = e % TN;
            wsm[kk][c] = k0 + kk < a.K ? load_as_float(a.w, DT, wbase + (int64_t)(k0 + kk) * a.N + c) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KC; ++kk) {
            const float4 wv = *reinterpret_cast<const float4*>(&wsm[kk][tx * 4]);
            float xv[RPT];
            if constexpr (RPT >= 4) {
#pragma unroll
                for (int r4 = 0; r4 < RPT; r4 += 4) {
                    const float4 v = *reinterpret_cast<const float4*>(&xs[kk][ty * RPT + r4]);
                    xv[r4] = v.x; xv[r4 + 1] = v.y; xv[r4 + 2] = v.z; xv[r4 + 3] = v.w;
                }
            } else {
#pragma unroll
                for (int r = 0; r < RPT; ++r) xv[r] = xs[kk][ty * RPT + r];
            }
#pragma unroll
            for (int r = 0; r < RPT; ++r) {
                acc[r][0] = __builtin_fmaf(xv[r], wv.x, acc[r][0]);
                acc[r][1] = __builtin_fmaf(xv[r], wv.y, acc[r][1]);
                acc[r][2] = __builtin_fmaf(xv[r], wv.z, acc[r][2]);
                acc[r][3] = __builtin_fmaf(xv[r], wv.w, acc[r][3]);
            }
        }
        __syncthreads();
    }
    // eight neighbouring lanes (tx % 8 = 0..7) hold the 32 columns of one word
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        uint32_t v = (acc[r][0] > 0.0f ? 1u : 0u) | (acc[r][1] > 0.0f ? 2u : 0u) |
                     (acc[r][2] > 0.0f ? 4u : 0u) | (acc[r][3] > 0.0f ? 8u : 0u);
        v <<= 4 * (tx & 7);
        v |= __shfl_xor(v, 1);
        v |= __shfl_xor(v, 2);
        v |= __shfl_xor(v, 4);
        const int64_t t = t0 + ty * RPT + r;
        if ((tx & 7) == 0 && t < a.T) {
            uint32_t* dst = row_dst(a, t, h);
            if (dst) dst[(n0 >> 5) + (tx >> 3)] = v;
        }
    }
}

template <int DT>
int launch_tiled(const EncArgs& a, hipStream_t st)
{
    const int tn = a.N % 128 == 0 ? 128 : (a.N % 64 == 0 ? 64 : 32);
    const dim3 grid((unsigned)ucm::ceil_div(a.T, 64), (unsigned)(a.N / tn), (unsigned)a.H);
    if (tn == 128) hipLaunchKernelGGL((encode_tiled_kernel<DT, 128>), grid, dim3(kThreads), 0, st, a);
    else if (tn == 64) hipLaunchKernelGGL((encode_tiled_kernel<DT, 64>), grid, dim3(kThreads), 0, st, a);
    else hipLaunchKernelGGL((encode_tiled_kernel<DT, 32>), grid, dim3(kThreads), 0, st, a);
    return ucm::launch_status("encode_tiled_kernel");
}

// Which matrix-core kernel: the wave-per-tile kernel costs about 4 us plus 12.5 ps per wave and
// k value (each wave gathers its own operand columns from L2); the LDS kernel has a floor of
// about 6 us plus 0.13 us per KiB of projection slice that every workgroup stages before its
// first tile (7 us at 64 x 64, 10 us at 128 x 128, 23-24 us for a 133 KiB slice), after which it
// streams rows at HBM rate.  Measured crossovers this reproduces: 128 -> 128 bits with 8 heads at
// ~4000 rows, 256 -> 256 with 4 heads and 512 -> 512 at ~5000-6000 rows, 64 -> 64 never below
// 16,384 rows.
bool small_eligible(const EncArgs& a, int x_dtype, int w_dtype)
{
    if (!mfma_eligible(a, x_dtype, w_dtype) || small_waves(a) > 0x7fffffff) return false;
    if (a.T <= kSmallRows && a.K <= 256) return true;
    constexpr size_t kStage = (size_t)kMfmaWaves * kStageBytes;
    const int bn = pick_slice(a.N, a.K, (size_t)160 * 1024 - kStage);
    if (bn == 0) return true;
    const double slice_kib = (double)bn * (a.K + kPad) * 2 / 1024.0;
    const double lds_floor_us = 6.0 + 0.13 * slice_kib;
    const double small_us = 4.0 + (double)small_waves(a) * a.K * 12.5e-6;
    return small_us < lds_floor_us;
}

// ---- the streaming kernel's time-out latch ----
// A wave of the streaming kernel whose bounded wait gave up sets a word in pinned host memory (one
// per device, allocated with the first streaming launch on it).  Every encode entry point reads that
// word first - a plain host read, no device call - and fails with UCM_ERROR while it is set: the
// codes of the launch that tripped it are undefined, so the caller must rebuild them and acknowledge
// with ucm_hash_encode_clear_stream_timeouts().
constexpr int kLatchDevices = 64;
std::mutex g_latch_mu;
unsigned int* g_latch_host[kLatchDevices] = {nullptr};  // pinned, mapped
unsigned int* g_latch_dev[kLatchDevices] = {nullptr};   // the same words as the device sees them
std::atomic<unsigned int> g_latch_forced[kLatchDevices];  // ucm_hash_encode_debug_trip_stream_latch()

int latch_device()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        dev = 0;  // no device at all: the latch still works for its host-side users
    }
    return dev >= 0 && dev < kLatchDevices ? dev : 0;
}

// Device address of the current device's flag word; null when pinned memory cannot be had (the
// kernel then only counts in g_stream_wait_timeouts).
unsigned int* stream_latch_flag()
{
    const int dev = latch_device();
    std::lock_guard<std::mutex> g(g_latch_mu);
    if (!g_latch_dev[dev]) {
        void* h = nullptr;
        void* d = nullptr;
        if (hipHostMalloc(&h, 64, hipHostMallocMapped) != hipSuccess || !h ||
            hipHostGetDevicePointer(&d, h, 0) != hipSuccess || !d) {
            (void)hipGetLastError();
            if (h) (void)hipHostFree(h);
            return nullptr;
        }
        *static_cast<volatile unsigned int*>(h) = 0;
        g_latch_host[dev] = static_cast<unsigned int*>(h);
        g_latch_dev[dev] = static_cast<unsigned int*>(d);
    }
    return g_latch_dev[dev];
}

bool stream_latch_tripped(int dev)
{
    if (g_latch_forced[dev].load(std::memory_order_relaxed)) return true;
    const volatile unsigned int* h = g_latch_host[dev];  // written once under the mutex, then constant
    return h && *h != 0;
}

int stream_latch_check()
{
    const int dev = latch_device();
    if (!stream_latch_tripped(dev)) return UCM_OK;
    return ucm::fail(UCM_ERROR,
                     "an earlier streaming encode on device %d gave up waiting for its workgroup's code exchange: "
                     "the codes that launch wrote are undefined; rebuild them, then call "
                     "ucm_hash_encode_clear_stream_timeouts()", dev);
}

int encode_common(EncArgs a, int x_dtype, int w_dtype, hipStream_t st)
{
    {
        const int lrc = stream_latch_check();
        if (lrc != UCM_OK) return lrc;
    }
    set_block_shift(a);
    int rc = check_shape(a, x_dtype, w_dtype);
    if (rc != UCM_OK) return rc;
    if (a.T == 0) return UCM_OK;

    if (small_eligible(a, x_dtype, w_dtype)) {
        EncJobs js{};
        js.job[0] = a;
        js.job[1] = a;
        js.waves0 = (int)small_waves(a);
        return x_dtype == UCM_DT_BF16 ? launch_small<bf16x8>(js, js.waves0, a.K, st)
                                      : launch_small<f16x8>(js, js.waves0, a.K, st);
    }
    if (wide_eligible(a, x_dtype, w_dtype)) {
        rc = x_dtype == UCM_DT_BF16 ? launch_wide<bf16x8>(a, st) : launch_wide<f16x8>(a, st);
        if (rc != UCM_EUNSUPPORTED) return rc;  // no large-LDS opt-in: the tiled kernel below
        ucm::clear_error();
    }
    if (stream_eligible(a, x_dtype, w_dtype)) {
        a.timeout_flag = stream_latch_flag();
        rc = x_dtype == UCM_DT_BF16 ? launch_stream<bf16x8>(a, st) : launch_stream<f16x8>(a, st);
        if (rc != UCM_EUNSUPPORTED) return rc;  // no large-LDS opt-in: the tiled kernel below
        ucm::clear_error();
    }
    if (mfma_eligible(a, x_dtype, w_dtype))
        return x_dtype == UCM_DT_BF16 ? dispatch_mfma<bf16x8>(a, st) : dispatch_mfma<f16x8>(a, st);
    // same element type on both sides, enough rows to fill a tile, grid within limits
    if (x_dtype == w_dtype && a.T >= 16 && a.H <= 65535 && ucm::ceil_div(a.T, 64) <= 0x7fffffff) {
        if (x_dtype == UCM_DT_F32) return launch_tiled<UCM_DT_F32>(a, st);
        if (x_dtype == UCM_DT_F16) return launch_tiled<UCM_DT_F16>(a, st);
        return launch_tiled<UCM_DT_BF16>(a, st);
    }
    const int64_t total = a.T * a.H * (a.N / 32);
    int64_t blocks = ucm::ceil_div(total, kThreads);
    if (blocks > 65535 * 16) blocks = 65535 * 16;
    hipLaunchKernelGGL(encode_fma_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, st, a, x_dtype,
                       w_dtype);
    return ucm::launch_status("encode_fma_kernel");
}

int check_cache(const void* slot, const uint32_t* cache, int64_t NB, int BS)
{
    UCM_REQUIRE(slot && cache, "null slot_mapping or cache");
    UCM_REQUIRE(NB > 0 && BS > 0, "bad cache shape");
    return UCM_OK;
}

}  // namespace

extern "C" int ucm_hash_encode(const void* x, int x_dtype, int64_t T, int32_t H, int32_t K,
                               int64_t x_stride_t, int64_t x_stride_h, const void* w, int w_dtype,
                               int32_t n_w, int32_t heads_per_w, int32_t N_bits, uint32_t* out,
                               int64_t out_stride_t, int64_t out_stride_h, ucm_stream_t stream)
{
    ucm::clear_error();
    UCM_REQUIRE(out, "null output");
    EncArgs a{};
    a.x = x; a.T = T; a.H = H; a.K = K; a.x_stride_t = x_stride_t; a.x_stride_h = x_stride_h;
    a.w = w; a.n_w = n_w; a.heads_per_w = heads_per_w; a.N = N_bits;
    a.out = out; a.out_stride_t = out_stride_t; a.out_stride_h = out_stride_h;
    return encode_common(a, x_dtype, w_dtype, (hipStream_t)stream);
}

extern "C" int64_t ucm_hash_encode_stream_timeouts(void)
{
    ucm::clear_error();
    unsigned int n = 0;
    const hipError_t e = hipMemcpyFromSymbol(&n, HIP_SYMBOL(g_stream_wait_timeouts), sizeof(n));
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return ucm::fail(UCM_ERROR, "reading the timeout counter: %s", hipGetErrorString(e));
    }
    return (int64_t)n;
}

extern "C" int ucm_hash_encode_clear_stream_timeouts(void)
{
    ucm::clear_error();
    const int dev = latch_device();
    g_latch_forced[dev].store(0, std::memory_order_relaxed);
    std::lock_guard<std::mutex> g(g_latch_mu);
    if (g_latch_host[dev]) *static_cast<volatile unsigned int*>(g_latch_host[dev]) = 0;
    return UCM_OK;
}

extern "C" int ucm_hash_encode_debug_trip_stream_latch(void)
{
    ucm::clear_error();
    g_latch_forced[latch_device()].store(1, std::memory_order_relaxed);
    return UCM_OK;
}

extern "C" int ucm_hash_encode_set_stream_threshold(int64_t rows)
{
    ucm::clear_error();
    t_stream_min_rows = rows > 0 ? rows : 0;
    return UCM_OK;
}

extern "C" int ucm_hash_encode_set_clock_probe(void* two_u64_in_device_memory)
{
    ucm::clear_error();
    if ((uintptr_t)two_u64_in_device_memory & 7) return ucm::fail(UCM_EPARAM, "ucm_hash_encode_set_clock_probe: the address is not 8-byte aligned");
    t_clock_probe = static_cast<unsigned long long*>(two_u64_in_device_memory);
    return UCM_OK;
}

extern "C" int ucm_hash_encode_cache(const void* x, int x_dtype, int64_t T, int32_t H, int32_t K,
                                     int64_t x_stride_t, int64_t x_stride_h, const void* w,
                                     int w_dtype, int32_t n_w, int32_t heads_per_w, int32_t N_bits,
                                     const void* slot_mapping, int slot_is_i64, uint32_t* cache,
                                     int64_t NB, int32_t BS, int64_t cs_block, int64_t cs_token,
                                     int64_t cs_head, ucm_stream_t stream)
{
    ucm::clear_error();
    int rc = check_cache(slot_mapping, cache, NB, BS);
    if (rc != UCM_OK) return rc;
    EncArgs a{};
    a.x = x; a.T = T; a.H = H; a.K = K; a.x_stride_t = x_stride_t; a.x_stride_h = x_stride_h;
    a.w = w; a.n_w = n_w; a.heads_per_w = heads_per_w; a.N = N_bits;
    a.slot = slot_mapping; a.slot_is_i64 = slot_is_i64; a.cache = cache; a.NB = NB; a.BS = BS;
    a.cs_block = cs_block; a.cs_token = cs_token; a.cs_head = cs_head;
    return encode_common(a, x_dtype, w_dtype, (hipStream_t)stream);
}

extern "C" int ucm_hash_encode_paged(const void* k_cache, int x_dtype, int64_t NBk, int32_t BS,
                                     int32_t H, int32_t K, int64_t ks_block, int64_t ks_token,
                                     int64_t ks_head, const int32_t* block_ids, int64_t n_blocks,
                                     int64_t n_tokens, const void* w, int w_dtype, int32_t n_w,
                                     int32_t heads_per_w, int32_t N_bits, uint32_t* cache,
                                     int64_t NB, int64_t cs_block, int64_t cs_token,
                                     int64_t cs_head, ucm_stream_t stream)
{
    ucm::clear_error();
    UCM_REQUIRE(cache && NB > 0 && BS > 0 && NBk > 0, "bad cache shape");
    UCM_REQUIRE(n_blocks >= 0 && n_tokens >= 0 && n_tokens <= n_blocks * (int64_t)BS,
                "n_tokens %lld does not fit %lld blocks of %d", (long long)n_tokens,
                (long long)n_blocks, (int)BS);
    UCM_REQUIRE(n_tokens == 0 || block_ids, "null block_ids");
    EncArgs a{};
    a.x = k_cache; a.T = n_tokens; a.H = H; a.K = K; a.x_stride_t = ks_token; a.x_stride_h = ks_head;
    a.src_blocks = block_ids; a.xs_block = ks_block;
    a.NBsrc = NBk < NB ? NBk : NB;  // an id must be valid in both caches
    a.w = w; a.n_w = n_w; a.heads_per_w = heads_per_w; a.N = N_bits;
    a.slot = nullptr; a.slot_is_i64 = 0; a.cache = cache; a.NB = NB; a.BS = BS;
    a.cs_block = cs_block; a.cs_token = cs_token; a.cs_head = cs_head;
    return encode_common(a, x_dtype, w_dtype, (hipStream_t)stream);
}

extern "C" int ucm_code_scatter(const uint32_t* codes, int64_t T, int32_t H, int32_t Wd,
                                int64_t in_stride_t, int64_t in_stride_h, const void* slot_mapping,
                                int slot_is_i64, uint32_t* cache, int64_t NB, int32_t BS,
                                int64_t cs_block, int64_t cs_token, int64_t cs_head,
                                ucm_stream_t stream)
{
    ucm::clear_error();
    UCM_REQUIRE(codes, "null codes");
    UCM_REQUIRE(T >= 0 && H > 0 && Wd > 0, "bad shape");
    int rc = check_cache(slot_mapping, cache, NB, BS);
    if (rc != UCM_OK) return rc;
    if (T == 0) return UCM_OK;
    EncArgs a{};
    a.slot = slot_mapping; a.slot_is_i64 = slot_is_i64; a.cache = cache; a.NB = NB; a.BS = BS;
    a.cs_block = cs_block; a.cs_token = cs_token; a.cs_head = cs_head;
    set_block_shift(a);
    const int64_t total = T * H * Wd;
    int64_t blocks = ucm::ceil_div(total, kThreads);
    if (blocks > 65535 * 16) blocks = 65535 * 16;
    hipLaunchKernelGGL(code_scatter_kernel, dim3((unsigned)blocks), dim3(kThreads), 0,
                       (hipStream_t)stream, codes, T, (int)H, (int)Wd, in_stride_t, in_stride_h, a);
    return ucm::launch_status("code_scatter_kernel");
}

// Encodes a step's new keys into the paged cache and its queries into a code tensor.  When both
// are small enough for the latency path they share one launch; two such pairs of input widths
// 512 and 64 (a latent-attention step) share one launch as well.
namespace ucm {
namespace {
// Fills the two jobs of a pair; has_keys = false when there are no new keys.
int build_pair(const PairSpec& p, EncArgs& kk, EncArgs& kq, bool& has_keys)
{
    kq = EncArgs{};
    kq.x = p.queries; kq.T = p.B; kq.H = p.Hq; kq.K = p.K; kq.x_stride_t = p.q_stride_b;
    kq.x_stride_h = p.q_stride_h; kq.w = p.w; kq.n_w = p.n_w;
    kq.heads_per_w = p.n_w > 1 ? p.Hq / p.Hkv : 0; kq.N = p.N_bits;
    if (p.q_group_mean && p.Hq > p.Hkv) {
        // one row per KV head: the mean of its Hq / Hkv query heads
        kq.H = p.Hkv;
        kq.gmean = p.Hq / p.Hkv;
        kq.x_stride_g = p.q_stride_h;
        kq.x_stride_h = p.q_stride_h * kq.gmean;
        kq.heads_per_w = p.n_w > 1 ? 1 : 0;
    } else if (p.q_reduce > 1) {
        // the reference's view(T, R, H / R, D).mean(1) (gsa_on_device.py:378-391): members of a group
        // lie H / R heads apart
        if (p.Hq % p.q_reduce) return ucm::fail(UCM_EPARAM, "%d query heads do not reduce by %d", p.Hq, p.q_reduce);
        kq.H = p.Hq / p.q_reduce;
        kq.gmean = p.q_reduce;
        kq.x_stride_g = p.q_stride_h * kq.H;
    }
    kq.out = p.q_codes; kq.out_stride_t = p.qc_stride_b; kq.out_stride_h = p.qc_stride_h;
    int rc = check_shape(kq, p.x_dtype, p.w_dtype);
    if (rc != UCM_OK) return rc;
    has_keys = p.T > 0;
    if (!has_keys) return UCM_OK;
    kk = EncArgs{};
    kk.x = p.keys; kk.T = p.T; kk.H = p.Hkv; kk.K = p.K; kk.x_stride_t = p.k_stride_t;
    kk.x_stride_h = p.k_stride_h; kk.w = p.w; kk.n_w = p.n_w; kk.heads_per_w = p.n_w > 1 ? 1 : 0;
    kk.N = p.N_bits; kk.slot = p.slot; kk.slot_is_i64 = p.slot_is_i64; kk.cache = p.cache;
    kk.NB = p.NB; kk.BS = p.BS; kk.cs_block = p.cs_block; kk.cs_token = p.cs_token;
    kk.cs_head = p.cs_head;
    rc = check_shape(kk, p.x_dtype, p.w_dtype);
    if (rc != UCM_OK) return rc;
    return check_cache(p.slot, p.cache, p.NB, p.BS);
}

bool pair_is_small(const PairSpec& p, const EncArgs& kk, const EncArgs& kq, bool has_keys)
{
    return has_keys && p.B > 0 && small_eligible(kk, p.x_dtype, p.w_dtype) &&
           small_eligible(kq, p.x_dtype, p.w_dtype);
}

// The queries alone through the small-row kernel (the only one that averages query groups).
int launch_queries_small(const PairSpec& p, EncArgs& kq, hipStream_t st)
{
    set_block_shift(kq);
    if (!mfma_eligible(kq, p.x_dtype, p.w_dtype) || small_waves(kq) > 0x7fffffff)
        return ucm::fail(UCM_EUNSUPPORTED,
                         "group-mean queries need bf16 / fp16 inputs of 64, 128, 256 or 512 dimensions, 16-byte aligned");
    if (kq.T == 0) return UCM_OK;
    EncJobs js{};
    js.job[0] = kq;
    js.job[1] = kq;
    js.waves0 = (int)small_waves(kq);
    return p.x_dtype == UCM_DT_BF16 ? launch_small<bf16x8>(js, js.waves0, p.K, st)
                                    : launch_small<f16x8>(js, js.waves0, p.K, st);
}

int launch_pair(const PairSpec& p, EncArgs& kk, EncArgs& kq, bool has_keys, hipStream_t st)
{
    if (kq.gmean > 1 && !(has_keys && pair_is_small(p, kk, kq, has_keys))) {
        if (has_keys) {
            const int rc = encode_common(kk, p.x_dtype, p.w_dtype, st);
            if (rc != UCM_OK) return rc;
        }
        return launch_queries_small(p, kq, st);
    }
    if (!has_keys) return encode_common(kq, p.x_dtype, p.w_dtype, st);
    if (pair_is_small(p, kk, kq, has_keys)) {
        EncJobs js{};
        set_block_shift(kk);
        set_block_shift(kq);
        js.job[0] = kk;
        js.job[1] = kq;
        js.waves0 = (int)small_waves(kk);
        const int64_t waves = js.waves0 + small_waves(kq);
        return p.x_dtype == UCM_DT_BF16 ? launch_small<bf16x8>(js, waves, p.K, st)
                                        : launch_small<f16x8>(js, waves, p.K, st);
    }
    const int rc = encode_common(kk, p.x_dtype, p.w_dtype, st);
    if (rc != UCM_OK) return rc;
    return encode_common(kq, p.x_dtype, p.w_dtype, st);
}
}  // namespace

int encode_pair(const PairSpec& p, hipStream_t st)
{
    EncArgs kk, kq;
    bool has_keys;
    const int lrc = stream_latch_check();
    if (lrc != UCM_OK) return lrc;
    const int rc = build_pair(p, kk, kq, has_keys);
    if (rc != UCM_OK) return rc;
    return launch_pair(p, kk, kq, has_keys, st);
}

int encode_two_pairs(const PairSpec& pa, const PairSpec& pb, hipStream_t st)
{
    EncArgs ka, qa, kb, qb;
    bool ha, hb;
    int rc = stream_latch_check();
    if (rc != UCM_OK) return rc;
    rc = build_pair(pa, ka, qa, ha);
    if (rc != UCM_OK) return rc;
    rc = build_pair(pb, kb, qb, hb);
    if (rc != UCM_OK) return rc;
    if (pa.K == 512 && pb.K == 64 && pa.x_dtype == pb.x_dtype && pair_is_small(pa, ka, qa, ha) &&
        pair_is_small(pb, kb, qb, hb)) {
        EncJobs4 js{};
        EncArgs* jobs[4] = {&ka, &qa, &kb, &qb};
        int64_t end = 0;
        for (int i = 0; i < 4; ++i) {
            set_block_shift(*jobs[i]);
            js.job[i] = *jobs[i];
            end += small_waves(*jobs[i]);
            js.end[i] = (int)end;
        }
        if (end <= 0x7fffffff) {
            if (pa.x_dtype == UCM_DT_BF16)
                hipLaunchKernelGGL((encode_small_mixed_kernel<bf16x8, 32, 4>), dim3((unsigned)end), dim3(64 * small_split(32)), 0, st, js);
            else
                hipLaunchKernelGGL((encode_small_mixed_kernel<f16x8, 32, 4>), dim3((unsigned)end), dim3(64 * small_split(32)), 0, st, js);
            return ucm::launch_status("encode_small_mixed_kernel");
        }
    }
    rc = launch_pair(pa, ka, qa, ha, st);
    if (rc != UCM_OK) return rc;
    return launch_pair(pb, kb, qb, hb, st);
}
}  // namespace ucm
