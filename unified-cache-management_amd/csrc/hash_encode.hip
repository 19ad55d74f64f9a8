// Sign-hash encoder for gfx950: codes = pack_lsb_first(x . W > 0), optionally scattered into
// the paged code cache.
//
// Follows the reference's HashEncoder (ucm/sparse/gsa_on_device/hash_encoder.py:359-370 for
// the arithmetic and bit order, :263-356 for the fused cache write, :136-195 for the code
// scatter).  Design for MI355X:
//   * bf16 / fp16 inputs go through v_mfma_f32_32x32x16_{bf16,f16}: a wave owns 32 rows, keeps
//     their K values in registers (A operand, one 16-byte load per lane and k-step) and walks
//     the hash columns 32 at a time; the projection matrix slice lives in LDS, transposed so a
//     B operand is one 16-byte LDS read;
//   * the sign of an accumulator register is a v_cmp whose 64-bit lane mask already IS two
//     packed output words (32 columns of two rows), so packing costs no shuffles;
//   * the row's words are written with one store, either to a dense [T,H,Wd] tensor or to
//     cache[slot/BS, slot%BS, h, :].
// Everything else (fp32 operands, odd shapes, unaligned rows) takes a plain FMA kernel.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerWave = 32;
constexpr int kRowsPerWg = 128;
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
    const void* w;
    int n_w, heads_per_w, N;
    // dense output
    uint32_t* out;
    int64_t out_stride_t, out_stride_h;
    // paged output (cache != null)
    const void* slot;
    int slot_is_i64;
    uint32_t* cache;
    int64_t NB;
    int BS;
    int64_t cs_block, cs_token, cs_head;
    int BN;        // hash columns per workgroup slice
    int bs_shift;  // log2(BS) when BS is a power of two, else -1
};

__device__ __forceinline__ int weight_index(const EncArgs& a, int h)
{
    int wi = a.heads_per_w > 0 ? h / a.heads_per_w : 0;
    return wi < a.n_w ? wi : a.n_w - 1;
}

// Destination of the code words of row (t, h), or null when the row must be skipped.
__device__ __forceinline__ uint32_t* row_dst(const EncArgs& a, int64_t t, int h)
{
    if (!a.cache) return a.out + t * a.out_stride_t + (int64_t)h * a.out_stride_h;
    const int64_t s = a.slot_is_i64 ? ((const int64_t*)a.slot)[t] : (int64_t)((const int32_t*)a.slot)[t];
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

// Sign-packs four accumulator registers of a 32x32 MFMA tile.  The 64-bit lane mask of
// "acc > 0" is two finished output words (32 columns of rows R and R+4); v_writelane_b32 drops
// each into the lane that owns the row, leaving the other lanes untouched.  The wait states
// between the vector compares that produce the masks and the lane writes that read them are
// inserted by hand: the compiler does not look inside inline assembly.
template <int R>
__device__ __forceinline__ uint32_t pack_rows4(uint32_t word, float a0, float a1, float a2, float a3)
{
    const unsigned long long m0 = __ballot(a0 > 0.0f), m1 = __ballot(a1 > 0.0f);
    const unsigned long long m2 = __ballot(a2 > 0.0f), m3 = __ballot(a3 > 0.0f);
    asm("s_nop 4\n\t"
        "v_writelane_b32 %0, %1, %9\n\ts_nop 0\n\t"
        "v_writelane_b32 %0, %2, %10\n\ts_nop 0\n\t"
        "v_writelane_b32 %0, %3, %11\n\ts_nop 0\n\t"
        "v_writelane_b32 %0, %4, %12\n\ts_nop 0\n\t"
        "v_writelane_b32 %0, %5, %13\n\ts_nop 0\n\t"
        "v_writelane_b32 %0, %6, %14\n\ts_nop 0\n\t"
        "v_writelane_b32 %0, %7, %15\n\ts_nop 0\n\t"
        "v_writelane_b32 %0, %8, %16"
        : "+v"(word)
        : "s"((uint32_t)m0), "s"((uint32_t)m1), "s"((uint32_t)m2), "s"((uint32_t)m3),
          "s"((uint32_t)(m0 >> 32)), "s"((uint32_t)(m1 >> 32)), "s"((uint32_t)(m2 >> 32)),
          "s"((uint32_t)(m3 >> 32)),
          "n"(R), "n"(R + 1), "n"(R + 2), "n"(R + 3), "n"(R + 4), "n"(R + 5), "n"(R + 6), "n"(R + 7));
    return word;
}

// Accumulator register v of lane l holds row 8*(v/4) + 4*(l/32) + v%4, column l%32 of the tile:
// registers 4g..4g+3 are rows 8g..8g+3 (low mask halves) and 8g+4..8g+7 (high halves).
__device__ __forceinline__ uint32_t pack_tile(const f32x16& acc)
{
    uint32_t word = 0;
    word = pack_rows4<0>(word, acc[0], acc[1], acc[2], acc[3]);
    word = pack_rows4<8>(word, acc[4], acc[5], acc[6], acc[7]);
    word = pack_rows4<16>(word, acc[8], acc[9], acc[10], acc[11]);
    word = pack_rows4<24>(word, acc[12], acc[13], acc[14], acc[15]);
    return word;
}

template <typename V>
struct Mfma;
template <>
struct Mfma<bf16x8> {
    static __device__ __forceinline__ f32x16 run(bf16x8 a, bf16x8 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Mfma<f16x8> {
    static __device__ __forceinline__ f32x16 run(f16x8 a, f16x8 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// V: 8-element vector type of the 16-bit input format.  KS = K / 16.
// grid = (row-tile workers, column slices, heads); a workgroup loads its W slice into LDS once
// and then walks row tiles of 128 rows (32 per wave) with a grid stride.
template <typename V, int KS>
__global__ __launch_bounds__(kThreads) void encode_mfma_kernel(EncArgs a)
{
    extern __shared__ uint16_t wt[];  // [BN][K + kPad], k contiguous
    constexpr int K = KS * 16;
    constexpr int KP = K + kPad;
    const int h = blockIdx.z;
    const int n0 = blockIdx.y * a.BN;
    const int bn = (a.N - n0 < a.BN) ? a.N - n0 : a.BN;  // columns in this slice
    const uint16_t* wsrc = (const uint16_t*)a.w + (int64_t)weight_index(a, h) * K * a.N;

    // W[k0..k0+8][n0+8j..+8] -> wt[8j+c][k0..k0+8]: each thread transposes 8x8 patches of 16-bit
    // elements in registers (byte permutes) and writes eight 16-byte LDS rows
    for (int idx = threadIdx.x; idx < (K / 8) * (bn / 8); idx += kThreads) {
        const int kq = idx / (bn / 8), j = idx % (bn / 8);
        const uint16_t* src = wsrc + (int64_t)(kq * 8) * a.N + n0 + 8 * j;
        u32x4 row[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) row[i] = *reinterpret_cast<const u32x4*>(src + (int64_t)i * a.N);
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
    }
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r = lane & 31, kb = lane >> 5;
    const uint16_t* xbase = (const uint16_t*)a.x + (int64_t)h * a.x_stride_h;
    const int64_t tiles = (a.T + kRowsPerWg - 1) / kRowsPerWg;
    const int nt_count = bn / 32;
    const int word0 = n0 / 32;

    // A operands of the wave's 32 rows of a tile; rows past T re-read the last row (discarded)
    auto load_tile = [&](int64_t tile, V (&dstv)[KS]) {
        int64_t t = tile * kRowsPerWg + wave * kRowsPerWave + r;
        if (t >= a.T) t = a.T - 1;
        const uint16_t* xr = xbase + t * a.x_stride_t + kb * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dstv[ks] = *reinterpret_cast<const V*>(xr + ks * 16);
    };
    constexpr bool kPrefetch = KS <= 16;  // the next tile's operands fit in registers
    V av[KS];
    V nx[kPrefetch ? KS : 1];
    if (blockIdx.x < tiles) load_tile(blockIdx.x, av);

    for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const int64_t row0 = tile * kRowsPerWg + wave * kRowsPerWave;
        const int64_t next = tile + gridDim.x;
        if constexpr (kPrefetch) {
            if (next < tiles) load_tile(next, nx);
        } else {
            if (tile != (int64_t)blockIdx.x) load_tile(tile, av);
        }
        const int64_t t = row0 + r;
        const bool row_ok = t < a.T;
        uint32_t* dst = (row_ok && lane < 32) ? row_dst(a, t, h) : nullptr;

        for (int nt0 = 0; nt0 < nt_count; nt0 += 4) {
            uint32_t words[4] = {0, 0, 0, 0};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int nt = nt0 + q;
                if (nt >= nt_count) break;
                f32x16 acc = {0};
                const uint16_t* bp = wt + (nt * 32 + r) * KP + kb * 8;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const V bv = *reinterpret_cast<const V*>(bp + ks * 16);
                    acc = Mfma<V>::run(av[ks], bv, acc);
                }
                // accumulator v of lane l is row 8*(v/4) + 4*(l/32) + v%4, column l%32
                const uint32_t word = pack_tile(acc);
                words[q] = word;
            }
            if (dst) {
                const int nq = (nt_count - nt0 < 4) ? nt_count - nt0 : 4;
                uint32_t* d = dst + word0 + nt0;
                if (nq == 4 && (((uintptr_t)d) & 15) == 0) {
                    u32x4 v = {words[0], words[1], words[2], words[3]};
                    *reinterpret_cast<u32x4*>(d) = v;
                } else {
                    for (int q = 0; q < nq; ++q) d[q] = words[q];
                }
            }
        }
        if constexpr (kPrefetch) {
            if (next < tiles) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) av[ks] = nx[ks];
            }
        }
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

template <typename V, int KS>
__global__ __launch_bounds__(64) void encode_small_kernel(EncJobs js)
{
    constexpr int K = KS * 16;
    const bool second = (int)blockIdx.x >= js.waves0;
    const EncArgs& a = second ? js.job[1] : js.job[0];
    int wv = second ? blockIdx.x - js.waves0 : blockIdx.x;
    const int ntiles = a.N / 32;
    const int nt = wv % ntiles;
    wv /= ntiles;
    const int h = wv % a.H;
    const int64_t row0 = (int64_t)(wv / a.H) * kRowsPerWave;

    const int lane = threadIdx.x;
    const int r = lane & 31, kb = lane >> 5;
    const uint16_t* wsrc =
        (const uint16_t*)a.w + (int64_t)weight_index(a, h) * K * a.N + nt * 32 + r;
    int64_t t = row0 + r;
    const bool row_ok = t < a.T;
    if (!row_ok) t = a.T - 1;
    const uint16_t* xr = (const uint16_t*)a.x + (int64_t)h * a.x_stride_h + t * a.x_stride_t + kb * 8;

    V av[KS];
    uint16_t bw[KS][8];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) av[ks] = *reinterpret_cast<const V*>(xr + ks * 16);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int i = 0; i < 8; ++i) bw[ks][i] = wsrc[(int64_t)(ks * 16 + kb * 8 + i) * a.N];

    f32x16 acc = {0};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        V bv;
        __builtin_memcpy(&bv, bw[ks], 16);
        acc = Mfma<V>::run(av[ks], bv, acc);
    }
    const uint32_t word = pack_tile(acc);
    if (row_ok && lane < 32) {
        uint32_t* dst = row_dst(a, t, h);
        if (dst) dst[nt] = word;
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
        const int64_t xo = t * a.x_stride_t + (int64_t)h * a.x_stride_h;
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

int num_cus()
{
    static int cached = 0;
    if (cached) return cached;
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
        prop.multiProcessorCount > 0)
        cached = prop.multiProcessorCount;
    else
        cached = 256;
    return cached;
}

// Widest slice of hash columns (a multiple of 32 that divides N) whose transposed LDS image
// stays within `cap` bytes; 0 when not even 32 columns fit.
int pick_slice(int N, int K, size_t cap)
{
    for (int bn = N; bn >= 32; bn -= 32)
        if (N % bn == 0 && (size_t)bn * (K + kPad) * 2 <= cap) return bn;
    return 0;
}

template <typename V, int KS>
int launch_mfma(EncArgs a, hipStream_t st)
{
    constexpr int K = KS * 16;
    // 0 = not tried, 1 = large LDS allocations allowed, -1 = refused by the runtime
    static int big_lds = 0;
    a.BN = pick_slice(a.N, K, 144 * 1024);
    if ((size_t)a.BN * (K + kPad) * 2 > 64 * 1024) {
        if (big_lds == 0) {
            const hipError_t e =
                hipFuncSetAttribute((const void*)encode_mfma_kernel<V, KS>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024);
            if (e != hipSuccess) (void)hipGetLastError();
            big_lds = (e == hipSuccess) ? 1 : -1;
        }
        if (big_lds < 0) a.BN = pick_slice(a.N, K, 64 * 1024);
    }
    if (a.BN == 0) return ucm::fail(UCM_EUNSUPPORTED, "no LDS slice fits K=%d", K);
    const size_t lds = (size_t)a.BN * (K + kPad) * 2;
    const int64_t tiles = (a.T + kRowsPerWg - 1) / kRowsPerWg;
    const int slices = a.N / a.BN;
    int64_t per = (int64_t)num_cus() * 4 / ((int64_t)slices * a.H);
    if (per < 1) per = 1;
    const dim3 grid((unsigned)(tiles < per ? tiles : per), (unsigned)slices, (unsigned)a.H);
    hipLaunchKernelGGL((encode_mfma_kernel<V, KS>), grid, dim3(kThreads), lds, st, a);
    return ucm::launch_status("encode_mfma_kernel");
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
    const bool aligned = (((uintptr_t)a.x | (uintptr_t)a.w) & 15) == 0 && a.x_stride_t % 8 == 0 &&
                         a.x_stride_h % 8 == 0;
    return same16 && k_ok && aligned;
}

int64_t small_waves(const EncArgs& a)
{
    return ucm::ceil_div(a.T, kRowsPerWave) * a.H * (a.N / 32);
}

template <typename V>
int launch_small(const EncJobs& js, int64_t waves, int K, hipStream_t st)
{
    const dim3 grid((unsigned)waves);
    switch (K) {
        case 64: hipLaunchKernelGGL((encode_small_kernel<V, 4>), grid, dim3(64), 0, st, js); break;
        case 128: hipLaunchKernelGGL((encode_small_kernel<V, 8>), grid, dim3(64), 0, st, js); break;
        case 256: hipLaunchKernelGGL((encode_small_kernel<V, 16>), grid, dim3(64), 0, st, js); break;
        default: return ucm::fail(UCM_ERROR, "internal: K %d has no small-row kernel", K);
    }
    return ucm::launch_status("encode_small_kernel");
}

void set_block_shift(EncArgs& a)
{
    a.bs_shift = -1;
    if (a.BS > 0 && (a.BS & (a.BS - 1)) == 0) a.bs_shift = __builtin_ctz((unsigned)a.BS);
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

bool small_eligible(const EncArgs& a, int x_dtype, int w_dtype)
{
    return mfma_eligible(a, x_dtype, w_dtype) && a.K <= 256 && a.T <= kSmallRows;
}

int encode_common(EncArgs a, int x_dtype, int w_dtype, hipStream_t st)
{
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
    if (mfma_eligible(a, x_dtype, w_dtype))
        return x_dtype == UCM_DT_BF16 ? dispatch_mfma<bf16x8>(a, st) : dispatch_mfma<f16x8>(a, st);
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

// Encodes the step's new keys into the paged cache and the step's queries into a dense
// tensor.  When both are small enough for the latency path they share one launch.
namespace ucm {
int encode_pair(const void* keys, int64_t T, int Hkv, int64_t k_stride_t, int64_t k_stride_h,
                const void* slot, int slot_is_i64, uint32_t* cache, int64_t NB, int BS,
                int64_t cs_block, int64_t cs_token, int64_t cs_head, const void* queries, int64_t B,
                int Hq, int64_t q_stride_b, int64_t q_stride_h, uint32_t* q_codes, int x_dtype,
                int K, const void* w, int w_dtype, int n_w, int N_bits, hipStream_t st)
{
    const int Wd = N_bits / 32;
    EncArgs kq{};
    kq.x = queries; kq.T = B; kq.H = Hq; kq.K = K; kq.x_stride_t = q_stride_b; kq.x_stride_h = q_stride_h;
    kq.w = w; kq.n_w = n_w; kq.heads_per_w = n_w > 1 ? Hq / Hkv : 0; kq.N = N_bits;
    kq.out = q_codes; kq.out_stride_t = (int64_t)Hq * Wd; kq.out_stride_h = Wd;
    int rc = check_shape(kq, x_dtype, w_dtype);
    if (rc != UCM_OK) return rc;
    if (T <= 0) return encode_common(kq, x_dtype, w_dtype, st);

    EncArgs kk{};
    kk.x = keys; kk.T = T; kk.H = Hkv; kk.K = K; kk.x_stride_t = k_stride_t; kk.x_stride_h = k_stride_h;
    kk.w = w; kk.n_w = n_w; kk.heads_per_w = n_w > 1 ? 1 : 0; kk.N = N_bits;
    kk.slot = slot; kk.slot_is_i64 = slot_is_i64; kk.cache = cache; kk.NB = NB; kk.BS = BS;
    kk.cs_block = cs_block; kk.cs_token = cs_token; kk.cs_head = cs_head;
    rc = check_shape(kk, x_dtype, w_dtype);
    if (rc != UCM_OK) return rc;
    rc = check_cache(slot, cache, NB, BS);
    if (rc != UCM_OK) return rc;
    if (B > 0 && small_eligible(kk, x_dtype, w_dtype) && small_eligible(kq, x_dtype, w_dtype)) {
        EncJobs js{};
        set_block_shift(kk);
        set_block_shift(kq);
        js.job[0] = kk;
        js.job[1] = kq;
        js.waves0 = (int)small_waves(kk);
        const int64_t waves = js.waves0 + small_waves(kq);
        return x_dtype == UCM_DT_BF16 ? launch_small<bf16x8>(js, waves, K, st)
                                      : launch_small<f16x8>(js, waves, K, st);
    }
    rc = encode_common(kk, x_dtype, w_dtype, st);
    if (rc != UCM_OK) return rc;
    return encode_common(kq, x_dtype, w_dtype, st);
}
}  // namespace ucm
