// Hamming scorer + deterministic block top-k for gfx950.
//
// Three kernels per call:
//   1. (group size > 4 only) plane_kernel: the G query codes of one KV head are reduced to
//      per-bit counts c_b, stored as binary bit planes, so that the group-summed distance of
//      a cached code k is   sum_b c_b + G*popc(k) - 2 * sum_p 2^p * popc(k & plane_p)
//      — exact integer arithmetic, 2*P+1 ops per word instead of 2*G.
//   2. block_score_*: every 16-byte piece of the paged code cache is read exactly once with
//      128-bit loads (one wave = 1 KiB contiguous), XOR+popcount in registers, summed across
//      the lanes that share a token, min-reduced per (block, KV head) with wave shuffles and
//      LDS atomics.  Result: one int32 similarity per (request, KV head, logical block).
//   3. select_kernel: per (request, KV head) an LDS radix search finds the k-th largest
//      score, ties are resolved towards the lower block index by an ordered prefix sum, and
//      the winners are compacted in ascending index order — no sort is needed for the
//      default output order.
//
// Semantics follow ucm/sparse/gsa_on_device/hamming_topk.py:15-54 and
// csrc/cuda/ham_dist/paged_ham_dist_mla.cu:148-247 of the reference (block min of the
// group-summed distance, sink/recent keep, +inf past seq_len), in the similarity form of
// its NPU op (csrc/ascend/hamming_dist_top_k/op_kernel/hamming_dist_top_k_base.h:150-347).
#include <hip/hip_ext.h>

#include <mutex>

#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWave = 64;
constexpr int kInf = 0x7fffffff;
constexpr int kMaxTileHeads = 1024;  // TB * Hkv bound of the LDS min table
constexpr int kMaxTile = 64;          // TB bound
constexpr int kSelLdsCap = 8192;     // block scores kept in LDS by select_kernel
constexpr int kSelSortCap = 2048;    // largest k for score-ordered output
constexpr int kMaxPlaneWords = 64;   // widest code the bit-plane kernels take

struct ScoreArgs {
    const uint32_t* q;
    int64_t q_stride_b, q_stride_h;
    const uint32_t* kc;
    int64_t NB;
    int BS, Hkv, Wd;
    int64_t ks_block, ks_token, ks_head;
    const int32_t* table;
    int table_stride, max_blocks;
    const int32_t* lens;
    int B, Hq, G, sink, recent;
    int TB;                  // logical blocks per workgroup
    int reduce_out;          // block_score_one / block_score_rows: write the maximum over the
                             // KV heads, scores then is [B][1][max_blocks]
    const uint32_t* planes;  // [B][Hkv][PMAX][Wd], planes mode only
    int32_t* scores;         // [B][Hkv][max_blocks]
    int sc_h, sc_j;          // block_score_one only: strides of head and block inside a request's
                             // Hkv * max_blocks scores (max_blocks, 1), or (1, Hkv) when the
                             // wave-per-row selection follows: the 8 scores of a block are then
                             // one 32-byte store instead of eight 4-byte stores into lines that
                             // other workgroups write too
    unsigned long long* clock_probe;  // strip scorers: see ucm_hamming_topk_set_clock_probe(); else null
};

__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); }
__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }

// Every read of cached codes goes through here.
template <class T>
__device__ __forceinline__ T code_load(const T* p)
{
    return __builtin_nontemporal_load(p);
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// popcount(x) + acc as the one instruction it is; as plain C++ the sum of many popcounts is
// re-associated into a tree with extra adds.
__device__ __forceinline__ int popc_add(uint32_t x, int acc)
{
    int r;
    asm("v_bcnt_u32_b32 %0, %1, %2" : "=v"(r) : "v"(x), "v"(acc));
    return r;
}

__device__ __forceinline__ int popc4(u32x4 v)
{
    return __popc(v.x) + __popc(v.y) + __popc(v.z) + __popc(v.w);
}

// Physical block of logical block j of request b, or -1 when the entry is unusable.
__device__ __forceinline__ int64_t physical_block(const ScoreArgs& a, int b, int j)
{
    int64_t pb = a.table ? (int64_t)a.table[(int64_t)b * a.table_stride + j]
                         : (int64_t)b * a.max_blocks + j;
    return (pb < 0 || pb >= a.NB) ? -1 : pb;
}

__device__ __forceinline__ int num_blocks_of(const ScoreArgs& a, int len)
{
    int n = len > 0 ? (len + a.BS - 1) / a.BS : 0;
    return n < a.max_blocks ? n : a.max_blocks;
}

// Writes the similarity of every (block, head) of the tile from the LDS min table.
__device__ __forceinline__ void write_tile_scores(const ScoreArgs& a, int b, int j0, int nb_tile,
                                                  int len, const int* smin)
{
    const int full = a.G * 32 * a.Wd;
    for (int i = threadIdx.x; i < nb_tile * a.Hkv; i += kThreads) {
        const int blk = i / a.Hkv, h = i % a.Hkv, j = j0 + blk;
        const int p0 = j * a.BS;
        const int p1 = (p0 + a.BS < len) ? p0 + a.BS : len;
        const bool forced = (p0 < a.sink) || (p1 > len - a.recent);
        int s;
        if (physical_block(a, b, j) < 0) s = -1;
        else if (forced) s = full;
        else s = full - smin[i];
        a.scores[((int64_t)b * a.Hkv + h) * a.max_blocks + j] = s;
    }
}

// ---------------------------------------------------------------------------------------
// Bit planes of the per-bit query counts (group size > 4).
// planes[b][h][p][w] bit i  =  bit p of  #{ g : q[b, h*G+g, w] has bit i set }.
// ---------------------------------------------------------------------------------------
// One workgroup per (request, KV head, 64 bits of the code): lane i of every wave owns bit i of
// the chunk, the four waves split the G query heads between them (all loads of a wave are
// independent and go out together), the partial counts meet in LDS and wave 0 turns each
// count bit into one 64-bit ballot, i.e. two plane words.
__global__ __launch_bounds__(kThreads) void plane_kernel(const uint32_t* __restrict__ q,
                                                         int64_t q_stride_b, int64_t q_stride_h,
                                                         int Hkv, int G, int Wd, int PMAX,
                                                         uint32_t* __restrict__ planes)
{
    __shared__ int part[kThreads];
    const int chunks = (Wd + 1) >> 1;
    const int chunk = blockIdx.x % chunks, bh = blockIdx.x / chunks;
    const int b = bh / Hkv, h = bh % Hkv;
    const int lane = lane_id(), wid = wave_id();
    const int w = chunk * 2 + (lane >> 5), sh = lane & 31;
    const bool ok = w < Wd;
    const uint32_t* qb = q + b * q_stride_b + (int64_t)h * G * q_stride_h + (ok ? w : 0);
    int cnt = 0;
    constexpr int kWaves = kThreads / kWave;
    int g = wid;
    for (; g + 7 * kWaves < G; g += 8 * kWaves) {
        uint32_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = qb[(int64_t)(g + u * kWaves) * q_stride_h];
#pragma unroll
        for (int u = 0; u < 8; ++u) cnt += (v[u] >> sh) & 1u;
    }
    for (; g < G; g += kWaves) cnt += (qb[(int64_t)g * q_stride_h] >> sh) & 1u;
    part[threadIdx.x] = cnt;
    __syncthreads();
    if (wid != 0) return;
    cnt = part[lane] + part[lane + kWave] + part[lane + 2 * kWave] + part[lane + 3 * kWave];
    if (!ok) cnt = 0;
    uint32_t* out = planes + ((int64_t)b * Hkv + h) * PMAX * Wd + chunk * 2;
    for (int p = 0; p < PMAX; ++p) {
        const unsigned long long m = __ballot((cnt >> p) & 1);
        if (lane == 0) out[p * Wd] = (uint32_t)m;
        if (lane == 32 && ok) out[p * Wd + 1] = (uint32_t)(m >> 32);
    }
}

// ---------------------------------------------------------------------------------------
// Fast block scorer.  Requirements (checked by the host): the [BS][Hkv][Wd] codes of a block
// are contiguous, Wd = 4*CPU, Hkv*CPU divides 64, BS*Hkv*CPU is a multiple of 64, all
// addresses 16-byte aligned.
//   CPU   : 16-byte pieces per code (1, 2 or 4)
//   DIRECT: true  -> G = GP query codes kept in registers, xor+popcount per query head
//           false -> GP = PMAX bit planes in registers
//   U     : 1 KiB runs a wave keeps in flight per step
// A workgroup owns TB consecutive logical blocks of one request.  A block is a sequence of
// 64-piece "runs" (1 KiB each); lane l of the wave that handles run r reads piece r*64+l, so
// each load instruction covers 1 KiB of contiguous memory.  Blocks with >= 4 runs are split
// over the four waves (split = 1), smaller blocks go whole to one wave (split = 0).  The
// loads of step s+1 are issued before the popcounts of step s, so every wave always has a
// batch in flight.  (head, piece-in-code) of a lane never changes, so its query material
// lives in registers for the whole kernel.
// ---------------------------------------------------------------------------------------
template <int CPU, bool DIRECT, int GP, int U>
__global__ __launch_bounds__(kThreads) void block_score_fast(ScoreArgs a, int split)
{
    __shared__ int smin[kMaxTileHeads];
    __shared__ long long pbs[kMaxTile];  // physical block per tile block, -1 = unusable
    const int b = blockIdx.y;
    const int j0 = blockIdx.x * a.TB;
    // table entries never depend on seq_len: read them while seq_len is still in flight
    if (threadIdx.x < a.TB && j0 + (int)threadIdx.x < a.max_blocks)
        pbs[threadIdx.x] = physical_block(a, b, j0 + threadIdx.x);
    const int len = a.lens[b];
    const int nblk = num_blocks_of(a, len);
    if (j0 >= nblk) return;
    const int nb_tile = (a.TB < nblk - j0) ? a.TB : nblk - j0;

    for (int i = threadIdx.x; i < nb_tile * a.Hkv; i += kThreads) smin[i] = kInf;

    const int period = a.Hkv * CPU;  // pieces per token
    const int lane = lane_id();
    const int lane_c = lane % period;
    const int h = lane_c / CPU, part = lane_c % CPU;
    const int period_shift = __builtin_ctz(period);

    uint32_t qr[GP][4];
    int ctot = 0;
    if (DIRECT) {
        const uint32_t* qp = a.q + b * a.q_stride_b + (int64_t)h * GP * a.q_stride_h + part * 4;
#pragma unroll
        for (int g = 0; g < GP; ++g)
#pragma unroll
            for (int w = 0; w < 4; ++w) qr[g][w] = qp[g * a.q_stride_h + w];
    } else {
        const uint32_t* pp = a.planes + ((int64_t)b * a.Hkv + h) * GP * a.Wd + part * 4;
#pragma unroll
        for (int p = 0; p < GP; ++p)
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                qr[p][w] = pp[p * a.Wd + w];
                ctot += __popc(qr[p][w]) << p;
            }
    }
    __syncthreads();

    const int rpb = (a.BS * period) >> 6;  // runs per block
    const int wid = wave_id();
    // this wave's blocks: blk_first, +blk_step ...; its runs inside a block: run_first, +run_step
    const int blk_first = split ? 0 : wid, blk_step = split ? 1 : 4;
    const int run_first = split ? wid : 0, run_step = split ? 4 : 1;
    const int rpw = split ? (rpb >> 2) : rpb;  // runs of one block handled by this wave
    const int bpb = (rpw + U - 1) / U;         // batches (steps) per block
    const int my_blocks = (nb_tile - blk_first + blk_step - 1) / blk_step;
    const int nsteps = my_blocks > 0 ? my_blocks * bpb : 0;

    auto issue = [&](int s, u32x4 (&kv)[U]) {
        const int bi = s / bpb, batch = s - bi * bpb;
        const int blk = blk_first + bi * blk_step;
        const long long pb = pbs[blk];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = batch * U + u;
            kv[u] = (u32x4)(0u);
            if (pb >= 0 && k < rpw) {
                const int run = run_first + k * run_step;
                const u32x4* src =
                    reinterpret_cast<const u32x4*>(a.kc + pb * a.ks_block) + (run << 6) + lane;
                kv[u] = code_load(src);
            }
        }
    };

    int m = kInf;
    auto consume = [&](int s, const u32x4 (&kv)[U]) {
        const int bi = s / bpb, batch = s - bi * bpb;
        const int blk = blk_first + bi * blk_step;
        const bool usable = pbs[blk] >= 0;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = batch * U + u;
            int d;
            if (DIRECT) {
                d = 0;
#pragma unroll
                for (int g = 0; g < GP; ++g)
                    d += __popc(kv[u].x ^ qr[g][0]) + __popc(kv[u].y ^ qr[g][1]) +
                         __popc(kv[u].z ^ qr[g][2]) + __popc(kv[u].w ^ qr[g][3]);
            } else {
                int acc = 0;
#pragma unroll
                for (int p = 0; p < GP; ++p)
                    acc += (__popc(kv[u].x & qr[p][0]) + __popc(kv[u].y & qr[p][1]) +
                            __popc(kv[u].z & qr[p][2]) + __popc(kv[u].w & qr[p][3]))
                           << p;
                d = ctot + a.G * popc4(kv[u]) - 2 * acc;
            }
            if (CPU >= 2) d += __shfl_xor(d, 1);
            if (CPU >= 4) d += __shfl_xor(d, 2);
            const int run = run_first + k * run_step;
            const int t = ((run << 6) + lane) >> period_shift;
            const int pos = (j0 + blk) * a.BS + t;
            if (usable && k < rpw && pos < len && d < m) m = d;
        }
        if (batch == bpb - 1) {  // last batch of the block: publish this wave's minimum
            int mm = m;
            for (int st = period; st < kWave; st <<= 1) {
                const int o = __shfl_xor(mm, st);
                mm = o < mm ? o : mm;
            }
            if (lane < period && part == 0) atomicMin(&smin[blk * a.Hkv + h], mm);
            m = kInf;
        }
    };

    u32x4 buf0[U], buf1[U];
    if (nsteps > 0) issue(0, buf0);
    for (int s = 0; s < nsteps; s += 2) {
        if (s + 1 < nsteps) issue(s + 1, buf1);
        consume(s, buf0);
        if (s + 1 < nsteps) {
            if (s + 2 < nsteps) issue(s + 2, buf0);
            consume(s + 1, buf1);
        }
    }
    __syncthreads();

    const int full = a.G * 32 * a.Wd;
    for (int i = threadIdx.x; i < nb_tile * a.Hkv; i += kThreads) {
        const int blk = i / a.Hkv, hh = i - blk * a.Hkv, j = j0 + blk;
        const int p0 = j * a.BS;
        const int p1 = (p0 + a.BS < len) ? p0 + a.BS : len;
        const bool forced = (p0 < a.sink) || (p1 > len - a.recent);
        int sc;
        if (pbs[blk] < 0) sc = -1;
        else if (forced) sc = full;
        else sc = full - smin[i];
        a.scores[((int64_t)b * a.Hkv + hh) * a.max_blocks + j] = sc;
    }
}

// ---------------------------------------------------------------------------------------
// One-block-per-workgroup scorer: the hot shape (a block of at least 4 KiB, split over the
// four waves).  Same arithmetic as block_score_fast with the head count a compile-time
// constant, so the lane -> (head, piece) map, the token of a piece and the wave reduction
// are all shifts and DPP-friendly shuffles.
//
// (Measured against it at 32 x 32,768 tokens, 16 KiB blocks: a grid of 256 workgroups of 16 waves,
// every wave resident, all small reads ahead of a barrier, then two whole blocks per wave with
// 16 KiB in flight and neither LDS nor barriers - 24.4 us against 22.8.  Time stamps of its waves:
// a compute unit answers its loads in issue order, so its 16 waves are served one after the other
// (first quarter of a block after 2.6 ... 15.8 us); every unit streams its 512 KB at about 30 GB/s,
// 7.8 TB/s together, but the XCDs differ by 10 % (their units end after 18.0 ... 20.0 us), which a
// static split pays at the tail and a grid of one-block workgroups, handed out as units free up,
// does not.)
// ---------------------------------------------------------------------------------------
template <int CPU, int HKV, bool DIRECT, int GP, bool EXACT>
__global__ __launch_bounds__(kThreads) void block_score_one(ScoreArgs a)
{
    // EXACT: the block is exactly 16 KiB (4 runs per wave): one batch of loads, no loop
    constexpr int PERIOD = HKV * CPU;  // pieces per token (a power of two <= 64)
    __shared__ int smin[kThreads / kWave][HKV];  // one row of partial minima per wave
    const int b = blockIdx.y, j = blockIdx.x;
    const int lane = lane_id();
    const int wid = wave_id();
    const int h = (lane % PERIOD) / CPU, part = lane % CPU;

    // The two request-level scalars do not depend on each other: both reads go out together
    // (without a table the entry read is a harmless second read of the length).
    // Selected with masks, not branches: a branch would put the reads on separate paths and
    // serialise their latencies.
    const uintptr_t has_table = a.table ? ~(uintptr_t)0 : 0;
    const uintptr_t ea = (reinterpret_cast<uintptr_t>(a.table + ((int64_t)b * a.table_stride + j)) & has_table) |
                         (reinterpret_cast<uintptr_t>(a.lens + b) & ~has_table);
    int entry = *reinterpret_cast<const int32_t*>(ea);
    int len = a.lens[b];
    // Scheduling fence: both scalars and the arguments the code loads need must be in
    // registers here, which makes the compiler fetch all of them up front (two dependent
    // rounds of scalar reads) instead of one after the other along the early-exit tests.
    // (Pointers stay out of it: one that passes through would lose its address space.)
    int64_t ks_block0 = a.ks_block, nb0 = a.NB, q_stride_b0 = a.q_stride_b;
    asm volatile("" : "+s"(entry), "+s"(len), "+s"(ks_block0), "+s"(nb0), "+s"(q_stride_b0));

    // query material next: it depends on nothing but the request index
    uint32_t qr[GP][4];
    int ctot = 0;
    if (DIRECT) {
        const uint32_t* qp = a.q + b * q_stride_b0 + (int64_t)h * GP * a.q_stride_h + part * 4;
#pragma unroll
        for (int g = 0; g < GP; ++g)
#pragma unroll
            for (int w = 0; w < 4; ++w) qr[g][w] = qp[g * a.q_stride_h + w];
    } else {
        const uint32_t* pp = a.planes + ((int64_t)b * HKV + h) * GP * a.Wd + part * 4;
#pragma unroll
        for (int p = 0; p < GP; ++p)
#pragma unroll
            for (int w = 0; w < 4; ++w) qr[p][w] = pp[p * a.Wd + w];
    }

    // physical block, or -1 when the entry is unusable; the address arithmetic sits in front of
    // the early exit so that every kernel argument is fetched in one go at the top
    int64_t pb = ((int64_t)entry & (int64_t)has_table) | (((int64_t)b * a.max_blocks + j) & ~(int64_t)has_table);
    if (pb < 0 || pb >= nb0) pb = -1;
    const int rpw = EXACT ? 4 : (a.BS * PERIOD) >> 8;  // runs per wave (a block has 4*rpw runs)
    const u32x4* base = reinterpret_cast<const u32x4*>(a.kc + (pb < 0 ? 0 : pb) * ks_block0) + lane;
    const int pos0 = j * a.BS;
    if (pos0 >= len) return;  // j >= ceil(len / BS); the grid never exceeds max_blocks

    // first batch of code loads goes out before anything waits
    u32x4 kv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) kv[u] = (u32x4)(0u);
    if (pb >= 0) {
        if (EXACT || rpw >= 4) {
#pragma unroll
            for (int u = 0; u < 4; ++u) kv[u] = code_load(base + ((wid + 4 * u) << 6));
        } else {
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (u < rpw) kv[u] = code_load(base + ((wid + 4 * u) << 6));
        }
    }
    if (!DIRECT) {
#pragma unroll
        for (int p = 0; p < GP; ++p)
#pragma unroll
            for (int w = 0; w < 4; ++w) ctot += __popc(qr[p][w]) << p;
    }

    int m = kInf;
    if (pb >= 0) {
        for (int k0 = 0; k0 < rpw; k0 += 4) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int d;
                if (DIRECT) {
                    // one accumulating popcount per word, chained: left to itself the compiler
                    // splits the sum into several chains and joins them with three-input adds
                    // (28 of 245 vector instructions per wave at four query heads)
                    d = __popc(kv[u].x ^ qr[0][0]);
                    d = popc_add(kv[u].y ^ qr[0][1], d);
                    d = popc_add(kv[u].z ^ qr[0][2], d);
                    d = popc_add(kv[u].w ^ qr[0][3], d);
#pragma unroll
                    for (int g = 1; g < GP; ++g) {
                        d = popc_add(kv[u].x ^ qr[g][0], d);
                        d = popc_add(kv[u].y ^ qr[g][1], d);
                        d = popc_add(kv[u].z ^ qr[g][2], d);
                        d = popc_add(kv[u].w ^ qr[g][3], d);
                    }
                } else {
                    int acc = 0;
#pragma unroll
                    for (int p = 0; p < GP; ++p)
                        acc += (__popc(kv[u].x & qr[p][0]) + __popc(kv[u].y & qr[p][1]) +
                                __popc(kv[u].z & qr[p][2]) + __popc(kv[u].w & qr[p][3]))
                               << p;
                    d = ctot + a.G * popc4(kv[u]) - 2 * acc;
                }
                if (CPU >= 2) d += __shfl_xor(d, 1);
                if (CPU >= 4) d += __shfl_xor(d, 2);
                const int t = (((wid + 4 * (k0 + u)) << 6) + lane) / PERIOD;
                if ((EXACT || k0 + u < rpw) && pos0 + t < len && d < m) m = d;
            }
            // next batch (blocks larger than 16 KiB)
            if (!EXACT && k0 + 4 < rpw) {
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    kv[u] = (u32x4)(0u);
                    if (k0 + 4 + u < rpw)
                        kv[u] = code_load(base + ((wid + 4 * (k0 + 4 + u)) << 6));
                }
            }
        }
#pragma unroll
        for (int st = PERIOD; st < kWave; st <<= 1) {
            const int o = __shfl_xor(m, st);
            m = o < m ? o : m;
        }
    }
    if (lane < PERIOD && part == 0) smin[wid][h] = m;
    __syncthreads();
    if (threadIdx.x < HKV) {
        int dmin = smin[0][threadIdx.x];
#pragma unroll
        for (int w = 1; w < kThreads / kWave; ++w) dmin = smin[w][threadIdx.x] < dmin ? smin[w][threadIdx.x] : dmin;
        const int full = a.G * 32 * a.Wd;
        const int p1 = (pos0 + a.BS < len) ? pos0 + a.BS : len;
        const bool forced = (pos0 < a.sink) || (p1 > len - a.recent);
        if (a.reduce_out) {
            // one list per request: the best head, i.e. the smallest distance over the heads
#pragma unroll
            for (int st = 1; st < HKV; st <<= 1) {
                const int o = __shfl_xor(dmin, st);
                dmin = o < dmin ? o : dmin;
            }
            if (threadIdx.x == 0)
                a.scores[(int64_t)b * a.max_blocks + j] = pb < 0 ? -1 : (forced ? full : full - dmin);
            return;
        }
        const int sc = pb < 0 ? -1 : (forced ? full : full - dmin);
        a.scores[(int64_t)b * HKV * a.max_blocks + (int64_t)threadIdx.x * a.sc_h + (int64_t)j * a.sc_j] = sc;
    }
}

// ---------------------------------------------------------------------------------------
// Small-block scorer: blocks of 1 or 2 KiB (RPB = 1 or 2 runs of 64 pieces), e.g. 64-token
// blocks of one 256-bit latent code.  A workgroup owns TB consecutive blocks; every wave takes
// 4/RPB whole blocks per round and issues their 4 loads at once, so no block is shared between
// waves (plain LDS stores, no atomics).  Head count and pieces per code are compile-time.
// ---------------------------------------------------------------------------------------
template <int CPU, int HKV, bool DIRECT, int GP, int RPB>
__global__ __launch_bounds__(kThreads) void block_score_small(ScoreArgs a)
{
    constexpr int PERIOD = HKV * CPU;
    constexpr int UB = 4 / RPB;  // blocks per wave and round
    __shared__ int smin[kMaxTileHeads];
    __shared__ long long pbs[kMaxTile];
    const int b = blockIdx.y;
    const int j0 = blockIdx.x * a.TB;
    if (threadIdx.x < a.TB && j0 + (int)threadIdx.x < a.max_blocks)
        pbs[threadIdx.x] = physical_block(a, b, j0 + threadIdx.x);
    const int lane = lane_id();
    const int wid = wave_id();
    const int h = (lane % PERIOD) / CPU, part = lane % CPU;

    uint32_t qr[GP][4];
    if (DIRECT) {
        const uint32_t* qp = a.q + b * a.q_stride_b + (int64_t)h * GP * a.q_stride_h + part * 4;
#pragma unroll
        for (int g = 0; g < GP; ++g)
#pragma unroll
            for (int w = 0; w < 4; ++w) qr[g][w] = qp[g * a.q_stride_h + w];
    } else {
        const uint32_t* pp = a.planes + ((int64_t)b * HKV + h) * GP * a.Wd + part * 4;
#pragma unroll
        for (int p = 0; p < GP; ++p)
#pragma unroll
            for (int w = 0; w < 4; ++w) qr[p][w] = pp[p * a.Wd + w];
    }
    const int len = a.lens[b];
    const int nblk = num_blocks_of(a, len);
    if (j0 >= nblk) return;
    const int nb_tile = (a.TB < nblk - j0) ? a.TB : nblk - j0;
    __syncthreads();  // pbs visible

    int ctot = 0;
    if (!DIRECT) {
#pragma unroll
        for (int p = 0; p < GP; ++p)
#pragma unroll
            for (int w = 0; w < 4; ++w) ctot += __popc(qr[p][w]) << p;
    }

    for (int blk0 = wid * UB; blk0 < nb_tile; blk0 += 4 * UB) {
        u32x4 kv[4];
        bool ok[UB];
#pragma unroll
        for (int ub = 0; ub < UB; ++ub) {
            const int blk = blk0 + ub;
            const long long pb = blk < nb_tile ? pbs[blk] : -1;
            ok[ub] = pb >= 0;
#pragma unroll
            for (int r = 0; r < RPB; ++r) {
                kv[ub * RPB + r] = (u32x4)(0u);
                if (ok[ub])
                    kv[ub * RPB + r] = code_load(
                        reinterpret_cast<const u32x4*>(a.kc + pb * a.ks_block) + (r << 6) + lane);
            }
        }
#pragma unroll
        for (int ub = 0; ub < UB; ++ub) {
            const int blk = blk0 + ub;
            int m = kInf;
#pragma unroll
            for (int r = 0; r < RPB; ++r) {
                const u32x4 k4 = kv[ub * RPB + r];
                int d;
                if (DIRECT) {
                    d = 0;
#pragma unroll
                    for (int g = 0; g < GP; ++g)
                        d = popc_add(k4.w ^ qr[g][3], popc_add(k4.z ^ qr[g][2], popc_add(k4.y ^ qr[g][1], popc_add(k4.x ^ qr[g][0], d))));
                } else {
                    int acc = 0;
#pragma unroll
                    for (int p = 0; p < GP; ++p)
                        acc += (__popc(k4.x & qr[p][0]) + __popc(k4.y & qr[p][1]) +
                                __popc(k4.z & qr[p][2]) + __popc(k4.w & qr[p][3]))
                               << p;
                    d = ctot + a.G * popc4(k4) - 2 * acc;
                }
                if (CPU >= 2) d += __shfl_xor(d, 1);
                if (CPU >= 4) d += __shfl_xor(d, 2);
                const int t = ((r << 6) + lane) / PERIOD;
                if ((j0 + blk) * a.BS + t < len && d < m) m = d;
            }
#pragma unroll
            for (int st = PERIOD; st < kWave; st <<= 1) {
                const int o = __shfl_xor(m, st);
                m = o < m ? o : m;
            }
            if (blk < nb_tile && lane < PERIOD && part == 0) smin[blk * HKV + h] = ok[ub] ? m : kInf;
        }
    }
    __syncthreads();

    const int full = a.G * 32 * a.Wd;
    for (int i = threadIdx.x; i < nb_tile * HKV; i += kThreads) {
        const int blk = i / HKV, hh = i % HKV, j = j0 + blk;
        const int p0 = j * a.BS;
        const int p1 = (p0 + a.BS < len) ? p0 + a.BS : len;
        const bool forced = (p0 < a.sink) || (p1 > len - a.recent);
        int sc;
        if (pbs[blk] < 0) sc = -1;
        else if (forced) sc = full;
        else sc = full - smin[i];
        a.scores[((int64_t)b * HKV + hh) * a.max_blocks + j] = sc;
    }
}

// ---------------------------------------------------------------------------------------
// Blocks of 1 to 8 KiB (16- to 64-token blocks of the usual head layouts) with the query codes
// compared directly (G = 1, 2, 4): every wave owns whole blocks — U = max(4, RPB) runs of 64
// pieces, i.e. U / RPB consecutive blocks — so its 4 or 8 loads go out together right after the
// two scalar reads, the block minimum never leaves the wave (register minimum over the runs,
// shuffles over the lanes of a head) and the kernel has no LDS, no barrier and no loop.  A
// workgroup is four such waves: the same 16 KiB in flight as the one-block kernel above, where
// a workgroup per 2 KiB block would spend most of its time in the prologue.
// ---------------------------------------------------------------------------------------
template <int CPU, int HKV, int GP, int RPB>
__global__ __launch_bounds__(kThreads) void block_score_rows(ScoreArgs a)
{
    constexpr int PERIOD = HKV * CPU;        // pieces per token (a power of two <= 64)
    constexpr int U = RPB > 4 ? RPB : 4;     // runs per wave
    constexpr int NBW = U / RPB;             // blocks per wave
    const int b = blockIdx.y;
    const int lane = lane_id();
    const int wid = wave_id();
    const int h = (lane % PERIOD) / CPU, part = lane % CPU;
    const int jw = (blockIdx.x * (kThreads / kWave) + wid) * NBW;  // the wave's first block

    // table entries of the wave's blocks and the length: independent scalar reads, selected with
    // masks (no table: the entry read is a harmless second read of the length)
    const uintptr_t has_table = a.table ? ~(uintptr_t)0 : 0;
    int entry[NBW];
#pragma unroll
    for (int bi = 0; bi < NBW; ++bi) {
        const int j = jw + bi < a.max_blocks ? jw + bi : a.max_blocks - 1;
        const uintptr_t ea = (reinterpret_cast<uintptr_t>(a.table + ((int64_t)b * a.table_stride + j)) & has_table) |
                             (reinterpret_cast<uintptr_t>(a.lens + b) & ~has_table);
        entry[bi] = *reinterpret_cast<const int32_t*>(ea);
    }
    const int len = a.lens[b];

    uint32_t qr[GP][4];
    {
        const uint32_t* qp = a.q + b * a.q_stride_b + (int64_t)h * GP * a.q_stride_h + part * 4;
#pragma unroll
        for (int g = 0; g < GP; ++g)
#pragma unroll
            for (int w = 0; w < 4; ++w) qr[g][w] = qp[g * a.q_stride_h + w];
    }
    if ((int64_t)jw * a.BS >= len) return;  // the whole wave lies past the request's last block

    // every load is issued, against block 0 when the entry is unusable (masked below): one
    // instruction stream, nothing waits before all of them are out
    int64_t pb[NBW];
    u32x4 kv[U];
#pragma unroll
    for (int bi = 0; bi < NBW; ++bi) {
        const int j = jw + bi;
        int64_t v = ((int64_t)entry[bi] & (int64_t)has_table) | (((int64_t)b * a.max_blocks + j) & ~(int64_t)has_table);
        if (j >= a.max_blocks || v < 0 || v >= a.NB) v = -1;
        pb[bi] = v;
        const u32x4* base = reinterpret_cast<const u32x4*>(a.kc + (v < 0 ? 0 : v) * a.ks_block) + lane;
#pragma unroll
        for (int r = 0; r < RPB; ++r) kv[bi * RPB + r] = code_load(base + (r << 6));
    }

    const int full = a.G * 32 * a.Wd;
#pragma unroll
    for (int bi = 0; bi < NBW; ++bi) {
        const int j = jw + bi;
        const int pos0 = j * a.BS;
        int m = kInf;
#pragma unroll
        for (int r = 0; r < RPB; ++r) {
            const u32x4 k4 = kv[bi * RPB + r];
            int d = 0;
#pragma unroll
            for (int g = 0; g < GP; ++g)
                d = popc_add(k4.w ^ qr[g][3], popc_add(k4.z ^ qr[g][2], popc_add(k4.y ^ qr[g][1], popc_add(k4.x ^ qr[g][0], d))));
            if (CPU >= 2) d += __shfl_xor(d, 1);
            if (CPU >= 4) d += __shfl_xor(d, 2);
            const int t = ((r << 6) + lane) / PERIOD;
            if (pos0 + t < len && d < m) m = d;
        }
#pragma unroll
        for (int st = PERIOD; st < kWave; st <<= 1) {
            const int o = __shfl_xor(m, st);
            m = o < m ? o : m;
        }
        if (a.reduce_out) {
            // one list per request: the smallest distance over the heads, one score per block
#pragma unroll
            for (int st = CPU; st < PERIOD; st <<= 1) {
                const int o = __shfl_xor(m, st);
                m = o < m ? o : m;
            }
            if (lane == 0 && j < a.max_blocks && pos0 < len) {
                const int p1 = (pos0 + a.BS < len) ? pos0 + a.BS : len;
                const bool forced = (pos0 < a.sink) || (p1 > len - a.recent);
                a.scores[(int64_t)b * a.max_blocks + j] = pb[bi] < 0 ? -1 : (forced ? full : full - m);
            }
            continue;
        }
        if (lane < PERIOD && part == 0 && j < a.max_blocks && pos0 < len) {
            const int p1 = (pos0 + a.BS < len) ? pos0 + a.BS : len;
            const bool forced = (pos0 < a.sink) || (p1 > len - a.recent);
            const int sc = pb[bi] < 0 ? -1 : (forced ? full : full - m);
            a.scores[((int64_t)b * HKV + h) * a.max_blocks + j] = sc;
        }
    }
}

// ---------------------------------------------------------------------------------------
// Blocks smaller than one 1 KiB run (e.g. 16-token blocks of one or two KV heads, the shape a
// tensor-parallel rank sees with the serving engine's default block size): a run of 64 pieces
// covers BPR = 2, 4 or 8 blocks, each read through its own table entry, and a wave owns four
// runs.  Directly compared query codes only (G = 1, 2, 4).  The lanes of one block reduce among
// themselves; no LDS, no barrier, no loop.
// ---------------------------------------------------------------------------------------
template <int CPU, int GP>
__global__ __launch_bounds__(kThreads) void block_score_tiny(ScoreArgs a, int bpr_shift)
{
    const int b = blockIdx.y;
    const int lane = lane_id();
    const int BPR = 1 << bpr_shift;
    const int LPB = kWave >> bpr_shift;      // pieces of one block
    const int PERIOD = a.Hkv * CPU;          // pieces of one token (a power of two <= LPB)
    const int sub = lane >> (6 - bpr_shift);  // the lane's block within a run
    const int lb = lane & (LPB - 1);          // its piece within that block
    const int pshift = __builtin_ctz((unsigned)PERIOD);
    const int h = (lb & (PERIOD - 1)) / CPU, part = lb % CPU;
    const int jw = (blockIdx.x * (kThreads / kWave) + wave_id()) * (4 * BPR);  // the wave's first block

    int entry[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int j = jw + u * BPR + sub;
        entry[u] = a.table ? a.table[(int64_t)b * a.table_stride + (j < a.max_blocks ? j : a.max_blocks - 1)] : 0;
    }
    const int len = a.lens[b];
    uint32_t qr[GP][4];
    {
        const uint32_t* qp = a.q + b * a.q_stride_b + (int64_t)h * GP * a.q_stride_h + part * 4;
#pragma unroll
        for (int g = 0; g < GP; ++g)
#pragma unroll
            for (int w = 0; w < 4; ++w) qr[g][w] = qp[g * a.q_stride_h + w];
    }
    if ((int64_t)jw * a.BS >= len) return;  // the whole wave lies past the request's last block

    int64_t pb[4];
    u32x4 kv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int j = jw + u * BPR + sub;
        int64_t v = a.table ? (int64_t)entry[u] : (int64_t)b * a.max_blocks + j;
        if (j >= a.max_blocks || v < 0 || v >= a.NB) v = -1;
        pb[u] = v;
        kv[u] = code_load(reinterpret_cast<const u32x4*>(a.kc + (v < 0 ? 0 : v) * a.ks_block) + lb);
    }
    const int full = a.G * 32 * a.Wd;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int j = jw + u * BPR + sub;
        const int pos0 = j * a.BS;
        int d = 0;
#pragma unroll
        for (int g = 0; g < GP; ++g)
            d = popc_add(kv[u].w ^ qr[g][3], popc_add(kv[u].z ^ qr[g][2], popc_add(kv[u].y ^ qr[g][1], popc_add(kv[u].x ^ qr[g][0], d))));
        if (CPU >= 2) d += __shfl_xor(d, 1);
        if (CPU >= 4) d += __shfl_xor(d, 2);
        int m = (pos0 + (lb >> pshift) < len) ? d : kInf;
        for (int st = PERIOD; st < LPB; st <<= 1) {  // over the block's tokens
            const int o = __shfl_xor(m, st);
            m = o < m ? o : m;
        }
        const int p1 = (pos0 + a.BS < len) ? pos0 + a.BS : len;
        const bool forced = (pos0 < a.sink) || (p1 > len - a.recent);
        const bool live = j < a.max_blocks && pos0 < len;
        if (a.reduce_out) {
            for (int st = CPU; st < PERIOD; st <<= 1) {  // over the heads
                const int o = __shfl_xor(m, st);
                m = o < m ? o : m;
            }
            if (lb == 0 && live)
                a.scores[(int64_t)b * a.max_blocks + j] = pb[u] < 0 ? -1 : (forced ? full : full - m);
        } else if (lb < PERIOD && part == 0 && live) {
            a.scores[((int64_t)b * a.Hkv + h) * a.max_blocks + j] = pb[u] < 0 ? -1 : (forced ? full : full - m);
        }
    }
}

// ---------------------------------------------------------------------------------------
// One KV head and codes of an even number of words that the 16-byte kernels above cannot take
// — above all the 18-word codes of a latent-attention cache (512 + 64 hash bits), where a
// 16-byte piece would straddle two tokens.  The unit is the 8-byte piece: L = Wd / 2 consecutive
// lanes hold one code and a wave covers TP = 64 / L tokens per pass (18 words: 9 lanes, 7
// tokens, 63 of 64 lanes busy).  Consecutive lanes read consecutive 8 bytes, so a pass is one
// contiguous run of TP * Wd * 4 bytes, and the query material of a lane (its two words of every
// query code, or of every bit plane) never changes.
// ---------------------------------------------------------------------------------------
template <bool DIRECT, int GP>
struct PairQuery {
    uint32_t m[GP][2];
    int ctot, G;

    // issues the loads of the lane's query material
    __device__ __forceinline__ void fetch(const ScoreArgs& a, int b, int w0)
    {
        G = a.G;
        if (DIRECT) {
            const uint32_t* qp = a.q + b * a.q_stride_b + w0;
#pragma unroll
            for (int g = 0; g < GP; ++g) {
                m[g][0] = qp[g * a.q_stride_h];
                m[g][1] = qp[g * a.q_stride_h + 1];
            }
        } else {
            const uint32_t* pl = a.planes + (int64_t)b * GP * a.Wd + w0;
#pragma unroll
            for (int p = 0; p < GP; ++p) {
                m[p][0] = pl[p * a.Wd];
                m[p][1] = pl[p * a.Wd + 1];
            }
        }
    }

    // first use of the material: call after the code loads are out
    __device__ __forceinline__ void finish()
    {
        ctot = 0;
        if (!DIRECT) {
#pragma unroll
            for (int p = 0; p < GP; ++p) ctot += (__popc(m[p][0]) + __popc(m[p][1])) << p;
        }
    }

    // group-summed distance of one 8-byte piece
    __device__ __forceinline__ int dist(u32x2 k) const
    {
        int d = 0;
        if (DIRECT) {
#pragma unroll
            for (int g = 0; g < GP; ++g) d += __popc(k.x ^ m[g][0]) + __popc(k.y ^ m[g][1]);
            return d;
        }
#pragma unroll
        for (int p = 0; p < GP; ++p) d += (__popc(k.x & m[p][0]) + __popc(k.y & m[p][1])) << p;
        return ctot + G * (__popc(k.x) + __popc(k.y)) - 2 * d;
    }
};

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kPairGroup = 5;  // passes whose shuffles are issued together

// Distances of the codes of kPairGroup passes, each summed over its code's lanes (valid in the
// code's first lane).  The shuffles of one tree step go out for all passes before the first
// result is used, so their latencies overlap.
template <class Q>
__device__ __forceinline__ void pair_group_sums(const Q& qm, const u32x2* kv, int* d, int p, int L)
{
#pragma unroll
    for (int u = 0; u < kPairGroup; ++u) d[u] = qm.dist(kv[u]);
    for (int o = 1; o < L; o <<= 1) {
        const int keep = (p + o < L) ? -1 : 0;
        int t[kPairGroup];
#pragma unroll
        for (int u = 0; u < kPairGroup; ++u) t[u] = __shfl_down(d[u], o);
#pragma unroll
        for (int u = 0; u < kPairGroup; ++u) d[u] += t[u] & keep;
    }
}

constexpr int kPairPasses = 2 * kPairGroup;  // passes a wave keeps in flight (64 tokens of 18 words: all)

// Block scores: a wave owns one block, a workgroup four consecutive ones.  The pieces of a code
// are summed over its L lanes by a shuffle tree clipped at the code's end, the block minimum is
// taken over the passes in registers and over the wave by shuffles: no LDS, no barrier.
template <bool DIRECT, int GP>
__global__ __launch_bounds__(kThreads) void block_score_pairs(ScoreArgs a, int L, int TP)
{
    const int b = blockIdx.y;
    const int lane = lane_id();
    const int j = blockIdx.x * (kThreads / kWave) + wave_id();
    const int slot = lane / L, p = lane - slot * L;
    const bool lane_ok = slot < TP;
    // the table entry, the length and the query material are independent reads: all are out
    // before the first of them is waited for
    const int jc = j < a.max_blocks ? j : a.max_blocks - 1;
    const int entry = a.table ? a.table[(int64_t)b * a.table_stride + jc] : 0;
    const int len = a.lens[b];
    PairQuery<DIRECT, GP> qm;
    qm.fetch(a, b, lane_ok ? 2 * p : 0);
    const int pos0 = j * a.BS;
    if (j >= a.max_blocks || pos0 >= len) return;
    int64_t pb = a.table ? (int64_t)entry : (int64_t)b * a.max_blocks + j;
    if (pb < 0 || pb >= a.NB) pb = -1;

    const u32x2* base = reinterpret_cast<const u32x2*>(a.kc + (pb < 0 ? 0 : pb) * a.ks_block);
    const int ntok = (a.BS < len - pos0) ? a.BS : len - pos0;
    int m = kInf;
    for (int t0 = 0; t0 < ntok; t0 += kPairPasses * TP) {
        u32x2 kv[kPairPasses];
#pragma unroll
        for (int u = 0; u < kPairPasses; ++u) {
            if (t0 + u * TP < ntok) {
                // idle lanes and lanes past the block re-read the pass's first piece
                const int tok = t0 + u * TP + slot;
                kv[u] = code_load(
                    base + ((tok < a.BS && lane_ok) ? tok * L + p : (t0 + u * TP) * L));
            } else {
                kv[u] = u32x2{0u, 0u};
            }
        }
        if (t0 == 0) qm.finish();
#pragma unroll
        for (int g = 0; g < kPairPasses; g += kPairGroup) {
            if (t0 + g * TP < ntok) {
                int d[kPairGroup];
                pair_group_sums(qm, kv + g, d, p, L);
#pragma unroll
                for (int u = 0; u < kPairGroup; ++u)
                    if (lane_ok && p == 0 && t0 + (g + u) * TP + slot < ntok && d[u] < m) m = d[u];
            }
        }
    }
#pragma unroll
    for (int st = 1; st < kWave; st <<= 1) {
        const int o = __shfl_xor(m, st);
        m = o < m ? o : m;
    }
    if (lane == 0) {
        const int full = a.G * 32 * a.Wd;
        const int p1 = (pos0 + a.BS < len) ? pos0 + a.BS : len;
        const bool forced = (pos0 < a.sink) || (p1 > len - a.recent);
        a.scores[(int64_t)b * a.max_blocks + j] = pb < 0 ? -1 : (forced ? full : full - m);
    }
}

// ---------------------------------------------------------------------------------------
// Token-per-lane kernels for the latent-attention layout (one KV head, WD = 2 * LC words per
// code, token-major, 16-byte aligned blocks) at block sizes that are multiples of 64 tokens.
// A wave owns one block and walks it in rounds of 64 tokens: the round's 64 * WD * 4 contiguous
// bytes are fetched with 16-byte loads (the next round's loads are issued before the current
// round is computed), written to a wave-private LDS strip as they lie, and read back one whole
// code per lane (8-byte reads at a stride of WD words: every bank is hit once per 16 lanes).
// With a complete code in the lane there is no cross-lane sum, no idle lane and one popcount
// accumulator per bit plane for the whole code, which halves the integer work of the
// piece-per-lane kernels; the bit planes are the same for all lanes and are read from LDS as
// broadcasts (padded to 8 words per code word).
// ---------------------------------------------------------------------------------------
// Bit-sliced adders: every bit position of a word is a counter of its own.
__device__ __forceinline__ void full_add(uint32_t x, uint32_t y, uint32_t z, uint32_t& sum, uint32_t& carry)
{
    const uint32_t t = x ^ y;
    sum = t ^ z;
    carry = (t & z) | (~t & x);  // majority(x, y, z)
}
__device__ __forceinline__ void half_add(uint32_t x, uint32_t y, uint32_t& sum, uint32_t& carry)
{
    sum = x ^ y;
    carry = x & y;
}

// Bit-sliced count of 16 words: n[p] bit i = bit p of the number of words with bit i set.
__device__ __forceinline__ void count16(const uint32_t (&x)[16], uint32_t (&n)[5])
{
    uint32_t s[6], c1[5];
#pragma unroll
    for (int i = 0; i < 5; ++i) full_add(x[3 * i], x[3 * i + 1], x[3 * i + 2], s[i], c1[i]);
    s[5] = x[15];
    // weight 1: six sums
    uint32_t a0, a1, k0, k1, k2;
    full_add(s[0], s[1], s[2], a0, k0);
    full_add(s[3], s[4], s[5], a1, k1);
    half_add(a0, a1, n[0], k2);
    // weight 2: c1[0..4], k0, k1, k2
    uint32_t b0, b1, m0, m1, m2, m3;
    full_add(c1[0], c1[1], c1[2], b0, m0);
    full_add(c1[3], c1[4], k0, b1, m1);
    uint32_t b2;
    full_add(b0, b1, k1, b2, m2);
    half_add(b2, k2, n[1], m3);
    // weight 4: m0..m3
    uint32_t d0, e0, e1;
    full_add(m0, m1, m2, d0, e0);
    half_add(d0, m3, n[2], e1);
    // weight 8: e0, e1
    half_add(e0, e1, n[3], n[4]);
}

template <int LC, bool DIRECT, int GP>
struct LaneCode {
    static constexpr int WD = 2 * LC;
    static constexpr int kRoundWords = 64 * WD;
    static constexpr int kVec = kRoundWords / 4;     // 16-byte pieces per round
    static constexpr int kLoads = (kVec + 63) / 64;  // loads per lane and round

    // Planes of request b into LDS as pl[word][8] and the per-piece constants
    // ctot[piece] = sum over the piece's two words and all planes of popc(plane word) << plane.
    // Every thread of the workgroup calls this; the caller synchronises afterwards.
    static __device__ __forceinline__ void stage_planes(const ScoreArgs& a, int b, uint32_t* pl, int* ctot)
    {
        if (DIRECT) return;
        const uint32_t* src = a.planes + (int64_t)b * GP * WD;
        for (int i = threadIdx.x; i < GP * WD; i += kThreads) {
            const int p = i / WD, w = i - p * WD;
            pl[w * 8 + p] = src[i];
        }
        if ((int)threadIdx.x >= kThreads - LC) {  // the last LC threads: one piece each
            const int piece = kThreads - 1 - threadIdx.x;
            int c = 0;
#pragma unroll
            for (int p = 0; p < GP; ++p)
                c += (__popc(src[p * WD + 2 * piece]) + __popc(src[p * WD + 2 * piece + 1])) << p;
            ctot[piece] = c;
        }
    }

    static __device__ __forceinline__ void load_round(const u32x4* src, int round, int lane, u32x4 (&v)[kLoads])
    {
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int i = u * 64 + lane;
            // lanes past the round's end re-read the load's first piece
            v[u] = code_load(src + round * kVec + (i < kVec ? i : u * 64));
        }
    }

    static __device__ __forceinline__ void store_round(u32x4* strip, int lane, const u32x4 (&v)[kLoads])
    {
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int i = u * 64 + lane;
            if (i < kVec) strip[i] = v[u];
        }
    }
};

template <int LC, bool DIRECT, int GP>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 8))) void block_score_lanes(ScoreArgs a)
{
    using LCd = LaneCode<LC, DIRECT, GP>;
    constexpr int WD = LCd::WD;
    __shared__ __align__(16) uint32_t strip[kThreads / kWave][LCd::kRoundWords];
    __shared__ __align__(16) uint32_t pl[DIRECT ? 8 : WD * 8];
    __shared__ int ctot[LC];
    const int b = blockIdx.y;
    const int lane = lane_id(), wid = wave_id();
    const int j = blockIdx.x * (kThreads / kWave) + wid;
    const int jc = j < a.max_blocks ? j : a.max_blocks - 1;
    const int entry = a.table ? a.table[(int64_t)b * a.table_stride + jc] : 0;
    const int len = a.lens[b];
    LCd::stage_planes(a, b, pl, ctot);
    if (!DIRECT) __syncthreads();
    const int pos0 = j * a.BS;
    if (j >= a.max_blocks || pos0 >= len) return;
    int64_t pb = a.table ? (int64_t)entry : (int64_t)b * a.max_blocks + j;
    if (pb < 0 || pb >= a.NB) pb = -1;
    const int ntok = (a.BS < len - pos0) ? a.BS : len - pos0;
    const int rounds = (ntok + 63) >> 6;
    const u32x4* src = reinterpret_cast<const u32x4*>(a.kc + (pb < 0 ? 0 : pb) * a.ks_block);
    u32x4* mine = reinterpret_cast<u32x4*>(strip[wid]);
    const uint32_t* row = strip[wid] + lane * WD;

    u32x4 cur[LCd::kLoads], nxt[LCd::kLoads];
    LCd::load_round(src, 0, lane, cur);
#pragma unroll
    for (int u = 0; u < LCd::kLoads; ++u) nxt[u] = cur[u];
    // wave-uniform query words (scalar registers) when the codes are compared directly
    const uint32_t* qp = a.q + b * a.q_stride_b;
    int base = 0;
    if (!DIRECT) {
#pragma unroll
        for (int i = 0; i < LC; ++i) base += ctot[i];
    }
    int m = kInf;
    for (int r = 0; r < rounds; ++r) {
        if (r + 1 < rounds) LCd::load_round(src, r + 1, lane, nxt);
        LCd::store_round(mine, lane, cur);
        // the planes are re-read from LDS every round: kept in registers across rounds they
        // would cost the kernel half of its resident waves
        asm volatile("" ::: "memory");
        int d = 0;
        if (DIRECT) {
#pragma unroll
            for (int i = 0; i < LC; ++i) {
                const u32x2 k = *reinterpret_cast<const u32x2*>(row + 2 * i);
#pragma unroll
                for (int g = 0; g < GP; ++g)
                    d = popc_add(k.y ^ qp[g * a.q_stride_h + 2 * i + 1], popc_add(k.x ^ qp[g * a.q_stride_h + 2 * i], d));
            }
        } else {
            int acc[GP], pk = 0;
#pragma unroll
            for (int p = 0; p < GP; ++p) acc[p] = 0;
#pragma unroll
            for (int i = 0; i < LC; ++i) {
                const u32x2 k = *reinterpret_cast<const u32x2*>(row + 2 * i);
                pk = popc_add(k.y, popc_add(k.x, pk));
                // the 8 plane slots of a code word as two 16-byte broadcast reads
                const u32x4* pw = reinterpret_cast<const u32x4*>(pl + (2 * i) * 8);
                const u32x4 x0 = pw[0], x1 = pw[1], y0 = pw[2], y1 = pw[3];
#pragma unroll
                for (int p = 0; p < GP; ++p)
                    acc[p] = popc_add(k.y & (p < 4 ? y0[p & 3] : y1[p & 3]), popc_add(k.x & (p < 4 ? x0[p & 3] : x1[p & 3]), acc[p]));
            }
            int x = 0;
#pragma unroll
            for (int p = 0; p < GP; ++p) x += acc[p] << p;
            d = base + a.G * pk - 2 * x;
        }
        if (r * 64 + lane < ntok && d < m) m = d;
#pragma unroll
        for (int u = 0; u < LCd::kLoads; ++u) cur[u] = nxt[u];
    }
#pragma unroll
    for (int st = 1; st < kWave; st <<= 1) {
        const int o = __shfl_xor(m, st);
        m = o < m ? o : m;
    }
    if (lane == 0) {
        const int full = a.G * 32 * a.Wd;
        const int p1 = (pos0 + a.BS < len) ? pos0 + a.BS : len;
        const bool forced = (pos0 < a.sink) || (p1 > len - a.recent);
        a.scores[(int64_t)b * a.max_blocks + j] = pb < 0 ? -1 : (forced ? full : full - m);
    }
}

// 64-token blocks of 16-word codes with bit planes (18-word codes have block_score_strip<18>; the
// figures below were taken with them): block_score_lanes' walk (a round of 64
// tokens through the wave's LDS strip, planes re-read from LDS) over a run of kLaneRun consecutive
// blocks per wave - the next block's codes are requested before the current one is computed - with
// the planes built by wave 0 of the workgroup while the first codes are in flight (up to 128 query
// heads): lane (w = lane % WD, g = lane / WD) counts, bit-sliced, word w of heads g, g + NG, ...
// 16 at a time, the NG lane groups meet in LDS.  No plane kernel runs.  (One block per wave with
// the planes built per workgroup was slower than the separate plane kernel: 22.7 against 16.1 +
// 4.4 us at 16 x 65,536 tokens; a run of four blocks shares one build between 16 blocks: 18.6 us;
// runs of two or eight blocks: 19.7 / 20.0 us.)
constexpr int kLanesRunBlocks = 4;  // block_score_lanes_run

template <int LC, int GP>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 8))) void block_score_lanes_run(ScoreArgs a)
{
    using LCd = LaneCode<LC, false, GP>;
    constexpr int kRun = kLanesRunBlocks;
    constexpr int WD = LCd::WD;
    constexpr int NG = kWave / WD;                        // lane groups (3 for 18 words)
    constexpr int NCH = (128 + 16 * NG - 1) / (16 * NG);  // rounds of 16 heads per lane
    __shared__ __align__(16) uint32_t strip[kThreads / kWave][LCd::kRoundWords];
    __shared__ __align__(16) uint32_t pl[WD * 8];
    __shared__ __align__(16) uint32_t ptmp[(NG - 1) * WD * 8];
    const int b = blockIdx.y;
    const int lane = lane_id(), wid = wave_id();
    const int j0 = (blockIdx.x * (kThreads / kWave) + wid) * kRun;
    // the run's table entries: lane i holds block j0 + i
    int my_entry = 0;
    {
        const int j = j0 + (lane < kRun ? lane : 0);
        const int jc = j < a.max_blocks ? j : a.max_blocks - 1;
        if (a.table) my_entry = a.table[(int64_t)b * a.table_stride + jc];
        else my_entry = b * a.max_blocks + jc;
    }
    const bool builder = wid == 0;
    const int pw = lane % WD, pg = lane / WD;
    uint32_t qx[NCH][16];
    if (builder) {
        const uint32_t* qb = a.q + b * a.q_stride_b + pw;
        const int qs = (int)a.q_stride_h;  // a request's query codes span far less than 2^31 words
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            if (c * 16 * NG < a.G) {
#pragma unroll
                for (int t = 0; t < 16; ++t) {
                    const int h = (c * 16 + t) * NG + pg;  // heads past the group re-read the last one
                    qx[c][t] = qb[(h < a.G ? h : a.G - 1) * qs];
                }
            }
        }
    }
    const int len = a.lens[b];
    int nblk = len > 0 ? (len + 63) >> 6 : 0;
    if (nblk > a.max_blocks) nblk = a.max_blocks;
    if ((int)blockIdx.x * (kThreads / kWave) * kRun >= nblk) return;  // the whole workgroup
    const int run = nblk - j0 < kRun ? nblk - j0 : kRun;  // <= 0: nothing to score
    auto block_src = [&](int i) -> const u32x4* {
        int64_t pb = __shfl(my_entry, i);
        if (pb < 0 || pb >= a.NB) pb = 0;  // scored as -1 below
        return reinterpret_cast<const u32x4*>(a.kc + pb * a.ks_block);
    };
    u32x4* mine = reinterpret_cast<u32x4*>(strip[wid]);
    const uint32_t* row = strip[wid] + lane * WD;
    // the first block's codes go out before anything waits for the planes
    u32x4 cur[LCd::kLoads], nxt[LCd::kLoads];
    LCd::load_round(block_src(0), 0, lane, cur);
#pragma unroll
    for (int u = 0; u < LCd::kLoads; ++u) nxt[u] = cur[u];
    if (builder) {
        uint32_t acc[8];
#pragma unroll
        for (int p = 0; p < 8; ++p) acc[p] = 0;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            if (c * 16 * NG < a.G) {
                uint32_t n[5], cy = 0;
#pragma unroll
                for (int t = 0; t < 16; ++t)
                    qx[c][t] = ((c * 16 + t) * NG + pg < a.G && pg < NG) ? qx[c][t] : 0u;
                count16(qx[c], n);
#pragma unroll
                for (int p = 0; p < 8; ++p) {
                    uint32_t sum, c2;
                    if (p < 5) full_add(acc[p], n[p], cy, sum, c2);
                    else half_add(acc[p], cy, sum, c2);
                    acc[p] = sum;
                    cy = c2;
                }
            }
        }
        if (pg > 0 && pg < NG) {
            u32x4* dst = reinterpret_cast<u32x4*>(ptmp + ((pg - 1) * WD + pw) * 8);
            dst[0] = u32x4{acc[0], acc[1], acc[2], acc[3]};
            dst[1] = u32x4{acc[4], acc[5], acc[6], acc[7]};
        }
        // the same wave reads what it has just written: LDS operations of a wave complete in order
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (pg == 0) {
#pragma unroll
            for (int g = 1; g < NG; ++g) {
                const u32x4* o4 = reinterpret_cast<const u32x4*>(ptmp + ((g - 1) * WD + pw) * 8);
                const u32x4 lo = o4[0], hi = o4[1];
                uint32_t cy = 0;
#pragma unroll
                for (int p = 0; p < 8; ++p) {
                    uint32_t sum, c2;
                    full_add(acc[p], p < 4 ? lo[p & 3] : hi[p & 3], cy, sum, c2);
                    acc[p] = sum;
                    cy = c2;
                }
            }
            u32x4* dst = reinterpret_cast<u32x4*>(pl + pw * 8);
            dst[0] = u32x4{acc[0], acc[1], acc[2], acc[3]};
            dst[1] = u32x4{acc[4], acc[5], acc[6], acc[7]};
        }
    }
    // a bare barrier: __syncthreads() would make every wave wait for its codes in flight
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (run <= 0) return;
    // sum over all code bits of the per-bit counts, from the planes in LDS
    int base = 0;
    {
        int c = 0;
        if (lane < WD) {
            const u32x4* w4 = reinterpret_cast<const u32x4*>(pl + lane * 8);
            const u32x4 lo = w4[0], hi = w4[1];
#pragma unroll
            for (int p = 0; p < 8; ++p) c += __popc(p < 4 ? lo[p & 3] : hi[p & 3]) << p;
        }
#pragma unroll
        for (int st = 1; st < 32; st <<= 1) c += __shfl_xor(c, st);
        base = __builtin_amdgcn_readfirstlane(c);
    }
    const int full = a.G * 32 * a.Wd;
    int result = 0;  // lane i: score of block j0 + i
    for (int r = 0; r < run; ++r) {
        if (r + 1 < run) LCd::load_round(block_src(r + 1), 0, lane, nxt);
        LCd::store_round(mine, lane, cur);
        asm volatile("" ::: "memory");  // the planes are re-read from LDS for every block
        int acc[GP], pk = 0;
#pragma unroll
        for (int p = 0; p < GP; ++p) acc[p] = 0;
#pragma unroll
        for (int i = 0; i < LC; ++i) {
            const u32x2 k = *reinterpret_cast<const u32x2*>(row + 2 * i);
            pk = popc_add(k.y, popc_add(k.x, pk));
            const u32x4* pw4 = reinterpret_cast<const u32x4*>(pl + (2 * i) * 8);
            const u32x4 x0 = pw4[0], x1 = pw4[1], y0 = pw4[2], y1 = pw4[3];
#pragma unroll
            for (int p = 0; p < GP; ++p)
                acc[p] = popc_add(k.y & (p < 4 ? y0[p & 3] : y1[p & 3]), popc_add(k.x & (p < 4 ? x0[p & 3] : x1[p & 3]), acc[p]));
        }
        asm volatile("" ::: "memory");  // the strip is rewritten by the next block
        int x = 0;
#pragma unroll
        for (int p = 0; p < GP; ++p) x += acc[p] << p;
        const int d = base + a.G * pk - 2 * x;
        const int pos0 = (j0 + r) << 6;
        const int ntok = (64 < len - pos0) ? 64 : len - pos0;
        int m = lane < ntok ? d : kInf;
#pragma unroll
        for (int st = 1; st < kWave; st <<= 1) {
            const int o = __shfl_xor(m, st);
            m = o < m ? o : m;
        }
        const int entry = __shfl(my_entry, r);
        const bool forced = (pos0 < a.sink) || (pos0 + ntok > len - a.recent);
        const int sc = (entry < 0 || entry >= a.NB) ? -1 : (forced ? full : full - m);
        if (lane == r) result = sc;
#pragma unroll
        for (int u = 0; u < LCd::kLoads; ++u) cur[u] = nxt[u];
    }
    if (lane < run) a.scores[(int64_t)b * a.max_blocks + j0 + lane] = result;
}

// 64-token blocks of 8-word codes against one KV head whose G query heads enter as per-bit counts
// (16 requests x 65,536 tokens, 128 query heads: 33 MB of codes in 16,384 blocks of 2 KiB).  Serves up
// to 15 and more than 128 query heads; 16 to 128 heads take block_score_strip<8>, whose weighted bit
// sums run on the matrix unit (9.5 against 10.8 us at 128 heads: this kernel's 2.8 million vector
// instructions are 11,000 issue cycles per SIMD, 5 of its microseconds at the 2.2 GHz measured inside
// these scorers).
//
// Arithmetic.  With c_b the number of query heads whose bit b is set, the group-summed distance
// of a cached code k is  sum_b c_b + G * popc(k) - 2 * sum_b k_b * c_b.  The last sum is a dot
// product of the code's bits with small integers, and v_dot8_u32_u4 multiplies eight 4-bit pairs
// per lane and instruction: k & (0x11111111 << j) holds bits j, j + 4, ... of a word as nibbles
// of value 2^j, the counts of those eight bits enter as two nibble digits (c = lo + 16 * hi), and
// an accumulator per (j, digit) carries the factor 2^j until the end of the code.  4 ands, 8 dot
// products and one popcount per code word (13 operations) against 17 with eight bit planes; up
// to 15 query heads need one digit (9 operations).  Exact: every intermediate is an integer far
// below 2^32.
//
// Loads.  Lane l of a wave takes 16-byte pieces l and 64 + l of a block (two instructions of 1 KiB
// contiguous each): half (l & 1) of the codes of tokens l >> 1 and 32 + (l >> 1); the two halves
// of a code meet with one lane swap.  A lane's weight words (its four code words x four bit
// residues x two digits) stay in 32 registers.  Whatever a wave asks of memory once the code
// loads of the whole grid are under way is answered microseconds later, the smallest scalar read
// included (measured: a table entry or a length requested behind the codes took 3 to 7 us).  So
// every read that needs the kernel arguments only goes out first and together - the run's table
// entries, the length, the builder's query words - and nothing at all is requested after the codes:
// no kernel argument, no dispatch-packet field (a private array indexed at run time is kept in
// LDS behind the flat thread id, which the compiler fetches from the dispatch packet right there).
//
// Weights.  Wave 0 of the workgroup builds them while the others wait: lane (w, g) counts word w
// of heads g, g + 8, ... bit-sliced with a carry-save adder tree, three bit-sliced additions join
// the lane groups, lane (w, (j, digit)) assembles one weight word and drops it into LDS.  No wave
// requests codes before the builder holds its query words (first barrier): queued behind the
// codes of the 31 other waves of its compute unit they took 5 us (median), and every wave of the
// workgroup then stood at the barrier that long.  The second barrier hands the weights over; both
// are bare s_barrier instructions - __syncthreads() makes a wave wait for its own loads in flight,
// i.e. for all of its codes.
constexpr int kDotRun = 4;    // blocks per wave
constexpr int kDotWaves = 8;  // waves per workgroup

// Minimum over the 64 lanes, valid in lane 63: butterflies inside a row of 16 lanes, then the
// last lane of a row broadcast into the next row(s).  Written out as v_min_i32 with a DPP operand
// (the compiler turns the builtin into a copy, a DPP move and a minimum per step); a DPP operand
// needs two idle cycles after the instruction that wrote it.
__device__ __forceinline__ int wave_min_lane63(int x)
{
    asm volatile("s_nop 1\n\t"
                 "v_min_i32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t"
                 "v_min_i32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t"
                 "v_min_i32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t"
                 "v_min_i32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t"
                 "v_min_i32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\ts_nop 1\n\t"
                 "v_min_i32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf"
                 : "+v"(x));
    return x;
}

// One LDS word, read and waited for in one statement (a register that an LDS read fills later,
// behind the compiler's back, may have been given to another value by then).
__device__ __forceinline__ int lds_flag_peek(const int* p)
{
    int v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)"
                 : "=v"(v)
                 : "v"((uint32_t)(uintptr_t)(const __attribute__((address_space(3))) int*)p)
                 : "memory");
    return v;
}

template <int ND>
__global__ __launch_bounds__(kDotWaves * kWave) void block_score_dot64(ScoreArgs a)
{
    constexpr int RUN = kDotRun;
    __shared__ __align__(16) uint32_t wl[64];  // weight word [w][j][digit]
    __shared__ int base_s;
    __shared__ int ready_s;  // set by the building wave once the weights are in LDS
    const int b = blockIdx.y;
    const int lane = lane_id(), wid = wave_id();
    const int j0 = (blockIdx.x * kDotWaves + wid) * RUN;
    // first round of reads: those that need the kernel arguments only
    const int len = a.lens[b];
    int my_entry;  // lane i: table entry of block j0 + i
    {
        const int j = j0 + (lane & 7);
        const int jc = j < a.max_blocks ? j : a.max_blocks - 1;
        if (a.table) my_entry = a.table[(int64_t)b * a.table_stride + jc];
        else my_entry = b * a.max_blocks + jc;
    }
    uint32_t x[16];
    const int qw = lane & 7, qg = lane >> 3;
    const uint32_t* qb = a.q + b * a.q_stride_b + qw;
    const int qs = (int)a.q_stride_h;  // a request's query codes span far less than 2^31 words
    const int G = a.G;
    if (wid == 0) {
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int h = t * 8 + qg;  // heads past the group re-read the last one, as zero
            x[t] = qb[(h < G ? h : G - 1) * qs];
        }
    }
    // everything the rest of the kernel takes from its arguments, now
    const int64_t NB = a.NB, ks_block = a.ks_block;
    const uint32_t* kc = a.kc;
    const int sink = a.sink, recent = a.recent, max_blocks = a.max_blocks;
    int32_t* scores = a.scores;
    asm volatile("" ::"s"(sink), "s"(recent), "s"(scores), "s"(NB), "s"(G), "s"(max_blocks));
    int nblk = len > 0 ? (len + 63) >> 6 : 0;
    if (nblk > max_blocks) nblk = max_blocks;
    if ((int)blockIdx.x * kDotWaves * RUN >= nblk) return;  // the whole workgroup
    const int run = nblk - j0 < RUN ? nblk - j0 : RUN;  // <= 0: nothing to score
    int entry[RUN];
#pragma unroll
    for (int i = 0; i < RUN; ++i) entry[i] = __builtin_amdgcn_readlane(my_entry, i);
    if (wid == 0) {
        uint32_t o = 0;
#pragma unroll
        for (int t = 0; t < 16; ++t) o |= x[t];
        asm volatile("" ::"v"(o));  // the query words are here
        if (lane == 0) ready_s = 0;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    // second round of reads: the codes.  A wave stands at its load instructions until the unit's queue has room
    // (a unit takes one 1 KiB instruction per 16 cycles and answers at its share of the memory
    // rate), for microseconds when 16 waves ask for 8 KiB each.  Nobody may wait for that: the
    // building wave builds first and requests its codes afterwards, and the weights are handed over
    // with a flag in LDS that the others poll once their own requests are out - a barrier would make
    // every wave wait for the slowest wave's requests (measured: weights ready after 1.8 ... 5.9 us).
    u32x4 v[RUN][2];
    auto request = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < RUN; ++i) {
            int64_t pb = entry[i];
            if (pb < 0 || pb >= NB) pb = 0;  // scored as -1 below
            const u32x4* src = reinterpret_cast<const u32x4*>(kc + pb * ks_block);
            v[i][0] = code_load(src + lane);
            v[i][1] = code_load(src + 64 + lane);
        }
    };
    if (wid != 0) request();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    if (wid == 0) {
        uint32_t acc[8];
#pragma unroll
        for (int p = 0; p < 8; ++p) acc[p] = 0;
        auto add16 = [&](int h0) __attribute__((always_inline)) {
            uint32_t n[5];
#pragma unroll
            for (int t = 0; t < 16; ++t) x[t] = (h0 + t * 8 + qg < G) ? x[t] : 0u;
            count16(x, n);
            uint32_t cy = 0;
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                uint32_t sum, c2;
                if (p < 5) full_add(acc[p], n[p], cy, sum, c2);
                else half_add(acc[p], cy, sum, c2);
                acc[p] = sum;
                cy = c2;
            }
        };
        // straight-line code for the first 128 heads: a load inside the loop below makes the
        // compiler wait for the codes at the loop's head
        add16(0);
        for (int h0 = 128; h0 < G; h0 += 128) {
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const int h = h0 + t * 8 + qg;
                x[t] = qb[(h < G ? h : G - 1) * qs];
            }
            add16(h0);
        }
        // the eight lane groups add up (every lane ends with the full counts of its word): the
        // partner lanes l ^ 8, l ^ 16, l ^ 32 through a row rotation and the two lane-swap
        // instructions - a lane exchange through the LDS pipe (ds_bpermute) costs some hundred
        // cycles, and 27 of them in a row kept seven waves waiting for this one
#pragma unroll
        for (int st = 8; st < kWave; st <<= 1) {
            uint32_t o[8], cy = 0;
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                if (st == 8) {
                    o[p] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)acc[p], 0x128, 0xf, 0xf, false);  // row_ror:8
                } else if (st == 16) {
                    const auto sw = __builtin_amdgcn_permlane16_swap(acc[p], acc[p], false, false);
                    o[p] = (lane & 16) ? sw[0] : sw[1];
                } else {
                    const auto sw = __builtin_amdgcn_permlane32_swap(acc[p], acc[p], false, false);
                    o[p] = (lane & 32) ? sw[0] : sw[1];
                }
            }
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                uint32_t sum, c2;
                full_add(acc[p], o[p], cy, sum, c2);
                acc[p] = sum;
                cy = c2;
            }
        }
        int c = 0;
#pragma unroll
        for (int p = 0; p < 8; ++p) c += __popc(acc[p]) << p;
        c += __builtin_amdgcn_update_dpp(0, c, 0xB1, 0xf, 0xf, false);   // quad_perm [1,0,3,2]
        c += __builtin_amdgcn_update_dpp(0, c, 0x4E, 0xf, 0xf, false);   // quad_perm [2,3,0,1]
        c += __builtin_amdgcn_update_dpp(0, c, 0x141, 0xf, 0xf, false);  // row_half_mirror: the other quad
        // lane (w, g = 2 * j + digit) assembles weight word [w][j][digit]: nibble n = that digit of
        // the count of bit 4 * n + j (both digits are computed, one is kept: no run-time index)
        const int jj = qg >> 1;
        uint32_t r0 = 0, r1 = 0;
#pragma unroll
        for (int pp = 0; pp < 4; ++pp) {
            r0 |= ((acc[pp] >> jj) & 0x11111111u) << pp;
            r1 |= ((acc[4 + pp] >> jj) & 0x11111111u) << pp;
        }
        wl[qw * 8 + qg] = (qg & 1) ? r1 : r0;
        if (lane == 0) base_s = c;  // sum over all code bits of the per-bit counts
        // LDS operations of a wave complete in order: the flag lands behind the weights
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) ready_s = 1;
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        request();
    } else {
        // the builder depends on nobody, so this ends; LDS reads do not wait for the codes in flight
        while (lds_flag_peek(&ready_s) == 0) __builtin_amdgcn_s_sleep(1);
    }
    if (run <= 0) return;
    u32x4 M[8];  // [w][j / 2] -> {lo, hi of j even; lo, hi of j odd} for the lane's four code words
    {
        const u32x4* src = reinterpret_cast<const u32x4*>(wl + (lane & 1) * 32);
#pragma unroll
        for (int i = 0; i < 8; ++i) M[i] = src[i];
    }
    const int base = base_s;
    const int full = G * 256;
    int result = 0;  // lane i: score of block j0 + i
#pragma unroll
    for (int i = 0; i < RUN; ++i) {
        int dd[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            int pk = 0;
            uint32_t lo[4] = {0, 0, 0, 0}, hi[4] = {0, 0, 0, 0};
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t k = v[i][h][w];
                pk = popc_add(k, pk);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t e = k & (0x11111111u << j);
                    lo[j] = __builtin_amdgcn_udot8(e, M[w * 2 + (j >> 1)][(j & 1) * 2], lo[j], false);
                    if (ND > 1) hi[j] = __builtin_amdgcn_udot8(e, M[w * 2 + (j >> 1)][(j & 1) * 2 + 1], hi[j], false);
                }
            }
            uint32_t t[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) t[j] = ND > 1 ? lo[j] + (hi[j] << 4) : lo[j];
            const uint32_t x8 = (((((t[0] << 1) + t[1]) << 1) + t[2]) << 1) + t[3];  // 8 * sum_b k_b * c_b
            dd[h] = G * pk - (int)(x8 >> 2);
            dd[h] += __builtin_amdgcn_update_dpp(0, dd[h], 0xB1, 0xf, 0xf, true);  // the code's other half
        }
        const int pos0 = (j0 + i) << 6;
        const int t0 = pos0 + (lane >> 1);
        int d = (i < run && t0 < len) ? dd[0] : kInf;
        const int d1 = (i < run && t0 + 32 < len) ? dd[1] : kInf;
        d = d1 < d ? d1 : d;
        const int m = __builtin_amdgcn_readlane(wave_min_lane63(d), 63) + base;
        const int ntok = (64 < len - pos0) ? 64 : len - pos0;
        const bool forced = (pos0 < sink) || (pos0 + ntok > len - recent);
        const int sc = (entry[i] < 0 || entry[i] >= NB) ? -1 : (forced ? full : full - m);
        if (lane == i) result = sc;
    }
    if (lane < run) scores[(int64_t)b * max_blocks + j0 + lane] = result;
}

// 64-token blocks of 18-word codes against one KV head whose G query heads enter as per-bit
// counts (the latent cache with position part: 16 requests x 65,536 tokens, 75 MB of codes in
// 16,384 blocks of 4.5 KiB).
//
// Arithmetic.  With c_b the number of query heads whose bit b is set, the group-summed distance of
// a code k is  sum_b c_b + sum_b k_b * t_b  with the signed weight t_b = G - 2 c_b: per request a
// matrix-vector product of the tokens' 576 code bits with one small-integer vector.  As vector
// work it costs 13 operations a code word and token at best (4-bit dot products, as in
// block_score_dot64): 270 a block and wave, 7.7 us a SIMD for the 16 blocks it gets - more than
// the 9.6 us the codes take to arrive allow for in a kernel that also has to start and end
// (measured: loads alone 12.6 us, arithmetic alone 9.7 us, together 16.1 to 16.7 us).  So the
// product runs on the matrix unit, exactly: v_mfma_f32_16x16x128 with FP4 (E2M1) operands, one
// instruction per code word.  A lane's word becomes 32 FP4 values with five operations -
// k & 0x1111.., k & 0x2222.., k & 0x4444.. and (k >> 1) & 0x4444.. hold bit 4 i + j in nibble i as
// 0.5, 1, 2, 2 - and |t_b| <= 128 is four base-4 digits whose products with those, digit x
// {2, 1, 1/2, 1/2} = 0 ... 6 in steps FP4 has, carry t_b's sign.  Lane l supplies row l % 16 for the
// K quarter l / 16, so token l is row l % 16 of quarter l / 16, and column 4 q + d of the other
// operand carries digit d in quarter q and zeros elsewhere: all 16 columns are used, the result
// register r of lane l is digit l % 4 of token 16 * ((l % 16) / 4) + 4 * (l / 16) + r.  Scaling by
// 4^digit, a sum over the four lanes of a quad and a minimum finish the block.  Every term is a
// small integer: the float accumulation is exact, and the scores equal the integer kernels' bit
// for bit.  (v_mfma_f32_32x32x64 with the same operands fills 8 of its 32 columns and measured
// 17.7 to 18.5 us, two accumulator chains 18.7 to 19.5: the instruction's own time is the limit
// there.  16x16x128: 15.0 to 15.4 us.)
//
// Codes.  A block goes from memory straight into the wave's LDS strip (load-to-LDS, five
// instructions of 1 KiB, the last one half masked): no register holds a code on its way, no LDS
// store instruction is issued.  The strip holds two blocks; a wave scores a run of four and
// requests block i + 2 the moment block i's reads are back.  Lane l reads token l's row (72 bytes
// apart: 16 consecutive lanes cover all banks) as nine 8-byte reads.  The 18 x 4 operand words of
// the weights stay in registers for the whole run.
//
// Build.  Lane (s, g) of wave v counts code word 8 v + s over heads g, g + 8, ... bit-sliced (up to
// 128 query heads), the eight lanes of a word add their counts with three DPP exchanges, subtract
// twice the sum from G (ten bit-sliced bits), take the magnitude, and lanes g < 4 assemble the
// four operand words of base-4 digit g: a wave takes its words from the query to the operands
// without LDS and without meeting another wave; waves 0 and 1 build eight words each, wave 2
// two, the others none.  (Before: three steps by all four waves with LDS and a barrier between
// them, 14.8 to 15.4 us; one wave doing all of it held the workgroup for 2.4 to 5 us.)
//
// Shape (18-word codes).  Eight waves per workgroup, a run of four blocks per wave, two blocks of a wave in LDS: two
// workgroups (147 KB of strips) and 16 waves on a compute unit, four to a SIMD.  A block costs its
// wave some 215 vector and 18 matrix instructions, about 1,150 issue cycles - 9 to 10 us per SIMD for
// its 16 blocks at the 2.1 to 2.3 GHz measured inside this kernel, most of the time the codes take to
// arrive - and with two waves to a SIMD (four
// waves per workgroup, runs of eight, four blocks in LDS - the same 147 KB in flight) a SIMD stood
// idle whenever both of its waves waited: 17.1 to 17.5 us with the codes from HBM against 15.4 us
// now (the whole call with the codes in the last-level cache: 18.0 to 19.8 against 16.4 to 17.5 us).
// The three building waves
// request their first blocks after the build - the five others' requests keep memory busy
// meanwhile (one block before the build: the same; two: 16.3 us).
constexpr int kStripWaves = 8;  // waves per workgroup
constexpr int kStripRun = 4;    // blocks per wave
constexpr int kStripSlots = 2;  // blocks of a wave in LDS
constexpr int strip_run(int wd) { return wd == 18 ? kStripRun : 4; }  // blocks per wave
constexpr int kStripFirst = 0;  // of those, a building wave requests before the weight build (at most kStripSlots)

// One block of NL KiB (+ half a KiB when TAIL) from `base` into LDS at byte address `lds`.
template <int NL, bool TAIL>
__device__ __forceinline__ void strip_issue_block(uint32_t lds, uint64_t base, uint32_t off, bool low_half)
{
    static_assert(NL == 4 || NL == 2, "a block of 64 codes of 8, 16 or 18 words");
    uint32_t keep;
    if (NL == 4) {
        asm volatile("s_mov_b32 %[keep], m0\n\ts_mov_b32 m0, %[lds]\n\ts_nop 0\n\t"
                     "global_load_lds_dwordx4 %[o], %[base] nt\n\t"
                     "global_load_lds_dwordx4 %[o], %[base] offset:1024 nt\n\t"
                     "global_load_lds_dwordx4 %[o], %[base] offset:2048 nt\n\t"
                     "global_load_lds_dwordx4 %[o], %[base] offset:3072 nt\n\t"
                     "s_mov_b32 m0, %[keep]\n\t"
                     : [keep] "=&s"(keep)
                     : [lds] "s"(lds), [base] "s"(base), [o] "v"(off)
                     : "memory");
    } else {
        asm volatile("s_mov_b32 %[keep], m0\n\ts_mov_b32 m0, %[lds]\n\ts_nop 0\n\t"
                     "global_load_lds_dwordx4 %[o], %[base] nt\n\t"
                     "global_load_lds_dwordx4 %[o], %[base] offset:1024 nt\n\t"
                     "s_mov_b32 m0, %[keep]\n\t"
                     : [keep] "=&s"(keep)
                     : [lds] "s"(lds), [base] "s"(base), [o] "v"(off)
                     : "memory");
    }
    if (TAIL) {
        if (low_half) {
            asm volatile("s_mov_b32 %[keep], m0\n\ts_add_u32 m0, %[lds], 4096\n\ts_nop 0\n\t"
                         "global_load_lds_dwordx4 %[o], %[base] nt\n\t"
                         "s_mov_b32 m0, %[keep]\n\t"
                         : [keep] "=&s"(keep)
                         : [lds] "s"(lds), [base] "s"(base), [o] "v"(off + 4096u)
                         : "memory", "scc");
        }
    }
}

typedef int i32x8s __attribute__((ext_vector_type(8)));
typedef float f32x4s __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2s __attribute__((ext_vector_type(2)));

// Four values, each replaced by its sum over the four lanes of a quad (two v_add_f32 with a DPP
// operand per value; a DPP operand needs two idle cycles after the instruction that wrote it, which
// the other three values' additions provide after the first).
__device__ __forceinline__ void quad_sum4(float& v0, float& v1, float& v2, float& v3)
{
    asm volatile("s_nop 1\n\t"
                 "v_add_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
                 "v_add_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
                 "v_add_f32_dpp %2, %2, %2 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
                 "v_add_f32_dpp %3, %3, %3 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
                 "v_add_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
                 "v_add_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
                 "v_add_f32_dpp %2, %2, %2 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
                 "v_add_f32_dpp %3, %3, %3 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf"
                 : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3));
}

// MODE 0: block scores.  MODE 1 / 2: the distance of every token as int32 / as fp16 - the reference scorer's
// own output (paged_ham_dist_mla.cu:204-210,235-241): an 8-byte piece is two code words, two matrix
// instructions into an accumulator of their own, and the piece sums are added in half precision in
// the reference's order; a quad's four lanes hold the same four tokens, its first lane writes them.
template <int WD, int MODE>
__device__ __forceinline__ void strip_body(const ScoreArgs& a, int max_seq_len, void* out)
{
    static_assert(WD == 18 || WD == 8, "64-token blocks of 18-word or 8-word codes");
    constexpr bool TOKENS = MODE != 0;
    // 8-word codes: blocks of 2 KiB, three of a wave in LDS (48 KB per workgroup).  Measured at 16 x 65,536
    // tokens and 128 query heads, codes from HBM: 9.5 to 9.6 us (runs of two blocks with two in LDS, eight
    // waves to a SIMD: 10.2 us; sixteen waves per workgroup, one workgroup and one build per compute unit: 10.1 us; four waves
    // per workgroup, four workgroups and builds per compute unit: 10.2 us;
    // the 4-bit dot products of block_score_dot64 on the vector unit: 10.8 to 11.0 us)
    constexpr int RUN = strip_run(WD), kSlots = WD == 18 ? kStripSlots : 3, kFirst = kStripFirst;
    constexpr int kBuilders = (WD + 7) / 8;  // waves that build weights, eight code words each
    // (fetched with the other arguments at the top: nothing is requested of the arguments once the codes flow)
    unsigned long long* const probe =
        (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x >= (kStripWaves - 1) * kWave) ? a.clock_probe : nullptr;
    unsigned long long probe_c0 = 0, probe_r0 = 0;
    if (probe) {
        probe_c0 = __builtin_readcyclecounter();
        probe_r0 = __builtin_amdgcn_s_memrealtime();
    }
    constexpr int kBlockWords = 64 * WD;
    constexpr int kLoadsPerBlock = WD == 18 ? 5 : 2;
    __shared__ __align__(16) uint32_t strip[kStripWaves][kSlots * kBlockWords];
    __shared__ __align__(16) uint32_t wB[WD * 4 * 4];    // operand words [w][digit][j]
    __shared__ __align__(16) uint32_t wzero[4];
    __shared__ int base_s;
    // per 8-byte piece: the sum over its bits of the per-bit counts, and a row of zeros for the lanes
    // that do not carry it
    __shared__ int cpiece[2 * (WD / 2)];
    const int b = blockIdx.y;
    const int lane = lane_id(), wid = wave_id();
    const int j0 = (blockIdx.x * kStripWaves + wid) * RUN;
    // first round of reads: those that need the kernel arguments only
    const int len = a.lens[b];
    int my_entry;  // lane i: table entry of block j0 + i
    {
        const int j = j0 + (lane & 7);
        const int jc = j < a.max_blocks ? j : a.max_blocks - 1;
        if (a.table) my_entry = a.table[(int64_t)b * a.table_stride + jc];
        else my_entry = b * a.max_blocks + jc;
    }
    // The build: lane (s, g) of wave v counts code word 8 v + s of heads g, g + 8, ... (16 of them,
    // 128 query heads), bit-sliced.  The eight head groups of a word are eight neighbouring lanes,
    // so they add up with three DPP exchanges and no LDS, and the same lanes turn the counts of
    // their word into its operand words: a wave builds its words from the query words to the end
    // without meeting another wave (waves 0 and 1 eight words each, wave 2 the last two).
    const int bs = lane >> 3, bg = lane & 7;
    const int word = wid * 8 + bs;
    const bool has_word = word < WD;
    const int G = a.G;
    uint32_t qx[16];
    if (wid < kBuilders) {
        const uint32_t* qb = a.q + b * a.q_stride_b + (has_word ? word : 0);
        const int qs = (int)a.q_stride_h;  // a request's query codes span far less than 2^31 words
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int h = bg + 8 * t;  // heads past the group re-read the last one, as zero
            qx[t] = qb[(h < G ? h : G - 1) * qs];
        }
    }
    if (threadIdx.x == 0) base_s = 0;
    if (threadIdx.x < 4) wzero[threadIdx.x] = 0;
    if (TOKENS && threadIdx.x < 2 * (WD / 2)) cpiece[threadIdx.x] = 0;
    // everything the rest of the kernel takes from its arguments, now
    const int64_t NB = a.NB, ks_block = a.ks_block;
    const uint32_t* kc = a.kc;
    const int sink = a.sink, recent = a.recent, max_blocks = a.max_blocks;
    int32_t* scores = a.scores;
    asm volatile("" ::"s"(sink), "s"(recent), "s"(scores), "s"(NB), "s"(G), "s"(max_blocks));
    int nblk = len > 0 ? (len + 63) >> 6 : 0;
    if (nblk > max_blocks) nblk = max_blocks;
    // per-token output: lane (column c, quarter q) holds tokens 16 (c / 4) + 4 q + r, r = 0..3, of a block;
    // the first lane of a quad writes them.  A block that is not read still gets its row: infinity,
    // or zero inside the sink and recent windows.
    const int tok0 = 16 * ((lane & 15) >> 2) + 4 * (lane >> 4);
    const bool by_four = TOKENS && (max_seq_len & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
    auto emit = [&](int i, bool usable, const float (&df)[4], const _Float16 (&dh)[4]) __attribute__((always_inline)) {
        const int pos0 = (j0 + i) << 6;
        if ((lane & 3) != 0 || pos0 + tok0 >= max_seq_len) return;
        const int64_t o = (int64_t)b * max_seq_len + pos0 + tok0;
        uint32_t iv[4];
        uint16_t hv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int pos = pos0 + tok0 + r;
            const bool keep = (pos < sink) || (pos >= len - recent && pos < len);
            const bool none = pos >= len || (!keep && !usable);
            iv[r] = (uint32_t)(none ? kInf : (keep ? 0 : (int)df[r]));  // exact: an integer below 2^24
            const _Float16 v = none ? (_Float16)__builtin_inff() : (keep ? (_Float16)0.0f : dh[r]);
            __builtin_memcpy(&hv[r], &v, 2);
        }
        if (MODE == 2) {
            if (by_four) {
                u32x2 w;
                w.x = hv[0] | ((uint32_t)hv[1] << 16);
                w.y = hv[2] | ((uint32_t)hv[3] << 16);
                *reinterpret_cast<u32x2*>((uint16_t*)out + o) = w;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (pos0 + tok0 + r < max_seq_len) ((uint16_t*)out)[o + r] = hv[r];
            }
        } else {
            if (by_four) {
                u32x4 w;
                w.x = iv[0]; w.y = iv[1]; w.z = iv[2]; w.w = iv[3];
                *reinterpret_cast<u32x4*>((int32_t*)out + o) = w;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (pos0 + tok0 + r < max_seq_len) ((int32_t*)out)[o + r] = (int32_t)iv[r];
            }
        }
    };
    auto emit_unread = [&](int first_i) __attribute__((always_inline)) {
        const float none_i[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        const _Float16 none_h[4] = {(_Float16)0.0f, (_Float16)0.0f, (_Float16)0.0f, (_Float16)0.0f};
#pragma unroll
        for (int i = 0; i < RUN; ++i)
            if (i >= first_i) emit(i, false, none_i, none_h);
    };
    if ((int)blockIdx.x * kStripWaves * RUN >= nblk) {  // the whole workgroup
        if (TOKENS) emit_unread(0);
        return;
    }
    const int run = nblk - j0 < RUN ? nblk - j0 : RUN;  // <= 0: nothing to score
    int entry[RUN];
#pragma unroll
    for (int i = 0; i < RUN; ++i) entry[i] = __builtin_amdgcn_readlane(my_entry, i);
    // base_s is zero for everybody (the waves get here within a few hundred nanoseconds of one
    // another, long before the query words)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane(
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint32_t*)strip[wid]);
    const uint32_t off = (uint32_t)lane * 16u;
    auto issue = [&](int i) __attribute__((always_inline)) {
        int64_t pb = entry[i];
        if (pb < 0 || pb >= NB) pb = 0;  // scored as -1 below
        strip_issue_block<(WD == 18 ? 4 : 2), (WD == 18)>(lds0 + (uint32_t)(i % kSlots) * (kBlockWords * 4),
                                                           reinterpret_cast<uint64_t>(kc + pb * ks_block), off, lane < 32);
    };
    if (wid < kBuilders) {
        {
            uint32_t o = 0;
#pragma unroll
            for (int t = 0; t < 16; ++t) o |= qx[t];
            asm volatile("" ::"v"(o));  // the query words are here: no code is requested before
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < kFirst; ++i)
            if (i < run) issue(i);
        __builtin_amdgcn_sched_barrier(0);
        uint32_t acc[8];
        {
            uint32_t n[5];
#pragma unroll
            for (int t = 0; t < 16; ++t) qx[t] = (bg + 8 * t < G && has_word) ? qx[t] : 0u;
            count16(qx, n);
#pragma unroll
            for (int p = 0; p < 8; ++p) acc[p] = p < 5 ? n[p] : 0u;
        }
        // the eight head groups of a word: lanes l ^ 1, l ^ 2 and the mirror lane of the other quad
#pragma unroll
        for (int st = 0; st < 3; ++st) {
            uint32_t o[8], cy = 0;
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                if (st == 0) o[p] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)acc[p], 0xB1, 0xf, 0xf, false);
                else if (st == 1) o[p] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)acc[p], 0x4E, 0xf, 0xf, false);
                else o[p] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)acc[p], 0x141, 0xf, 0xf, false);
            }
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                uint32_t sum, c2;
                full_add(acc[p], o[p], cy, sum, c2);
                acc[p] = sum;
                cy = c2;
            }
        }
        // signed weight of every bit, t = G - 2 c (|t| <= G <= 128), bit-sliced: ten-bit
        // subtraction, then the magnitude
        uint32_t mag[8], sgn;
        {
            uint32_t diff[10], br = 0;
#pragma unroll
            for (int i = 0; i < 10; ++i) {
                const uint32_t g = ((G >> i) & 1) ? ~0u : 0u;
                const uint32_t u = (i >= 1 && i <= 8) ? acc[i - 1] : 0u;
                diff[i] = g ^ u ^ br;
                br = (~g & (u | br)) | (u & br);
            }
            sgn = diff[9];
            uint32_t cy = sgn;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t m = diff[i] ^ sgn;
                mag[i] = m ^ cy;
                cy = m & cy;
            }
        }
        // lane g < 4 assembles base-4 digit g of the magnitude (selected, not indexed: an array
        // indexed at run time would be kept in LDS)
        const int p2 = bg & 3;
        const uint32_t a0 = p2 == 0 ? mag[0] : p2 == 1 ? mag[2] : p2 == 2 ? mag[4] : mag[6];
        const uint32_t a1 = p2 == 0 ? mag[1] : p2 == 1 ? mag[3] : p2 == 2 ? mag[5] : mag[7];
        const uint32_t both = a0 & a1;
        // FP4 (E2M1) code of digit * {2, 1, 1/2, 1/2} for bit residue j = 0, 1, 2, 3 - the code
        // operand holds such a bit as 0.5, 1, 2, 2 - nibble i of word j for code bit 4 i + j
        auto pack = [&](uint32_t b0, uint32_t b1, uint32_t b2, int j) {
            constexpr uint32_t M = 0x11111111u;
            return ((b0 >> j) & M) | (((b1 >> j) & M) << 1) | (((b2 >> j) & M) << 2) | (((sgn >> j) & M) << 3);
        };
        u32x4 bw;
        bw.x = pack(both, a1, a0 | a1, 0);   // 0, 2, 4, 6 -> codes 0, 4, 6, 7
        bw.y = pack(both, a0 & ~a1, a1, 1);  // 0, 1, 2, 3 -> codes 0, 2, 4, 5
        bw.z = pack(a0, a1, 0u, 2);          // 0, 1/2, 1, 3/2 -> codes 0, 1, 2, 3
        bw.w = pack(a0, a1, 0u, 3);
        if (has_word && bg < 4) *reinterpret_cast<u32x4*>(wB + (word * 4 + p2) * 4) = bw;
        if (has_word && bg == 0) {
            int c = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) c += __popc(acc[i]) << i;
            atomicAdd(&base_s, c);  // sum over all code bits of the per-bit counts
            if (TOKENS) atomicAdd(&cpiece[word >> 1], c);
        }
    } else {
#pragma unroll
        for (int i = 0; i < kSlots; ++i)
            if (i < run) issue(i);
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    const int first = wid < kBuilders ? kFirst : kSlots;
#pragma unroll
    for (int i = 0; i < kSlots; ++i)
        if (i >= first && i < run) issue(i);
    if (run <= 0) {
        if (TOKENS) emit_unread(0);
        return;
    }
    const int base = base_s;
    // the first lane of a quad adds the piece's constant: it reads the row of constants, the others the zeros
    const int* cp_row = cpiece + ((lane & 3) == 0 ? 0 : WD / 2);
    const int full = G * 32 * WD;
    // v_mfma_f32_16x16x128 with FP4 operands, one per code word: 16 rows x 128 values of A times
    // 128 x 16 of B.  Lane l supplies row l % 16 of A / column l % 16 of B for the K quarter l / 16,
    // so token l (its word as four masked copies = 32 FP4 values) is row l % 16, quarter l / 16, and
    // column 4 q + d carries digit d for the tokens of quarter q: zeros outside quarter q.  Result
    // register r of lane l is row 4 * (l / 16) + r of column l % 16.
    const int col = lane & 15, quarter = lane >> 4;
    u32x4 Bw[WD];
    {
        const bool live = (col >> 2) == quarter;
        const uint32_t* src = live ? wB + (col & 3) * 4 : wzero;
        const int stride = live ? 16 : 0;
#pragma unroll
        for (int w = 0; w < WD; ++w) Bw[w] = *reinterpret_cast<const u32x4*>(src + w * stride);
    }
    const float dscale = (col & 3) == 0 ? 1.0f : (col & 3) == 1 ? 4.0f : (col & 3) == 2 ? 16.0f : 64.0f;
    // tok0 + r: the token of result register r
    int result = 0;  // lane i: score of block j0 + i
#pragma unroll
    for (int i = 0; i < RUN; ++i) {
        if (i >= run) break;
        // block i's codes have landed: loads complete in order, and at most the kSlots - 1 blocks
        // requested behind it may still be under way
        {
            const int behind = run - 1 - i < kSlots - 1 ? run - 1 - i : kSlots - 1;
            if (behind >= 3) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * kLoadsPerBlock) : "memory");
            else if (behind == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kLoadsPerBlock) : "memory");
            else if (behind == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoadsPerBlock) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        const uint32_t* row = strip[wid] + (i % kSlots) * kBlockWords + lane * WD;
        uint32_t k[WD];
        if (WD % 4 == 0) {
            // rows of 32 bytes: 16-byte reads (two lanes to a bank; 8-byte reads would put four there)
#pragma unroll
            for (int w = 0; w < WD / 4; ++w) {
                const u32x4 kk = *reinterpret_cast<const u32x4*>(row + 4 * w);
                k[4 * w] = kk.x;
                k[4 * w + 1] = kk.y;
                k[4 * w + 2] = kk.z;
                k[4 * w + 3] = kk.w;
            }
        } else {
#pragma unroll
            for (int w = 0; w < WD / 2; ++w) {
                const u32x2 kk = *reinterpret_cast<const u32x2*>(row + 2 * w);
                k[2 * w] = kk.x;
                k[2 * w + 1] = kk.y;
            }
        }
        f32x4s c = {0.0f, 0.0f, 0.0f, 0.0f};
        float df[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        f16x2s dh01 = {(_Float16)0.0f, (_Float16)0.0f}, dh23 = dh01;
#pragma unroll
        for (int w = 0; w < WD; ++w) {
            const i32x8s A = {(int)(k[w] & 0x11111111u), (int)(k[w] & 0x22222222u), (int)(k[w] & 0x44444444u),
                              (int)((k[w] >> 1) & 0x44444444u), 0, 0, 0, 0};
            const i32x8s B = {(int)Bw[w].x, (int)Bw[w].y, (int)Bw[w].z, (int)Bw[w].w, 0, 0, 0, 0};
            if (TOKENS && (w & 1) == 0) c = f32x4s{0.0f, 0.0f, 0.0f, 0.0f};
            c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, c, 4, 4, 0, 0, 0, 0);  // FP4 x FP4, scales off
            if (TOKENS && (w & 1) == 1) {
                // the piece's sum per token: scale by 4^digit, the piece's constant in one lane of the
                // quad, the sum over the quad.  Small integers: every step is exact in fp32.
                const float cpf = (float)cp_row[w >> 1];
                float v0 = c[0] * dscale + cpf, v1 = c[1] * dscale + cpf, v2 = c[2] * dscale + cpf, v3 = c[3] * dscale + cpf;
                quad_sum4(v0, v1, v2, v3);
                if (MODE == 2) {
                    // two tokens to an instruction: packed conversion (round to nearest even) and packed addition
                    dh01 = dh01 + f16x2s{(_Float16)v0, (_Float16)v1};
                    dh23 = dh23 + f16x2s{(_Float16)v2, (_Float16)v3};
                } else {
                    df[0] += v0;
                    df[1] += v1;
                    df[2] += v2;
                    df[3] += v3;
                }
            }
        }
        if (i + kSlots < run) {
            // this strip slot is free once its last reads are back
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            issue(i + kSlots);
        }
        if (TOKENS) {
            const _Float16 dh[4] = {dh01.x, dh01.y, dh23.x, dh23.y};
            emit(i, entry[i] >= 0 && entry[i] < NB, df, dh);
            continue;
        }
        // sum_b k_b t_b of a token = sum over its four digit columns of 4^digit * column: scale, add
        // across the four lanes of a quad, then the minimum over this lane's four tokens
        const int pos0 = (j0 + i) << 6;
        const int ntok = (64 < len - pos0) ? 64 : len - pos0;
        float mn = 3.0e38f;
        {
            float v[4] = {c[0] * dscale, c[1] * dscale, c[2] * dscale, c[3] * dscale};
            quad_sum4(v[0], v[1], v[2], v[3]);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (tok0 + r >= ntok) v[r] = 3.0e38f;  // the last block of a request
                mn = v[r] < mn ? v[r] : mn;
            }
        }
        const int d = (int)mn;  // exact: every term is an integer below 2^24 (all masked: saturates)
        const int m = __builtin_amdgcn_readlane(wave_min_lane63(d), 63) + base;
        const bool forced = (pos0 < sink) || (pos0 + ntok > len - recent);
        const int sc = (entry[i] < 0 || entry[i] >= NB) ? -1 : (forced ? full : full - m);
        if (lane == i) result = sc;
    }
    if (TOKENS) emit_unread(run);
    else if (lane < run) scores[(int64_t)b * max_blocks + j0 + lane] = result;
    // the last wave of the first workgroup: shader cycles and 100 MHz ticks of its life
    if (probe && threadIdx.x == kStripWaves * kWave - 1) {
        probe[0] = __builtin_readcyclecounter() - probe_c0;
        probe[1] = __builtin_amdgcn_s_memrealtime() - probe_r0;
    }
}

template <int WD>
__global__ __launch_bounds__(kStripWaves * kWave) __attribute__((amdgpu_waves_per_eu(4, 8))) void block_score_strip(ScoreArgs a)
{
    strip_body<WD, 0>(a, 0, nullptr);
}

template <int WD, bool F16>
__global__ __launch_bounds__(kStripWaves * kWave) __attribute__((amdgpu_waves_per_eu(4, 8))) void token_score_strip(ScoreArgs a, int max_seq_len, void* out)
{
    strip_body<WD, F16 ? 2 : 1>(a, max_seq_len, out);
}

// ---------------------------------------------------------------------------------------
// Generic block scorer: any strides, code width, head count and group size.  One thread per
// (token, head) code, word-by-word loads; query codes staged in LDS.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void block_score_generic(ScoreArgs a)
{
    extern __shared__ uint32_t dyn[];
    __shared__ int smin[kMaxTileHeads];
    uint32_t* qs = dyn;  // [Hq][Wd]
    const int b = blockIdx.y;
    const int len = a.lens[b];
    const int nblk = num_blocks_of(a, len);
    const int j0 = blockIdx.x * a.TB;
    if (j0 >= nblk) return;
    const int nb_tile = (a.TB < nblk - j0) ? a.TB : nblk - j0;

    for (int i = threadIdx.x; i < nb_tile * a.Hkv; i += kThreads) smin[i] = kInf;
    for (int i = threadIdx.x; i < a.Hq * a.Wd; i += kThreads)
        qs[i] = a.q[b * a.q_stride_b + (int64_t)(i / a.Wd) * a.q_stride_h + (i % a.Wd)];
    __syncthreads();

    const int units = a.BS * a.Hkv;
    for (int blk = 0; blk < nb_tile; ++blk) {
        const int64_t pb = physical_block(a, b, j0 + blk);
        if (pb < 0) continue;
        const uint32_t* base = a.kc + pb * a.ks_block;
        for (int u = threadIdx.x; u < units; u += kThreads) {
            const int t = u / a.Hkv, h = u % a.Hkv;
            if ((j0 + blk) * a.BS + t >= len) continue;
            const uint32_t* kp = base + t * a.ks_token + h * a.ks_head;
            int d = 0;
            for (int w = 0; w < a.Wd; ++w) {
                const uint32_t kw = kp[w];
                for (int g = 0; g < a.G; ++g) d += __popc(kw ^ qs[(h * a.G + g) * a.Wd + w]);
            }
            atomicMin(&smin[blk * a.Hkv + h], d);
        }
    }
    __syncthreads();
    write_tile_scores(a, b, j0, nb_tile, len, smin);
}

// ---------------------------------------------------------------------------------------
// Selection.
// ---------------------------------------------------------------------------------------
struct SelectArgs {
    const int32_t* scores;  // [B][Hkv][max_blocks]
    int sc_h, sc_j;         // select_wave_kernel only: head / block strides inside a request's scores
    int32_t* reduced;       // [B][max_blocks] scratch for head-reduced rows beyond the LDS cap
    const int32_t* table;
    int table_stride, max_blocks;
    const int32_t* lens;
    int BS, Hkv, Ho, k, full, key_bits;
    uint32_t flags;
    int32_t* out_idx;    // [B][Ho][k]
    int32_t* out_score;  // may be null
    // Replacement block table and sequence lengths of a decode step (null = not asked for; needs
    // Ho == 1 and physical ids): row b of new_table gets the selected ids in its first k entries
    // and 0 in all others up to max_blocks; a request shorter than thr_len keeps its own row and
    // length; new_lens[b] = len - ceil(max(len - topk_tok, 0) / BS) * BS otherwise.
    int32_t* new_table;
    int new_table_stride;
    int32_t* new_lens;
    int thr_len, topk_tok;
};

// The first part of that epilogue, shared by the selection kernels: `tid` of `nthreads` threads
// own a row.  Returns true when the row is complete (short request or no blocks) and the
// selection can be skipped; otherwise entries [kk, max_blocks) are zeroed and the caller
// fills [0, kk).
__device__ __forceinline__ bool plugin_row_prologue(const SelectArgs& a, int b, int len, int kk, int tid,
                                                    int nthreads)
{
    int32_t* row = a.new_table + (int64_t)b * a.new_table_stride;
    const bool keep = a.thr_len > 0 && len < a.thr_len;
    if (tid == 0) {
        int over = len - a.topk_tok;
        over = over < 0 ? 0 : over;
        a.new_lens[b] = keep ? len : len - ((over + a.BS - 1) / a.BS) * a.BS;
    }
    if (keep) {
        const int32_t* src = a.table + (int64_t)b * a.table_stride;
        for (int j = tid; j < a.max_blocks; j += nthreads) row[j] = src[j];
        return true;
    }
    for (int j = kk + tid; j < a.max_blocks; j += nthreads) row[j] = 0;
    return kk == 0;
}

// Inclusive prefix sum over the 64 lanes with DPP operands (row shifts inside a row of 16 lanes -
// a lane without a source adds 0 - then the last lane of a row broadcast into the next row(s)):
// six additions a few cycles apart, where six lane exchanges through the LDS pipe cost some
// hundred cycles each, one after the other.
__device__ __forceinline__ int wave_incl_scan(int v)
{
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
    return v;
}
// Maximum over the 64 lanes, valid in lane 63 (see wave_min_lane63).
__device__ __forceinline__ int wave_max_lane63(int x)
{
    asm volatile("s_nop 1\n\t"
                 "v_max_i32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t"
                 "v_max_i32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t"
                 "v_max_i32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t"
                 "v_max_i32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t"
                 "v_max_i32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\ts_nop 1\n\t"
                 "v_max_i32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf"
                 : "+v"(x));
    return x;
}

// Exclusive prefix sum of one int per thread over the 256-thread workgroup; *total gets the
// sum.  `wsum` is a 4-entry LDS array.
__device__ __forceinline__ int block_exclusive_scan(int v, int* wsum, int* total)
{
    const int inc = wave_incl_scan(v);
    __syncthreads();  // protects wsum from the previous use
    if (lane_id() == kWave - 1) wsum[threadIdx.x >> 6] = inc;
    __syncthreads();
    int base = 0;
    const int w = threadIdx.x >> 6;
    for (int i = 0; i < w; ++i) base += wsum[i];
    *total = wsum[0] + wsum[1] + wsum[2] + wsum[3];
    return base + inc - v;
}

__global__ __launch_bounds__(kThreads) void select_kernel(SelectArgs a)
{
    __shared__ int sbuf[kSelLdsCap];
    __shared__ int hist[256];
    __shared__ int wsum[4];
    __shared__ int sh_digit, sh_need;
    __shared__ int sel_idx[kSelSortCap];
    __shared__ int sel_key[kSelSortCap];

    const int b = blockIdx.x / a.Ho, ho = blockIdx.x % a.Ho;
    const int tid = threadIdx.x;
    const int len = a.lens[b];
    int n = len > 0 ? (len + a.BS - 1) / a.BS : 0;
    if (n > a.max_blocks) n = a.max_blocks;
    int32_t* oi = a.out_idx + ((int64_t)b * a.Ho + ho) * a.k;
    int32_t* os = a.out_score ? a.out_score + ((int64_t)b * a.Ho + ho) * a.k : nullptr;
    const int kk = a.k < n ? a.k : n;

    for (int i = kk + tid; i < a.k; i += kThreads) {
        oi[i] = -1;
        if (os) os[i] = 0;
    }
    if (n == 0) return;

    // stage the row (reduced over heads when asked) where every pass can re-read it
    const bool reduce = (a.flags & UCM_TOPK_REDUCE_HEADS) && a.Hkv > 1;
    const int32_t* row = a.scores + ((int64_t)b * a.Hkv + (reduce ? 0 : ho)) * a.max_blocks;
    const int* s;
    if (n <= kSelLdsCap) {
        for (int j = tid; j < n; j += kThreads) {
            int v = row[j];
            if (reduce)
                for (int h = 1; h < a.Hkv; ++h) {
                    const int o = row[(int64_t)h * a.max_blocks + j];
                    v = o > v ? o : v;
                }
            sbuf[j] = v;
        }
        s = sbuf;
    } else if (reduce) {
        int32_t* red = a.reduced + (int64_t)b * a.max_blocks;
        for (int j = tid; j < n; j += kThreads) {
            int v = row[j];
            for (int h = 1; h < a.Hkv; ++h) {
                const int o = row[(int64_t)h * a.max_blocks + j];
                v = o > v ? o : v;
            }
            red[j] = v;
        }
        __threadfence_block();
        s = red;
    } else {
        s = row;
    }
    __syncthreads();

    // ---- radix search for the kk-th largest key (key = score + 1 >= 0) ----
    uint32_t prefix = 0;  // decided high digits
    int need = kk;        // how many still to take among keys matching the prefix
    int shift = ((a.key_bits + 7) / 8) * 8;
    while (shift > 0) {
        shift -= 8;
        hist[tid] = 0;
        __syncthreads();
        for (int j = tid; j < n; j += kThreads) {
            const uint32_t key = (uint32_t)(s[j] + 1);
            if ((key >> (shift + 8)) == prefix) atomicAdd(&hist[(key >> shift) & 255], 1);
        }
        __syncthreads();
        if (tid < kWave) {
            // lane l owns digits 255-4l .. 252-4l (descending), so an inclusive scan over
            // lanes walks the digits from the largest down
            const int d0 = 255 - 4 * tid;
            const int c0 = hist[d0], c1 = hist[d0 - 1], c2 = hist[d0 - 2], c3 = hist[d0 - 3];
            const int mine = c0 + c1 + c2 + c3;
            const int inc = wave_incl_scan(mine);
            const int above = inc - mine;  // keys with a larger digit than any of mine
            if (above < need && need <= inc) {
                int acc = above, digit = d0, cnt = c0;
                if (acc + cnt < need) { acc += cnt; digit = d0 - 1; cnt = c1; }
                if (acc + cnt < need) { acc += cnt; digit = d0 - 2; cnt = c2; }
                if (acc + cnt < need) { acc += cnt; digit = d0 - 3; cnt = c3; }
                sh_digit = digit;
                sh_need = need - acc;
            }
        }
        __syncthreads();
        prefix = (prefix << 8) | (uint32_t)sh_digit;
        need = sh_need;
        __syncthreads();
    }
    const int thr = (int)prefix - 1;  // threshold score; `need` ties at thr are taken

    // ---- ordered compaction: thread t owns indices [t*E, (t+1)*E) ----
    const int E = (n + kThreads - 1) / kThreads;
    const int jb = tid * E;
    const int je = (jb + E < n) ? jb + E : n;
    int eq = 0, gt = 0;
    for (int j = jb; j < je; ++j) {
        const int v = s[j];
        eq += (v == thr);
        gt += (v > thr);
    }
    int tot;
    const int eq_before = block_exclusive_scan(eq, wsum, &tot);
    int eq_take = need - eq_before;
    eq_take = eq_take < 0 ? 0 : (eq_take > eq ? eq : eq_take);
    int pos = block_exclusive_scan(gt + eq_take, wsum, &tot);

    const bool score_order = (a.flags & UCM_TOPK_SCORE_ORDER) != 0;
    int eq_seen = 0;
    for (int j = jb; j < je; ++j) {
        const int v = s[j];
        bool take = v > thr;
        if (v == thr) {
            take = eq_seen < eq_take;
            ++eq_seen;
        }
        if (!take || pos >= a.k) continue;
        if (score_order) {
            sel_idx[pos] = j;
            sel_key[pos] = v;
        } else {
            oi[pos] = (a.flags & UCM_TOPK_RETURN_PHYSICAL)
                          ? (a.table ? a.table[(int64_t)b * a.table_stride + j]
                                     : b * a.max_blocks + j)
                          : j;
            if (os) os[pos] = (a.flags & UCM_TOPK_DISTANCE) ? a.full - v : v;
        }
        ++pos;
    }
    if (!score_order) return;

    // ---- score order: rank by counting among the kk winners (index order breaks ties;
    // sel_idx is ascending, so "earlier position" == "lower index") ----
    __syncthreads();
    for (int i = tid; i < kk; i += kThreads) {
        const int v = sel_key[i];
        int rank = 0;
        for (int m = 0; m < kk; ++m) {
            const int o = sel_key[m];
            rank += (o > v) || (o == v && m < i);
        }
        const int j = sel_idx[i];
        oi[rank] = (a.flags & UCM_TOPK_RETURN_PHYSICAL)
                       ? (a.table ? a.table[(int64_t)b * a.table_stride + j] : b * a.max_blocks + j)
                       : j;
        if (os) os[rank] = (a.flags & UCM_TOPK_DISTANCE) ? a.full - v : v;
    }
}

// ---------------------------------------------------------------------------------------
// Wave-level selection for rows of at most 64*EL block scores (index-ordered output only).
// One wave per (request, KV head) row, no LDS and no barriers: a binary search on the score
// value with ballot counts finds the k-th largest score, two wave prefix sums place the winners
// in ascending index order, ties to the lower index.  Same results as select_kernel.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ int wave_excl_scan(int v, int* total)
{
    const int inc = wave_incl_scan(v);
    *total = __builtin_amdgcn_readlane(inc, kWave - 1);
    return inc - v;
}

template <int EL>
__global__ __launch_bounds__(kThreads) void select_wave_kernel(SelectArgs a, int rows_total)
{
    // (a wave past the last row reads the last row and leaves below: with the exit up here the
    // kernel's arguments would be fetched in two rounds, the row count first)
    const int rowid_raw = blockIdx.x * (kThreads / kWave) + wave_id();
    const int rowid = rowid_raw < rows_total ? rowid_raw : rows_total - 1;
    const int b = rowid / a.Ho, ho = rowid % a.Ho;
    const int lane = lane_id();
    const int len = a.lens[b];
    // the row's scores go out before the length is known (in-range positions only, masked
    // below): one round trip to memory instead of two
    int raw[EL];
    {
        const bool red = (a.flags & UCM_TOPK_REDUCE_HEADS) && a.Hkv > 1;
        const int32_t* r0 = a.scores + (int64_t)b * a.Hkv * a.max_blocks + (int64_t)(red ? 0 : ho) * a.sc_h;
#pragma unroll
        for (int e = 0; e < EL; ++e) {
            const int j = lane * EL + e;
            raw[e] = r0[(int64_t)(j < a.max_blocks ? j : 0) * a.sc_j];
        }
    }
    // physical block ids of the whole row, fetched alongside the scores: the output loop then
    // has no load (and no round trip to memory) per selected element
    const bool physical = (a.flags & UCM_TOPK_RETURN_PHYSICAL) != 0;
    int tab[EL];
    if (physical && a.table) {
        const int32_t* t0 = a.table + (int64_t)b * a.table_stride;
#pragma unroll
        for (int e = 0; e < EL; ++e) {
            const int j = lane * EL + e;
            tab[e] = t0[j < a.max_blocks ? j : 0];
        }
    } else {
#pragma unroll
        for (int e = 0; e < EL; ++e) tab[e] = physical ? b * a.max_blocks + lane * EL + e : lane * EL + e;
    }
    if (rowid_raw >= rows_total) return;
    int n = len > 0 ? (len + a.BS - 1) / a.BS : 0;
    if (n > a.max_blocks) n = a.max_blocks;
    int32_t* oi = a.out_idx + ((int64_t)b * a.Ho + ho) * a.k;
    int32_t* os = a.out_score ? a.out_score + ((int64_t)b * a.Ho + ho) * a.k : nullptr;
    const int kk = a.k < n ? a.k : n;
    if (a.new_table) {
        if (plugin_row_prologue(a, b, len, kk, lane, kWave)) return;
        oi = a.new_table + (int64_t)b * a.new_table_stride;
        os = nullptr;
    } else {
        for (int i = kk + lane; i < a.k; i += kWave) {
            oi[i] = -1;
            if (os) os[i] = 0;
        }
        if (n == 0) return;
    }
    const bool reduce = (a.flags & UCM_TOPK_REDUCE_HEADS) && a.Hkv > 1;
    const int32_t* row = a.scores + (int64_t)b * a.Hkv * a.max_blocks + (int64_t)(reduce ? 0 : ho) * a.sc_h;
    int v[EL];
#pragma unroll
    for (int e = 0; e < EL; ++e) v[e] = raw[e];
    if (reduce) {
        // maximum over the KV heads, CH heads at a time with all of their loads in flight
        // (heads past the last re-read head 0, which changes nothing)
        constexpr int CH = EL <= 4 ? 8 : 2;
        for (int h0 = 1; h0 < a.Hkv; h0 += CH) {
            int o[CH][EL];
#pragma unroll
            for (int u = 0; u < CH; ++u) {
                const int hh = h0 + u < a.Hkv ? h0 + u : 0;
#pragma unroll
                for (int e = 0; e < EL; ++e) {
                    const int j = lane * EL + e;
                    o[u][e] = row[(int64_t)hh * a.sc_h + (int64_t)(j < a.max_blocks ? j : 0) * a.sc_j];
                }
            }
#pragma unroll
            for (int u = 0; u < CH; ++u)
#pragma unroll
                for (int e = 0; e < EL; ++e) v[e] = o[u][e] > v[e] ? o[u][e] : v[e];
        }
    }
#pragma unroll
    for (int e = 0; e < EL; ++e)
        if (lane * EL + e >= n) v[e] = -0x7fffffff;  // below every real score (>= -1): never selected
    auto count_ge = [&](int t) {
        int c = 0;
#pragma unroll
        for (int e = 0; e < EL; ++e) c += __popcll(__ballot(v[e] >= t));
        return c;
    };
    // the search runs between the row's smallest and largest score (count_ge(lo) >= kk always
    // holds: every one of the n >= kk real scores is >= the smallest)
    int lo = 0x7fffffff, hi = -0x7fffffff;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
        if (lane * EL + e < n) lo = v[e] < lo ? v[e] : lo;
        hi = v[e] > hi ? v[e] : hi;
    }
    lo = __builtin_amdgcn_readlane(wave_min_lane63(lo), 63);
    hi = __builtin_amdgcn_readlane(wave_max_lane63(hi), 63);
    while (lo < hi) {
        const int mid = lo + ((hi - lo + 1) >> 1);
        if (count_ge(mid) >= kk) lo = mid;
        else hi = mid - 1;
    }
    const int thr = lo;
    const int need = kk - count_ge(thr + 1);  // ties at thr to take, lowest indices first
    int eq = 0, gt = 0;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
        eq += (v[e] == thr);
        gt += (v[e] > thr);
    }
    int tot;
    const int eq_before = wave_excl_scan(eq, &tot);
    int eq_take = need - eq_before;
    eq_take = eq_take < 0 ? 0 : (eq_take > eq ? eq : eq_take);
    int pos = wave_excl_scan(gt + eq_take, &tot);
    int eq_seen = 0;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
        bool take = v[e] > thr;
        if (v[e] == thr) {
            take = eq_seen < eq_take;
            ++eq_seen;
        }
        if (take && pos < a.k) {
            oi[pos] = tab[e];
            if (os) os[pos] = (a.flags & UCM_TOPK_DISTANCE) ? a.full - v[e] : v[e];
            ++pos;
        }
    }
}

// Rows of 257 to 4096 block scores, index-ordered output: one workgroup per row, EL = 2 to 16
// scores per thread.  Same algorithm as select_wave_kernel<16>, but a wave there runs some 2000
// instructions back to back for its row (7 us, however few rows there are); here each wave has
// a quarter of the row and the four partial counts of a search step meet in LDS (two buffers
// in turn, one barrier per step).
template <int EL>
__global__ __launch_bounds__(kThreads) void select_group_kernel(SelectArgs a)
{
    constexpr int kWaves = kThreads / kWave;
    __shared__ int cnt[2][kWaves];
    __shared__ int ext[2][kWaves];
    __shared__ int wsum[kWaves];
    const int b = blockIdx.x / a.Ho, ho = blockIdx.x % a.Ho;
    const int tid = threadIdx.x, lane = lane_id(), wid = wave_id();
    const bool reduce = (a.flags & UCM_TOPK_REDUCE_HEADS) && a.Hkv > 1;
    const int32_t* row = a.scores + ((int64_t)b * a.Hkv + (reduce ? 0 : ho)) * a.max_blocks;
    const int len = a.lens[b];  // asked for with the scores: one round trip to memory
    int v[EL], tab[EL];
#pragma unroll
    for (int e = 0; e < EL; ++e) {
        const int j = tid * EL + e;
        v[e] = row[j < a.max_blocks ? j : 0];
    }
    const bool physical = (a.flags & UCM_TOPK_RETURN_PHYSICAL) != 0;
    if (physical && a.table) {
        const int32_t* t0 = a.table + (int64_t)b * a.table_stride;
#pragma unroll
        for (int e = 0; e < EL; ++e) {
            const int j = tid * EL + e;
            tab[e] = t0[j < a.max_blocks ? j : 0];
        }
    } else {
#pragma unroll
        for (int e = 0; e < EL; ++e) tab[e] = physical ? b * a.max_blocks + tid * EL + e : tid * EL + e;
    }
    int n = len > 0 ? (len + a.BS - 1) / a.BS : 0;
    if (n > a.max_blocks) n = a.max_blocks;
    int32_t* oi = a.out_idx + ((int64_t)b * a.Ho + ho) * a.k;
    int32_t* os = a.out_score ? a.out_score + ((int64_t)b * a.Ho + ho) * a.k : nullptr;
    const int kk = a.k < n ? a.k : n;
    if (a.new_table) {
        if (plugin_row_prologue(a, b, len, kk, tid, kThreads)) return;  // the same for every thread
        oi = a.new_table + (int64_t)b * a.new_table_stride;
        os = nullptr;
    } else {
        for (int i = kk + tid; i < a.k; i += kThreads) {
            oi[i] = -1;
            if (os) os[i] = 0;
        }
        if (n == 0) return;  // the same for every thread of the row
    }
    if (reduce) {
        for (int h0 = 1; h0 < a.Hkv; h0 += 8) {
            int o[8][EL];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int hh = h0 + u < a.Hkv ? h0 + u : 0;
#pragma unroll
                for (int e = 0; e < EL; ++e) {
                    const int j = tid * EL + e;
                    o[u][e] = row[(int64_t)hh * a.max_blocks + (j < a.max_blocks ? j : 0)];
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int e = 0; e < EL; ++e) v[e] = o[u][e] > v[e] ? o[u][e] : v[e];
        }
    }
    int lo = 0x7fffffff, hi = -0x7fffffff;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
        if (tid * EL + e >= n) v[e] = -0x7fffffff;  // below every real score (>= -1): never selected
        else lo = v[e] < lo ? v[e] : lo;
        hi = v[e] > hi ? v[e] : hi;
    }
    lo = wave_min_lane63(lo);
    hi = wave_max_lane63(hi);
    if (lane == kWave - 1) {
        ext[0][wid] = lo;
        ext[1][wid] = hi;
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        lo = ext[0][w] < lo ? ext[0][w] : lo;
        hi = ext[1][w] > hi ? ext[1][w] : hi;
    }
    lo = __builtin_amdgcn_readfirstlane(lo);
    hi = __builtin_amdgcn_readfirstlane(hi);
    // count of scores >= t over the whole row; `step` alternates the LDS buffer
    int step = 0;
    auto count_ge = [&](int t) {
        int c = 0;
#pragma unroll
        for (int e = 0; e < EL; ++e) c += __popcll(__ballot(v[e] >= t));
        int* buf = cnt[step & 1];
        ++step;
        if (lane == 0) buf[wid] = c;
        __syncthreads();
        return buf[0] + buf[1] + buf[2] + buf[3];
    };
    while (lo < hi) {  // count_ge(lo) >= kk always holds
        const int mid = lo + ((hi - lo + 1) >> 1);
        if (count_ge(mid) >= kk) lo = mid;
        else hi = mid - 1;
    }
    const int thr = lo;
    const int need = kk - count_ge(thr + 1);  // ties at thr to take, lowest indices first
    int eq = 0, gt = 0;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
        eq += (v[e] == thr);
        gt += (v[e] > thr);
    }
    int tot;
    const int eq_before = block_exclusive_scan(eq, wsum, &tot);
    int eq_take = need - eq_before;
    eq_take = eq_take < 0 ? 0 : (eq_take > eq ? eq : eq_take);
    int pos = block_exclusive_scan(gt + eq_take, wsum, &tot);
    int eq_seen = 0;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
        bool take = v[e] > thr;
        if (v[e] == thr) {
            take = eq_seen < eq_take;
            ++eq_seen;
        }
        if (take && pos < a.k) {
            oi[pos] = tab[e];
            if (os) os[pos] = (a.flags & UCM_TOPK_DISTANCE) ? a.full - v[e] : v[e];
            ++pos;
        }
    }
}

// ---------------------------------------------------------------------------------------
// Per-token scores in the reference scorer's output shape.
// ---------------------------------------------------------------------------------------
struct TokenArgs {
    ScoreArgs s;
    int max_seq_len, reduce_heads, out_is_f16;
    void* out;
};

// fp16 accumulation exactly as paged_ham_dist_mla.cu:204-210,235-241: the code is cut into
// 64-bit pieces when Wd is even (:384-387) and 32-bit pieces otherwise; each piece's
// group-summed popcount is converted to half and added in half precision, piece 0 first.
__global__ __launch_bounds__(kThreads) void token_score_kernel(TokenArgs t)
{
    extern __shared__ uint32_t dyn[];
    const ScoreArgs& a = t.s;
    uint32_t* qs = dyn;
    const int b = blockIdx.y;
    for (int i = threadIdx.x; i < a.Hq * a.Wd; i += kThreads)
        qs[i] = a.q[b * a.q_stride_b + (int64_t)(i / a.Wd) * a.q_stride_h + (i % a.Wd)];
    __syncthreads();
    const int p = blockIdx.x * kThreads + threadIdx.x;
    if (p >= t.max_seq_len) return;
    const int len = a.lens[b];
    const bool is_inf = p >= len;
    const bool keep = (p < a.sink) || (p >= len - a.recent && p < len);
    const int j = p / a.BS, tok = p % a.BS;
    const int Ho = t.reduce_heads ? 1 : a.Hkv;
    const int piece = (a.Wd % 2 == 0) ? 2 : 1;  // words per fp16 accumulation step

    int red_i = kInf;
    _Float16 red_h = (_Float16)__builtin_inff();
    for (int h = 0; h < a.Hkv; ++h) {
        int di = kInf;
        _Float16 dh = (_Float16)__builtin_inff();
        if (!is_inf) {
            if (keep) {
                di = 0;
                dh = (_Float16)0.0f;
            } else {
                const int64_t pb = (j < a.max_blocks) ? physical_block(a, b, j) : -1;
                if (pb >= 0) {
                    const uint32_t* kp = a.kc + pb * a.ks_block + tok * a.ks_token + h * a.ks_head;
                    di = 0;
                    dh = (_Float16)0.0f;
                    for (int w0 = 0; w0 < a.Wd; w0 += piece) {
                        int part = 0;
                        for (int w = w0; w < w0 + piece; ++w) {
                            const uint32_t kw = kp[w];
                            for (int g = 0; g < a.G; ++g)
                                part += __popc(kw ^ qs[(h * a.G + g) * a.Wd + w]);
                        }
                        di += part;
                        dh = dh + (_Float16)(float)part;
                    }
                }
            }
        }
        if (t.reduce_heads) {
            red_i = di < red_i ? di : red_i;
            red_h = dh < red_h ? dh : red_h;
        } else {
            const int64_t o = ((int64_t)b * Ho + h) * t.max_seq_len + p;
            if (t.out_is_f16) {
                uint16_t u;
                __builtin_memcpy(&u, &dh, 2);
                ((uint16_t*)t.out)[o] = u;
            } else {
                ((int32_t*)t.out)[o] = di;
            }
        }
    }
    if (t.reduce_heads) {
        const int64_t o = (int64_t)b * t.max_seq_len + p;
        if (t.out_is_f16) {
            uint16_t u;
            __builtin_memcpy(&u, &red_h, 2);
            ((uint16_t*)t.out)[o] = u;
        } else {
            ((int32_t*)t.out)[o] = red_i;
        }
    }
}

__global__ void update_seq_lens_kernel(const int32_t* lens, int B, int topk_tok, int BS,
                                       int32_t* out)
{
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= B) return;
    int over = lens[b] - topk_tok;
    over = over < 0 ? 0 : over;
    out[b] = lens[b] - ((over + BS - 1) / BS) * BS;
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

int planes_for_group(int G)
{
    int p = 0;
    while ((1 << p) <= G) ++p;  // bit width of G
    return p <= 4 ? 4 : 8;
}

struct Workspace {
    int32_t* scores;
    int32_t* reduced;
    uint32_t* planes;
    size_t bytes;
};

Workspace carve(void* base, int B, int Hkv, int max_blocks)
{
    Workspace w;
    size_t off = 0;
    w.scores = (int32_t*)((char*)base + off);
    off += align_up((size_t)B * Hkv * max_blocks * 4, 256);
    w.reduced = (int32_t*)((char*)base + off);
    off += align_up((size_t)B * max_blocks * 4, 256);
    w.planes = (uint32_t*)((char*)base + off);
    // worst case: 8 planes, widest code handled by a plane path (kMaxPlaneWords words)
    off += align_up((size_t)B * Hkv * 8 * kMaxPlaneWords * 4, 256);
    w.bytes = off;
    return w;
}

// Profiling hook: when set, the block-score launch carries these events as the kernel's own
// start/stop markers (timestamps of the dispatch itself, without the launch latency an event
// recorded on the stream would add).
thread_local unsigned long long* g_clock_probe = nullptr;  // see ucm_hamming_topk_set_clock_probe()
thread_local hipEvent_t g_prof_before = nullptr;
thread_local hipEvent_t g_prof_after = nullptr;

// Which kernels the last call on this thread launched (ucm_hamming_last_dispatch): a dispatch
// regression to a general kernel gives the same results and would otherwise only show as time.
struct DispatchNote {
    const char* planes;   // "plane_kernel" when the bit planes were built
    const char* score;    // scoring kernel family
    int sp[5];            // its template arguments, -1 = unused
    const char* select;   // selection kernel family
    int sel_el;
    int score_launches;   // scoring kernels launched (one, unless the dispatch is broken)
};
thread_local DispatchNote g_note = {nullptr, nullptr, {-1, -1, -1, -1, -1}, nullptr, -1, 0};

void note_reset() { g_note = DispatchNote{nullptr, nullptr, {-1, -1, -1, -1, -1}, nullptr, -1, 0}; }
void note_score(const char* family, int a = -1, int b = -1, int c = -1, int d = -1, int e = -1)
{
    g_note.score = family;
    g_note.sp[0] = a; g_note.sp[1] = b; g_note.sp[2] = c; g_note.sp[3] = d; g_note.sp[4] = e;
}
void note_select(const char* family, int el = -1)
{
    g_note.select = family;
    g_note.sel_el = el;
}

template <typename K, typename... Args>
void launch_score_threads(K kernel, dim3 grid, int threads, size_t lds, hipStream_t st, Args... args)
{
    ++g_note.score_launches;
    if (g_prof_before && g_prof_after)
        hipExtLaunchKernelGGL(kernel, grid, dim3(threads), lds, st, g_prof_before, g_prof_after, 0,
                              args...);
    else
        hipLaunchKernelGGL(kernel, grid, dim3(threads), lds, st, args...);
}

template <typename K, typename... Args>
void launch_score(K kernel, dim3 grid, size_t lds, hipStream_t st, Args... args)
{
    launch_score_threads(kernel, grid, kThreads, lds, st, args...);
}

template <int CPU, bool DIRECT, int GP>
void launch_fast(const ScoreArgs& a, int split, int u, dim3 grid, hipStream_t st)
{
    note_score("block_score_fast", CPU, DIRECT, GP, u >= 4 ? 4 : (u >= 2 ? 2 : 1));
    if (u >= 4)
        launch_score(block_score_fast<CPU, DIRECT, GP, 4>, grid, 0, st, a, split);
    else if (u >= 2)
        launch_score(block_score_fast<CPU, DIRECT, GP, 2>, grid, 0, st, a, split);
    else
        launch_score(block_score_fast<CPU, DIRECT, GP, 1>, grid, 0, st, a, split);
}

template <int CPU>
bool dispatch_fast(const ScoreArgs& a, int pmax, int split, int u, dim3 grid, hipStream_t st)
{
    if (a.G == 1) launch_fast<CPU, true, 1>(a, split, u, grid, st);
    else if (a.G == 2) launch_fast<CPU, true, 2>(a, split, u, grid, st);
    else if (a.G == 4) launch_fast<CPU, true, 4>(a, split, u, grid, st);
    else if (pmax == 4) launch_fast<CPU, false, 4>(a, split, u, grid, st);
    else launch_fast<CPU, false, 8>(a, split, u, grid, st);
    return true;
}

template <int CPU, int HKV, bool EXACT>
void dispatch_one_e(const ScoreArgs& a, int pmax, dim3 grid, hipStream_t st)
{
    // (measured at the config 2 shape with eight query heads per KV head, 31.2 us with the plane
    // kernel in front: the eight heads compared directly 42.3 us; the planes built by wave 0 of every
    // workgroup behind a barrier 31.3 us - what the plane kernel costs, the scorer then loses)
    const bool dir = a.G == 1 || a.G == 2 || a.G == 4;
    note_score("block_score_one", CPU, HKV, dir, dir ? a.G : (pmax <= 5 ? pmax : 8), EXACT);
    if (a.G == 1) launch_score(block_score_one<CPU, HKV, true, 1, EXACT>, grid, 0, st, a);
    else if (a.G == 2) launch_score(block_score_one<CPU, HKV, true, 2, EXACT>, grid, 0, st, a);
    else if (a.G == 4) launch_score(block_score_one<CPU, HKV, true, 4, EXACT>, grid, 0, st, a);
    else if (pmax == 4) launch_score(block_score_one<CPU, HKV, false, 4, EXACT>, grid, 0, st, a);
    else if (pmax == 5) launch_score(block_score_one<CPU, HKV, false, 5, EXACT>, grid, 0, st, a);
    else launch_score(block_score_one<CPU, HKV, false, 8, EXACT>, grid, 0, st, a);
}

template <int CPU, int HKV>
void dispatch_one_g(const ScoreArgs& a, int pmax, dim3 grid, hipStream_t st)
{
    if (((int64_t)a.BS * HKV * CPU) >> 8 == 4) dispatch_one_e<CPU, HKV, true>(a, pmax, grid, st);
    else dispatch_one_e<CPU, HKV, false>(a, pmax, grid, st);
}

template <int CPU, int HKV, int RPB>
void dispatch_small_g(const ScoreArgs& a, int pmax, dim3 grid, hipStream_t st)
{
    const bool dir = a.G == 1 || a.G == 2 || a.G == 4;
    note_score("block_score_small", CPU, HKV, dir, dir ? a.G : (pmax == 4 ? 4 : 8), RPB);
    if (a.G == 1) launch_score(block_score_small<CPU, HKV, true, 1, RPB>, grid, 0, st, a);
    else if (a.G == 2) launch_score(block_score_small<CPU, HKV, true, 2, RPB>, grid, 0, st, a);
    else if (a.G == 4) launch_score(block_score_small<CPU, HKV, true, 4, RPB>, grid, 0, st, a);
    else if (pmax == 4) launch_score(block_score_small<CPU, HKV, false, 4, RPB>, grid, 0, st, a);
    else launch_score(block_score_small<CPU, HKV, false, 8, RPB>, grid, 0, st, a);
}

// Blocks of 1 or 2 KiB with 1, 2 or 4 KV heads; false when no instance exists.
template <int CPU>
bool dispatch_small(const ScoreArgs& a, int rpb, int pmax, dim3 grid, hipStream_t st)
{
    if (rpb != 1 && rpb != 2) return false;
    switch (a.Hkv) {
        case 1: if (rpb == 1) dispatch_small_g<CPU, 1, 1>(a, pmax, grid, st); else dispatch_small_g<CPU, 1, 2>(a, pmax, grid, st); return true;
        case 2: if (rpb == 1) dispatch_small_g<CPU, 2, 1>(a, pmax, grid, st); else dispatch_small_g<CPU, 2, 2>(a, pmax, grid, st); return true;
        case 4: if (rpb == 1) dispatch_small_g<CPU, 4, 1>(a, pmax, grid, st); else dispatch_small_g<CPU, 4, 2>(a, pmax, grid, st); return true;
        default: return false;
    }
}

template <int CPU, int HKV, int RPB>
void dispatch_rows_g(const ScoreArgs& a, dim3 grid, hipStream_t st)
{
    note_score("block_score_rows", CPU, HKV, a.G, RPB);
    if (a.G == 1) launch_score(block_score_rows<CPU, HKV, 1, RPB>, grid, 0, st, a);
    else if (a.G == 2) launch_score(block_score_rows<CPU, HKV, 2, RPB>, grid, 0, st, a);
    else launch_score(block_score_rows<CPU, HKV, 4, RPB>, grid, 0, st, a);
}

template <int CPU, int HKV>
bool dispatch_rows_h(const ScoreArgs& a, int rpb, int B, hipStream_t st)
{
    const int nbw = rpb > 4 ? 1 : 4 / rpb;  // blocks per wave
    const dim3 grid((unsigned)ucm::ceil_div(a.max_blocks, 4 * nbw), (unsigned)B);
    switch (rpb) {
        case 1: dispatch_rows_g<CPU, HKV, 1>(a, grid, st); return true;
        case 2: dispatch_rows_g<CPU, HKV, 2>(a, grid, st); return true;
        case 4: dispatch_rows_g<CPU, HKV, 4>(a, grid, st); return true;
        case 8: dispatch_rows_g<CPU, HKV, 8>(a, grid, st); return true;
        default: return false;
    }
}

// Blocks of 1, 2, 4 or 8 KiB, group size 1, 2 or 4, 1 to 16 KV heads; false when no instance exists.
template <int CPU>
bool dispatch_rows(const ScoreArgs& a, int rpb, int B, hipStream_t st)
{
    if (!(a.G == 1 || a.G == 2 || a.G == 4)) return false;
    switch (a.Hkv) {
        case 1: return dispatch_rows_h<CPU, 1>(a, rpb, B, st);
        case 2: return dispatch_rows_h<CPU, 2>(a, rpb, B, st);
        case 4: return dispatch_rows_h<CPU, 4>(a, rpb, B, st);
        case 8: return dispatch_rows_h<CPU, 8>(a, rpb, B, st);
        case 16: if (CPU <= 4) return dispatch_rows_h<CPU, 16>(a, rpb, B, st); return false;
        default: return false;
    }
}

// true when a block_score_one instance exists for this (pieces per code, KV heads) pair
template <int CPU>
bool dispatch_one(const ScoreArgs& a, int pmax, dim3 grid, hipStream_t st)
{
    switch (a.Hkv) {
        case 1: dispatch_one_g<CPU, 1>(a, pmax, grid, st); return true;
        case 2: dispatch_one_g<CPU, 2>(a, pmax, grid, st); return true;
        case 4: dispatch_one_g<CPU, 4>(a, pmax, grid, st); return true;
        case 8: dispatch_one_g<CPU, 8>(a, pmax, grid, st); return true;
        case 16: if (CPU <= 4) { dispatch_one_g<CPU, 16>(a, pmax, grid, st); return true; } return false;
        default: return false;
    }
}

bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

// Blocks of 128, 256 or 512 bytes in the layout of the 16-byte-piece kernels, query codes
// compared directly.
bool tiny_layout(const ScoreArgs& a, const uint32_t* k_cache, bool direct)
{
    const int cpu = a.Wd / 4;
    if (!direct || a.Wd % 4 || !(cpu == 1 || cpu == 2 || cpu == 4)) return false;
    const int64_t pieces = (int64_t)a.BS * a.Hkv * cpu;
    return a.ks_head == a.Wd && a.ks_token == (int64_t)a.Hkv * a.Wd && a.ks_block % 4 == 0 &&
           (reinterpret_cast<uintptr_t>(k_cache) & 15) == 0 && is_pow2(a.Hkv * cpu) &&
           is_pow2((int)pieces) && pieces >= 8 && pieces < kWave && a.Hkv * cpu <= pieces;
}

template <int CPU>
void launch_tiny(const ScoreArgs& a, int bshift, dim3 grid, hipStream_t st)
{
    note_score("block_score_tiny", CPU, a.G == 1 || a.G == 2 ? a.G : 4);
    if (a.G == 1) launch_score(block_score_tiny<CPU, 1>, grid, 0, st, a, bshift);
    else if (a.G == 2) launch_score(block_score_tiny<CPU, 2>, grid, 0, st, a, bshift);
    else launch_score(block_score_tiny<CPU, 4>, grid, 0, st, a, bshift);
}

// Layout and shapes the code-per-lane kernels take (on top of pairs_layout): 18-word codes
// with any group size, 8- and 16-word codes with bit planes (directly compared codes of those
// widths have the 16-byte-piece kernels).
bool lanes_layout(const ScoreArgs& a, const uint32_t* k_cache, bool direct)
{
    const bool width = a.Wd == 18 || (!direct && (a.Wd == 16 || a.Wd == 8));
    return width && a.BS % 64 == 0 && a.ks_block % 4 == 0 &&
           (reinterpret_cast<uintptr_t>(k_cache) & 15) == 0;
}

template <int LC>
void launch_lanes_run(const ScoreArgs& a, int pmax, dim3 grid, hipStream_t st)
{
    switch (pmax) {
        case 4: launch_score(block_score_lanes_run<LC, 4>, grid, 0, st, a); break;
        case 5: launch_score(block_score_lanes_run<LC, 5>, grid, 0, st, a); break;
        case 6: launch_score(block_score_lanes_run<LC, 6>, grid, 0, st, a); break;
        case 7: launch_score(block_score_lanes_run<LC, 7>, grid, 0, st, a); break;
        default: launch_score(block_score_lanes_run<LC, 8>, grid, 0, st, a); break;
    }
}

template <int LC>
void dispatch_lanes(const ScoreArgs& a, int pmax, dim3 grid, hipStream_t st)
{
    const bool dir = LC == 9 && (a.G == 1 || a.G == 2 || a.G == 4);
    note_score("block_score_lanes", LC, dir, dir ? a.G : (pmax < 4 ? 4 : (pmax > 8 ? 8 : pmax)));
    if (LC == 9 && a.G == 1) launch_score(block_score_lanes<9, true, 1>, grid, 0, st, a);
    else if (LC == 9 && a.G == 2) launch_score(block_score_lanes<9, true, 2>, grid, 0, st, a);
    else if (LC == 9 && a.G == 4) launch_score(block_score_lanes<9, true, 4>, grid, 0, st, a);
    else if (pmax == 4) launch_score(block_score_lanes<LC, false, 4>, grid, 0, st, a);
    else if (pmax == 5) launch_score(block_score_lanes<LC, false, 5>, grid, 0, st, a);
    else if (pmax == 6) launch_score(block_score_lanes<LC, false, 6>, grid, 0, st, a);
    else if (pmax == 7) launch_score(block_score_lanes<LC, false, 7>, grid, 0, st, a);
    else launch_score(block_score_lanes<LC, false, 8>, grid, 0, st, a);
}

// Layout the 8-byte-piece kernels take: one KV head, an even code width of at most
// kMaxPlaneWords words, the tokens of a block back to back, 8-byte aligned blocks.
bool pairs_layout(const ScoreArgs& a, const uint32_t* k_cache)
{
    return a.Hkv == 1 && a.Wd % 2 == 0 && a.Wd <= kMaxPlaneWords && a.ks_token == a.Wd &&
           a.ks_block % 2 == 0 && (reinterpret_cast<uintptr_t>(k_cache) & 7) == 0;
}

int common_checks(const uint32_t* q, const uint32_t* kc, const int32_t* lens, int64_t NB, int BS,
                  int Hkv, int Wd, int B, int Hq, int max_blocks)
{
    UCM_REQUIRE(q && kc && lens, "null input pointer");
    UCM_REQUIRE(B >= 0 && B <= 65535, "batch %d out of range [0, 65535]", B);
    UCM_REQUIRE(NB > 0 && BS > 0 && Hkv > 0 && Wd > 0 && Hq > 0, "non-positive shape");
    UCM_REQUIRE(Hq % Hkv == 0, "query heads %d not a multiple of KV heads %d", Hq, Hkv);
    UCM_REQUIRE(Hq / Hkv <= 255, "group size %d above 255", Hq / Hkv);
    UCM_REQUIRE(max_blocks > 0, "max_blocks must be positive");
    UCM_REQUIRE((int64_t)max_blocks * BS <= INT32_MAX, "max_blocks * BS overflows int32");
    UCM_REQUIRE((int64_t)Hq * Wd * 4 <= 48 * 1024, "query codes of one request exceed 48 KiB");
    return UCM_OK;
}

}  // namespace

extern "C" size_t ucm_hamming_topk_workspace_bytes(int32_t B, int32_t Hkv, int32_t max_blocks)
{
    if (B <= 0 || Hkv <= 0 || max_blocks <= 0) return 256;
    return carve(nullptr, B, Hkv, max_blocks).bytes;
}

namespace {

// Outputs of a decode step in the form the serving engine's attention reads them (see
// SelectArgs): replaces out_idx / out_score when given.
struct StepOut {
    int32_t* new_table;
    int32_t new_table_stride;
    int32_t* new_lens;
    int32_t thr_len, topk_tok;
};

int hamming_topk_run(const uint32_t* q_codes, int64_t q_stride_b, int64_t q_stride_h,
                     const uint32_t* k_cache, int64_t NB, int32_t BS, int32_t Hkv, int32_t Wd,
                     int64_t ks_block, int64_t ks_token, int64_t ks_head, const int32_t* block_table,
                     int32_t table_stride, int32_t max_blocks, const int32_t* seq_lens, int32_t B,
                     int32_t Hq, int32_t k, int32_t sink_tok, int32_t recent_tok, uint32_t flags,
                     int32_t* out_idx, int32_t* out_score, void* workspace, size_t workspace_bytes,
                     ucm_stream_t stream, const StepOut* step_out)
{
    note_reset();
    int rc = common_checks(q_codes, k_cache, seq_lens, NB, BS, Hkv, Wd, B, Hq, max_blocks);
    if (rc != UCM_OK) return rc;
    if (step_out) {
        UCM_REQUIRE(step_out->new_table && step_out->new_lens && block_table, "null table or length output");
        UCM_REQUIRE(step_out->new_table_stride >= max_blocks, "new table rows of %d entries for %d blocks",
                    step_out->new_table_stride, max_blocks);
        UCM_REQUIRE((flags & UCM_TOPK_RETURN_PHYSICAL) && !(flags & UCM_TOPK_SCORE_ORDER) &&
                        ((flags & UCM_TOPK_REDUCE_HEADS) || Hkv == 1),
                    "a replacement table is one list of physical ids per request");
        if (max_blocks > 4096)
            return ucm::fail(UCM_EUNSUPPORTED, "replacement tables support at most 4096 blocks per request");
    } else {
        UCM_REQUIRE(out_idx, "out_idx is null");
    }
    UCM_REQUIRE(k > 0, "k must be positive");
    UCM_REQUIRE(!block_table || table_stride >= max_blocks, "table_stride %d < max_blocks %d",
                table_stride, max_blocks);
    UCM_REQUIRE(sink_tok >= 0 && recent_tok >= 0, "negative sink/recent");
    UCM_REQUIRE(Hkv <= kMaxTileHeads, "more than %d KV heads", kMaxTileHeads);
    if ((flags & UCM_TOPK_SCORE_ORDER) && k > kSelSortCap)
        return ucm::fail(UCM_EUNSUPPORTED, "score-ordered output supports k <= %d", kSelSortCap);
    if (B == 0) return UCM_OK;
    const Workspace ws = carve(workspace, B, Hkv, max_blocks);
    UCM_REQUIRE(workspace && workspace_bytes >= ws.bytes, "workspace too small: %zu < %zu",
                workspace_bytes, ws.bytes);
    UCM_REQUIRE(((uintptr_t)workspace & 15) == 0, "workspace not 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;

    ScoreArgs a;
    a.q = q_codes; a.q_stride_b = q_stride_b; a.q_stride_h = q_stride_h;
    a.kc = k_cache; a.NB = NB; a.BS = BS; a.Hkv = Hkv; a.Wd = Wd;
    a.ks_block = ks_block; a.ks_token = ks_token; a.ks_head = ks_head;
    a.table = block_table; a.table_stride = table_stride; a.max_blocks = max_blocks;
    a.lens = seq_lens; a.B = B; a.Hq = Hq; a.G = Hq / Hkv; a.sink = sink_tok;
    a.recent = recent_tok; a.planes = ws.planes; a.scores = ws.scores; a.reduce_out = 0;
    a.sc_h = max_blocks; a.sc_j = 1; a.clock_probe = g_clock_probe;
    // the wave-per-row selection (same test as at its launch below) reads either layout
    const bool wave_select = !(flags & UCM_TOPK_SCORE_ORDER) && max_blocks <= 256;
    bool reduced_scores = false;  // the score kernel already took the maximum over the heads

    // fast path eligibility
    const int cpu = Wd / 4;
    const bool fast = (Wd % 4 == 0) && (cpu == 1 || cpu == 2 || cpu == 4) && ks_head == Wd &&
                      ks_token == (int64_t)Hkv * Wd && (ks_block % 4 == 0) &&
                      (((uintptr_t)k_cache & 15) == 0) && is_pow2(Hkv * cpu) &&
                      Hkv * cpu <= 64 && ((int64_t)BS * Hkv * cpu) % 64 == 0;
    const int64_t block_bytes = (int64_t)BS * Hkv * Wd * 4;
    int TB = (int)(16384 / block_bytes);
    if (TB < 1) TB = 1;
    while (TB > 1 && TB * Hkv > kMaxTileHeads) TB >>= 1;
    // keep at least ~8 workgroups per CU in flight when the problem allows it
    while (TB > 1 && (int64_t)B * ucm::ceil_div(max_blocks, TB) < 2048) TB >>= 1;
    if (TB > kMaxTile) TB = kMaxTile;
    while (TB > 1 && TB * Hkv > kMaxTileHeads) TB >>= 1;
    a.TB = TB;
    const dim3 grid((unsigned)ucm::ceil_div(max_blocks, TB), (unsigned)B);

    // one KV head, 16-word codes and bit planes: a wave per block of 8-byte pieces beats a
    // workgroup per 4 KiB block of 16-byte pieces (37 against 68 us at 16 x 65,536 tokens)
    const bool direct_g = a.G == 1 || a.G == 2 || a.G == 4;
    const bool one_head_planes = Hkv == 1 && !direct_g && pairs_layout(a, k_cache) &&
                                 (Wd >= 16 || lanes_layout(a, k_cache, false));
    if (fast && !one_head_planes) {
        int pmax = planes_for_group(a.G);
        const bool direct = a.G == 1 || a.G == 2 || a.G == 4;
        {
            // 16 to 31 query heads per KV head need five planes, not eight; the one-block-per-workgroup
            // kernel has that variant (config 2 shape with 128 query heads: 46.7 us with eight planes)
            const int rpb0 = (int)(((int64_t)BS * Hkv * cpu) >> 6);
            const bool to_one = rpb0 >= 4 && rpb0 % 4 == 0 &&
                                (Hkv == 1 || Hkv == 2 || Hkv == 4 || Hkv == 8 || (Hkv == 16 && cpu <= 4));
            if (!direct && to_one && a.G >= 16 && a.G < 32) pmax = 5;
        }
        if (!direct) {
            g_note.planes = "plane_kernel";
            hipLaunchKernelGGL(plane_kernel, dim3(B * Hkv * ((Wd + 1) / 2)), dim3(kThreads), 0, st, q_codes,
                               q_stride_b, q_stride_h, Hkv, a.G, Wd, pmax, ws.planes);
            rc = ucm::launch_status("plane_kernel");
            if (rc != UCM_OK) return rc;
        }
        const int rpb = (int)(((int64_t)BS * Hkv * cpu) >> 6);
        const int split = (rpb >= 4 && rpb % 4 == 0) ? 1 : 0;
        const int rpw = split ? rpb / 4 : rpb;
        const int u = rpw;
        // blocks of >= 4 KiB: one block per workgroup with the head count compiled in
        bool done = false;
        // blocks of at most 8 KiB with directly compared query codes: whole blocks per wave
        if (direct && rpb <= 8) {
            a.reduce_out = ((flags & UCM_TOPK_REDUCE_HEADS) && Hkv > 1) ? 1 : 0;
            if (cpu == 1) done = dispatch_rows<1>(a, rpb, B, st);
            else if (cpu == 2) done = dispatch_rows<2>(a, rpb, B, st);
            else done = dispatch_rows<4>(a, rpb, B, st);
            reduced_scores = done && a.reduce_out;
            a.reduce_out = 0;
        }
        if (!done && split && Hkv <= 16) {
            a.TB = 1;
            a.reduce_out = ((flags & UCM_TOPK_REDUCE_HEADS) && Hkv > 1) ? 1 : 0;
            if (wave_select && !a.reduce_out && Hkv > 1) {
                a.sc_h = 1;
                a.sc_j = Hkv;
            }
            const dim3 grid1((unsigned)max_blocks, (unsigned)B);
            if (cpu == 1) done = dispatch_one<1>(a, pmax, grid1, st);
            else if (cpu == 2) done = dispatch_one<2>(a, pmax, grid1, st);
            else done = dispatch_one<4>(a, pmax, grid1, st);
            reduced_scores = done && a.reduce_out;
            a.reduce_out = 0;
            if (!done) {
                a.sc_h = max_blocks;
                a.sc_j = 1;
            }
        }
        if (!done) a.TB = TB;
        if (!done && !split) {
            // 16 blocks per workgroup: every wave gets two rounds of 4 loads
            int tbs = 16;
            if (tbs > kMaxTile) tbs = kMaxTile;
            while (tbs > 1 && tbs * Hkv > kMaxTileHeads) tbs >>= 1;
            a.TB = tbs;
            const dim3 grids((unsigned)ucm::ceil_div(max_blocks, tbs), (unsigned)B);
            if (cpu == 1) done = dispatch_small<1>(a, rpb, pmax, grids, st);
            else if (cpu == 2) done = dispatch_small<2>(a, rpb, pmax, grids, st);
            else done = dispatch_small<4>(a, rpb, pmax, grids, st);
            if (!done) a.TB = TB;
        }
        if (!done) {
            if (cpu == 1) dispatch_fast<1>(a, pmax, split, u, grid, st);
            else if (cpu == 2) dispatch_fast<2>(a, pmax, split, u, grid, st);
            else dispatch_fast<4>(a, pmax, split, u, grid, st);
        }
    } else if (tiny_layout(a, k_cache, direct_g)) {
        // blocks below 1 KiB with directly compared query codes: several blocks per run of 64 pieces
        const int pieces = BS * Hkv * cpu;
        int bshift = 0;
        while ((pieces << bshift) < kWave) ++bshift;
        a.reduce_out = ((flags & UCM_TOPK_REDUCE_HEADS) && Hkv > 1) ? 1 : 0;
        reduced_scores = a.reduce_out != 0;
        const dim3 tgrid((unsigned)ucm::ceil_div(max_blocks, (kThreads / kWave) * (4 << bshift)), (unsigned)B);
        if (cpu == 1) launch_tiny<1>(a, bshift, tgrid, st);
        else if (cpu == 2) launch_tiny<2>(a, bshift, tgrid, st);
        else launch_tiny<4>(a, bshift, tgrid, st);
        a.reduce_out = 0;
    } else if (pairs_layout(a, k_cache)) {
        const int L = Wd / 2, TP = kWave / L;
        int pmax = 0;
        while ((1 << pmax) <= a.G) ++pmax;  // bit planes that hold the counts 0..G
        if (pmax < 4) pmax = 4;
        const bool direct = a.G == 1 || a.G == 2 || a.G == 4;
        // 64-token blocks of 8-word codes: the scorer builds its weights (per-bit counts) itself
        const bool planes_inside = !direct && Wd == 8 && BS == 64 && pmax <= 8 && lanes_layout(a, k_cache, direct);
        // the other code-per-lane shapes build them in wave 0 of every workgroup (up to 128 query heads)
        const bool planes_in_lanes = !direct && !planes_inside && a.G <= 128 && BS == 64 && (Wd == 16 || Wd == 18) &&
                                     lanes_layout(a, k_cache, direct);
        if (!direct && !planes_inside && !planes_in_lanes) {
            g_note.planes = "plane_kernel";
            hipLaunchKernelGGL(plane_kernel, dim3(B * ((Wd + 1) / 2)), dim3(kThreads), 0, st, q_codes,
                               q_stride_b, q_stride_h, 1, a.G, Wd, pmax, ws.planes);
            rc = ucm::launch_status("plane_kernel");
            if (rc != UCM_OK) return rc;
        }
        const dim3 pgrid((unsigned)ucm::ceil_div(max_blocks, kThreads / kWave), (unsigned)B);
        // 18-word codes (and 8- or 16-word codes with bit planes) in blocks of 64, 128, ...
        // tokens: a whole code per lane
        if (planes_inside && a.G >= 16 && a.G <= 128) {
            // the weighted bit sums on the matrix unit, as for 18-word codes
            note_score("block_score_strip8");
            const dim3 g64((unsigned)ucm::ceil_div(max_blocks, kStripWaves * strip_run(8)), (unsigned)B);
            launch_score_threads(block_score_strip<8>, g64, kStripWaves * kWave, 0, st, a);
        } else if (planes_inside) {
            // one nibble digit of the per-bit counts up to 15 query heads, two up to 255
            const int nd = a.G <= 15 ? 1 : 2;
            note_score("block_score_dot64", nd);
            const dim3 g64((unsigned)ucm::ceil_div(max_blocks, kDotWaves * kDotRun), (unsigned)B);
            ++g_note.score_launches;
            const dim3 threads(kDotWaves * kWave);
            if (g_prof_before && g_prof_after) {
                if (nd == 1) hipExtLaunchKernelGGL(block_score_dot64<1>, g64, threads, 0, st, g_prof_before, g_prof_after, 0, a);
                else hipExtLaunchKernelGGL(block_score_dot64<2>, g64, threads, 0, st, g_prof_before, g_prof_after, 0, a);
            } else {
                if (nd == 1) hipLaunchKernelGGL(block_score_dot64<1>, g64, threads, 0, st, a);
                else hipLaunchKernelGGL(block_score_dot64<2>, g64, threads, 0, st, a);
            }
        } else if (planes_in_lanes && Wd == 18) {
            note_score("block_score_strip18");
            const dim3 g64((unsigned)ucm::ceil_div(max_blocks, kStripWaves * kStripRun), (unsigned)B);
            launch_score_threads(block_score_strip<18>, g64, kStripWaves * kWave, 0, st, a);
        } else if (planes_in_lanes) {
            note_score("block_score_lanes_run", Wd / 2, pmax);
            const dim3 g64((unsigned)ucm::ceil_div(max_blocks, (kThreads / kWave) * kLanesRunBlocks), (unsigned)B);
            launch_lanes_run<8>(a, pmax, g64, st);  // 16-word codes
        } else if (lanes_layout(a, k_cache, direct)) {
            if (Wd == 18) dispatch_lanes<9>(a, pmax, pgrid, st);
            else if (Wd == 16) dispatch_lanes<8>(a, pmax, pgrid, st);
            else dispatch_lanes<4>(a, pmax, pgrid, st);
        } else {
            note_score("block_score_pairs", direct, direct ? a.G : (pmax > 8 ? 8 : pmax));
            if (a.G == 1) launch_score(block_score_pairs<true, 1>, pgrid, 0, st, a, L, TP);
            else if (a.G == 2) launch_score(block_score_pairs<true, 2>, pgrid, 0, st, a, L, TP);
            else if (a.G == 4) launch_score(block_score_pairs<true, 4>, pgrid, 0, st, a, L, TP);
            else if (pmax == 4) launch_score(block_score_pairs<false, 4>, pgrid, 0, st, a, L, TP);
            else if (pmax == 5) launch_score(block_score_pairs<false, 5>, pgrid, 0, st, a, L, TP);
            else if (pmax == 6) launch_score(block_score_pairs<false, 6>, pgrid, 0, st, a, L, TP);
            else if (pmax == 7) launch_score(block_score_pairs<false, 7>, pgrid, 0, st, a, L, TP);
            else launch_score(block_score_pairs<false, 8>, pgrid, 0, st, a, L, TP);
        }
    } else {
        note_score("block_score_generic");
        launch_score(block_score_generic, grid, (size_t)Hq * Wd * 4, st, a);
    }
    rc = ucm::launch_status("block_score");
    if (rc != UCM_OK) return rc;

    SelectArgs s;
    s.scores = ws.scores; s.sc_h = a.sc_h; s.sc_j = a.sc_j; s.reduced = ws.reduced; s.table = block_table;
    s.table_stride = table_stride; s.max_blocks = max_blocks; s.lens = seq_lens; s.BS = BS;
    s.Hkv = reduced_scores ? 1 : Hkv; s.Ho = (flags & UCM_TOPK_REDUCE_HEADS) ? 1 : Hkv; s.k = k;
    s.full = a.G * 32 * Wd;
    s.key_bits = 1;
    while ((1ll << s.key_bits) <= (int64_t)s.full + 1) ++s.key_bits;
    s.flags = flags; s.out_idx = out_idx; s.out_score = out_score;
    s.new_table = step_out ? step_out->new_table : nullptr;
    s.new_table_stride = step_out ? step_out->new_table_stride : 0;
    s.new_lens = step_out ? step_out->new_lens : nullptr;
    s.thr_len = step_out ? step_out->thr_len : 0;
    s.topk_tok = step_out ? step_out->topk_tok : 0;
    const int rows_total = B * s.Ho;
    const dim3 wgrid((unsigned)ucm::ceil_div(rows_total, kThreads / kWave));
    if (!(flags & UCM_TOPK_SCORE_ORDER) && max_blocks <= 256) {
        // up to 256 blocks a wave per row stays ahead of a workgroup per row (config 2 step:
        // 32.7 against 33.3 us)
        note_select("select_wave_kernel", 4);
        hipLaunchKernelGGL(select_wave_kernel<4>, wgrid, dim3(kThreads), 0, st, s, rows_total);
        return ucm::launch_status("select_wave_kernel");
    }
    if (!(flags & UCM_TOPK_SCORE_ORDER) && max_blocks <= 4096) {
        const dim3 rgrid((unsigned)rows_total);
        note_select("select_group_kernel", max_blocks <= 512 ? 2 : (max_blocks <= 1024 ? 4 : (max_blocks <= 2048 ? 8 : 16)));
        if (max_blocks <= 512)
            hipLaunchKernelGGL(select_group_kernel<2>, rgrid, dim3(kThreads), 0, st, s);
        else if (max_blocks <= 1024)
            hipLaunchKernelGGL(select_group_kernel<4>, rgrid, dim3(kThreads), 0, st, s);
        else if (max_blocks <= 2048)
            hipLaunchKernelGGL(select_group_kernel<8>, rgrid, dim3(kThreads), 0, st, s);
        else
            hipLaunchKernelGGL(select_group_kernel<16>, rgrid, dim3(kThreads), 0, st, s);
        return ucm::launch_status("select_group_kernel");
    }
    note_select("select_kernel");
    hipLaunchKernelGGL(select_kernel, dim3(B * s.Ho), dim3(kThreads), 0, st, s);
    return ucm::launch_status("select_kernel");
}

}  // namespace

extern "C" int ucm_hamming_topk(const uint32_t* q_codes, int64_t q_stride_b, int64_t q_stride_h,
                                const uint32_t* k_cache, int64_t NB, int32_t BS, int32_t Hkv,
                                int32_t Wd, int64_t ks_block, int64_t ks_token, int64_t ks_head,
                                const int32_t* block_table, int32_t table_stride,
                                int32_t max_blocks, const int32_t* seq_lens, int32_t B,
                                int32_t Hq, int32_t k, int32_t sink_tok, int32_t recent_tok,
                                uint32_t flags, int32_t* out_idx, int32_t* out_score,
                                void* workspace, size_t workspace_bytes, ucm_stream_t stream)
{
    ucm::clear_error();
    return hamming_topk_run(q_codes, q_stride_b, q_stride_h, k_cache, NB, BS, Hkv, Wd, ks_block, ks_token,
                            ks_head, block_table, table_stride, max_blocks, seq_lens, B, Hq, k, sink_tok,
                            recent_tok, flags, out_idx, out_score, workspace, workspace_bytes, stream,
                            nullptr);
}

/* One GQA decode step as the reference's plugin performs it, see ucm_hip.h. */
extern "C" int ucm_gsa_decode_step(const void* new_keys, int64_t T, int64_t k_stride_t, int64_t k_stride_h,
                                   const void* slot_mapping, int slot_is_i64, const void* queries,
                                   int64_t q_stride_b, int64_t q_stride_h, int x_dtype, int32_t K,
                                   const void* w, int w_dtype, int32_t n_w, int32_t N_bits,
                                   uint32_t* k_cache, int64_t NB, int32_t BS, int32_t Hkv,
                                   int64_t ks_block, int64_t ks_token, int64_t ks_head,
                                   const int32_t* block_table, int32_t table_stride, int32_t max_blocks,
                                   const int32_t* seq_lens, int32_t B, int32_t Hq, int32_t topk_tok,
                                   int32_t sink_tok, int32_t recent_tok, int32_t seq_len_threshold,
                                   uint32_t* q_codes, int32_t* new_block_table, int32_t new_table_stride,
                                   int32_t* new_seq_lens, void* workspace, size_t workspace_bytes,
                                   ucm_stream_t stream)
{
    ucm::clear_error();
    UCM_REQUIRE(Hkv > 0 && Hq > 0 && Hq % Hkv == 0, "bad head counts");
    UCM_REQUIRE(N_bits > 0 && N_bits % 32 == 0, "hash_bits must be a multiple of 32");
    UCM_REQUIRE(n_w == 1 || n_w == Hkv, "n_w must be 1 or the number of KV heads");
    UCM_REQUIRE(q_codes, "q_codes is null");
    // the reference's own checks (hamming_topk.py:30-31)
    UCM_REQUIRE(BS > 0 && topk_tok > 0 && topk_tok % BS == 0, "topk_token %d is no multiple of the block size %d",
                topk_tok, BS);
    UCM_REQUIRE(recent_tok > 0 && topk_tok > sink_tok + recent_tok, "topk_token must exceed sink + recent > 0");
    const int32_t Wd = N_bits / 32;
    ucm::PairSpec spec{new_keys, T, Hkv, k_stride_t, k_stride_h, slot_mapping, slot_is_i64,
                       k_cache, NB, BS, ks_block, ks_token, ks_head, queries, B, Hq,
                       q_stride_b, q_stride_h, q_codes, (int64_t)Hkv * Wd, Wd, x_dtype, K, w,
                       w_dtype, n_w, N_bits};
    spec.q_group_mean = 1;
    int rc = ucm::encode_pair(spec, (hipStream_t)stream);
    if (rc != UCM_OK) return rc;
    const StepOut so{new_block_table, new_table_stride, new_seq_lens, seq_len_threshold, topk_tok};
    return hamming_topk_run(q_codes, (int64_t)Hkv * Wd, Wd, k_cache, NB, BS, Hkv, Wd, ks_block, ks_token,
                            ks_head, block_table, table_stride, max_blocks, seq_lens, B, Hkv, topk_tok / BS,
                            sink_tok, recent_tok, UCM_TOPK_REDUCE_HEADS | UCM_TOPK_RETURN_PHYSICAL, nullptr,
                            nullptr, workspace, workspace_bytes, stream, &so);
}

// ---------------------------------------------------------------------------------------
// ucm_hamming_topk_static: the same operator for callers that cannot allocate.  Its block
// scores, head-reduced rows and bit planes live in a fixed device array instead of a caller's
// workspace.  The array's name is only a host-side handle: each GPU holds its own copy, whose
// address is resolved once per device and passed to the kernels like any workspace.
// ---------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[UCM_TOPK_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {nullptr};

// Device address of `scratch` on the calling thread's current device.
int static_scratch(void** out)
{
    int dev = -1;
    UCM_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return ucm::fail(UCM_EUNSUPPORTED, "device %d out of range", dev);
    std::lock_guard<std::mutex> g(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return ucm::hip_fail(e, "hipGetSymbolAddress(scratch)");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return UCM_OK;
}
}  // namespace

extern "C" int ucm_hamming_topk_static(const uint32_t* q_codes, int64_t q_stride_b, int64_t q_stride_h,
                                       const uint32_t* k_cache, int64_t NB, int32_t BS, int32_t Hkv,
                                       int32_t Wd, int64_t ks_block, int64_t ks_token, int64_t ks_head,
                                       const int32_t* block_table, int32_t table_stride,
                                       int32_t max_blocks, const int32_t* seq_lens, int32_t B,
                                       int32_t Hq, int32_t k, int32_t sink_tok, int32_t recent_tok,
                                       uint32_t flags, int32_t* out_idx, int32_t* out_score,
                                       ucm_stream_t stream)
{
    ucm::clear_error();
    UCM_REQUIRE(B >= 0 && Hkv > 0 && max_blocks > 0, "non-positive shape");
    const size_t need = B > 0 ? carve(nullptr, B, Hkv, max_blocks).bytes : 0;
    if (need > (size_t)UCM_TOPK_STATIC_SCRATCH_BYTES)
        return ucm::fail(UCM_EPARAM,
                         "B=%d x Hkv=%d x max_blocks=%d needs %zu bytes of scratch, the static "
                         "entry point holds %zu: use ucm_hamming_topk with a workspace",
                         B, Hkv, max_blocks, need, (size_t)UCM_TOPK_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc != UCM_OK) return rc;
    // Nothing in the scratch has to start at zero: every kernel writes the cells it later reads.
    return ucm_hamming_topk(q_codes, q_stride_b, q_stride_h, k_cache, NB, BS, Hkv, Wd, ks_block, ks_token,
                            ks_head, block_table, table_stride, max_blocks, seq_lens, B, Hq, k, sink_tok,
                            recent_tok, flags, out_idx, out_score, ws, (size_t)UCM_TOPK_STATIC_SCRATCH_BYTES,
                            stream);
}

extern "C" int ucm_sparse_decode_step(const void* new_keys, int64_t T, int64_t k_stride_t,
                                      int64_t k_stride_h, const void* slot_mapping,
                                      int slot_is_i64, const void* queries, int64_t q_stride_b,
                                      int64_t q_stride_h, int x_dtype, int32_t K, const void* w,
                                      int w_dtype, int32_t n_w, int32_t N_bits, uint32_t* k_cache,
                                      int64_t NB, int32_t BS, int32_t Hkv, int64_t ks_block,
                                      int64_t ks_token, int64_t ks_head,
                                      const int32_t* block_table, int32_t table_stride,
                                      int32_t max_blocks, const int32_t* seq_lens, int32_t B,
                                      int32_t Hq, int32_t k, int32_t sink_tok, int32_t recent_tok,
                                      uint32_t flags, uint32_t* q_codes, int32_t* out_idx,
                                      int32_t* out_score, void* workspace, size_t workspace_bytes,
                                      ucm_stream_t stream)
{
    ucm::clear_error();
    UCM_REQUIRE(Hkv > 0 && Hq > 0 && Hq % Hkv == 0, "bad head counts");
    UCM_REQUIRE(N_bits > 0 && N_bits % 32 == 0, "hash_bits must be a multiple of 32");
    UCM_REQUIRE(n_w == 1 || n_w == Hkv, "n_w must be 1 or the number of KV heads");
    UCM_REQUIRE(q_codes, "q_codes is null");
    const int32_t Wd = N_bits / 32;
    const ucm::PairSpec spec{new_keys, T, Hkv, k_stride_t, k_stride_h, slot_mapping, slot_is_i64,
                             k_cache, NB, BS, ks_block, ks_token, ks_head, queries, B, Hq,
                             q_stride_b, q_stride_h, q_codes, (int64_t)Hq * Wd, Wd, x_dtype, K, w,
                             w_dtype, n_w, N_bits};
    int rc = ucm::encode_pair(spec, (hipStream_t)stream);
    if (rc != UCM_OK) return rc;
    return ucm_hamming_topk(q_codes, (int64_t)Hq * Wd, Wd, k_cache, NB, BS, Hkv, Wd, ks_block,
                            ks_token, ks_head, block_table, table_stride, max_blocks, seq_lens, B,
                            Hq, k, sink_tok, recent_tok, flags, out_idx, out_score, workspace,
                            workspace_bytes, stream);
}

extern "C" int ucm_sparse_decode_step_mla(
    const void* new_nope, int64_t nope_stride_t, const void* new_rope, int64_t rope_stride_t, int64_t T,
    const void* slot_mapping, int slot_is_i64, const void* q_nope, int64_t qn_stride_b,
    int64_t qn_stride_h, const void* q_rope, int64_t qr_stride_b, int64_t qr_stride_h, int x_dtype,
    int32_t K_nope, int32_t K_rope, const void* w_nope, const void* w_rope, int w_dtype,
    int32_t N_nope_bits, int32_t N_rope_bits, uint32_t* k_cache, int64_t NB, int32_t BS,
    int64_t ks_block, int64_t ks_token, const int32_t* block_table, int32_t table_stride,
    int32_t max_blocks, const int32_t* seq_lens, int32_t B, int32_t Hq, int32_t k, int32_t sink_tok,
    int32_t recent_tok, uint32_t flags, uint32_t* q_codes, int32_t* out_idx, int32_t* out_score,
    void* workspace, size_t workspace_bytes, ucm_stream_t stream)
{
    ucm::clear_error();
    UCM_REQUIRE(Hq > 0, "bad head count");
    UCM_REQUIRE(N_nope_bits > 0 && N_nope_bits % 32 == 0 && N_rope_bits > 0 && N_rope_bits % 32 == 0,
                "hash_bits of both parts must be multiples of 32");
    UCM_REQUIRE(q_codes && k_cache, "q_codes or k_cache is null");
    const int32_t Wn = N_nope_bits / 32, Wd = Wn + N_rope_bits / 32;
    UCM_REQUIRE(ks_token >= Wd, "cache rows of %lld words do not hold %d-word codes", (long long)ks_token, Wd);
    // nope part: words [0, Wn) of every code; rope part: words [Wn, Wd)
    const ucm::PairSpec nope{new_nope, T, 1, nope_stride_t, 0, slot_mapping, slot_is_i64, k_cache, NB, BS,
                             ks_block, ks_token, ks_token, q_nope, B, Hq, qn_stride_b, qn_stride_h,
                             q_codes, (int64_t)Hq * Wd, Wd, x_dtype, K_nope, w_nope, w_dtype, 1,
                             N_nope_bits};
    const ucm::PairSpec rope{new_rope, T, 1, rope_stride_t, 0, slot_mapping, slot_is_i64, k_cache + Wn, NB,
                             BS, ks_block, ks_token, ks_token, q_rope, B, Hq, qr_stride_b, qr_stride_h,
                             q_codes + Wn, (int64_t)Hq * Wd, Wd, x_dtype, K_rope, w_rope, w_dtype, 1,
                             N_rope_bits};
    const int rc = ucm::encode_two_pairs(nope, rope, (hipStream_t)stream);
    if (rc != UCM_OK) return rc;
    return ucm_hamming_topk(q_codes, (int64_t)Hq * Wd, Wd, k_cache, NB, BS, 1, Wd, ks_block, ks_token,
                            ks_token, block_table, table_stride, max_blocks, seq_lens, B, Hq, k,
                            sink_tok, recent_tok, flags, out_idx, out_score, workspace,
                            workspace_bytes, stream);
}

/* One latent-attention decode step as the reference's plugin performs it, see ucm_hip.h. */
extern "C" int ucm_gsa_decode_step_mla(
    const void* new_nope, int64_t nope_stride_t, const void* new_rope, int64_t rope_stride_t, int64_t T,
    const void* slot_mapping, int slot_is_i64, const void* q_nope, int64_t qn_stride_b,
    int64_t qn_stride_h, const void* q_rope, int64_t qr_stride_b, int64_t qr_stride_h, int x_dtype,
    int32_t K_nope, int32_t K_rope, const void* w_nope, const void* w_rope, int w_dtype,
    int32_t N_nope_bits, int32_t N_rope_bits, uint32_t* k_cache, int64_t NB, int32_t BS,
    int64_t ks_block, int64_t ks_token, const int32_t* block_table, int32_t table_stride,
    int32_t max_blocks, const int32_t* seq_lens, int32_t B, int32_t Hq, int32_t reduction_head_num,
    int32_t topk_tok, int32_t sink_tok, int32_t recent_tok, int32_t seq_len_threshold, uint32_t* q_codes,
    int32_t* new_block_table, int32_t new_table_stride, int32_t* new_seq_lens, void* workspace,
    size_t workspace_bytes, ucm_stream_t stream)
{
    ucm::clear_error();
    UCM_REQUIRE(Hq > 0 && reduction_head_num >= 1 && Hq % reduction_head_num == 0,
                "%d query heads do not reduce by %d", Hq, reduction_head_num);
    UCM_REQUIRE(N_nope_bits > 0 && N_nope_bits % 32 == 0 && N_rope_bits > 0 && N_rope_bits % 32 == 0,
                "hash_bits of both parts must be multiples of 32");
    UCM_REQUIRE(q_codes && k_cache, "q_codes or k_cache is null");
    // the reference's own checks (hamming_topk.py:30-31)
    UCM_REQUIRE(BS > 0 && topk_tok > 0 && topk_tok % BS == 0, "topk_token %d is no multiple of the block size %d",
                topk_tok, BS);
    UCM_REQUIRE(recent_tok > 0 && topk_tok > sink_tok + recent_tok, "topk_token must exceed sink + recent > 0");
    const int32_t Wn = N_nope_bits / 32, Wd = Wn + N_rope_bits / 32;
    UCM_REQUIRE(ks_token >= Wd, "cache rows of %lld words do not hold %d-word codes", (long long)ks_token, Wd);
    const int32_t Hr = Hq / reduction_head_num;  // rows that are hashed and scored
    ucm::PairSpec nope{new_nope, T, 1, nope_stride_t, 0, slot_mapping, slot_is_i64, k_cache, NB, BS,
                       ks_block, ks_token, ks_token, q_nope, B, Hq, qn_stride_b, qn_stride_h,
                       q_codes, (int64_t)Hr * Wd, Wd, x_dtype, K_nope, w_nope, w_dtype, 1, N_nope_bits};
    ucm::PairSpec rope{new_rope, T, 1, rope_stride_t, 0, slot_mapping, slot_is_i64, k_cache + Wn, NB,
                       BS, ks_block, ks_token, ks_token, q_rope, B, Hq, qr_stride_b, qr_stride_h,
                       q_codes + Wn, (int64_t)Hr * Wd, Wd, x_dtype, K_rope, w_rope, w_dtype, 1, N_rope_bits};
    nope.q_reduce = rope.q_reduce = reduction_head_num;
    const int rc = ucm::encode_two_pairs(nope, rope, (hipStream_t)stream);
    if (rc != UCM_OK) return rc;
    const StepOut so{new_block_table, new_table_stride, new_seq_lens, seq_len_threshold, topk_tok};
    return hamming_topk_run(q_codes, (int64_t)Hr * Wd, Wd, k_cache, NB, BS, 1, Wd, ks_block, ks_token, ks_token,
                            block_table, table_stride, max_blocks, seq_lens, B, Hr, topk_tok / BS, sink_tok,
                            recent_tok, UCM_TOPK_RETURN_PHYSICAL, nullptr, nullptr, workspace, workspace_bytes,
                            stream, &so);
}

extern "C" int64_t ucm_hamming_last_dispatch(char* buf, size_t cap)
{
    char tmp[256];
    int n = 0;
    if (g_note.planes) n += snprintf(tmp + n, sizeof(tmp) - n, "%s+", g_note.planes);
    if (g_note.score) {
        n += snprintf(tmp + n, sizeof(tmp) - n, "%s", g_note.score);
        for (int i = 0; i < 5 && g_note.sp[i] >= 0; ++i)
            n += snprintf(tmp + n, sizeof(tmp) - n, "%c%d", i == 0 ? '<' : ',', g_note.sp[i]);
        if (g_note.sp[0] >= 0) n += snprintf(tmp + n, sizeof(tmp) - n, ">");
    }
    if (g_note.select) {
        n += snprintf(tmp + n, sizeof(tmp) - n, "+%s", g_note.select);
        if (g_note.sel_el >= 0) n += snprintf(tmp + n, sizeof(tmp) - n, "<%d>", g_note.sel_el);
    }
    if (g_note.score_launches > 1) n += snprintf(tmp + n, sizeof(tmp) - n, " (%d scoring launches)", g_note.score_launches);
    tmp[n] = 0;
    if (buf && cap) {
        snprintf(buf, cap, "%s", tmp);
    }
    return n;
}

extern "C" int ucm_hamming_topk_set_clock_probe(void* two_u64_in_device_memory)
{
    ucm::clear_error();
    UCM_REQUIRE((reinterpret_cast<uintptr_t>(two_u64_in_device_memory) & 7) == 0, "the address is not 8-byte aligned");
    g_clock_probe = static_cast<unsigned long long*>(two_u64_in_device_memory);
    return UCM_OK;
}

extern "C" int ucm_hamming_topk_set_profile_events(void* before, void* after)
{
    ucm::clear_error();
    UCM_REQUIRE((before == nullptr) == (after == nullptr), "pass both events or neither");
    g_prof_before = (hipEvent_t)before;
    g_prof_after = (hipEvent_t)after;
    return UCM_OK;
}

namespace {

// Per-token scores for the usual layout (token-major codes whose words are a multiple of four,
// Hkv * Wd / 4 a power of two): one workgroup per (request, logical block).  A thread keeps the
// (head, 16-byte piece) it is responsible for and walks the block's tokens, so its loads are
// 16 bytes wide and a wave reads 1 KiB of contiguous codes per instruction, and the G query
// pieces of its head stay in registers.  Pieces of a wider code are summed across neighbouring
// lanes; the block's distances are collected in LDS and written out as one contiguous run per
// head.  Used when G * bits <= 2048, where every partial sum is an integer that fp16 holds
// exactly, so the reference's piecewise half-precision accumulation equals the exact sum.
template <int G>
__global__ __launch_bounds__(kThreads) void token_score_fast(TokenArgs t, int tb_shift)
{
    extern __shared__ uint32_t dyn[];  // [Hkv][tile tokens] distances
    __shared__ int64_t pbs[32];        // physical block of each of the tile's blocks, or -1
    const ScoreArgs& a = t.s;
    // the tile: 1 << tb_shift consecutive logical blocks (more than one only for power-of-two
    // block sizes, so that a workgroup has at least 128 tokens and ~16 KiB of codes to read)
    const int TBK = 1 << tb_shift, TT = a.BS << tb_shift;
    const int bs_shift = tb_shift ? __builtin_ctz((unsigned)a.BS) : 31;  // 31: every token -> block 0
    const int b = blockIdx.y, j0 = blockIdx.x << tb_shift;
    const int P = a.Wd >> 2, HP = a.Hkv * P;
    const int sub = threadIdx.x & (HP - 1);
    const int p_shift = __builtin_ctz(P), hp_shift = __builtin_ctz(HP);
    const int h = sub >> p_shift, part = sub & (P - 1);
    // one block per workgroup: its table entry is a scalar read, no LDS and no extra barrier
    int64_t pb0 = -1;
    if (tb_shift == 0) {
        pb0 = j0 < a.max_blocks ? physical_block(a, b, j0) : -1;
    } else if ((int)threadIdx.x < TBK) {
        const int j = j0 + threadIdx.x;
        pbs[threadIdx.x] = j < a.max_blocks ? physical_block(a, b, j) : -1;
    }
    uint32_t qw[G][4];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            qw[g][i] = a.q[b * a.q_stride_b + (int64_t)(h * G + g) * a.q_stride_h + part * 4 + i];
    const int len = a.lens[b];
    if (tb_shift) __syncthreads();
    const int step = kThreads >> hp_shift;
    // four passes of loads go out together (tokens past the tile re-read its last token; an
    // unusable block reads block 0 and is masked at the output)
    for (int tt0 = threadIdx.x >> hp_shift; tt0 < TT; tt0 += 4 * step) {
        u32x4 kw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            int tt = tt0 + u * step;
            tt = tt < TT ? tt : TT - 1;
            const int64_t pb = tb_shift ? pbs[tt >> bs_shift] : pb0;
            const int tok = tb_shift ? (tt & (a.BS - 1)) : tt;
            kw[u] = code_load(reinterpret_cast<const u32x4*>(
                a.kc + (pb < 0 ? 0 : pb) * a.ks_block + (int64_t)tok * a.ks_token + sub * 4));
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int tt = tt0 + u * step;
            int d = 0;
#pragma unroll
            for (int g = 0; g < G; ++g)
                d = popc_add(kw[u].w ^ qw[g][3], popc_add(kw[u].z ^ qw[g][2], popc_add(kw[u].y ^ qw[g][1], popc_add(kw[u].x ^ qw[g][0], d))));
            for (int o = 1; o < P; o <<= 1) d += __shfl_xor(d, o);
            if (part == 0 && tt < TT) dyn[h * TT + tt] = (uint32_t)d;
        }
    }
    __syncthreads();
    // with the KV-head reduction (the reference's GQA call, hamming_topk.py:33) one row per
    // request holds the minimum over the heads; the sums are exact here, so the minimum of
    // the integers is the minimum of the reference's half values
    const int rows_out = t.reduce_heads ? 1 : a.Hkv;
    // Four positions per thread and one 8- or 16-byte store where the rows allow it (block size and
    // row length multiples of four, aligned output): a quarter of the store instructions, and all
    // threads of the workgroup take part instead of one thread per token and head in turn.
    const bool by_four = ((a.BS | t.max_seq_len) & 3) == 0 && (reinterpret_cast<uintptr_t>(t.out) & 15) == 0;
    if (by_four) {
        const int TQ = TT >> 2;
        for (int i = threadIdx.x; i < rows_out * TQ; i += kThreads) {
            const int hh = i / TQ, tt = (i - hh * TQ) << 2;
            const int pos = j0 * a.BS + tt;
            if (pos >= t.max_seq_len) continue;
            u32x4 d = *reinterpret_cast<const u32x4*>(dyn + hh * TT + tt);
            if (t.reduce_heads)
                for (int h2 = 1; h2 < a.Hkv; ++h2) {
                    const u32x4 o2 = *reinterpret_cast<const u32x4*>(dyn + h2 * TT + tt);
                    d.x = o2.x < d.x ? o2.x : d.x;
                    d.y = o2.y < d.y ? o2.y : d.y;
                    d.z = o2.z < d.z ? o2.z : d.z;
                    d.w = o2.w < d.w ? o2.w : d.w;
                }
            const bool have = (tb_shift ? pbs[tt >> bs_shift] : pb0) >= 0;
            const int64_t o = ((int64_t)b * rows_out + hh) * t.max_seq_len + pos;
            const uint32_t dv[4] = {d.x, d.y, d.z, d.w};
            if (t.out_is_f16) {
                uint16_t hv[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int pe = pos + e;
                    const bool is_inf = pe >= len;
                    const bool keep = (pe < a.sink) || (pe >= len - a.recent && pe < len);
                    const _Float16 v = is_inf ? (_Float16)__builtin_inff()
                                              : (keep ? (_Float16)0.0f : (have ? (_Float16)(float)(int)dv[e] : (_Float16)__builtin_inff()));
                    __builtin_memcpy(&hv[e], &v, 2);
                }
                u32x2 w;
                w.x = hv[0] | ((uint32_t)hv[1] << 16);
                w.y = hv[2] | ((uint32_t)hv[3] << 16);
                *reinterpret_cast<u32x2*>((uint16_t*)t.out + o) = w;
            } else {
                u32x4 w;
                uint32_t iv[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int pe = pos + e;
                    const bool is_inf = pe >= len;
                    const bool keep = (pe < a.sink) || (pe >= len - a.recent && pe < len);
                    iv[e] = (uint32_t)(is_inf ? kInf : (keep ? 0 : (have ? (int)dv[e] : kInf)));
                }
                w.x = iv[0]; w.y = iv[1]; w.z = iv[2]; w.w = iv[3];
                *reinterpret_cast<u32x4*>((int32_t*)t.out + o) = w;
            }
        }
        return;
    }
    for (int hh = 0; hh < rows_out; ++hh) {
        for (int tt = threadIdx.x; tt < TT; tt += kThreads) {
            const int pos = j0 * a.BS + tt;
            if (pos >= t.max_seq_len) continue;
            const bool is_inf = pos >= len;
            const bool keep = (pos < a.sink) || (pos >= len - a.recent && pos < len);
            const bool have = (tb_shift ? pbs[tt >> bs_shift] : pb0) >= 0;
            int d = (int)dyn[hh * TT + tt];
            if (t.reduce_heads)
                for (int h2 = 1; h2 < a.Hkv; ++h2) {
                    const int o2 = (int)dyn[h2 * TT + tt];
                    d = o2 < d ? o2 : d;
                }
            const int64_t o = ((int64_t)b * rows_out + hh) * t.max_seq_len + pos;
            if (t.out_is_f16) {
                const _Float16 v = is_inf ? (_Float16)__builtin_inff()
                                          : (keep ? (_Float16)0.0f : (have ? (_Float16)(float)d : (_Float16)__builtin_inff()));
                uint16_t u;
                __builtin_memcpy(&u, &v, 2);
                ((uint16_t*)t.out)[o] = u;
            } else {
                ((int32_t*)t.out)[o] = is_inf ? kInf : (keep ? 0 : (have ? d : kInf));
            }
        }
    }
}

// Per-token scores of the hot shape: 128-bit codes, HKV heads, a block of exactly 16 KiB
// (1024 / HKV tokens), row length a multiple of four.  One workgroup per (request, logical block),
// laid out as block_score_one: lane l of wave w reads pieces (w + 4u) * 64 + l, u = 0..3 - 1 KiB
// per wave and instruction, all four before anything waits - and owns head l % HKV, whose G query
// codes stay in registers.  The request's scalars are read together at the top, without branches
// between them.  A distance goes to LDS once (row stride padded so that the 64 lanes of a store
// fall into 64 banks) and leaves as four positions per thread in one 8- or 16-byte store.  Every
// sum is an integer that fp16 holds exactly (G * 128 <= 2048), so the piecewise half-precision
// accumulation of paged_ham_dist_mla.cu:204-241 equals the exact sum.
template <int G, int HKV>
__global__ __launch_bounds__(kThreads) void token_score_one(TokenArgs t)
{
    constexpr int BSC = 1024 / HKV;               // tokens of a block
    constexpr int PAD = 64 / HKV < 4 ? 4 : 64 / HKV;
    constexpr int STRIDE = BSC + PAD;             // words between the rows of two heads
    constexpr int TQ = BSC / 4;                   // groups of four positions per head
    __shared__ __attribute__((aligned(16))) uint32_t dist[HKV * STRIDE];
    const ScoreArgs& a = t.s;
    const int b = blockIdx.y, j = blockIdx.x;
    const int lane = lane_id();
    const int wid = wave_id();
    const int h = lane % HKV;

    // the grid covers max_seq_len, which may reach past the table's row: such a block reads the
    // row's last entry and does not use it
    const int jt = j < a.max_blocks ? j : a.max_blocks - 1;
    const uintptr_t has_table = a.table ? ~(uintptr_t)0 : 0;
    const uintptr_t ea = (reinterpret_cast<uintptr_t>(a.table + ((int64_t)b * a.table_stride + jt)) & has_table) |
                         (reinterpret_cast<uintptr_t>(a.lens + b) & ~has_table);
    int entry = *reinterpret_cast<const int32_t*>(ea);
    int len = a.lens[b];
    int64_t ks_block0 = a.ks_block, nb0 = a.NB, q_stride_b0 = a.q_stride_b;
    asm volatile("" : "+s"(entry), "+s"(len), "+s"(ks_block0), "+s"(nb0), "+s"(q_stride_b0));

    uint32_t qr[G][4];
    {
        const uint32_t* qp = a.q + b * q_stride_b0 + (int64_t)h * G * a.q_stride_h;
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int w = 0; w < 4; ++w) qr[g][w] = qp[g * a.q_stride_h + w];
    }
    int64_t pb = ((int64_t)entry & (int64_t)has_table) | (((int64_t)b * a.max_blocks + j) & ~(int64_t)has_table);
    if (j >= a.max_blocks || pb < 0 || pb >= nb0) pb = -1;
    const int pos0 = j * BSC;
    const bool reads = pb >= 0 && pos0 < len;
    if (reads) {
        const u32x4* base = reinterpret_cast<const u32x4*>(a.kc + pb * ks_block0) + lane;
        u32x4 kv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) kv[u] = code_load(base + ((wid + 4 * u) << 6));
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            int d = __popc(kv[u].x ^ qr[0][0]);
            d = popc_add(kv[u].y ^ qr[0][1], d);
            d = popc_add(kv[u].z ^ qr[0][2], d);
            d = popc_add(kv[u].w ^ qr[0][3], d);
#pragma unroll
            for (int g = 1; g < G; ++g) {
                d = popc_add(kv[u].x ^ qr[g][0], d);
                d = popc_add(kv[u].y ^ qr[g][1], d);
                d = popc_add(kv[u].z ^ qr[g][2], d);
                d = popc_add(kv[u].w ^ qr[g][3], d);
            }
            const int tok = (((wid + 4 * u) << 6) + lane) / HKV;
            dist[h * STRIDE + tok] = (uint32_t)d;
        }
    }
    __syncthreads();
    // with the KV-head reduction (the reference's GQA call, hamming_topk.py:33) one row per request
    // holds the minimum over the heads
    const int rows_out = t.reduce_heads ? 1 : HKV;
    // a block between the sink and the recent window, all of it below the length: plain distances
    const bool interior = reads && pos0 >= a.sink && pos0 + BSC <= len - a.recent;
    for (int i = threadIdx.x; i < rows_out * TQ; i += kThreads) {
        const int hh = i / TQ, tt = (i % TQ) << 2;
        const int pos = pos0 + tt;
        if (pos >= t.max_seq_len) continue;
        u32x4 d = (u32x4)(0u);
        if (reads) {
            d = *reinterpret_cast<const u32x4*>(dist + hh * STRIDE + tt);
            if (t.reduce_heads) {
#pragma unroll
                for (int h2 = 1; h2 < HKV; ++h2) {
                    const u32x4 o2 = *reinterpret_cast<const u32x4*>(dist + h2 * STRIDE + tt);
                    d.x = o2.x < d.x ? o2.x : d.x;
                    d.y = o2.y < d.y ? o2.y : d.y;
                    d.z = o2.z < d.z ? o2.z : d.z;
                    d.w = o2.w < d.w ? o2.w : d.w;
                }
            }
        }
        const uint32_t dv[4] = {d.x, d.y, d.z, d.w};
        const int64_t o = ((int64_t)b * rows_out + hh) * t.max_seq_len + pos;
        if (t.out_is_f16) {
            uint16_t hv[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int pe = pos + e;
                const bool none = !interior && (pe >= len || (!reads && !(pe < a.sink) && !(pe >= len - a.recent)));
                const bool keep = !interior && ((pe < a.sink) || (pe >= len - a.recent));
                const _Float16 v = none ? (_Float16)__builtin_inff() : (keep ? (_Float16)0.0f : (_Float16)(float)(int)dv[e]);
                __builtin_memcpy(&hv[e], &v, 2);
            }
            u32x2 w;
            w.x = hv[0] | ((uint32_t)hv[1] << 16);
            w.y = hv[2] | ((uint32_t)hv[3] << 16);
            *reinterpret_cast<u32x2*>((uint16_t*)t.out + o) = w;
        } else {
            uint32_t iv[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int pe = pos + e;
                const bool none = !interior && (pe >= len || (!reads && !(pe < a.sink) && !(pe >= len - a.recent)));
                const bool keep = !interior && ((pe < a.sink) || (pe >= len - a.recent));
                iv[e] = (uint32_t)(none ? kInf : (keep ? 0 : (int)dv[e]));
            }
            u32x4 w;
            w.x = iv[0]; w.y = iv[1]; w.z = iv[2]; w.w = iv[3];
            *reinterpret_cast<u32x4*>((int32_t*)t.out + o) = w;
        }
    }
    // (Streaming stores measured against these plain ones at 32 x 32,768 tokens: 0.4 us less with all
    // heads written, 16.8 MB, and 1.5 us more with the one reduced row; plain stores also leave the
    // scores in the cache for the selection that reads them next.)
}

// Per-token scores for the 8-byte-piece layout (one KV head, even code width).  A lane's piece
// is exactly one step of the reference's half-precision accumulation, so the first lane of a
// code collects the piece sums of its L lanes in order and adds them as the reference does; any
// group size is exact (bit planes from the workspace above 8 query heads).  A wave owns one
// logical block and writes every position of it below max_seq_len.
template <bool DIRECT, int GP, bool F16>
__global__ __launch_bounds__(kThreads) void token_score_pairs(TokenArgs t, int L, int TP)
{
    const ScoreArgs& a = t.s;
    const int b = blockIdx.y;
    const int lane = lane_id();
    const int j = blockIdx.x * (kThreads / kWave) + wave_id();
    const int pos0 = j * a.BS;
    if (pos0 >= t.max_seq_len) return;
    const int slot = lane / L, p = lane - slot * L;
    const bool lane_ok = slot < TP;
    const int jc = j < a.max_blocks ? j : a.max_blocks - 1;
    const int entry = a.table ? a.table[(int64_t)b * a.table_stride + jc] : 0;
    const int len = a.lens[b];
    PairQuery<DIRECT, GP> qm;
    qm.fetch(a, b, lane_ok ? 2 * p : 0);
    int64_t pb = a.table ? (int64_t)entry : (int64_t)b * a.max_blocks + j;
    if (j >= a.max_blocks || pb < 0 || pb >= a.NB) pb = -1;
    const int nout = (a.BS < t.max_seq_len - pos0) ? a.BS : t.max_seq_len - pos0;
    int ntok = len - pos0;  // tokens whose codes are read
    ntok = pb < 0 ? 0 : (ntok < 0 ? 0 : (ntok > nout ? nout : ntok));

    const u32x2* base = reinterpret_cast<const u32x2*>(a.kc + (pb < 0 ? 0 : pb) * a.ks_block);
    const int64_t obase = (int64_t)b * t.max_seq_len + pos0;
    const bool writer = lane_ok && p == 0;
    // what a position holds when it has no distance of its own
    auto fixed = [&](int pos, bool& none, bool& keep) {
        keep = (pos < a.sink) || (pos >= len - a.recent && pos < len);
        none = pos >= len || (!keep && pb < 0);
    };
    for (int t0 = 0; t0 < nout; t0 += kPairPasses * TP) {
        u32x2 kv[kPairPasses];
#pragma unroll
        for (int u = 0; u < kPairPasses; ++u) {
            if (t0 + u * TP < ntok) {
                const int tok = t0 + u * TP + slot;
                kv[u] = code_load(
                    base + ((tok < a.BS && lane_ok) ? tok * L + p : (t0 + u * TP) * L));
            } else {
                kv[u] = u32x2{0u, 0u};
            }
        }
        if (t0 == 0) qm.finish();
        if (F16) {
            // two passes share every shuffle and every (packed) half add: the halves of a
            // register are the piece sums of token `tok` and of token `tok + TP`; the shuffles of
            // all pass pairs go out together
            constexpr int NP = kPairPasses / 2;
            f16x2 acc[NP];
            uint32_t mine[NP];
#pragma unroll
            for (int v = 0; v < NP; ++v) {
                acc[v].x = (_Float16)(float)qm.dist(kv[2 * v]);
                acc[v].y = (_Float16)(float)qm.dist(kv[2 * v + 1]);
                __builtin_memcpy(&mine[v], &acc[v], 4);
            }
            if (t0 < ntok) {
                for (int o = 1; o < L; ++o) {
                    uint32_t x[NP];
#pragma unroll
                    for (int v = 0; v < NP; ++v) x[v] = (uint32_t)__shfl_down((int)mine[v], o);
#pragma unroll
                    for (int v = 0; v < NP; ++v) {
                        f16x2 xv;
                        __builtin_memcpy(&xv, &x[v], 4);
                        acc[v] = acc[v] + xv;
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < kPairPasses; ++u) {
                const int tok = t0 + u * TP + slot;
                if (t0 + u * TP < nout && writer && tok < nout) {
                    bool none, keep;
                    fixed(pos0 + tok, none, keep);
                    const _Float16 d = (u & 1) ? acc[u >> 1].y : acc[u >> 1].x;
                    const _Float16 v = none ? (_Float16)__builtin_inff() : (keep ? (_Float16)0.0f : d);
                    uint16_t bits;
                    __builtin_memcpy(&bits, &v, 2);
                    ((uint16_t*)t.out)[obase + tok] = bits;
                }
            }
        } else {
#pragma unroll
            for (int g = 0; g < kPairPasses; g += kPairGroup) {
                if (t0 + g * TP >= nout) continue;
                int d[kPairGroup];
                pair_group_sums(qm, kv + g, d, p, L);
#pragma unroll
                for (int u = 0; u < kPairGroup; ++u) {
                    const int tok = t0 + (g + u) * TP + slot;
                    if (writer && tok < nout) {
                        bool none, keep;
                        fixed(pos0 + tok, none, keep);
                        ((int32_t*)t.out)[obase + tok] = none ? kInf : (keep ? 0 : d[u]);
                    }
                }
            }
        }
    }
}

// Per-token scores, a whole code per lane (see block_score_lanes): the lane adds its code's
// 8-byte piece sums in half precision in the reference's order without any cross-lane step, and
// the 64 results of a round leave as one contiguous run.
template <int LC, bool DIRECT, int GP, bool F16>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 8))) void token_score_lanes(TokenArgs t)
{
    using LCd = LaneCode<LC, DIRECT, GP>;
    constexpr int WD = LCd::WD;
    __shared__ __align__(16) uint32_t strip[kThreads / kWave][LCd::kRoundWords];
    __shared__ __align__(16) uint32_t pl[DIRECT ? 8 : WD * 8];
    __shared__ int ctot[LC];
    const ScoreArgs& a = t.s;
    const int b = blockIdx.y;
    const int lane = lane_id(), wid = wave_id();
    const int j = blockIdx.x * (kThreads / kWave) + wid;
    const int jc = j < a.max_blocks ? j : a.max_blocks - 1;
    const int entry = a.table ? a.table[(int64_t)b * a.table_stride + jc] : 0;
    const int len = a.lens[b];
    LCd::stage_planes(a, b, pl, ctot);
    if (!DIRECT) __syncthreads();
    const int pos0 = j * a.BS;
    if (pos0 >= t.max_seq_len) return;
    int64_t pb = a.table ? (int64_t)entry : (int64_t)b * a.max_blocks + j;
    if (j >= a.max_blocks || pb < 0 || pb >= a.NB) pb = -1;
    const int nout = (a.BS < t.max_seq_len - pos0) ? a.BS : t.max_seq_len - pos0;
    int ntok = len - pos0;  // tokens whose codes are read
    ntok = pb < 0 ? 0 : (ntok < 0 ? 0 : (ntok > nout ? nout : ntok));
    const int rounds_in = (ntok + 63) >> 6, rounds_out = (nout + 63) >> 6;
    const u32x4* src = reinterpret_cast<const u32x4*>(a.kc + (pb < 0 ? 0 : pb) * a.ks_block);
    u32x4* mine = reinterpret_cast<u32x4*>(strip[wid]);
    const uint32_t* row = strip[wid] + lane * WD;
    const uint32_t* qp = a.q + b * a.q_stride_b;
    const int64_t obase = (int64_t)b * t.max_seq_len + pos0;

    u32x4 cur[LCd::kLoads], nxt[LCd::kLoads];
    LCd::load_round(src, 0, lane, cur);  // block 0 when there is nothing to read: harmless
#pragma unroll
    for (int u = 0; u < LCd::kLoads; ++u) nxt[u] = cur[u];
    for (int r = 0; r < rounds_out; ++r) {
        int di = 0;
        _Float16 dh = (_Float16)0.0f;
        if (r < rounds_in) {
            if (r + 1 < rounds_in) LCd::load_round(src, r + 1, lane, nxt);
            LCd::store_round(mine, lane, cur);
            asm volatile("" ::: "memory");  // planes re-read per round, see block_score_lanes
#pragma unroll
            for (int i = 0; i < LC; ++i) {
                const u32x2 k = *reinterpret_cast<const u32x2*>(row + 2 * i);
                int part = 0;
                if (DIRECT) {
#pragma unroll
                    for (int g = 0; g < GP; ++g)
                        part += __popc(k.x ^ qp[g * a.q_stride_h + 2 * i]) +
                                __popc(k.y ^ qp[g * a.q_stride_h + 2 * i + 1]);
                } else {
                    int x = 0;
#pragma unroll
                    for (int p = 0; p < GP; ++p)
                        x += (__popc(k.x & pl[(2 * i) * 8 + p]) + __popc(k.y & pl[(2 * i + 1) * 8 + p])) << p;
                    part = ctot[i] + a.G * (__popc(k.x) + __popc(k.y)) - 2 * x;
                }
                di += part;
                if (F16) dh = dh + (_Float16)(float)part;
            }
#pragma unroll
            for (int u = 0; u < LCd::kLoads; ++u) cur[u] = nxt[u];
        }
        const int tok = r * 64 + lane;
        if (tok < nout) {
            const int pos = pos0 + tok;
            const bool keep = (pos < a.sink) || (pos >= len - a.recent && pos < len);
            const bool none = pos >= len || (!keep && pb < 0);
            if (F16) {
                const _Float16 v = none ? (_Float16)__builtin_inff() : (keep ? (_Float16)0.0f : dh);
                uint16_t bits;
                __builtin_memcpy(&bits, &v, 2);
                ((uint16_t*)t.out)[obase + tok] = bits;
            } else {
                ((int32_t*)t.out)[obase + tok] = none ? kInf : (keep ? 0 : di);
            }
        }
    }
}

template <int LC, bool DIRECT, int GP>
void launch_token_lanes(const TokenArgs& t, dim3 grid, hipStream_t st)
{
    if (t.out_is_f16)
        hipLaunchKernelGGL((token_score_lanes<LC, DIRECT, GP, true>), grid, dim3(kThreads), 0, st, t);
    else
        hipLaunchKernelGGL((token_score_lanes<LC, DIRECT, GP, false>), grid, dim3(kThreads), 0, st, t);
}

template <int LC>
void dispatch_token_lanes_planes(const TokenArgs& t, int pmax, dim3 grid, hipStream_t st)
{
    switch (pmax) {
        case 4: launch_token_lanes<LC, false, 4>(t, grid, st); break;
        case 5: launch_token_lanes<LC, false, 5>(t, grid, st); break;
        case 6: launch_token_lanes<LC, false, 6>(t, grid, st); break;
        case 7: launch_token_lanes<LC, false, 7>(t, grid, st); break;
        default: launch_token_lanes<LC, false, 8>(t, grid, st); break;
    }
}

template <bool DIRECT, int GP>
void launch_token_pairs(const TokenArgs& t, int L, int TP, dim3 grid, hipStream_t st)
{
    if (t.out_is_f16)
        hipLaunchKernelGGL((token_score_pairs<DIRECT, GP, true>), grid, dim3(kThreads), 0, st, t, L, TP);
    else
        hipLaunchKernelGGL((token_score_pairs<DIRECT, GP, false>), grid, dim3(kThreads), 0, st, t, L, TP);
}

// bit planes that hold the counts 0..G
int exact_planes(int G)
{
    int p = 0;
    while ((1 << p) <= G) ++p;
    return p < 4 ? 4 : p;
}

size_t score_plane_bytes(int B, int Wd) { return align_up((size_t)B * 8 * Wd * 4, 256); }

}  // namespace

extern "C" size_t ucm_hamming_score_workspace_bytes(int32_t B, int32_t Hq, int32_t Wd)
{
    (void)Hq;
    if (B <= 0 || Wd <= 0) return 256;
    return score_plane_bytes(B, Wd);
}

extern "C" int ucm_hamming_score(const uint32_t* q_codes, int64_t q_stride_b, int64_t q_stride_h,
                                 const uint32_t* k_cache, int64_t NB, int32_t BS, int32_t Hkv,
                                 int32_t Wd, int64_t ks_block, int64_t ks_token, int64_t ks_head,
                                 const int32_t* block_table, int32_t table_stride,
                                 int32_t max_blocks, const int32_t* seq_lens, int32_t B,
                                 int32_t Hq, int32_t max_seq_len, int32_t sink_tok,
                                 int32_t recent_tok, int reduce_heads, void* out, int out_is_f16,
                                 void* workspace, size_t workspace_bytes, ucm_stream_t stream)
{
    ucm::clear_error();
    note_reset();
    int rc = common_checks(q_codes, k_cache, seq_lens, NB, BS, Hkv, Wd, B, Hq, max_blocks);
    if (rc != UCM_OK) return rc;
    UCM_REQUIRE(out, "out is null");
    UCM_REQUIRE(max_seq_len > 0, "max_seq_len must be positive");
    UCM_REQUIRE(!block_table || table_stride >= max_blocks, "table_stride %d < max_blocks %d",
                table_stride, max_blocks);
    if (B == 0) return UCM_OK;
    TokenArgs t;
    ScoreArgs& a = t.s;
    a.q = q_codes; a.q_stride_b = q_stride_b; a.q_stride_h = q_stride_h;
    a.kc = k_cache; a.NB = NB; a.BS = BS; a.Hkv = Hkv; a.Wd = Wd;
    a.ks_block = ks_block; a.ks_token = ks_token; a.ks_head = ks_head;
    a.table = block_table; a.table_stride = table_stride; a.max_blocks = max_blocks;
    a.lens = seq_lens; a.B = B; a.Hq = Hq; a.G = Hq / Hkv; a.sink = sink_tok;
    a.recent = recent_tok; a.TB = 1; a.reduce_out = 0; a.planes = nullptr; a.scores = nullptr;
    a.clock_probe = g_clock_probe;
    t.max_seq_len = max_seq_len; t.reduce_heads = reduce_heads; t.out_is_f16 = out_is_f16;
    t.out = out;
    const int G = a.G;
    const bool fast = Wd % 4 == 0 && is_pow2(Wd / 4) && is_pow2(Hkv * (Wd / 4)) &&
                      Hkv * (Wd / 4) <= kThreads && ks_head == Wd && ks_token == (int64_t)Hkv * Wd &&
                      ks_block % 4 == 0 && (reinterpret_cast<uintptr_t>(k_cache) & 15) == 0 &&
                      (G == 1 || G == 2 || G == 4 || G == 8) && (int64_t)G * Wd * 32 <= 2048 &&
                      (int64_t)BS * Hkv * 4 <= 48 * 1024 && ucm::ceil_div(max_seq_len, BS) <= 0x7fffffff;
    if (fast && Wd == 4 && (Hkv == 4 || Hkv == 8) && (int64_t)BS * Hkv == 1024 && max_seq_len % 4 == 0 &&
        (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
        const dim3 ogrid((unsigned)ucm::ceil_div(max_seq_len, BS), (unsigned)B);
        hipStream_t st = (hipStream_t)stream;
        note_score("token_score_one", G, Hkv);
#define UCM_TOKEN_ONE(GG)                                                                      \
    do {                                                                                       \
        if (Hkv == 8) hipLaunchKernelGGL((token_score_one<GG, 8>), ogrid, dim3(kThreads), 0, st, t); \
        else hipLaunchKernelGGL((token_score_one<GG, 4>), ogrid, dim3(kThreads), 0, st, t);      \
    } while (0)
        if (G == 1) UCM_TOKEN_ONE(1);
        else if (G == 2) UCM_TOKEN_ONE(2);
        else if (G == 4) UCM_TOKEN_ONE(4);
        else UCM_TOKEN_ONE(8);
#undef UCM_TOKEN_ONE
        return ucm::launch_status("token_score_one");
    }
    if (fast) {
        // small blocks (power-of-two sizes): several per workgroup, until it has at least 128
        // tokens and 16 KiB of codes to read
        int tbs = 0;
        if (is_pow2(BS))
            while (tbs < 5 && ((BS << tbs) < 128 || ((int64_t)BS << tbs) * Hkv * Wd * 4 < 16384)) ++tbs;
        while (tbs > 0 && ((size_t)BS << tbs) * Hkv * 4 > 48 * 1024) --tbs;
        const dim3 fgrid((unsigned)ucm::ceil_div(ucm::ceil_div(max_seq_len, BS), 1 << tbs), (unsigned)B);
        const size_t lds = ((size_t)BS << tbs) * Hkv * 4;
        hipStream_t st = (hipStream_t)stream;
        note_score("token_score_fast", G);
        if (G == 1) hipLaunchKernelGGL(token_score_fast<1>, fgrid, dim3(kThreads), lds, st, t, tbs);
        else if (G == 2) hipLaunchKernelGGL(token_score_fast<2>, fgrid, dim3(kThreads), lds, st, t, tbs);
        else if (G == 4) hipLaunchKernelGGL(token_score_fast<4>, fgrid, dim3(kThreads), lds, st, t, tbs);
        else hipLaunchKernelGGL(token_score_fast<8>, fgrid, dim3(kThreads), lds, st, t, tbs);
        return ucm::launch_status("token_score_fast");
    }
    const bool direct = G == 1 || G == 2 || G == 4 || G == 8;
    const bool have_planes = workspace && workspace_bytes >= score_plane_bytes(B, Wd) &&
                             (reinterpret_cast<uintptr_t>(workspace) & 15) == 0;
    // 64-token blocks of 18-word codes above four query heads (or three) and of 8-word codes with 16 to 128:
    // the scorer builds its weights itself
    const bool run18 = Wd == 18 && BS == 64 && G <= 128 && !(G <= 4 && direct) && lanes_layout(a, k_cache, false);
    const bool run8 = Wd == 8 && BS == 64 && G >= 16 && G <= 128 && lanes_layout(a, k_cache, false);
    if (pairs_layout(a, k_cache) && (direct || have_planes || run18 || run8)) {
        hipStream_t st = (hipStream_t)stream;
        const int L = Wd / 2, TP = kWave / L;
        const int nblk = ucm::ceil_div(max_seq_len, BS);
        const dim3 pgrid((unsigned)ucm::ceil_div(nblk, kThreads / kWave), (unsigned)B);
        // 18-word codes in blocks of 64, 128, ... tokens: a whole code per lane
        const bool lanes = lanes_layout(a, k_cache, G <= 4 && direct);
        if (lanes && G <= 4 && direct) {
            note_score("token_score_lanes", 9, 1, G);
            if (G == 1) launch_token_lanes<9, true, 1>(t, pgrid, st);
            else if (G == 2) launch_token_lanes<9, true, 2>(t, pgrid, st);
            else launch_token_lanes<9, true, 4>(t, pgrid, st);
            return ucm::launch_status("token_score_lanes");
        }
        if (run18 || run8) {
            // the weighted bit sums of every 8-byte piece on the matrix unit; no plane kernel, no workspace
            const dim3 rgrid((unsigned)ucm::ceil_div(nblk, kStripWaves * strip_run(Wd)), (unsigned)B);
            const dim3 threads(kStripWaves * kWave);
            note_score("token_score_strip", Wd, out_is_f16 ? 1 : 0);
            if (Wd == 18) {
                if (out_is_f16) hipLaunchKernelGGL((token_score_strip<18, true>), rgrid, threads, 0, st, a, max_seq_len, out);
                else hipLaunchKernelGGL((token_score_strip<18, false>), rgrid, threads, 0, st, a, max_seq_len, out);
            } else {
                if (out_is_f16) hipLaunchKernelGGL((token_score_strip<8, true>), rgrid, threads, 0, st, a, max_seq_len, out);
                else hipLaunchKernelGGL((token_score_strip<8, false>), rgrid, threads, 0, st, a, max_seq_len, out);
            }
            return ucm::launch_status("token_score_strip");
        }
        // 8 query heads: bit planes when the caller brought the workspace for them
        if (direct && !(lanes && have_planes)) {
            note_score("token_score_pairs", 1, G);
            if (G == 1) launch_token_pairs<true, 1>(t, L, TP, pgrid, st);
            else if (G == 2) launch_token_pairs<true, 2>(t, L, TP, pgrid, st);
            else if (G == 4) launch_token_pairs<true, 4>(t, L, TP, pgrid, st);
            else launch_token_pairs<true, 8>(t, L, TP, pgrid, st);
        } else {
            const int pmax = exact_planes(G);
            a.planes = static_cast<uint32_t*>(workspace);
            g_note.planes = "plane_kernel";
            hipLaunchKernelGGL(plane_kernel, dim3(B * ((Wd + 1) / 2)), dim3(kThreads), 0, st, q_codes,
                               q_stride_b, q_stride_h, 1, G, Wd, pmax, static_cast<uint32_t*>(workspace));
            rc = ucm::launch_status("plane_kernel");
            if (rc != UCM_OK) return rc;
            if (lanes) {
                note_score("token_score_lanes", Wd / 2, 0, pmax > 8 ? 8 : pmax);
                if (Wd == 18) dispatch_token_lanes_planes<9>(t, pmax, pgrid, st);
                else if (Wd == 16) dispatch_token_lanes_planes<8>(t, pmax, pgrid, st);
                else dispatch_token_lanes_planes<4>(t, pmax, pgrid, st);
                return ucm::launch_status("token_score_lanes");
            }
            note_score("token_score_pairs", 0, pmax > 8 ? 8 : pmax);
            switch (pmax) {
                case 4: launch_token_pairs<false, 4>(t, L, TP, pgrid, st); break;
                case 5: launch_token_pairs<false, 5>(t, L, TP, pgrid, st); break;
                case 6: launch_token_pairs<false, 6>(t, L, TP, pgrid, st); break;
                case 7: launch_token_pairs<false, 7>(t, L, TP, pgrid, st); break;
                default: launch_token_pairs<false, 8>(t, L, TP, pgrid, st); break;
            }
        }
        return ucm::launch_status("token_score_pairs");
    }
    const dim3 grid((unsigned)ucm::ceil_div(max_seq_len, kThreads), (unsigned)B);
    note_score("token_score_kernel");
    hipLaunchKernelGGL(token_score_kernel, grid, dim3(kThreads), (size_t)Hq * Wd * 4,
                       (hipStream_t)stream, t);
    return ucm::launch_status("token_score_kernel");
}

extern "C" int ucm_update_seq_lens(const int32_t* seq_lens, int32_t B, int32_t topk_tok,
                                   int32_t BS, int32_t* out, ucm_stream_t stream)
{
    ucm::clear_error();
    UCM_REQUIRE(seq_lens && out, "null pointer");
    UCM_REQUIRE(BS > 0 && B >= 0, "bad sizes");
    if (B == 0) return UCM_OK;
    hipLaunchKernelGGL(update_seq_lens_kernel, dim3((unsigned)ucm::ceil_div(B, 256)), dim3(256), 0,
                       (hipStream_t)stream, seq_lens, B, topk_tok, BS, out);
    return ucm::launch_status("update_seq_lens_kernel");
}
