// Bucketed linear layer: the first layer of the layer stacks, where every position uses the
// weights of its own bucket only.  The reference evaluates all `count` layers as one wide GEMM and
// then keeps one block per position (model/modules/stacked_linear.py:38-66); here the positions
// are grouped by bucket first and each group meets only its own [out, in] weight block, an eighth
// of the arithmetic and no wide intermediate.  fp32 MFMA (v_mfma_f32_32x32x2_f32) on tiles of 32
// positions; out <= 32.
//
//   k_bucket_order     positions grouped by bucket (ascending inside a group), cut into tiles of 32
//   k_bucket_fwd       y[pos, :] = bias_b + W_b x[pos]           tile x waves that split `in`
//   k_bucket_bwd_x     gx[pos, :] = W_b^T gy[pos]                tile x column ranges
//   k_bucket_bwd_w     gW_b = sum over the bucket's positions of gy[pos] (x) x[pos], gbias_b likewise,
//                      in a fixed order                         bucket x 64-column block, 8 waves
#include "common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kOrderThreads = 1024;
constexpr int kTile = 32;
constexpr int kMaxCount = 64;

constexpr size_t kPartialBytes = 8 << 20;   // partial weight gradients of narrow layers (k_bucket_bwd_w in splits)
constexpr int kBwdSplits = 8;

struct BucketLayout {
    size_t order, bucket_off, ntiles, tiles, partial, end;
    int max_tiles;
};

inline size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

bool bucket_layout(int B, int count, BucketLayout* L) {
    if (B <= 0 || count <= 0 || count > kMaxCount) return false;
    L->max_tiles = (B + kTile - 1) / kTile + count;
    size_t off = 0;
    L->order = off;
    off += up256((size_t)B * sizeof(uint32_t));
    L->bucket_off = off;
    off += up256((size_t)(count + 1) * sizeof(uint32_t));
    L->ntiles = off;
    off += 256;
    L->tiles = off;
    off += up256((size_t)L->max_tiles * 2 * sizeof(uint32_t));
    L->partial = off;
    off += kPartialBytes;
    L->end = off;
    return true;
}

// Single workgroup.  order[] = the positions of bucket 0 ascending, then bucket 1, ...; positions
// whose bucket is outside [0, count) are left out.  tiles[2t] = first index into order, tiles[2t+1]
// = bucket << 8 | positions in the tile.
// The kernel is one workgroup, so every latency it waits for is run time: a thread keeps the buckets
// of kOrderAhead positions in registers (loads issued together), counts with ballots, and the
// workgroup synchronises three times per block of kOrderThreads * kOrderAhead positions, not per step.
//   counts   per (step, wave, bucket) to LDS, ranks inside the ballot kept in registers
//   prefix   wave w turns the counts of buckets w, w + NW, ... into places, in (step, wave) order
//   place    order[place of (step, wave, bucket) + rank] = position
// The lanes of the wave that hold the same bucket as this one (valid lanes only): one ballot per bit
// of the bucket number instead of one per bucket.
__device__ __forceinline__ u64 same_bucket(int c, bool valid, int nbits) {
    u64 m = __ballot(valid);
    for (int j = 0; j < nbits; ++j) {
        const bool bit = (c >> j) & 1;
        const u64 bj = __ballot(valid && bit);
        m &= bit ? bj : ~bj;
    }
    return m;
}

template <int kOrderAhead>
__global__ __launch_bounds__(kOrderThreads) void k_bucket_order(const int64_t* __restrict__ bucket,
                                                                uint32_t* __restrict__ order,
                                                                uint32_t* __restrict__ bucket_off,
                                                                uint32_t* __restrict__ ntiles,
                                                                uint32_t* __restrict__ tiles, int B, int count) {
    constexpr int NW = kOrderThreads / 64;
    constexpr int NS = kOrderAhead * NW;             // (step, wave) pairs of a block, in position order
    extern __shared__ uint32_t cnt_s[];              // [count][NS]
    __shared__ uint32_t total_s[kMaxCount];          // positions per bucket
    __shared__ uint32_t cursor_s[kMaxCount];         // next free place of each bucket
    __shared__ uint32_t tile_base_s[kMaxCount + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid < kMaxCount) total_s[tid] = 0;
    __syncthreads();
    // totals.  The first block's buckets stay in registers for the
    // second pass (a batch of up to kOrderThreads * kOrderAhead positions is read from memory once).
    constexpr int NB = kOrderThreads * kOrderAhead;
    const int nbits = count > 1 ? 32 - __clz(count - 1) : 0;
    const u64 lt = (1ull << lane) - 1ull;
    int first[kOrderAhead];
#pragma unroll
    for (int u = 0; u < kOrderAhead; ++u) {
        const int b = u * kOrderThreads + tid;
        first[u] = b < B ? (int)bucket[b] : -1;
    }
    for (int b0 = 0; b0 < B; b0 += NB) {
        int cs[kOrderAhead];
#pragma unroll
        for (int u = 0; u < kOrderAhead; ++u) {
            const int b = b0 + u * kOrderThreads + tid;
            cs[u] = b0 == 0 ? first[u] : (b < B ? (int)bucket[b] : -1);
        }
#pragma unroll
        for (int u = 0; u < kOrderAhead; ++u) {
            if (b0 + u * kOrderThreads >= B) break;
            const bool valid = cs[u] >= 0 && cs[u] < count;
            const u64 m = same_bucket(cs[u], valid, nbits);
            if (valid && (m & lt) == 0) atomicAdd(&total_s[cs[u]], (uint32_t)__popcll(m));   // first of its group
        }
    }
    __syncthreads();
    if (tid == 0) {
        uint32_t base = 0, tb = 0;
        for (int k = 0; k < count; ++k) {
            bucket_off[k] = base;
            cursor_s[k] = base;
            tile_base_s[k] = tb;
            base += total_s[k];
            tb += (total_s[k] + kTile - 1) / kTile;
        }
        bucket_off[count] = base;
        tile_base_s[count] = tb;
        *ntiles = tb;
    }
    __syncthreads();
    for (int k = 0; k < count; ++k) {
        const uint32_t nt = tile_base_s[k + 1] - tile_base_s[k];
        for (uint32_t t = tid; t < nt; t += kOrderThreads) {
            tiles[2 * (tile_base_s[k] + t)] = (cursor_s[k]) + t * kTile;
            tiles[2 * (tile_base_s[k] + t) + 1] = ((uint32_t)k << 8) | min((uint32_t)kTile, total_s[k] - t * kTile);
        }
    }
    // places, ascending position inside a bucket
    for (int b0 = 0; b0 < B; b0 += NB) {
        int cs[kOrderAhead];
        uint32_t rank[kOrderAhead];
#pragma unroll
        for (int u = 0; u < kOrderAhead; ++u) {
            const int b = b0 + u * kOrderThreads + tid;
            cs[u] = b0 == 0 ? first[u] : (b < B ? (int)bucket[b] : -1);
        }
        for (int i = tid; i < count * NS; i += kOrderThreads) cnt_s[i] = 0;
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kOrderAhead; ++u) {
            const bool valid = cs[u] >= 0 && cs[u] < count;
            const u64 m = same_bucket(cs[u], valid, nbits);
            rank[u] = (uint32_t)__popcll(m & lt);
            if (valid && rank[u] == 0) cnt_s[cs[u] * NS + u * NW + wave] = (uint32_t)__popcll(m);
        }
        __syncthreads();
        for (int k = wave; k < count; k += NW) {
            constexpr int PER = NS / 64;
            uint32_t v[PER], sum = 0;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                v[i] = cnt_s[k * NS + lane * PER + i];
                sum += v[i];
            }
            uint32_t incl = sum;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const uint32_t t = __shfl_up(incl, off);
                if (lane >= off) incl += t;
            }
            uint32_t run = cursor_s[k] + incl - sum;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                cnt_s[k * NS + lane * PER + i] = run;
                run += v[i];
            }
            if (lane == 63) cursor_s[k] = run;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kOrderAhead; ++u) {
            const int c = cs[u];
            if (c >= 0 && c < count)
                order[cnt_s[c * NS + u * NW + wave] + rank[u]] = (uint32_t)(b0 + u * kOrderThreads + tid);
        }
        __syncthreads();
    }
}

__device__ __forceinline__ f32x16 mfma4(const vecf<4>& a, const vecf<4>& b, f32x16 acc) {
#pragma unroll
    for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[s], b.v[s], acc, 0, 0, 0);
    return acc;
}

// row of the 32x32 result that accumulator register v of this lane holds
__device__ __forceinline__ int acc_row(int v, int lane) { return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3); }

// One workgroup per tile, KS waves; wave w walks columns [w * in / KS, (w + 1) * in / KS) of x and W
// eight at a time: lanes 0-31 supply the first four, lanes 32-63 the next four (the order of the
// terms of a dot product is free as long as both operands agree).
template <int KS>
__global__ __launch_bounds__(KS * 64) void k_bucket_fwd(const float* __restrict__ x, const float* __restrict__ W,
                                                         const float* __restrict__ bias, float* __restrict__ y,
                                                         const uint32_t* __restrict__ order,
                                                         const uint32_t* __restrict__ ntiles,
                                                         const uint32_t* __restrict__ tiles, int in, int out) {
    __shared__ float red[KS > 1 ? (KS - 1) * 16 * 64 : 1];
    const int t = blockIdx.x;
    if ((uint32_t)t >= *ntiles) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t start = tiles[2 * t], info = tiles[2 * t + 1];
    const int n = (int)(info & 255u), bk = (int)(info >> 8);
    const int r = lane & 31, h = lane >> 5;
    const uint32_t pos = order[start + (r < n ? r : 0)];
    const int kw = in / KS;
    const float* xa = x + (size_t)pos * in + wave * kw + 4 * h;
    const bool jok = r < out;
    const float* wb = W + ((size_t)bk * out + (jok ? r : 0)) * in + wave * kw + 4 * h;
    f32x16 acc = {0};
    constexpr int PF = 4;
    int k = 0;
    for (; k + 8 * PF <= kw; k += 8 * PF) {
        vecf<4> a[PF], b[PF];
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            a[u] = ldv<4>(xa + k + 8 * u);
            b[u] = ldv<4>(wb + k + 8 * u);
        }
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            if (!jok) b[u] = vzero<4>();
            acc = mfma4(a[u], b[u], acc);
        }
    }
    for (; k < kw; k += 8) {
        vecf<4> a = ldv<4>(xa + k), b = ldv<4>(wb + k);
        if (!jok) b = vzero<4>();
        acc = mfma4(a, b, acc);
    }
    if (KS > 1) {
        if (wave > 0) {
#pragma unroll
            for (int v = 0; v < 16; ++v) red[((wave - 1) * 16 + v) * 64 + lane] = acc[v];
        }
        __syncthreads();
        if (wave > 0) return;
        for (int w = 0; w < KS - 1; ++w)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] = acc[v] + red[(w * 16 + v) * 64 + lane];
    }
    if (!jok) return;
    const float bj = bias[bk * out + r];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int i = acc_row(v, lane);
        if (i < n) y[(size_t)order[start + i] * out + r] = acc[v] + bj;
    }
}

// The same for wide layers (in % (64 KS) == 0), with the tile of x taken through LDS.  The MFMA
// operand wants one row of x per lane, which as a global load touches 32 rows x 32 bytes per
// instruction; here a wave loads 4 rows x 256 contiguous bytes per instruction, parks 32 rows x 64
// columns in its own LDS strip and reads the operand layout back from there.  The terms of every
// dot product meet in the same order as in k_bucket_fwd, so the two kernels give the same bits.
template <int KS>
__global__ __launch_bounds__(KS * 64) void k_bucket_fwd_lds(const float* __restrict__ x, const float* __restrict__ W,
                                                             const float* __restrict__ bias, float* __restrict__ y,
                                                             const uint32_t* __restrict__ order,
                                                             const uint32_t* __restrict__ ntiles,
                                                             const uint32_t* __restrict__ tiles, int in, int out) {
    constexpr int CK = 64;          // columns per step
    constexpr int LD = CK + 4;      // padded row of the strip, floats
    constexpr int kStrip = 32 * LD;
    constexpr int kRed = KS > 1 ? (KS - 1) * 16 * 64 : 1;
    __shared__ __attribute__((aligned(16))) float lds[KS * kStrip > kRed ? KS * kStrip : kRed];
    const int t = blockIdx.x;
    if ((uint32_t)t >= *ntiles) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t start = tiles[2 * t], info = tiles[2 * t + 1];
    const int n = (int)(info & 255u), bk = (int)(info >> 8);
    const int r = lane & 31, h = lane >> 5;
    const int kw = in / KS;
    const int srow = lane >> 4, scol = 4 * (lane & 15);
    const float* xs[8];
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int i = srow + 4 * it;
        xs[it] = x + (size_t)order[start + (i < n ? i : 0)] * in + wave * kw + scol;
    }
    const bool jok = r < out;
    const float* wb = W + ((size_t)bk * out + (jok ? r : 0)) * in + wave * kw + 4 * h;
    float* strip = lds + wave * kStrip;
    f32x16 acc = {0};
    // the activations of step k + 1 (from HBM) are requested before the matrix operations of step k;
    // the weights (L2-resident) are requested at the top of their own step
    vecf<4> v[8], b[8];
#pragma unroll
    for (int it = 0; it < 8; ++it) v[it] = ldv4_stream(xs[it]);
    for (int k = 0; k < kw; k += CK) {
#pragma unroll
        for (int u = 0; u < 8; ++u) b[u] = ldv<4>(wb + k + 8 * u);
#pragma unroll
        for (int it = 0; it < 8; ++it) stv<4>(strip + (srow + 4 * it) * LD + scol, v[it]);
        __syncthreads();
        if (k + CK < kw) {
#pragma unroll
            for (int it = 0; it < 8; ++it) v[it] = ldv4_stream(xs[it] + k + CK);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const vecf<4> a = ldv<4>(strip + r * LD + 8 * u + 4 * h);
            if (!jok) b[u] = vzero<4>();
            acc = mfma4(a, b[u], acc);
        }
        __syncthreads();
    }
    if (KS > 1) {
        if (wave > 0) {
#pragma unroll
            for (int v = 0; v < 16; ++v) lds[((wave - 1) * 16 + v) * 64 + lane] = acc[v];
        }
        __syncthreads();
        if (wave > 0) return;
        for (int w = 0; w < KS - 1; ++w)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] = acc[v] + lds[(w * 16 + v) * 64 + lane];
    }
    if (!jok) return;
    const float bj = bias[bk * out + r];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int i = acc_row(v, lane);
        if (i < n) y[(size_t)order[start + i] * out + r] = acc[v] + bj;
    }
}

// gx[pos, c0 + 32 q + j] = sum_o gy[pos, o] * W_b[o, c0 + 32 q + j].  Workgroup = (tile, column range);
// lanes 0-31 supply outputs o = 0..15, lanes 32-63 o = 16..31.
__global__ __launch_bounds__(64) void k_bucket_bwd_x(const float* __restrict__ gy, const float* __restrict__ W,
                                                     float* __restrict__ gx, const uint32_t* __restrict__ order,
                                                     const uint32_t* __restrict__ ntiles,
                                                     const uint32_t* __restrict__ tiles, int in, int out, int nsplit) {
    const int t = blockIdx.x;
    if ((uint32_t)t >= *ntiles) return;
    const int lane = threadIdx.x;
    const uint32_t start = tiles[2 * t], info = tiles[2 * t + 1];
    const int n = (int)(info & 255u), bk = (int)(info >> 8);
    const int r = lane & 31, h = lane >> 5;
    const uint32_t pos = order[start + (r < n ? r : 0)];
    float a[16];
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        const int o = 16 * h + s;
        a[s] = (r < n && o < out) ? gy[(size_t)pos * out + o] : 0.0f;
    }
    uint32_t rowpos[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int i = acc_row(v, lane);
        rowpos[v] = i < n ? order[start + i] : 0xffffffffu;
    }
    const int nblk = in / 32;
    const int q0 = (int)((long long)blockIdx.y * nblk / nsplit), q1 = (int)((long long)(blockIdx.y + 1) * nblk / nsplit);
    const float* wb = W + (size_t)bk * out * in + r;
    for (int q = q0; q < q1; ++q) {
        float b[16];
#pragma unroll
        for (int s = 0; s < 16; ++s) {
            const int o = 16 * h + s;
            b[s] = o < out ? wb[(size_t)o * in + 32 * q] : 0.0f;
        }
        f32x16 acc = {0};
#pragma unroll
        for (int s = 0; s < 16; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
#pragma unroll
        for (int v = 0; v < 16; ++v)
            if (rowpos[v] != 0xffffffffu) gx[(size_t)rowpos[v] * in + 32 * q + r] = acc[v];
    }
}

// gW_b[o, c] = sum over the bucket's positions of gy[pos, o] * x[pos, c]; workgroup = (bucket, block of
// 64 columns), its KW waves take every KW-th run of 64 positions and their sums are added in wave
// order, so the result is the same on every run.  Two positions per MFMA step, lanes 0-31 the even
// one of the pair; the position numbers of a run arrive in one coalesced load.
constexpr int kBwdWaves = 8;
#ifndef NNUEFT_BWDW_PF
#define NNUEFT_BWDW_PF 32
#endif
#ifndef NNUEFT_BWDW_COLS
#define NNUEFT_BWDW_COLS 64
#endif
#ifndef NNUEFT_BWDW_WIDE_SPLITS
#define NNUEFT_BWDW_WIDE_SPLITS 2
#endif
constexpr int kBwdCols = NNUEFT_BWDW_COLS;   // 64 or 32 columns per workgroup
__global__ __launch_bounds__(kBwdWaves * 64) void k_bucket_bwd_w(const float* __restrict__ x,
                                                                 const float* __restrict__ gy,
                                                                 float* __restrict__ gW, float* __restrict__ gbias,
                                                                 const uint32_t* __restrict__ order,
                                                                 const uint32_t* __restrict__ bucket_off, int in,
                                                                 int out, int nsplit, int rows_total) {
    // nsplit > 1: workgroup z takes every nsplit-th group of kBwdWaves runs and writes its sums to
    // gW + z * rows_total * in (gbias + z * rows_total): partial results that k_bucket_bwd_w_sum adds up
    // in the order of z.  A narrow layer has too few (bucket, column block) pairs to fill the chip.
    __shared__ float red[(kBwdWaves - 1) * 33 * 64];
    const int bk = blockIdx.y, q = blockIdx.x, z = blockIdx.z;
    gW += (size_t)z * rows_total * in;
    gbias += (size_t)z * rows_total;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, h = lane >> 5;
    const uint32_t beg = bucket_off[bk], end = bucket_off[bk + 1];
    const bool ook = r < out;
    const int c0 = kBwdCols * q + r;
    const bool c1ok = kBwdCols == 64 && c0 + 32 < in;
    f32x16 acc0 = {0}, acc1 = {0};
    float bsum = 0.0f;
    for (uint32_t e0 = beg + 64u * (uint32_t)(z * kBwdWaves + wave); e0 < end; e0 += 64u * kBwdWaves * (uint32_t)nsplit) {
        const uint32_t mine = e0 + lane < end ? order[e0 + lane] : 0xffffffffu;
        constexpr int PF = NNUEFT_BWDW_PF;
#pragma unroll
        for (int u0 = 0; u0 < 32; u0 += PF) {
            float a[PF], b0[PF], b1[PF];
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                const uint32_t pe = (uint32_t)__builtin_amdgcn_readlane((int)mine, 2 * (u0 + u));
                const uint32_t po = (uint32_t)__builtin_amdgcn_readlane((int)mine, 2 * (u0 + u) + 1);
                const uint32_t pos = h ? po : pe;
                a[u] = 0.0f;
                b0[u] = 0.0f;
                b1[u] = 0.0f;
                if (pos != 0xffffffffu) {
                    if (ook) a[u] = gy[(size_t)pos * out + r];
                    b0[u] = x[(size_t)pos * in + c0];
                    if (c1ok) b1[u] = x[(size_t)pos * in + c0 + 32];
                }
            }
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b0[u], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b1[u], acc1, 0, 0, 0);
                bsum += a[u];
            }
        }
    }
    if (wave > 0) {
        float* dst = red + (size_t)(wave - 1) * 33 * 64;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            dst[v * 64 + lane] = acc0[v];
            dst[(16 + v) * 64 + lane] = acc1[v];
        }
        dst[32 * 64 + lane] = bsum;
    }
    __syncthreads();
    if (wave > 0) return;
    for (int w = 0; w < kBwdWaves - 1; ++w) {
        const float* src = red + (size_t)w * 33 * 64;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            acc0[v] = acc0[v] + src[v * 64 + lane];
            acc1[v] = acc1[v] + src[(16 + v) * 64 + lane];
        }
        bsum = bsum + src[32 * 64 + lane];
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int o = acc_row(v, lane);
        if (o < out) {
            gW[((size_t)bk * out + o) * in + c0] = acc0[v];
            if (c1ok) gW[((size_t)bk * out + o) * in + c0 + 32] = acc1[v];
        }
    }
    if (q == 0) {
        // even-position sums sit in lanes 0-31, odd ones in lanes 32-63
        const float other = __shfl_xor(bsum, 32);
        if (h == 0 && ook) gbias[bk * out + r] = bsum + other;
    }
}

// gW[i] = chain over the splits of part[z, i], likewise gbias; one thread per element.
__global__ __launch_bounds__(256) void k_bucket_bwd_w_sum(const float* __restrict__ part_w,
                                                          const float* __restrict__ part_b, float* __restrict__ gW,
                                                          float* __restrict__ gbias, int nw, int nb, int nsplit) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < nw) {
        float v[kBwdSplits];
#pragma unroll
        for (int z = 0; z < kBwdSplits; ++z) v[z] = z < nsplit ? part_w[(size_t)z * nw + i] : 0.0f;
        float t = v[0];
#pragma unroll
        for (int z = 1; z < kBwdSplits; ++z)
            if (z < nsplit) t = t + v[z];
        gW[i] = t;
    } else if (i - nw < nb) {
        const int j = i - nw;
        float t = part_b[j];
        for (int z = 1; z < nsplit; ++z) t = t + part_b[(size_t)z * nb + j];
        gbias[j] = t;
    }
}

int check_args(int B, int in, int out, int count) {
    if (B <= 0 || in <= 0 || out <= 0 || count <= 0) return NNUEFT_E_ARG;
    if (out > 32 || count > kMaxCount || in % 32 != 0) return NNUEFT_E_UNSUPPORTED;
    return 0;
}

int launch_order(const int64_t* bucket, char* ws, const BucketLayout& L, int B, int count, hipStream_t st) {
    // counts of a block in LDS: count x steps x waves words, at most 32 KB
    if (count <= 32) {
        const size_t lds = (size_t)count * 16 * (kOrderThreads / 64) * sizeof(uint32_t);
        hipLaunchKernelGGL(k_bucket_order<16>, dim3(1), dim3(kOrderThreads), lds, st, bucket,
                           (uint32_t*)(ws + L.order), (uint32_t*)(ws + L.bucket_off), (uint32_t*)(ws + L.ntiles),
                           (uint32_t*)(ws + L.tiles), B, count);
    } else {
        const size_t lds = (size_t)count * 4 * (kOrderThreads / 64) * sizeof(uint32_t);
        hipLaunchKernelGGL(k_bucket_order<4>, dim3(1), dim3(kOrderThreads), lds, st, bucket,
                           (uint32_t*)(ws + L.order), (uint32_t*)(ws + L.bucket_off), (uint32_t*)(ws + L.ntiles),
                           (uint32_t*)(ws + L.tiles), B, count);
    }
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

}  // namespace

extern "C" size_t nnueft_bucket_linear_workspace_bytes(int B, int count) {
    BucketLayout L;
    return bucket_layout(B, count, &L) ? L.end : 0;
}

extern "C" int nnueft_bucket_linear_group(const int64_t* bucket, int B, int count, void* workspace,
                                          size_t workspace_bytes, void* stream) {
    if (!bucket) return NNUEFT_E_ARG;
    BucketLayout L;
    if (!bucket_layout(B, count, &L)) return NNUEFT_E_ARG;
    if (!workspace || !aligned256(workspace) || workspace_bytes < L.end) return NNUEFT_E_WORKSPACE;
    return launch_order(bucket, (char*)workspace, L, B, count, (hipStream_t)stream);
}

extern "C" int nnueft_bucket_linear_fwd(const float* x, const int64_t* bucket, const float* W, const float* bias,
                                        float* y, int B, int in, int out, int count, void* workspace,
                                        size_t workspace_bytes, int workspace_grouped, void* stream) {
    const int bad = check_args(B, in, out, count);
    if (bad) return bad;
    if (!x || !bucket || !W || !bias || !y) return NNUEFT_E_ARG;
    if (!aligned16(x) || !aligned16(W)) return NNUEFT_E_UNSUPPORTED;
    BucketLayout L;
    if (!bucket_layout(B, count, &L)) return NNUEFT_E_ARG;
    if (!workspace || !aligned256(workspace) || workspace_bytes < L.end) return NNUEFT_E_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    char* ws = (char*)workspace;
    if (!workspace_grouped) {
        const int rc = launch_order(bucket, ws, L, B, count, st);
        if (rc) return rc;
    }
    const uint32_t* order = (const uint32_t*)(ws + L.order);
    const uint32_t* ntiles = (const uint32_t*)(ws + L.ntiles);
    const uint32_t* tiles = (const uint32_t*)(ws + L.tiles);
    if (in % 512 == 0 && in >= 1024 && aligned16(x) && aligned16(W))
        hipLaunchKernelGGL(k_bucket_fwd_lds<8>, dim3(L.max_tiles), dim3(512), 0, st, x, W, bias, y, order, ntiles,
                           tiles, in, out);
    else if (in % 256 == 0)
        hipLaunchKernelGGL(k_bucket_fwd<8>, dim3(L.max_tiles), dim3(512), 0, st, x, W, bias, y, order, ntiles, tiles, in,
                           out);
    else if (in % 128 == 0)
        hipLaunchKernelGGL(k_bucket_fwd<4>, dim3(L.max_tiles), dim3(256), 0, st, x, W, bias, y, order, ntiles, tiles, in,
                           out);
    else
        hipLaunchKernelGGL(k_bucket_fwd<1>, dim3(L.max_tiles), dim3(64), 0, st, x, W, bias, y, order, ntiles, tiles, in,
                           out);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

extern "C" int nnueft_bucket_linear_bwd(const float* x, const int64_t* bucket, const float* W, const float* gy,
                                        float* gx, float* gW, float* gbias, int B, int in, int out, int count,
                                        void* workspace, size_t workspace_bytes, int workspace_grouped,
                                        void* stream) {
    const int bad = check_args(B, in, out, count);
    if (bad) return bad;
    if (!x || !bucket || !W || !gy || !gW || !gbias) return NNUEFT_E_ARG;
    BucketLayout L;
    if (!bucket_layout(B, count, &L)) return NNUEFT_E_ARG;
    if (!workspace || !aligned256(workspace) || workspace_bytes < L.end) return NNUEFT_E_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    char* ws = (char*)workspace;
    if (!workspace_grouped) {
        const int rc = launch_order(bucket, ws, L, B, count, st);
        if (rc) return rc;
    }
    const uint32_t* order = (const uint32_t*)(ws + L.order);
    if (gx) {
        const int nblk = in / 32;
        const int nsplit = nblk >= 24 ? 8 : 1;
        hipLaunchKernelGGL(k_bucket_bwd_x, dim3(L.max_tiles, nsplit), dim3(64), 0, st, gy, W, gx, order,
                           (const uint32_t*)(ws + L.ntiles), (const uint32_t*)(ws + L.tiles), in, out, nsplit);
        NNUEFT_LAUNCH_CHECK();
    }
    const int colblocks = (in + kBwdCols - 1) / kBwdCols;
    const int rows_total = count * out;
    // too few (bucket, column block) pairs to fill the chip: several workgroups per pair, partial sums,
    // then their chain
    int nsplit = colblocks * count < 128 ? kBwdSplits : (colblocks * count < 1024 ? NNUEFT_BWDW_WIDE_SPLITS : 1);
    while (nsplit > 1 && (size_t)nsplit * rows_total * ((size_t)in + 1) * sizeof(float) > kPartialBytes) nsplit >>= 1;
    if (nsplit > 1) {
        float* part_w = (float*)(ws + L.partial);
        float* part_b = part_w + (size_t)nsplit * rows_total * in;
        hipLaunchKernelGGL(k_bucket_bwd_w, dim3(colblocks, count, nsplit), dim3(kBwdWaves * 64), 0, st, x, gy, part_w,
                           part_b, order, (const uint32_t*)(ws + L.bucket_off), in, out, nsplit, rows_total);
        NNUEFT_LAUNCH_CHECK();
        const int nw = rows_total * in, nb = rows_total;
        hipLaunchKernelGGL(k_bucket_bwd_w_sum, dim3((nw + nb + 255) / 256), dim3(256), 0, st, part_w, part_b, gW, gbias,
                           nw, nb, nsplit);
        NNUEFT_LAUNCH_CHECK();
        return 0;
    }
    hipLaunchKernelGGL(k_bucket_bwd_w, dim3(colblocks, count, 1), dim3(kBwdWaves * 64), 0, st, x, gy, gW, gbias, order,
                       (const uint32_t*)(ws + L.bucket_off), in, out, 1, rows_total);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}
