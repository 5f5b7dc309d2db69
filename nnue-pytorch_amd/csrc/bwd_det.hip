// Deterministic backward: a stable counting sort of the (table row, position) pairs of a batch,
// then a segmented reduction that writes every row of the weight gradient exactly once.
//
// Pipeline (all on the caller's stream, no host synchronisation):
//   k_bwd_rows      double only: per-position upstream rows G[2,B,out_cols] + bias partial sums
//   k_tile_colsum   sparse only: bias partial sums of gout
//   k_chunk_hist    per chunk of positions, how often each table row is named     cnt[chunk,row]
//   k_col_scan      exclusive scan of cnt over the chunks; per-row totals and white-perspective share
//   k_row_scan      exclusive scan of the totals -> segment offsets; work split for the reduction
//   k_fill          every slot writes its position id to its place: segment offset + chunk offset
//                   + rank inside the chunk, ranks taken position by position so the list of a
//                   row ends up in ascending (perspective, position) order
//   k_seg_reduce    persistent waves, one task = (table row, column slice): white chain, black
//                   chain, sum, store.  Rows are dealt to the 8 XCDs in contiguous ranges of equal
//                   work and walked one column slice at a time, so the upstream rows a XCD gathers
//                   (those of the positions of one king bucket, one slice wide) stay in its L2.
//                   A row named by more than NNUEFT_ROW_SPLIT slots (a king bucket that holds a
//                   large part of the batch has many) is cut at the window boundaries instead: one
//                   task per (row, perspective, window, slice) writes that window's sum, and a XCD
//                   takes whole (perspective, window) pairs, so what it gathers is one slice of
//                   one window's upstream rows.  The last columns of the rows (the 8 PSQT columns
//                   behind a whole number of 64-lane slices) are reduced 32 rows per wave
//   k_split_combine the window sums of a split row: chain over the windows, white + black; its first
//                   workgroups chain the tile partial sums of the bias gradient
//   k_bias_final    the same chain as a launch of its own where no row can be split (strict order)
#include <atomic>

#include <algorithm>
#include <cstdlib>

#include "gather.h"
#include "internal.h"

namespace {

#ifndef NNUEFT_SORT_CHUNK
#define NNUEFT_SORT_CHUNK 128
#endif
constexpr int kChunk = NNUEFT_SORT_CHUNK;        // positions per sort chunk
#ifndef NNUEFT_SEG_U
#define NNUEFT_SEG_U 8
#endif
#ifndef NNUEFT_SEG_NQ
#define NNUEFT_SEG_NQ 3
#endif
#ifndef NNUEFT_SEG_WAVES
#define NNUEFT_SEG_WAVES 320
#endif
constexpr int kRowsUnroll = NNUEFT_SEG_U;  // rows in flight per lane group in the segmented reduction
using nnueft_blocked::kXcd;
constexpr int kWavesPerXcd = NNUEFT_SEG_WAVES;  // persistent waves per XCD in the segmented reduction
#ifndef NNUEFT_LONG_ROW
#define NNUEFT_LONG_ROW 256
#endif
constexpr int kLongRow = NNUEFT_LONG_ROW;  // table rows named by at least this many slots are reduced first
#ifndef NNUEFT_FILL_U
#define NNUEFT_FILL_U 8
#endif
#ifndef NNUEFT_FILL_THREADS
#define NNUEFT_FILL_THREADS 1024
#endif
constexpr int kFillThreads = NNUEFT_FILL_THREADS;   // all of them load the cursors, one wave hands out the ranks
#ifndef NNUEFT_RUN_U
#define NNUEFT_RUN_U 32
#endif
// rows in flight per lane in the 64-lane-slice chains (window sums of split rows, long rows): a chain of thousands of
// slots is as many dependent steps as its slots over this number (16 -> 32: the strict order's reduction on game-like
// lists 1.02 -> 0.94 ms at L1 = 3072, 75 -> 67 us at L1 = 128; nothing elsewhere)
constexpr int kRunUnroll = NNUEFT_RUN_U;
#ifndef NNUEFT_TAIL_U
#define NNUEFT_TAIL_U 8
#endif
constexpr int kTailUnroll = NNUEFT_TAIL_U;
constexpr int kTailMax = 8;   // most trailing vectors that are handled that way  // slots in flight per lane where a wave reduces the last columns of many rows   // rows in flight per lane in the chain of one window of a split row
#ifndef NNUEFT_NARROW_AVG
#define NNUEFT_NARROW_AVG 64
#endif
constexpr int kNarrowAvg = NNUEFT_NARROW_AVG;   // slots per row of a XCD's row range from which it is walked in 64-lane slices
constexpr uint32_t kSplitFlag = 0x80000000u;   // on a row's slot count between k_col_scan and k_row_scan

// Work split of the segmented reduction, written by k_row_scan (uint32 words).
constexpr int kSchedCtr = 0;       // kXcd * kSchedQueues task counters, 32 words (128 bytes) apart
constexpr int kSchedQueues = 16;   // room for that many counters per XCD
constexpr int kSchedNLong = kXcd * kSchedQueues * 32;         // long_rows[0 .. n_long): long rows that are not split
constexpr int kSchedNSplit = kSchedNLong + 1;  // long_rows[R - n_split .. R), from the back: split rows, in three classes:
constexpr int kSchedNRemote = kSchedNSplit + 1;   // the first n_remote: window sums by (perspective, window) pair, any XCD
constexpr int kSchedNLocal = kSchedNRemote + 1;   // the next n_local: window sums inside their XCD's walk of its row range
                                                  // (the rest: more rows than there is room for window sums; reduced whole)
constexpr int kSchedRowSplit = kSchedNLocal + 1;  // the threshold the lists were sorted for
constexpr int kSchedRowLo = kSchedRowSplit + 1;   // kXcd + 1 range bounds
constexpr int kSchedLocalCnt = kSchedRowLo + kXcd + 1;   // kXcd counts: the local split rows of each XCD's range
// What the tables of the reduction out of LDS tiles were made for (0: they were not made, or not for these lists): set
// by that path's sort, cleared by k_row_scan, so that a reduction never reads tables that are not there.
constexpr int kSchedChainTag = kSchedLocalCnt + kXcd;
constexpr int kSchedWords = kSchedChainTag + 1;
// Window sums are kept for this many split rows at most (uniform positions split 32 rows, game-like ones a few hundred);
// further ones are reduced by one wave per 64-lane slice, window by window in the same order, so the bits are the same.
#ifndef NNUEFT_SPLIT_CAP
#define NNUEFT_SPLIT_CAP 384
#endif
constexpr int kSplitCap = NNUEFT_SPLIT_CAP;
constexpr int kLocalMax = 64;        // most local split rows per XCD (a wave keeps them one per lane)
// A split row is local only while its windows are short chains (this many slots a window on average, at most):
// inside the walk a window is one task at its row's place, and a long task late in the walk is a tail; the
// (perspective, window) path starts its tasks first and cuts them into 64-lane slices.  Measured on game-like
// lists at L1 = 1024, B = 8192 (rows of up to 256 slots a window local): reduction 121 -> 186 us.
#ifndef NNUEFT_LOCAL_PER_WINDOW
#define NNUEFT_LOCAL_PER_WINDOW 48
#endif
constexpr uint32_t kLocalPerWindow = NNUEFT_LOCAL_PER_WINDOW;

struct DetLayout {
    size_t G, partial, cnt, wcount, seg_off, long_rows, split_local, sched, list, chain, runs, end;
    bool chain_shape;   // the shape can take the strict-order reduction out of LDS tiles (its tables are in the sort block)
    size_t sort_begin, sort_end;   // cnt .. list: what the sort writes and the reduction reads (one block)
    int cpp;     // chunks per perspective
    int nchunks; // n_persp * cpp
    int ntiles;  // bias tiles
    int wch;     // chunks per window of a split row
    int nwin;    // windows
    int max_split;   // most rows that can be split
    int row_split;   // the threshold this layout was made for
};

inline size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

// row_split: a table row named by more slots than this is summed window by window; 0 = no row is.
// Floats from one upstream row of G to the next where the library lays G out itself (the two-perspective backward):
// whole 128-byte lines, so that a wave's 1 KB load touches 8 lines, not 9.
#ifndef NNUEFT_G_PAD
#define NNUEFT_G_PAD 1
#endif
inline int g_pitch_of(int out_cols) { return NNUEFT_G_PAD ? (out_cols + 31) / 32 * 32 : out_cols; }

bool det_layout(int B, int K, int R, int out_cols, int n_persp, int row_split, DetLayout* L) {
    if (B <= 0 || K <= 0 || R <= 0 || out_cols <= 0 || (n_persp != 1 && n_persp != 2) || row_split < 0) return false;
    L->row_split = row_split;
    L->cpp = (B + kChunk - 1) / kChunk;
    L->nchunks = n_persp * L->cpp;
    L->ntiles = (B + NNUEFT_BIAS_TILE - 1) / NNUEFT_BIAS_TILE;
    size_t off = 0;
    L->G = off;
    off += up256(n_persp == 2 ? (size_t)2 * B * g_pitch_of(out_cols) * sizeof(float) : 0);
    L->partial = off;
    off += up256((size_t)L->ntiles * out_cols * sizeof(float));
    L->sort_begin = off;
    L->cnt = off;
    off += up256((size_t)L->nchunks * R * sizeof(uint32_t));
    L->wcount = off;
    off += up256((size_t)R * sizeof(uint32_t));
    L->seg_off = off;
    off += up256(((size_t)R + 1) * sizeof(uint32_t));
    L->long_rows = off;
    off += up256((size_t)R * sizeof(uint32_t));
    L->split_local = off;
    off += up256((size_t)kXcd * kLocalMax * sizeof(uint32_t));
    L->sched = off;
    off += up256((size_t)kSchedWords * sizeof(uint32_t));
    L->list = off;
    off += up256((size_t)n_persp * B * K * sizeof(uint32_t));
    // the two-perspective backward in the strict order takes wide rows out of LDS tiles (bwd_chain.hip) where the
    // device allows; the tables of that path are part of what the sort writes (last, so that the other tables lie
    // at the same places whatever the threshold)
    L->chain = off;
    const size_t chain_bytes = n_persp == 2 && row_split == 0 ? nnueft_chain::shape_workspace(B, K, R, out_cols, n_persp) : 0;
    L->chain_shape = chain_bytes != 0;
    off += chain_bytes;
    L->sort_end = off;
    static_assert(NNUEFT_ROW_WINDOW_MIN % kChunk == 0, "windows are whole sort chunks");
    const int wpos = nnueft_window_positions(B);
    L->wch = wpos / kChunk;
    L->nwin = (B + wpos - 1) / wpos;
    const long long most = row_split > 0 ? ((long long)n_persp * B * K) / ((long long)row_split + 1) : 0;
    if (most > 0x3fffffffLL) return false;
    // window sums are kept for kSplitCap rows at most (and no table has more split rows than rows)
    L->max_split = (int)std::min<long long>(std::min<long long>(most, R), kSplitCap);
    L->runs = off;
    off += up256((size_t)L->max_split * n_persp * L->nwin * out_cols * sizeof(float));
    L->end = off;
    return true;
}

template <int VW>
__device__ __forceinline__ vecf<VW> ldv_once(const float* p) {
    if constexpr (VW == 4) return ldv4_stream(p);
    else return ldv<VW>(p);
}

// ---------------------------------------------------------------------------------------------
// Upstream rows of the two sparse-linear outputs of a position, and the bias partial sums.
// One wave per (tile of NNUEFT_BIAS_TILE positions, column slice); a lane keeps its columns and
// walks the tile's positions in order, which is the order of the bias chain.
template <int VW>
__global__ __launch_bounds__(64) void k_bwd_rows(const float* __restrict__ us, const float* __restrict__ them,
                                                 const int64_t* __restrict__ psqt_idx,
                                                 const float* __restrict__ bias, float max_act,
                                                 const float* __restrict__ grad_l0,
                                                 const float* __restrict__ grad_wpsqt,
                                                 const float* __restrict__ grad_bpsqt,
                                                 const float* __restrict__ saved, float* __restrict__ G,
                                                 float* __restrict__ partial, int B, int L1, int n_psqt, int group,
                                                 int ntiles, int nslices, int g_pitch) {
    // `group` lanes share a tile (64 for wide rows; narrow rows put 64 / group tiles into one wave)
    const int lane = threadIdx.x;
    const int s = blockIdx.x % nslices;          // launched 1-D: the slices of a tile are neighbours
    const int tile = (blockIdx.x / nslices) * (64 / group) + lane / group;
    const int ql = lane % group;
    if (tile >= ntiles) return;
    const int h = L1 >> 1;
    const int hv = h / VW;
    const size_t out_cols = (size_t)L1 + n_psqt;
    const int b0 = tile * NNUEFT_BIAS_TILE;
    const int b1 = min(b0 + NNUEFT_BIAS_TILE, B);
    float* Gw = G;
    float* Gb = G + (size_t)B * g_pitch;

    const int q = s * group + ql;
    if (q < hv) {
        const int c = q * VW;
        vecf<VW> part0 = vzero<VW>(), part1 = vzero<VW>();
        const vecf<VW> bias0 = ldv<VW>(bias + c), bias1 = ldv<VW>(bias + h + c);
        for (int b = b0; b < b1; ++b) {
            const float u = us[b], t = them[b];
            const float* sw = saved + (size_t)b * L1;
            const float* sb = saved + ((size_t)B + b) * L1;
            // read once: streaming loads, so they do not displace the rows the next kernel gathers
            const vecf<VW> sw0 = ldv_once<VW>(sw + c), sw1 = ldv_once<VW>(sw + h + c);
            const vecf<VW> sb0 = ldv_once<VW>(sb + c), sb1 = ldv_once<VW>(sb + h + c);
            const vecf<VW> g0 = ldv_once<VW>(grad_l0 + (size_t)b * L1 + c);
            const vecf<VW> g1 = ldv_once<VW>(grad_l0 + (size_t)b * L1 + h + c);
            vecf<VW> gw0, gw1, gb0, gb1;
#pragma unroll
            for (int i = 0; i < VW; ++i) {
                float xw0, xw1, xb0, xb1;
                mix4(u, t, sw0.v[i], sw1.v[i], sb0.v[i], sb1.v[i], bias0.v[i], bias1.v[i], xw0, xw1, xb0, xb1);
                grad4(u, t, xw0, xw1, xb0, xb1, g0.v[i], g1.v[i], max_act, gw0.v[i], gw1.v[i], gb0.v[i], gb1.v[i]);
                part0.v[i] = part0.v[i] + (gw0.v[i] + gb0.v[i]);
                part1.v[i] = part1.v[i] + (gw1.v[i] + gb1.v[i]);
            }
            stv<VW>(Gw + (size_t)b * g_pitch + c, gw0);
            stv<VW>(Gw + (size_t)b * g_pitch + h + c, gw1);
            stv<VW>(Gb + (size_t)b * g_pitch + c, gb0);
            stv<VW>(Gb + (size_t)b * g_pitch + h + c, gb1);
        }
        stv<VW>(partial + (size_t)tile * out_cols + c, part0);
        stv<VW>(partial + (size_t)tile * out_cols + h + c, part1);
    }
    if (s == 0) {
        for (int j = ql; j < n_psqt; j += group) {
            float part = 0.0f;
            for (int b = b0; b < b1; ++b) {
                const bool hit = psqt_idx[b] == (int64_t)j;
                const float gw = hit ? grad_wpsqt[b] : 0.0f;
                const float gb = hit ? grad_bpsqt[b] : 0.0f;
                Gw[(size_t)b * g_pitch + L1 + j] = gw;
                Gb[(size_t)b * g_pitch + L1 + j] = gb;
                part = part + (gw + gb);
            }
            partial[(size_t)tile * out_cols + L1 + j] = part;
        }
    }
}

// partial[tile, c] = chain over the tile's positions of gout[b, c]
__global__ __launch_bounds__(256) void k_tile_colsum(const float* __restrict__ gout, float* __restrict__ partial,
                                                     int B, int out_cols) {
    const int tile = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= out_cols) return;
    const int b0 = tile * NNUEFT_BIAS_TILE;
    const int b1 = min(b0 + NNUEFT_BIAS_TILE, B);
    float part = 0.0f;
    for (int b = b0; b < b1; ++b) part = part + gout[(size_t)b * out_cols + c];
    partial[(size_t)tile * out_cols + c] = part;
}

// gbias[c] = chain over the tiles of partial[tile, c].  The adds are one dependent chain; the loads
// are not, so they are issued a batch ahead.
__device__ __forceinline__ void bias_final_block(const float* __restrict__ partial, float* __restrict__ gbias,
                                                 int ntiles, int out_cols, uint32_t* __restrict__ sched, int block) {
    // the last kernel of the backward also rewinds the task counters, so the sorted lists can serve
    // another reduction (a second backward through the same graph)
    if (sched && block == 0)
        for (int i = threadIdx.x; i < kXcd * kSchedQueues; i += 64) sched[kSchedCtr + i * 32] = 0;
    if (!partial) return;   // the rows-only reduction: nothing but the rewind
    const int c = block * 64 + threadIdx.x;
    if (c >= out_cols) return;
    constexpr int PF = 64;
    float total = 0.0f;
    int t = 0;
    for (; t + PF <= ntiles; t += PF) {
        float v[PF];
#pragma unroll
        for (int u = 0; u < PF; ++u) v[u] = partial[(size_t)(t + u) * out_cols + c];
#pragma unroll
        for (int u = 0; u < PF; ++u) total = total + v[u];
    }
    for (; t < ntiles; ++t) total = total + partial[(size_t)t * out_cols + c];
    gbias[c] = total;
}

__global__ __launch_bounds__(64) void k_bias_final(const float* __restrict__ partial, float* __restrict__ gbias,
                                                   int ntiles, int out_cols, uint32_t* __restrict__ sched) {
    bias_final_block(partial, gbias, ntiles, out_cols, sched, (int)blockIdx.x);
}

// ---------------------------------------------------------------------------------------------
// Sort.  Chunk c covers positions [ (c % cpp) * kChunk, +kChunk ) of perspective c / cpp; chunks
// are numbered in the order their slots are to appear inside a row's list.  Table rows are
// handled `range` at a time so the per-chunk counters fit in LDS whatever R is.

__device__ __forceinline__ const int32_t* chunk_indices(const int32_t* widx, const int32_t* bidx, int c, int cpp,
                                                        int B, int K, int* pos0, int* npos, int* persp) {
    const int p = c / cpp;
    const int cc = c - p * cpp;
    *persp = p;
    *pos0 = cc * kChunk;
    *npos = min(kChunk, B - *pos0);
    return (p ? bidx : widx) + (size_t)(*pos0) * K;
}

__global__ __launch_bounds__(256) void k_chunk_hist(const int32_t* __restrict__ widx,
                                                    const int32_t* __restrict__ bidx, uint32_t* __restrict__ cnt,
                                                    int B, int K, int R, int cpp, int range, const uint32_t* __restrict__ only_if) {
    if (only_if && *only_if == 0) return;   // the batch went to the reduction out of LDS tiles
    extern __shared__ uint32_t lds_u32[];
    const int c = blockIdx.x;
    const int r0 = blockIdx.y * range;
    const int nr = min(range, R - r0);
    int pos0, npos, p;
    const int32_t* ix = chunk_indices(widx, bidx, c, cpp, B, K, &pos0, &npos, &p);
    for (int j = threadIdx.x; j < nr; j += 256) lds_u32[j] = 0;
    __syncthreads();
    const int nslots = npos * K;
    constexpr int PF = 16;   // index loads in flight per thread: a chunk of 128 lists of 32 is one batch
    for (int i0 = threadIdx.x; i0 < nslots; i0 += 256 * PF) {
        int rr[PF];
#pragma unroll
        for (int u = 0; u < PF; ++u) rr[u] = i0 + u * 256 < nslots ? ix[i0 + u * 256] - r0 : -1;
#pragma unroll
        for (int u = 0; u < PF; ++u)
            if (rr[u] >= 0 && rr[u] < nr) atomicAdd(&lds_u32[rr[u]], 1u);
    }
    __syncthreads();
    uint32_t* dst = cnt + (size_t)c * R + r0;
    if ((R & 3) == 0 && (r0 & 3) == 0 && (nr & 3) == 0) {
        const uint4* src4 = reinterpret_cast<const uint4*>(lds_u32);
        uint4* dst4 = reinterpret_cast<uint4*>(dst);
        for (int j = threadIdx.x; j < (nr >> 2); j += 256) dst4[j] = src4[j];
    } else {
        for (int j = threadIdx.x; j < nr; j += 256) dst[j] = lds_u32[j];
    }
}

// Per table row: chunk counts -> exclusive offsets; total and white share.
__global__ __launch_bounds__(64) void k_col_scan(uint32_t* __restrict__ cnt, uint32_t* __restrict__ wcount,
                                                 uint32_t* __restrict__ seg_off, int R, int cpp, int nchunks,
                                                 uint32_t row_split, const uint32_t* __restrict__ only_if) {
    if (only_if && *only_if == 0) return;   // the batch went to the reduction out of LDS tiles
    const int r = blockIdx.x * 64 + threadIdx.x;
    if (r >= R) return;
    constexpr int PF = 16;
    uint32_t run = 0, white = 0;
    int c = 0;
    for (; c + PF <= nchunks; c += PF) {
        uint32_t t[PF];
#pragma unroll
        for (int u = 0; u < PF; ++u) t[u] = cnt[(size_t)(c + u) * R + r];
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            if (c + u == cpp) white = run;
            cnt[(size_t)(c + u) * R + r] = run;
            run += t[u];
        }
    }
    for (; c < nchunks; ++c) {
        if (c == cpp) white = run;
        const uint32_t t = cnt[(size_t)c * R + r];
        cnt[(size_t)c * R + r] = run;
        run += t;
    }
    if (nchunks == cpp) white = run;
    wcount[r] = white;
    seg_off[r] = (row_split != 0 && run > row_split) ? (run | kSplitFlag) : run;
}

// floor(kXcd * w / denom) for w < denom, without a 64-bit division
__device__ __forceinline__ int xcd_of(unsigned long long w, unsigned long long denom) {
    int x = 0;
#pragma unroll
    for (int k = 1; k < kXcd; ++k) x += (w * kXcd >= (unsigned long long)k * denom) ? 1 : 0;
    return x;
}

// What a row's slots weigh less in its row range than their number: all of them for a split row (its windows
// are tasks of their own).  A row named by kHeavyRow slots or more sits in a table block that much of the batch
// names, where the upstream rows of a slice overflow the L2 and a slot costs a trip to memory: such slots count
// kHeavyFactor times (a negative return), so the XCDs that own crowded blocks get shorter ranges.
#ifndef NNUEFT_HEAVY_ROW
#define NNUEFT_HEAVY_ROW 64
#endif
#ifndef NNUEFT_HEAVY_F
#define NNUEFT_HEAVY_F 3
#endif
constexpr int kHeavyRow = NNUEFT_HEAVY_ROW;
constexpr int kHeavyFactor = NNUEFT_HEAVY_F;
__device__ __forceinline__ uint32_t slots_elsewhere(uint32_t raw) {
    const uint32_t len = raw & ~kSplitFlag;
    if (raw & kSplitFlag) return len;
    // (wraps below zero: the caller subtracts it, which adds the surcharge)
    if (len >= (uint32_t)kHeavyRow && len < (uint32_t)kLongRow) return 0u - len * (uint32_t)(kHeavyFactor - 1);
    return 0u;
}

// Single workgroup: seg_off (holding per-row totals) -> exclusive offsets, seg_off[R] = grand total.
// Also the work split of the segmented reduction: the split rows (flagged by k_col_scan), the other
// rows named by >= kLongRow slots (their chains are long and start first), and kXcd contiguous row
// ranges of equal weight (kRowWeight per row, plus its slots unless the row is split: those are
// reduced elsewhere).
#ifndef NNUEFT_ROW_WEIGHT
#define NNUEFT_ROW_WEIGHT 8
#endif
constexpr uint32_t kRowWeight = NNUEFT_ROW_WEIGHT;   // cost of a task that finds nothing to add, in slots
constexpr int kScanThreads = 1024;
constexpr int kLongClasses = 8;   // long rows by length: [kLongRow, 2 kLongRow), [2 kLongRow, 4 kLongRow), ...
__device__ __forceinline__ int long_class(uint32_t len) {
    const int c = (31 - __clz((int)(len / (uint32_t)kLongRow)));
    return c < kLongClasses - 1 ? c : kLongClasses - 1;
}
__global__ __launch_bounds__(kScanThreads) void k_row_scan(uint32_t* __restrict__ seg_off,
                                                           uint32_t* __restrict__ long_rows,
                                                           uint32_t* __restrict__ split_local,
                                                           uint32_t* __restrict__ sched, int R, int cap,
                                                           uint32_t row_split, uint32_t split_cap, uint32_t local_len, const uint32_t* __restrict__ only_if) {
    if (only_if && *only_if == 0) return;   // the batch went to the reduction out of LDS tiles
    extern __shared__ uint32_t stage[];   // `cap` row lengths, turned into offsets in place
    // two running sums: all slots, and what slots_elsewhere() takes off the weight of the row ranges
    __shared__ uint32_t wave_tot[2][kScanThreads / 64];
    __shared__ uint32_t carry_s[2], total_s[2], n_split_s;
    __shared__ uint32_t long_cnt[kLongClasses];
    __shared__ uint32_t lo_s[kXcd + 1];
    const int tid = threadIdx.x;
    if (tid == 0) {
        carry_s[0] = 0;
        carry_s[1] = 0;
        n_split_s = 0;
    }
    if (tid < kLongClasses) long_cnt[tid] = 0;
    if (tid <= kXcd) lo_s[tid] = (uint32_t)R;
    if (tid < kXcd * kSchedQueues) sched[kSchedCtr + tid * 32] = 0;
    // The row ranges need the two totals before the scan reaches the rows.  A table that fits the
    // staging buffer gets them from the scan's own first step; a larger one is summed here first.
    const bool one_pass = R <= cap;
    if (!one_pass) {
        uint32_t s0 = 0, s1 = 0;
        for (int i = tid; i < R; i += kScanThreads) {
            const uint32_t raw = seg_off[i];
            s0 += raw & ~kSplitFlag;
            s1 += slots_elsewhere(raw);
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            s0 += __shfl_down(s0, off);
            s1 += __shfl_down(s1, off);
        }
        if ((tid & 63) == 0) {
            wave_tot[0][tid >> 6] = s0;
            wave_tot[1][tid >> 6] = s1;
        }
        __syncthreads();
        if (tid < 2) {
            uint32_t t = 0;
            for (int w = 0; w < kScanThreads / 64; ++w) t += wave_tot[tid][w];
            total_s[tid] = t;
        }
    }
    __syncthreads();
    for (int base = 0; base < R; base += cap) {
        const int n = min(cap, R - base);
        // coalesced loads, 24 in flight per thread (a 24 576-row table is one batch)
        constexpr int PFS = 24;
        for (int i0 = tid; i0 < n; i0 += kScanThreads * PFS) {
            uint32_t v[PFS];
#pragma unroll
            for (int u = 0; u < PFS; ++u) v[u] = (i0 + u * kScanThreads < n) ? seg_off[base + i0 + u * kScanThreads] : 0;
#pragma unroll
            for (int u = 0; u < PFS; ++u)
                if (i0 + u * kScanThreads < n) stage[i0 + u * kScanThreads] = v[u];
        }
        __syncthreads();
        // a thread scans `per` consecutive rows (odd count: its LDS reads then spread over all banks)
        const int per = ((n + kScanThreads - 1) / kScanThreads) | 1;
        const int i_beg = min(tid * per, n), i_end = min(i_beg + per, n);
        uint32_t local[2] = {0, 0};
        for (int i = i_beg; i < i_end; ++i) {
            const uint32_t raw = stage[i];
            local[0] += raw & ~kSplitFlag;
            local[1] += slots_elsewhere(raw);
        }
        uint32_t incl[2] = {local[0], local[1]};
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const uint32_t t = __shfl_up(incl[k], off);
                if ((tid & 63) >= off) incl[k] += t;
            }
        }
        if ((tid & 63) == 63) {
            wave_tot[0][tid >> 6] = incl[0];
            wave_tot[1][tid >> 6] = incl[1];
        }
        __syncthreads();
        uint32_t run[2], all[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            run[k] = carry_s[k] + incl[k] - local[k];
            all[k] = 0;
            for (int w = 0; w < kScanThreads / 64; ++w) {
                const uint32_t x = wave_tot[k][w];
                if (w < (tid >> 6)) run[k] += x;
                all[k] += x;
            }
            if (!one_pass) all[k] = total_s[k];
        }
        // XCD of a row = floor(kXcd * weight of the rows before it / weight of all rows), weight =
        // kRowWeight + its slots (none for a split row, kHeavyFactor times for a heavy one); a range begins
        // where that number goes up
        const unsigned long long denom = (unsigned long long)(all[0] - all[1]) + (unsigned long long)R * kRowWeight;
        int x_cur = 0;
        if (i_beg < i_end) {
            x_cur = xcd_of((unsigned long long)(run[0] - run[1]) + (unsigned long long)(base + i_beg) * kRowWeight, denom);
            if (base + i_beg == 0)
                for (int k = 0; k <= x_cur; ++k) lo_s[k] = 0;
        }
        // 8 w >= thr  <=>  the rows before this one weigh at least (x_cur + 1) eighths of the total
        unsigned long long thr = (unsigned long long)(x_cur + 1) * denom;
        for (int i = i_beg; i < i_end; ++i) {
            const uint32_t raw = stage[i];
            const uint32_t len = raw & ~kSplitFlag;
            stage[i] = run[0];
            // a row is in at most one of the two lists, so they cannot meet inside long_rows[0..R)
            if (raw & kSplitFlag) {
                long_rows[R - 1 - (int)atomicAdd(&n_split_s, 1u)] = (uint32_t)(base + i);
            } else if (len >= (uint32_t)kLongRow) {
                atomicAdd(&long_cnt[long_class(len)], 1u);
            }
            run[1] += slots_elsewhere(raw);
            run[0] += len;
            const int r_next = base + i + 1;
            if (r_next < R) {
                const unsigned long long w8 =
                    ((unsigned long long)(run[0] - run[1]) + (unsigned long long)r_next * kRowWeight) * kXcd;
                while (x_cur < kXcd - 1 && w8 >= thr) {
                    lo_s[++x_cur] = (uint32_t)r_next;
                    thr += denom;
                }
            }
        }
        __syncthreads();
        if (tid == kScanThreads - 1) {
            carry_s[0] = run[0];
            carry_s[1] = run[1];
        }
        for (int i = tid; i < n; i += kScanThreads) seg_off[base + i] = stage[i];
        __syncthreads();
    }
    // The long rows, longest class first: their chains are the longest tasks of the reduction and are dealt to
    // the XCDs in this order.
    if (tid == 0) {
        seg_off[R] = carry_s[0];
        uint32_t at = 0;
        for (int c = kLongClasses - 1; c >= 0; --c) {
            const uint32_t n = long_cnt[c];
            long_cnt[c] = at;   // from here on the class's cursor
            at += n;
        }
        sched[kSchedNLong] = at;
        sched[kSchedNSplit] = n_split_s;
    }
    __syncthreads();
    const uint32_t total = carry_s[0];
    for (int i = tid; i < R; i += kScanThreads) {
        // (a table scanned in one pass still has its offsets staged in LDS)
        const uint32_t a = one_pass ? stage[i] : seg_off[i];
        const uint32_t b = i + 1 == R ? total : one_pass ? stage[i + 1] : seg_off[i + 1];
        const uint32_t len = b - a;
        if (len >= (uint32_t)kLongRow && !(row_split != 0 && len > row_split))
            long_rows[atomicAdd(&long_cnt[long_class(len)], 1u)] = (uint32_t)i;
    }
    if (tid <= kXcd) sched[kSchedRowLo + tid] = lo_s[tid];
    // The split rows in three classes (see kSchedNRemote).  A split row is local when its XCD's row range is
    // sparse (few slots per row: the range is walked in wide slices and the upstream rows its rows name stay in
    // that XCD's L2 meanwhile, the split row's among them), it is not too long, and the XCD has room for it.
    __shared__ uint32_t sparse_s[kXcd], loc_cnt_s[kXcd], n_remote_s, n_local_s, slot_s[2];
    if (tid < kXcd) {
        const uint32_t lo = lo_s[tid], hi = lo_s[tid + 1];
        const uint32_t a = lo >= (uint32_t)R ? total : one_pass ? stage[lo] : seg_off[lo];
        const uint32_t b = hi >= (uint32_t)R ? total : one_pass ? stage[hi] : seg_off[hi];
        sparse_s[tid] = hi > lo && (b - a) / (hi - lo) <= (uint32_t)kNarrowAvg;
        loc_cnt_s[tid] = 0;
    }
    if (tid == 0) {
        n_remote_s = 0;
        n_local_s = 0;
        slot_s[0] = 0;
        slot_s[1] = 0;
    }
    __syncthreads();
    const uint32_t n_split = n_split_s;
    constexpr int SPT = 4;   // split rows a thread classifies; beyond kScanThreads * SPT of them none is local
    uint32_t row_of[SPT];
    int cls[SPT];            // 0 remote, 1 local, 2 reduced whole
    int xcd_of_row[SPT];
    const bool classify = n_split <= (uint32_t)(kScanThreads * SPT);
#pragma unroll
    for (int u = 0; u < SPT; ++u) {
        const uint32_t k = (uint32_t)(tid + u * kScanThreads);
        cls[u] = -1;
        row_of[u] = 0;
        xcd_of_row[u] = 0;
        if (classify && k < n_split) {
            const uint32_t r = long_rows[R - 1 - (int)k];
            row_of[u] = r;
            int x = 0;
            for (int q = 1; q < kXcd; ++q) x += r >= lo_s[q] ? 1 : 0;
            xcd_of_row[u] = x;
            const uint32_t a = one_pass ? stage[r] : seg_off[r];
            const uint32_t b = r + 1 == (uint32_t)R ? total : one_pass ? stage[r + 1] : seg_off[r + 1];
            cls[u] = 0;
            if (sparse_s[x] && b - a <= local_len) {
                // room among the window sums and in the XCD's list (first come, first served: which rows are
                // local only moves work, never a bit of the result)
                if (atomicAdd(&n_local_s, 1u) < split_cap) {
                    if (atomicAdd(&loc_cnt_s[x], 1u) < (uint32_t)kLocalMax) cls[u] = 1;
                    else atomicSub(&n_local_s, 1u);
                } else {
                    atomicSub(&n_local_s, 1u);
                }
            }
        }
    }
    __syncthreads();
    const uint32_t n_local = min(n_local_s, split_cap);
    const uint32_t n_remote = classify ? min(n_split - n_local, split_cap - n_local) : min(n_split, split_cap);
    if (tid < kXcd) loc_cnt_s[tid] = 0;
    __syncthreads();
    if (classify) {
        // the list again, class by class: remote, local, whole
#pragma unroll
        for (int u = 0; u < SPT; ++u) {
            if (cls[u] < 0) continue;
            uint32_t slot;
            if (cls[u] == 1) {
                slot = n_remote + atomicAdd(&slot_s[1], 1u);
                split_local[xcd_of_row[u] * kLocalMax + (int)atomicAdd(&loc_cnt_s[xcd_of_row[u]], 1u)] = slot;
            } else {
                const uint32_t i = atomicAdd(&slot_s[0], 1u);
                slot = i < n_remote ? i : n_local + i;
            }
            long_rows[R - 1 - (int)slot] = row_of[u];
        }
    }
    __syncthreads();
    if (tid < kXcd) sched[kSchedLocalCnt + tid] = classify ? min(loc_cnt_s[tid], (uint32_t)kLocalMax) : 0u;
    if (tid == 0) {
        sched[kSchedNRemote] = n_remote;
        sched[kSchedNLocal] = classify ? n_local : 0u;
        sched[kSchedRowSplit] = row_split;
        sched[kSchedChainTag] = 0;
    }
}

// Every slot of the chunk writes its position id.  Ranks inside the chunk are handed out position
// by position (one LDS atomic per position and slot group), so a row's list is in position order.
// LDS: `range` cursors, then (when they fit) the chunk's index lists staged by all four waves.
__global__ __launch_bounds__(kFillThreads) void k_fill(const int32_t* __restrict__ widx, const int32_t* __restrict__ bidx,
                                              const uint32_t* __restrict__ cnt,
                                              const uint32_t* __restrict__ seg_off, uint32_t* __restrict__ list,
                                              int B, int K, int R, int cpp, int range, int stage, const uint32_t* __restrict__ only_if) {
    if (only_if && *only_if == 0) return;   // the batch went to the reduction out of LDS tiles
    extern __shared__ uint32_t lds_u32[];
    __shared__ uint32_t idle[64];
    if (threadIdx.x < 64) idle[threadIdx.x] = 0;
    const int c = blockIdx.x;
    const int r0 = blockIdx.y * range;
    const int nr = min(range, R - r0);
    int pos0, npos, p;
    const int32_t* ix = chunk_indices(widx, bidx, c, cpp, B, K, &pos0, &npos, &p);
    const uint32_t* coff = cnt + (size_t)c * R + r0;
    // cursors = segment offset + offset of this chunk inside the segment.  The workgroup waits for
    // every batch of loads, so the batches are made as large as registers allow: four rows per load
    // where the two arrays are 16-byte aligned, twelve loads of each array in flight per thread.
    if ((R & 3) == 0 && (r0 & 3) == 0 && (nr & 3) == 0) {
        constexpr int PF = 6;
        const uint4* so4 = reinterpret_cast<const uint4*>(seg_off + r0);
        const uint4* co4 = reinterpret_cast<const uint4*>(coff);
        uint4* lds4 = reinterpret_cast<uint4*>(lds_u32);
        const int nr4 = nr >> 2;
        for (int j0 = threadIdx.x; j0 < nr4; j0 += kFillThreads * PF) {
            uint4 a[PF], b[PF];
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                const int j = j0 + u * kFillThreads;
                if (j < nr4) {
                    a[u] = so4[j];
                    b[u] = co4[j];
                }
            }
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                const int j = j0 + u * kFillThreads;
                if (j < nr4) lds4[j] = make_uint4(a[u].x + b[u].x, a[u].y + b[u].y, a[u].z + b[u].z, a[u].w + b[u].w);
            }
        }
    } else {
        constexpr int PF = 8;
        for (int j0 = threadIdx.x; j0 < nr; j0 += kFillThreads * PF) {
            uint32_t a[PF], b[PF];
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                const int j = j0 + u * kFillThreads;
                a[u] = j < nr ? seg_off[r0 + j] : 0;
                b[u] = j < nr ? coff[j] : 0;
            }
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                const int j = j0 + u * kFillThreads;
                if (j < nr) lds_u32[j] = a[u] + b[u];
            }
        }
    }
    int32_t* staged = reinterpret_cast<int32_t*>(lds_u32 + range);
    if (stage)
        for (int i = threadIdx.x; i < npos * K; i += kFillThreads) staged[i] = ix[i];
    __syncthreads();
    if (threadIdx.x >= 64) return;
    const int lane = threadIdx.x;
    const uint32_t id0 = (uint32_t)p * (uint32_t)B + (uint32_t)pos0;
    if (K <= 64) {
        // One slot group per position.  LDS executes a wave's atomics in the order they were issued, so the ranks
        // of four positions are asked for before the first is needed; a lane with nothing to add adds 0 to a word
        // of its own, which keeps the four atomics free of branches.
        constexpr int U = NNUEFT_FILL_U;
        for (int i0 = 0; i0 < npos; i0 += U) {
            uint32_t* at[U];
            uint32_t one[U], slot[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int i = i0 + u;
                int r = -1;
                if (i < npos && lane < K) r = (stage ? staged[i * K + lane] : ix[(size_t)i * K + lane]) - r0;
                const bool ok = r >= 0 && r < nr;
                at[u] = ok ? &lds_u32[r] : &idle[lane];
                one[u] = ok ? 1u : 0u;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) slot[u] = atomicAdd(at[u], one[u]);
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (one[u]) list[slot[u]] = id0 + (uint32_t)(i0 + u);
        }
        return;
    }
    // all slot groups of a position before the next position
    for (int i = 0; i < npos; ++i) {
        for (int k0 = 0; k0 < K; k0 += 64) {
            int r = -1;
            if (k0 + lane < K) r = (stage ? staged[i * K + k0 + lane] : ix[(size_t)i * K + k0 + lane]) - r0;
            if (r >= 0 && r < nr) {
                const uint32_t slot = atomicAdd(&lds_u32[r], 1u);
                list[slot] = id0 + (uint32_t)i;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Segmented reduction.  list[seg_off[r] .. +wcount[r]) are the white-perspective rows of G naming
// table row r, the rest of the segment the black ones.  gW[r] = white chain (+ black chain).
// `pre`: the caller already holds list[beg + lane] of a segment of at most 64 slots in `pre_my`.
// The columns of a lane in slice s of slice_v vectors.
template <int VW, int NQ>
__device__ __forceinline__ void seg_cols(int (&col)[NQ], bool (&act)[NQ], int s, int lane, int out_cols, int slice_v) {
    const int nv = out_cols / VW;
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        const int w = m * 64 + lane;
        const int q = s * slice_v + w;
        act[m] = w < slice_v && q < nv;
        col[m] = act[m] ? q * VW : 0;
    }
}

// acc[0] = chain from +0 over list[beg .. mid), acc[1] = the same over list[mid .. end).
template <int VW, int NQ, int U>
__device__ __forceinline__ void seg_chains(vecf<VW> (&acc)[2][NQ], const float* __restrict__ G,
                                           const uint32_t* __restrict__ list, uint32_t beg, uint32_t mid, uint32_t end,
                                           const int (&col)[NQ], int lane, int g_pitch, bool pre = false, int pre_my = 0) {
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
        for (int m = 0; m < NQ; ++m) acc[p][m] = vzero<VW>();
    }
    if (pre) {
        const uint32_t nw = mid - beg, n = end - beg;
        const u64 all = n >= 64 ? ~0ull : ((1ull << n) - 1ull);
        const u64 white = nw >= 64 ? ~0ull : ((1ull << nw) - 1ull);
        chain_rows<VW, NQ, U>(acc[0], G, (size_t)g_pitch, col, pre_my, white);
        chain_rows<VW, NQ, U>(acc[1], G, (size_t)g_pitch, col, pre_my, all & ~white);
    } else {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const uint32_t e_beg = p ? mid : beg, e_end = p ? end : mid;
            for (uint32_t e0 = e_beg; e0 < e_end; e0 += 64) {
                const uint32_t n = min(64u, e_end - e0);
                const int my = lane < (int)n ? (int)list[e0 + lane] : 0;
                const u64 mask = n >= 64 ? ~0ull : ((1ull << n) - 1ull);
                chain_rows<VW, NQ, U>(acc[p], G, (size_t)g_pitch, col, my, mask);
            }
        }
    }
}

template <int VW, int NQ, int U>
__device__ __forceinline__ void seg_reduce_task(const float* __restrict__ G, const uint32_t* __restrict__ list,
                                                uint32_t beg, uint32_t mid, uint32_t end, float* __restrict__ dst,
                                                int s, int lane, int out_cols, int g_pitch, int slice_v, int two_persp,
                                                bool pre = false, int pre_my = 0) {
    int col[NQ];
    bool act[NQ];
    seg_cols<VW, NQ>(col, act, s, lane, out_cols, slice_v);
    vecf<VW> acc[2][NQ];
    seg_chains<VW, NQ, U>(acc, G, list, beg, mid, end, col, lane, g_pitch, pre, pre_my);
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        if (!act[m]) continue;
        if (two_persp) vadd<VW>(acc[0][m], acc[1][m]);
        stv_stream<VW>(dst + col[m], acc[0][m]);
    }
}

// The last few columns of a row (the 8 PSQT columns behind 3072 others) do not fill a slice of their own:
// a wave that walked one row's list for them would pay a whole task for 32 bytes per slot.  Here a wave
// takes 64 / g consecutive rows at once, g lanes per row, every lane group walking its own row's list
// (U slots in flight per lane, the next U list entries fetched meanwhile).  Same chains, same order.
template <int VW, int U>
__device__ __forceinline__ void tail_rows_task(const float* __restrict__ G, const uint32_t* __restrict__ list,
                                               const uint32_t* __restrict__ seg_off,
                                               const uint32_t* __restrict__ wcount, float* __restrict__ gW,
                                               uint32_t r0, uint32_t r1, int lane, int out_cols, int g_pitch, int tail_v,
                                               int g, int two_persp, uint32_t row_split) {
    const int sub = lane % g;
    const uint32_t row = r0 + (uint32_t)(lane / g);
    bool on = row < r1 && sub < tail_v;
    uint32_t bounds[3] = {0, 0, 0};
    if (on) {
        bounds[0] = seg_off[row];
        bounds[2] = seg_off[row + 1];
        bounds[1] = bounds[0] + wcount[row];
        const uint32_t len = bounds[2] - bounds[0];
        // long or split: done elsewhere, tail included
        if (len >= (uint32_t)kLongRow || (row_split != 0 && len > row_split)) on = false;
    }
    if (!on) bounds[0] = bounds[1] = bounds[2] = 0;
    const size_t col = (size_t)(out_cols / VW - tail_v + (on ? sub : 0)) * VW;
    const float* src = G + col;
    vecf<VW> acc[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        acc[p] = vzero<VW>();
        uint32_t e = bounds[p];
        const uint32_t e_end = bounds[p + 1];
        uint32_t nid[U];
#pragma unroll
        for (int u = 0; u < U; ++u) nid[u] = e + u < e_end ? list[e + u] : 0u;
        while (__any(e < e_end)) {
            vecf<VW> v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = e + u < e_end ? ldv<VW>(src + (size_t)nid[u] * g_pitch) : vzero<VW>();
#pragma unroll
            for (int u = 0; u < U; ++u) nid[u] = e + U + u < e_end ? list[e + U + u] : 0u;
            // a chain that started at +0 never holds -0, so adding the +0 of a lane that has run out changes no bit
#pragma unroll
            for (int u = 0; u < U; ++u) vadd<VW>(acc[p], v[u]);
            e += U;
        }
    }
    if (on) {
        if (two_persp) vadd<VW>(acc[0], acc[1]);
        stv_stream<VW>(gW + (size_t)row * out_cols + col, acc[0]);
    }
}

// Atomics on one address complete one after the other, some tens of nanoseconds each, so a single
// counter that every task of a XCD goes through bounds the run time of the kernel.  Each XCD
// therefore has kQueues counters; counter q hands out the tasks q, q + kQueues, q + 2 kQueues, ...
#ifndef NNUEFT_SEG_QUEUES
#define NNUEFT_SEG_QUEUES 8
#endif
constexpr int kQueues = NNUEFT_SEG_QUEUES;
__device__ __forceinline__ uint32_t next_task(uint32_t* ctr, int lane) {
    uint32_t t = 0;
    if (lane == 0) t = atomicAdd(ctr, 1u);
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)t);
}

// What the reduction needs to know about the windows of split rows.
struct RunPlan {
    const uint32_t* cnt;   // [nchunks, R] offset of a chunk inside the row's segment
    float* runs;           // [split row, perspective, window, out_cols] window sums
    int R, cpp, nchunks, wch, nwin, n_persp;
    int nslices, slice_v;  // 64-lane slices
    int tail_v, tail_g;    // trailing vectors of a row that tail_rows_task reduces (0: none), lanes per row there
    int g_pitch;           // floats from one row of G to the next
    uint32_t row_split;    // rows named by more slots than this are the split ones (0: none)
    const uint32_t* split_local;   // [kXcd, kLocalMax] the local split rows of each XCD, as places in the split list
};

// The window (perspective p, window w) of split row r: its part [beg, end) of the sorted list.
__device__ __forceinline__ void window_bounds(const RunPlan& rp, const uint32_t* __restrict__ seg_off, uint32_t r, uint32_t p,
                                              uint32_t w, uint32_t* beg, uint32_t* end) {
    const uint32_t c0 = p * (uint32_t)rp.cpp + w * (uint32_t)rp.wch;
    const uint32_t c1 = min(c0 + (uint32_t)rp.wch, (p + 1u) * (uint32_t)rp.cpp);
    const uint32_t seg = seg_off[r];
    *beg = seg + rp.cnt[(size_t)c0 * rp.R + r];
    *end = c1 == (uint32_t)rp.nchunks ? seg_off[r + 1] : seg + rp.cnt[(size_t)c1 * rp.R + r];
}

// A split row reduced whole by one wave per 64-lane slice: per perspective the chain over its windows of the window
// sums (each a chain from +0 over the window's slots), white + black: the order k_split_combine gives the rows whose
// window sums are kept, so the same bits.
template <int VW, int U>
__device__ __forceinline__ void split_row_whole(const RunPlan& rp, const float* __restrict__ G,
                                                const uint32_t* __restrict__ list, const uint32_t* __restrict__ seg_off,
                                                uint32_t r, float* __restrict__ dst, int s, int lane, int out_cols) {
    int col[1];
    bool act[1];
    seg_cols<VW, 1>(col, act, s, lane, out_cols, rp.slice_v);
    vecf<VW> tot = vzero<VW>();
    for (uint32_t p = 0; p < (uint32_t)rp.n_persp; ++p) {
        vecf<VW> run = vzero<VW>();
        for (uint32_t w = 0; w < (uint32_t)rp.nwin; ++w) {
            uint32_t beg, end;
            window_bounds(rp, seg_off, r, p, w, &beg, &end);
            vecf<VW> acc[2][1];
            seg_chains<VW, 1, U>(acc, G, list, beg, end, end, col, lane, rp.g_pitch);
            vadd<VW>(run, acc[0][0]);
        }
        if (p == 0) tot = run;
        else vadd<VW>(tot, run);
    }
    if (act[0]) stv_stream<VW>(dst + col[0], tot);
}

// Persistent waves.  A wave takes tasks from its home queue of its XCD, then from the XCD's other
// queues, until none is left (a counter only grows, so every wave leaves every loop).  Task order per XCD: the
// windows of the split rows, (perspective, window) pair after pair of those dealt to it, slice by
// slice; the long rows dealt to it (the 64-lane slices of a row together); then its row range, slice by slice.
template <int VW, int NQ>
__global__ __launch_bounds__(64) void k_seg_reduce(const float* __restrict__ G, const uint32_t* __restrict__ list,
                                                   const uint32_t* __restrict__ seg_off,
                                                   const uint32_t* __restrict__ wcount,
                                                   const uint32_t* __restrict__ long_rows,
                                                   uint32_t* __restrict__ sched, float* __restrict__ gW,
                                                   int out_cols, int nslices, int slice_v, int two_persp,
                                                   RunPlan rp, const uint32_t* __restrict__ only_if) {
    const int lane = threadIdx.x;
    const int xcd = blockIdx.x % kXcd;
    if (sched[kSchedRowSplit] != rp.row_split) return;   // the lists were sorted for another threshold
    // (asked behind the threshold: the flag lies in tables that only a sort for the strict order makes)
    if (only_if && *only_if == 0) return;   // the batch went to the reduction out of LDS tiles
    const uint32_t n_long = sched[kSchedNLong], n_split = sched[kSchedNSplit];
    const uint32_t n_remote = sched[kSchedNRemote], n_stored = n_remote + sched[kSchedNLocal];
    const uint32_t n_whole = n_split - n_stored;
    const uint32_t npairs = (uint32_t)(rp.n_persp * rp.nwin);
    const uint32_t my_pairs = npairs > (uint32_t)xcd ? (npairs - xcd + kXcd - 1) / kXcd : 0;
    const uint32_t pair_tasks = (uint32_t)rp.nslices * n_remote;
    const uint32_t run_tasks = my_pairs * pair_tasks;
    const uint32_t my_long = n_long > (uint32_t)xcd ? (n_long - xcd + kXcd - 1) / kXcd : 0;
    const uint32_t my_whole = n_whole > (uint32_t)xcd ? (n_whole - xcd + kXcd - 1) / kXcd : 0;
    const uint32_t lo = sched[kSchedRowLo + xcd], hi = sched[kSchedRowLo + xcd + 1];
    const uint32_t nreg = hi - lo;
    // long rows: 64-lane slices with kRunUnroll rows in flight (a chain of hundreds of slots is bound by how
    // many of its loads are in flight; three times as many waves share the row)
    const uint32_t long_slices = (uint32_t)rp.nslices;
    const uint32_t whole_end = run_tasks + my_whole * long_slices;
    const uint32_t long_end = whole_end + my_long * long_slices;
    // A range whose rows are named by many slots each belongs to a table block that a large part of
    // the batch sits in: one wide slice of all those positions' upstream rows would not fit the L2,
    // so such a range is walked in 64-lane slices (the results do not depend on the slicing).
    const uint32_t narrow_slices = (uint32_t)(rp.nslices - (rp.tail_v ? 1 : 0));   // the tail has tasks of its own
    const bool narrow = nreg > 0 && (seg_off[hi] - seg_off[lo]) / nreg > (uint32_t)kNarrowAvg && narrow_slices > (uint32_t)nslices;
    const uint32_t walk_slices = narrow ? narrow_slices : (uint32_t)nslices;
    const uint32_t tail_rows = rp.tail_v ? 64u / (uint32_t)rp.tail_g : 1u;
    const uint32_t tail_tasks = rp.tail_v ? (nreg + tail_rows - 1) / tail_rows : 0u;
    // The local split rows of this range, one per lane in row order: in the walk of a slice such a row stands for
    // npairs tasks, one per (perspective, window), at the row's place among the others (whose upstream rows are
    // those of the same positions, in this XCD's L2 at that time).
    const uint32_t nloc = min(sched[kSchedLocalCnt + xcd], (uint32_t)kLocalMax);
    uint32_t loc_r = 0xffffffffu, loc_j = 0, loc_pos = 0xffffffffu;
    if (nloc) {
        uint32_t my_j = 0, my_r = 0xffffffffu;
        if ((uint32_t)lane < nloc) {
            my_j = rp.split_local[xcd * kLocalMax + lane];
            my_r = long_rows[(uint32_t)rp.R - 1u - my_j];
        }
        uint32_t rank = 0;
        for (uint32_t k = 0; k < nloc; ++k) rank += (uint32_t)__builtin_amdgcn_readlane((int)my_r, (int)k) < my_r ? 1u : 0u;
        for (uint32_t q = 0; q < nloc; ++q) {
            const int src = __ffsll((long long)__ballot((uint32_t)lane < nloc && rank == q)) - 1;
            const uint32_t r = (uint32_t)__builtin_amdgcn_readlane((int)my_r, src);
            const uint32_t j = (uint32_t)__builtin_amdgcn_readlane((int)my_j, src);
            if ((uint32_t)lane == q) {
                loc_r = r;
                loc_j = j;
            }
        }
        if ((uint32_t)lane < nloc) loc_pos = (loc_r - lo) + (uint32_t)lane * (npairs - 1u);
    }
    const uint32_t nexp = nreg + nloc * (npairs - 1u);          // tasks of a slice of the walk
    const uint32_t walk_end = long_end + tail_tasks + nexp * walk_slices;
    const uint32_t loc_tail = rp.tail_v ? nloc * npairs : 0u;   // the trailing columns of the local rows' windows
    const uint32_t ntasks = walk_end + loc_tail;
    static_assert(kQueues <= kSchedQueues, "counters per XCD");
    const int home = (blockIdx.x / kXcd) % kQueues;

  for (int qi = 0; qi < kQueues; ++qi) {
    const uint32_t q = (uint32_t)((home + qi) % kQueues);
    uint32_t* ctr = sched + kSchedCtr + (xcd * kSchedQueues + (int)q) * 32;
    const uint32_t nq = ntasks > q ? (ntasks - q + kQueues - 1) / kQueues : 0;
    uint32_t next = next_task(ctr, lane);
    while (next < nq) {
        const uint32_t t = q + next * kQueues;
        next = next_task(ctr, lane);   // in flight while this task runs
        if (t < run_tasks) {
            const uint32_t pl = t / pair_tasks;
            const uint32_t rem = t - pl * pair_tasks;
            const uint32_t s = rem / n_remote;
            const uint32_t j = rem - s * n_remote;
            const uint32_t pair = (uint32_t)xcd + pl * kXcd;
            const uint32_t p = pair / (uint32_t)rp.nwin, w = pair - p * (uint32_t)rp.nwin;
            const uint32_t r = long_rows[(uint32_t)rp.R - 1u - j];
            uint32_t beg, end;
            window_bounds(rp, seg_off, r, p, w, &beg, &end);
            float* dst = rp.runs + ((size_t)(j * (uint32_t)rp.n_persp + p) * rp.nwin + w) * out_cols;
            seg_reduce_task<VW, 1, kRunUnroll>(G, list, beg, end, end, dst, (int)s, lane, out_cols, rp.g_pitch, rp.slice_v, 0);
            continue;
        }
        if (t < whole_end) {
            const uint32_t u = t - run_tasks;
            const uint32_t i = u / long_slices;
            const int s = (int)(u - i * long_slices);
            const uint32_t r = long_rows[(uint32_t)rp.R - 1u - (n_stored + (uint32_t)xcd + i * kXcd)];
            split_row_whole<VW, kRunUnroll>(rp, G, list, seg_off, r, gW + (size_t)r * out_cols, s, lane, out_cols);
            continue;
        }
        if (t < long_end) {
            const uint32_t u = t - whole_end;
            const uint32_t i = u / long_slices;
            const int s = (int)(u - i * long_slices);
            const uint32_t r = long_rows[xcd + i * kXcd];
            const uint32_t beg = seg_off[r], end = seg_off[r + 1];
            seg_reduce_task<VW, 1, kRunUnroll>(G, list, beg, beg + wcount[r], end, gW + (size_t)r * out_cols, s, lane,
                                               out_cols, rp.g_pitch, rp.slice_v, two_persp);
            continue;
        }
        uint32_t u = t - long_end;
        if (u < tail_tasks) {   // first: they are few and each is a long chain of short steps
            const uint32_t r0 = lo + u * tail_rows;
            tail_rows_task<VW, kTailUnroll>(G, list, seg_off, wcount, gW, r0, hi, lane, out_cols, rp.g_pitch, rp.tail_v, rp.tail_g,
                                            two_persp, rp.row_split);
            continue;
        }
        if (t >= walk_end) {
            // trailing columns of a local split row's window: the last 64-lane slice
            const uint32_t v = t - walk_end;
            const uint32_t i = v / npairs, pw = v - i * npairs;
            const uint32_t r = (uint32_t)__builtin_amdgcn_readlane((int)loc_r, (int)i);
            const uint32_t j = (uint32_t)__builtin_amdgcn_readlane((int)loc_j, (int)i);
            const uint32_t p = pw / (uint32_t)rp.nwin, w = pw - p * (uint32_t)rp.nwin;
            uint32_t beg, end;
            window_bounds(rp, seg_off, r, p, w, &beg, &end);
            float* dst = rp.runs + ((size_t)(j * (uint32_t)rp.n_persp + p) * rp.nwin + w) * out_cols;
            seg_reduce_task<VW, 1, kRunUnroll>(G, list, beg, end, end, dst, rp.nslices - 1, lane, out_cols, rp.g_pitch, rp.slice_v, 0);
            continue;
        }
        u -= tail_tasks;
        const int s = (int)(u / nexp);
        uint32_t v = u - (uint32_t)s * nexp;
        if (nloc) {
            // local rows that begin at or before place v of the slice
            const uint32_t k = (uint32_t)__popcll(__ballot(loc_pos <= v));
            if (k) {
                const uint32_t pos = (uint32_t)__builtin_amdgcn_readlane((int)loc_pos, (int)k - 1);
                if (v < pos + npairs) {
                    const uint32_t pw = v - pos;
                    const uint32_t r = (uint32_t)__builtin_amdgcn_readlane((int)loc_r, (int)k - 1);
                    const uint32_t j = (uint32_t)__builtin_amdgcn_readlane((int)loc_j, (int)k - 1);
                    const uint32_t p = pw / (uint32_t)rp.nwin, w = pw - p * (uint32_t)rp.nwin;
                    uint32_t beg, end;
                    window_bounds(rp, seg_off, r, p, w, &beg, &end);
                    float* dst = rp.runs + ((size_t)(j * (uint32_t)rp.n_persp + p) * rp.nwin + w) * out_cols;
                    if (narrow)
                        seg_reduce_task<VW, 1, kRunUnroll>(G, list, beg, end, end, dst, s, lane, out_cols, rp.g_pitch, rp.slice_v, 0);
                    else
                        seg_reduce_task<VW, NQ, kRowsUnroll>(G, list, beg, end, end, dst, s, lane, out_cols, rp.g_pitch, slice_v, 0);
                    continue;
                }
                v -= k * (npairs - 1u);
            }
        }
        const uint32_t r = lo + v;
        const uint32_t beg = seg_off[r], end = seg_off[r + 1];
        const uint32_t len = end - beg;
        // long or split: done elsewhere
        if (len >= (uint32_t)kLongRow || (rp.row_split != 0 && len > rp.row_split)) continue;
        // a segment of 64 slots at most: one load brings the white and the black part of the list
        const bool pre = len <= 64u;
        const int my = (pre && (uint32_t)lane < len) ? (int)list[beg + lane] : 0;
        float* dst = gW + (size_t)r * out_cols;
        if (narrow)
            seg_reduce_task<VW, 1, kRunUnroll>(G, list, beg, beg + wcount[r], end, dst, s, lane, out_cols, rp.g_pitch,
                                               rp.slice_v, two_persp, pre, my);
        else
            seg_reduce_task<VW, NQ, kRowsUnroll>(G, list, beg, beg + wcount[r], end, dst, s, lane, out_cols, rp.g_pitch,
                                                 slice_v, two_persp, pre, my);
    }
  }
}

// gW[r] of a split row = (chain over the windows of its white window sums) + (the same, black).
// One wave per (split row, 64-lane slice); an empty window's sum is +0, which changes no bit of a
// chain that started at +0.
// The first `nbias` workgroups of slice 0 are the last step of the bias gradient instead (and rewind the task
// counters): one launch less behind the reduction.
template <int VW>
__global__ __launch_bounds__(64) void k_split_combine(const uint32_t* __restrict__ long_rows,
                                                      uint32_t* __restrict__ sched, float* __restrict__ gW,
                                                      int out_cols, RunPlan rp, const float* __restrict__ partial,
                                                      float* __restrict__ gbias, int ntiles, int nbias) {
    const int lane = threadIdx.x;
    if (blockIdx.x < (unsigned)nbias) {
        // (every workgroup reads n_split below; the rewind touches the task counters only)
        if (blockIdx.y == 0) bias_final_block(partial, gbias, ntiles, out_cols, sched, (int)blockIdx.x);
        return;
    }
    if (sched[kSchedRowSplit] != rp.row_split) return;   // the lists were sorted for another threshold
    const uint32_t n_split = sched[kSchedNRemote] + sched[kSchedNLocal];   // the rows whose window sums were kept
    const int q = blockIdx.y * 64 + lane;
    if (q >= out_cols / VW) return;
    const int col = q * VW;
    const uint32_t stride = gridDim.x - (uint32_t)nbias;
    for (uint32_t j = blockIdx.x - (uint32_t)nbias; j < n_split; j += stride) {
        const uint32_t r = long_rows[(uint32_t)rp.R - 1u - j];
        vecf<VW> tot = vzero<VW>();
        for (int p = 0; p < rp.n_persp; ++p) {
            const float* src = rp.runs + (size_t)(j * (uint32_t)rp.n_persp + p) * rp.nwin * out_cols + col;
            vecf<VW> v[NNUEFT_ROW_WINDOWS];
#pragma unroll
            for (int w = 0; w < NNUEFT_ROW_WINDOWS; ++w)
                v[w] = w < rp.nwin ? ldv<VW>(src + (size_t)w * out_cols) : vzero<VW>();
            vecf<VW> acc = vzero<VW>();
#pragma unroll
            for (int w = 0; w < NNUEFT_ROW_WINDOWS; ++w)
                if (w < rp.nwin) vadd<VW>(acc, v[w]);
            if (p == 0) tot = acc;
            else vadd<VW>(tot, acc);
        }
        stv_stream<VW>(gW + (size_t)r * out_cols + col, tot);
    }
}

// Table rows per sort pass and whether the chunk's index lists are staged in LDS by k_fill.
bool lds_plan(int max_lds, int R, int K, int* range_out, int* stage_out, size_t* hist_bytes, size_t* fill_bytes) {
    if (max_lds < 16 * 1024) return false;
    // what the sort kernels declare statically (scan sums, counters, the spare words of k_fill) comes out of the
    // same budget as the dynamic part planned here
    constexpr int kStaticLds = 1024;
    max_lds -= kStaticLds;
    const size_t stage_bytes = (size_t)kChunk * K * sizeof(int32_t);
    const int stage = stage_bytes <= (size_t)max_lds / 4;
    const size_t avail = (size_t)max_lds - (stage ? stage_bytes : 0);
    int range = (int)(avail / sizeof(uint32_t));
    range = min(range, 32768);
    range = min(range, (R + 255) / 256 * 256);
    range = range / 256 * 256;
    if (range <= 0) return false;
    *range_out = range;
    *stage_out = stage;
    *hist_bytes = (size_t)range * sizeof(uint32_t);
    *fill_bytes = *hist_bytes + (stage ? stage_bytes : 0);
    return true;
}

// The three sort kernels may ask for all of a workgroup's LDS; that permission is a property of
// the loaded kernel on a device, so it is given once per device, on the first sort there.
constexpr int kMaxDevices = 64;
std::atomic<int> g_lds_allowed[kMaxDevices];

int allow_full_lds(int device, int max_lds) {
    if (device < 0 || device >= kMaxDevices) return NNUEFT_E_UNSUPPORTED;
    if (g_lds_allowed[device].load(std::memory_order_acquire) == max_lds) return 0;
    if (max_lds > 48 * 1024) {
        const void* kernels[3] = {(const void*)k_row_scan, (const void*)k_chunk_hist, (const void*)k_fill};
        for (const void* k : kernels) {
            // what a kernel declares statically comes out of the same budget
            hipFuncAttributes fa{};
            hipError_t e = hipFuncGetAttributes(&fa, k);
            if (e != hipSuccess) return (int)e;
            e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, max_lds - (int)fa.sharedSizeBytes);
            if (e != hipSuccess) return (int)e;
        }
    }
    g_lds_allowed[device].store(max_lds, std::memory_order_release);
    return 0;
}

// The sort: everything the reduction needs to know about the index lists (it reads no gradient).
// `sorted` is the block [L.sort_begin, L.sort_end) of the layout, wherever the caller keeps it.
// Whether this call takes the strict-order reduction out of LDS tiles: the shape and the threshold say so (the
// layout), and the device.
bool chain_in_use(const DetLayout& L, const nnueft_dev::DeviceInfo& d) {
    // NNUEFT_STRICT_LDS=0 in the environment keeps every batch on the segmented reduction (for comparing the two)
    static const bool enabled = [] {
        const char* e = getenv("NNUEFT_STRICT_LDS");
        return !(e && e[0] == '0');
    }();
    return enabled && L.chain_shape && L.row_split == 0 && nnueft_chain::device_ok(d);
}

int det_sort(const int32_t* widx, const int32_t* bidx, int B, int K, int R, int n_persp, char* sorted,
             const DetLayout& L, hipStream_t st) {
    char* ws = sorted - L.sort_begin;
    uint32_t* cnt = (uint32_t*)(ws + L.cnt);
    uint32_t* wcount = (uint32_t*)(ws + L.wcount);
    uint32_t* seg_off = (uint32_t*)(ws + L.seg_off);
    uint32_t* long_rows = (uint32_t*)(ws + L.long_rows);
    uint32_t* split_local = (uint32_t*)(ws + L.split_local);
    uint32_t* sched = (uint32_t*)(ws + L.sched);
    uint32_t* list = (uint32_t*)(ws + L.list);

    int device = 0;
    const nnueft_dev::DeviceInfo* info = nullptr;
    int rc = nnueft_dev::device_info(&device, &info);
    if (rc) return rc;
    int range = 0, stage = 0;
    size_t hist_bytes = 0, fill_bytes = 0;
    if (!lds_plan(info->max_lds, R, K, &range, &stage, &hist_bytes, &fill_bytes)) return NNUEFT_E_UNSUPPORTED;
    const int nranges = (R + range - 1) / range;
    // rows the single-workgroup row scan stages in LDS at a time (`range` fits by construction)
    const int scan_cap = max(kScanThreads, min(range, (R + kScanThreads - 1) / kScanThreads * kScanThreads));
    rc = allow_full_lds(device, info->max_lds);
    if (rc) return rc;
    // with the tables of the LDS-tiled reduction made first, the kernels below run only for a batch it cannot take
    const uint32_t* only_if = nullptr;
    if (chain_in_use(L, *info)) {
        rc = nnueft_chain::sort(widx, bidx, B, K, R, n_persp, ws + L.chain, sched + kSchedRowSplit, sched + kSchedChainTag, st);
        if (rc) return rc;
        only_if = nnueft_chain::fallback_flag(ws + L.chain, B, R, n_persp);
    }
    hipLaunchKernelGGL(k_chunk_hist, dim3(L.nchunks, nranges), dim3(256), hist_bytes, st, widx, bidx, cnt, B, K, R,
                       L.cpp, range, only_if);
    NNUEFT_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_col_scan, dim3((R + 63) / 64), dim3(64), 0, st, cnt, wcount, seg_off, R, L.cpp,
                       L.nchunks, (uint32_t)L.row_split, only_if);
    NNUEFT_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_row_scan, dim3(1), dim3(kScanThreads), (size_t)scan_cap * sizeof(uint32_t), st, seg_off,
                       long_rows, split_local, sched, R, scan_cap, (uint32_t)L.row_split, (uint32_t)L.max_split,
                       kLocalPerWindow * (uint32_t)(L.nchunks / L.cpp) * (uint32_t)L.nwin, only_if);
    NNUEFT_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_fill, dim3(L.nchunks, nranges), dim3(kFillThreads), fill_bytes, st, widx, bidx, cnt, seg_off, list,
                       B, K, R, L.cpp, range, stage, only_if);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

// The reduction over the sorted lists, and the last step of the bias gradient.
int det_reduce(const float* G, int g_pitch, float* gW, float* gbias, int B, int R, int out_cols, int n_persp, char* ws,
               char* sorted, const DetLayout& L, hipStream_t st) {
    char* sw = sorted - L.sort_begin;
    uint32_t* cnt = (uint32_t*)(sw + L.cnt);
    uint32_t* wcount = (uint32_t*)(sw + L.wcount);
    uint32_t* seg_off = (uint32_t*)(sw + L.seg_off);
    uint32_t* long_rows = (uint32_t*)(sw + L.long_rows);
    uint32_t* sched = (uint32_t*)(sw + L.sched);
    uint32_t* list = (uint32_t*)(sw + L.list);
    float* partial = (float*)(ws + L.partial);

    // the strict order out of LDS tiles where the sort made its tables; the kernels below then run only for a
    // batch that path could not take
    const uint32_t* only_if = nullptr;
    {
        int device = 0;
        const nnueft_dev::DeviceInfo* info = nullptr;
        int rc = nnueft_dev::device_info(&device, &info);
        if (rc) return rc;
        if (chain_in_use(L, *info) && g_pitch % 4 == 0 && aligned16(G)) {
            rc = nnueft_chain::reduce(G, g_pitch, gW, B, R, out_cols, n_persp, sw + L.chain, sched + kSchedChainTag, st);
            if (rc) return rc;
            only_if = nnueft_chain::fallback_flag(sw + L.chain, B, R, n_persp);
        } else if (chain_in_use(L, *info)) {
            return NNUEFT_E_UNSUPPORTED;   // the sort left the lists to the other path, which needs 16-byte rows
        }
    }
    const bool vec = (out_cols % 4 == 0) && (g_pitch % 4 == 0) && aligned16(G) && aligned16(gW);
    const int VWr = vec ? 4 : 1;
    const int nv = out_cols / VWr;
    const int NQ = nv > 64 ? NNUEFT_SEG_NQ : 1;
    // up to kTailMax vectors beyond a whole number of 64-lane slices are reduced many rows at a time
    int tail_v = (nv > 64 && nv % 64 <= kTailMax) ? nv % 64 : 0;
#ifdef NNUEFT_NO_TAIL
    tail_v = 0;
#endif
    int tail_g = 1;
    while (tail_g < tail_v) tail_g *= 2;
    const int nv_main = nv - tail_v;
    const int nslices = (nv_main + 64 * NQ - 1) / (64 * NQ);
    // equal slices, rounded up to whole 128-byte lines so no two waves share a cache line of a row
    const int line_v = 128 / (VWr * (int)sizeof(float));
    const int slice_v = ((nv_main + nslices - 1) / nslices + line_v - 1) / line_v * line_v;
    if ((long long)R * nslices > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
    const int two = n_persp == 2;
    RunPlan rp;
    rp.cnt = cnt;
    rp.runs = (float*)(ws + L.runs);
    rp.R = R;
    rp.cpp = L.cpp;
    rp.nchunks = L.nchunks;
    rp.wch = L.wch;
    rp.nwin = L.nwin;
    rp.n_persp = n_persp;
    rp.nslices = (nv + 63) / 64;
    // (with a tail: whole 64-lane slices and the tail as the last one, which the row ranges leave out)
    rp.slice_v = tail_v ? 64 : ((nv + rp.nslices - 1) / rp.nslices + line_v - 1) / line_v * line_v;
    rp.tail_v = tail_v;
    rp.tail_g = tail_g;
    rp.g_pitch = g_pitch;
    rp.row_split = (uint32_t)L.row_split;
    rp.split_local = (const uint32_t*)(sw + L.split_local);
    if ((long long)L.max_split * rp.nslices * NNUEFT_ROW_WINDOWS > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
#define SEG_LAUNCH(VW_, NQ_)                                                                                      \
    hipLaunchKernelGGL((k_seg_reduce<VW_, NQ_>), dim3(kXcd * kWavesPerXcd), dim3(64), 0, st, G, list, seg_off,      \
                       wcount, long_rows, sched, gW, out_cols, nslices, slice_v, two, rp, only_if)
    if (vec && NQ > 1) SEG_LAUNCH(4, NNUEFT_SEG_NQ);
    else if (vec) SEG_LAUNCH(4, 1);
    else if (NQ > 1) SEG_LAUNCH(1, NNUEFT_SEG_NQ);
    else SEG_LAUNCH(1, 1);
#undef SEG_LAUNCH
    NNUEFT_LAUNCH_CHECK();
    if (L.max_split > 0) {
        const int nbias = (out_cols + 63) / 64;
        const int ntiles = (B + NNUEFT_BIAS_TILE - 1) / NNUEFT_BIAS_TILE;
        const float* part = gbias ? partial : nullptr;
        const dim3 cgrid((unsigned)(nbias + min(L.max_split, 1024)), (unsigned)rp.nslices);
        if (vec)
            hipLaunchKernelGGL(k_split_combine<4>, cgrid, dim3(64), 0, st, long_rows, sched, gW, out_cols, rp, part,
                               gbias, ntiles, nbias);
        else
            hipLaunchKernelGGL(k_split_combine<1>, cgrid, dim3(64), 0, st, long_rows, sched, gW, out_cols, rp, part,
                               gbias, ntiles, nbias);
        NNUEFT_LAUNCH_CHECK();
        return 0;
    }
    return nnueft_det::launch_bias_final(gbias ? partial : nullptr, gbias, B, out_cols, sched, st);
}

}  // namespace

namespace nnueft_det {

constexpr long long kRowsScalarBelow = 2048;   // waves of 16-byte lanes below which k_bwd_rows uses 4-byte lanes

int launch_bwd_rows(const float* us, const float* them, const int64_t* psqt_idx, const float* bias, float max_act,
                    const float* grad_l0, const float* grad_wpsqt, const float* grad_bpsqt, const float* saved,
                    float* G, int g_pitch, float* partial, int B, int L1, int n_psqt, hipStream_t st) {
    const int out_cols = L1 + n_psqt;
    const int ntiles = (B + NNUEFT_BIAS_TILE - 1) / NNUEFT_BIAS_TILE;
    bool vec = (L1 % 8 == 0) && (out_cols % 4 == 0) && (g_pitch % 4 == 0) && aligned16(grad_l0) && aligned16(saved) &&
               aligned16(bias) && aligned16(G) && aligned16(partial);
    // a tile is one chain over its positions: with few tiles and narrow rows, 16-byte lanes leave most of the
    // chip without a wave; 4-byte lanes give four times the waves (config 2: 128 -> 512 waves, 44 -> 30 us)
    if (vec && (long long)ntiles * ((L1 / 8 + 63) / 64) < kRowsScalarBelow) vec = false;
    const int hv = (L1 / 2) / (vec ? 4 : 1);
    int group = 64;
    while (group > 8 && group / 2 >= hv) group /= 2;   // lanes per tile: 64, 32, 16 or 8
    const int tiles_per_wave = 64 / group;
    const int nslices = max(1, (hv + group - 1) / group);
    if ((long long)((ntiles + tiles_per_wave - 1) / tiles_per_wave) * nslices > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
    const dim3 grid((unsigned)((ntiles + tiles_per_wave - 1) / tiles_per_wave) * nslices);
    if (vec)
        hipLaunchKernelGGL(k_bwd_rows<4>, grid, dim3(64), 0, st, us, them, psqt_idx, bias, max_act, grad_l0,
                           grad_wpsqt, grad_bpsqt, saved, G, partial, B, L1, n_psqt, group, ntiles, nslices, g_pitch);
    else
        hipLaunchKernelGGL(k_bwd_rows<1>, grid, dim3(64), 0, st, us, them, psqt_idx, bias, max_act, grad_l0,
                           grad_wpsqt, grad_bpsqt, saved, G, partial, B, L1, n_psqt, group, ntiles, nslices, g_pitch);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

int launch_tile_colsum(const float* gout, float* partial, int B, int out_cols, hipStream_t st) {
    const int ntiles = (B + NNUEFT_BIAS_TILE - 1) / NNUEFT_BIAS_TILE;
    hipLaunchKernelGGL(k_tile_colsum, dim3(ntiles, (out_cols + 255) / 256), dim3(256), 0, st, gout, partial, B, out_cols);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

int launch_bias_final(const float* partial, float* gbias, int B, int out_cols, uint32_t* sched, hipStream_t st) {
    const int ntiles = (B + NNUEFT_BIAS_TILE - 1) / NNUEFT_BIAS_TILE;
    hipLaunchKernelGGL(k_bias_final, dim3((out_cols + 63) / 64), dim3(64), 0, st, partial, gbias, ntiles, out_cols,
                       sched);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

}  // namespace nnueft_det

extern "C" size_t nnueft_det_workspace_bytes(int B, int K, int R, int out_cols, int n_persp, int row_split) {
    DetLayout L;
    if (!det_layout(B, K, R, out_cols, n_persp, row_split, &L)) return 0;
    return L.end;
}

extern "C" size_t nnueft_det_sort_bytes(int B, int K, int R, int out_cols, int n_persp) {
    DetLayout L;
    if (!det_layout(B, K, R, out_cols, n_persp, 0, &L)) return 0;
    return L.sort_end - L.sort_begin;
}

extern "C" int nnueft_det_sort(const int32_t* widx, const int32_t* bidx, int B, int K, int R, int out_cols,
                               int n_persp, int row_split, void* sorted_lists, size_t sorted_bytes, void* stream) {
    if (!widx || (n_persp == 2 && !bidx)) return NNUEFT_E_ARG;
    if ((long long)B * K > 0x3fffffffLL || (long long)B > 0x3fffffffLL) return NNUEFT_E_UNSUPPORTED;
    DetLayout L;
    if (!det_layout(B, K, R, out_cols, n_persp, row_split, &L)) return NNUEFT_E_ARG;
    if (!sorted_lists || !aligned256(sorted_lists) || sorted_bytes < L.sort_end - L.sort_begin)
        return NNUEFT_E_WORKSPACE;
    return det_sort(widx, n_persp == 2 ? bidx : widx, B, K, R, n_persp, (char*)sorted_lists, L, (hipStream_t)stream);
}

extern "C" int nnueft_det_upstream_pitch(int out_cols) { return out_cols > 0 ? g_pitch_of(out_cols) : 0; }

extern "C" int nnueft_det_reduce_rows_pitched(const float* G, int g_pitch, float* gW, int B, int K, int R, int out_cols,
                                              int n_persp, int row_split, void* workspace, size_t workspace_bytes,
                                              void* sorted_lists, void* stream) {
    if (!G || !gW || g_pitch < out_cols) return NNUEFT_E_ARG;
    if ((long long)B * K > 0x3fffffffLL || (long long)B > 0x3fffffffLL) return NNUEFT_E_UNSUPPORTED;
    DetLayout L;
    if (!det_layout(B, K, R, out_cols, n_persp, row_split, &L)) return NNUEFT_E_ARG;
    if (!workspace || !aligned256(workspace) || workspace_bytes < L.end) return NNUEFT_E_WORKSPACE;
    if (!sorted_lists || !aligned256(sorted_lists)) return NNUEFT_E_WORKSPACE;
    return det_reduce(G, g_pitch, gW, nullptr, B, R, out_cols, n_persp, (char*)workspace, (char*)sorted_lists, L,
                      (hipStream_t)stream);
}

extern "C" int nnueft_det_reduce_rows(const float* G, float* gW, int B, int K, int R, int out_cols, int n_persp,
                                      int row_split, void* workspace, size_t workspace_bytes, void* sorted_lists,
                                      void* stream) {
    return nnueft_det_reduce_rows_pitched(G, out_cols, gW, B, K, R, out_cols, n_persp, row_split, workspace,
                                          workspace_bytes, sorted_lists, stream);
}

extern "C" int nnueft_sparse_bwd_det(const int32_t* idx, const float* gout, float* gW, float* gbias, int B, int K,
                                     int R, int out_cols, int row_split, void* workspace, size_t workspace_bytes,
                                     void* stream) {
    if (B <= 0 || K <= 0 || R <= 0 || out_cols <= 0 || row_split < 0) return NNUEFT_E_ARG;
    if (!idx || !gout || !gW || !gbias) return NNUEFT_E_ARG;
    if ((long long)B * K > 0x7fffffffLL || (long long)B > 0x3fffffffLL) return NNUEFT_E_UNSUPPORTED;
    DetLayout L;
    if (!det_layout(B, K, R, out_cols, 1, row_split, &L)) return NNUEFT_E_ARG;
    if (!workspace || !aligned256(workspace) || workspace_bytes < L.end) return NNUEFT_E_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    char* ws = (char*)workspace;
    hipLaunchKernelGGL(k_tile_colsum, dim3(L.ntiles, (out_cols + 255) / 256), dim3(256), 0, st, gout,
                       (float*)(ws + L.partial), B, out_cols);
    NNUEFT_LAUNCH_CHECK();
    const int rc = det_sort(idx, idx, B, K, R, 1, ws + L.sort_begin, L, st);
    if (rc) return rc;
    return det_reduce(gout, out_cols, gW, gbias, B, R, out_cols, 1, ws, ws + L.sort_begin, L, st);
}

extern "C" int nnueft_double_bwd_det(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                                     const int64_t* psqt_idx, const float* bias, float max_act,
                                     const float* grad_l0,
                                     const float* grad_wpsqt, const float* grad_bpsqt, const float* saved,
                                     float* gW, float* gbias, int B, int K, int R, int L1, int n_psqt, int row_split,
                                     void* workspace, size_t workspace_bytes, void* sorted_lists, void* stream,
                                     void* aux_stream) {
    if (B <= 0 || K <= 0 || R <= 0 || L1 <= 0 || (L1 & 1) || n_psqt < 0 || row_split < 0) return NNUEFT_E_ARG;
    if (!us || !them || !widx || !bidx || !psqt_idx || !bias || !grad_l0 || !grad_wpsqt || !grad_bpsqt || !saved ||
        !gW || !gbias)
        return NNUEFT_E_ARG;
    if ((long long)B * K > 0x3fffffffLL || (long long)B > 0x3fffffffLL) return NNUEFT_E_UNSUPPORTED;
    const int out_cols = L1 + n_psqt;
    DetLayout L;
    if (!det_layout(B, K, R, out_cols, 2, row_split, &L)) return NNUEFT_E_ARG;
    if (!workspace || !aligned256(workspace) || workspace_bytes < L.end) return NNUEFT_E_WORKSPACE;
    if (sorted_lists && !aligned256(sorted_lists)) return NNUEFT_E_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    char* ws = (char*)workspace;
    float* G = (float*)(ws + L.G);
    float* partial = (float*)(ws + L.partial);
    // The sort reads only the index lists, the upstream rows only the activations: with a second
    // stream they run side by side and meet before the reduction.
    hipStream_t aux = (hipStream_t)aux_stream;
    const bool two_streams = aux && aux != st;
    hipEvent_t forked = nullptr, joined = nullptr;
    if (two_streams) {
        int device = 0;
        const nnueft_dev::DeviceInfo* info = nullptr;
        int rc = nnueft_dev::device_info(&device, &info);
        if (rc == 0) rc = nnueft_dev::thread_events(device, &forked, &joined);
        if (rc) return rc;
    }
    if (sorted_lists) {
        // the caller ran nnueft_det_sort on these lists already; if on aux_stream, it may still be
        // running there: only the reduction has to wait for it, the upstream rows do not
        const int rc = nnueft_det::launch_bwd_rows(us, them, psqt_idx, bias, max_act, grad_l0, grad_wpsqt, grad_bpsqt,
                                                   saved, G, g_pitch_of(out_cols), partial, B, L1, n_psqt, st);
        if (rc) return rc;
        if (two_streams) {
            hipError_t e = hipEventRecord(joined, aux);
            if (e == hipSuccess) e = hipStreamWaitEvent(st, joined, 0);
            if (e != hipSuccess) return (int)e;
        }
        return det_reduce(G, g_pitch_of(out_cols), gW, gbias, B, R, out_cols, 2, ws, (char*)sorted_lists, L, st);
    }
    if (two_streams) {
        hipError_t e = hipEventRecord(forked, st);
        if (e == hipSuccess) e = hipStreamWaitEvent(aux, forked, 0);
        if (e != hipSuccess) return (int)e;
    }
    int rc = det_sort(widx, bidx, B, K, R, 2, ws + L.sort_begin, L, two_streams ? aux : st);
    hipError_t sorted = hipSuccess;
    if (two_streams) sorted = hipEventRecord(joined, aux);
    // the upstream rows go onto the caller's stream before it is made to wait for the sort
    if (rc == 0)
        rc = nnueft_det::launch_bwd_rows(us, them, psqt_idx, bias, max_act, grad_l0, grad_wpsqt, grad_bpsqt, saved, G,
                                         g_pitch_of(out_cols), partial, B, L1, n_psqt, st);
    if (two_streams) {
        // always rejoin, also after a failed launch: the caller's stream must not run ahead of the other one
        if (sorted == hipSuccess) sorted = hipStreamWaitEvent(st, joined, 0);
        if (rc == 0 && sorted != hipSuccess) rc = (int)sorted;
    }
    if (rc) return rc;
    return det_reduce(G, g_pitch_of(out_cols), gW, gbias, B, R, out_cols, 2, ws, ws + L.sort_begin, L, st);
}
