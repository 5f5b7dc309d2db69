// Deterministic backward: a stable counting sort of the (table row, position) pairs of a batch,
// then a segmented reduction that writes every row of the weight gradient exactly once.
//
// Pipeline (all on the caller's stream, no host synchronisation):
//   k_bwd_rows      double only: per-position upstream rows G[2,B,out_cols] + bias partial sums
//   k_tile_colsum   sparse only: bias partial sums of gout
//   k_chunk_hist    per chunk of positions, how often each table row is named     cnt[chunk,row]
//   k_col_scan      exclusive scan of cnt over the chunks; per-row totals and white-perspective share
//   k_row_scan      exclusive scan of the totals -> segment offsets; rows ordered longest first
//   k_fill          every slot writes its position id to its place: segment offset + chunk offset
//                   + rank inside the chunk, ranks taken position by position so the list of a
//                   row ends up in ascending (perspective, position) order
//   k_seg_reduce    one wave per (row, column slice): white chain, black chain, sum, store
//   k_bias_final    chain over the tile partial sums
#include "gather.h"

namespace {

constexpr int kChunk = 128;        // positions per sort chunk
constexpr int kRowsUnroll = 8;     // rows in flight per lane group in the segmented reduction

struct DetLayout {
    size_t G, partial, cnt, wcount, seg_off, row_order, list, end;
    int cpp;     // chunks per perspective
    int nchunks; // n_persp * cpp
    int ntiles;  // bias tiles
};

inline size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

bool det_layout(int B, int K, int R, int out_cols, int n_persp, DetLayout* L) {
    if (B <= 0 || K <= 0 || R <= 0 || out_cols <= 0 || (n_persp != 1 && n_persp != 2)) return false;
    L->cpp = (B + kChunk - 1) / kChunk;
    L->nchunks = n_persp * L->cpp;
    L->ntiles = (B + NNUEFT_BIAS_TILE - 1) / NNUEFT_BIAS_TILE;
    size_t off = 0;
    L->G = off;
    off += up256(n_persp == 2 ? (size_t)2 * B * out_cols * sizeof(float) : 0);
    L->partial = off;
    off += up256((size_t)L->ntiles * out_cols * sizeof(float));
    L->cnt = off;
    off += up256((size_t)L->nchunks * R * sizeof(uint32_t));
    L->wcount = off;
    off += up256((size_t)R * sizeof(uint32_t));
    L->seg_off = off;
    off += up256(((size_t)R + 1) * sizeof(uint32_t));
    L->row_order = off;
    off += up256((size_t)R * sizeof(uint32_t));
    L->list = off;
    off += up256((size_t)n_persp * B * K * sizeof(uint32_t));
    L->end = off;
    return true;
}

// ---------------------------------------------------------------------------------------------
// Upstream rows of the two sparse-linear outputs of a position, and the bias partial sums.
// One wave per (tile of NNUEFT_BIAS_TILE positions, column slice); a lane keeps its columns and
// walks the tile's positions in order, which is the order of the bias chain.
template <int VW>
__global__ __launch_bounds__(64) void k_bwd_rows(const float* __restrict__ us, const float* __restrict__ them,
                                                 const int64_t* __restrict__ psqt_idx, float max_act,
                                                 const float* __restrict__ grad_l0,
                                                 const float* __restrict__ grad_wpsqt,
                                                 const float* __restrict__ grad_bpsqt,
                                                 const float* __restrict__ saved, float* __restrict__ G,
                                                 float* __restrict__ partial, int B, int L1, int n_psqt) {
    const int lane = threadIdx.x;
    const int tile = blockIdx.x;
    const int s = blockIdx.y;
    const int h = L1 >> 1;
    const int hv = h / VW;
    const size_t out_cols = (size_t)L1 + n_psqt;
    const int b0 = tile * NNUEFT_BIAS_TILE;
    const int b1 = min(b0 + NNUEFT_BIAS_TILE, B);
    float* Gw = G;
    float* Gb = G + (size_t)B * out_cols;

    const int q = s * 64 + lane;
    if (q < hv) {
        const int c = q * VW;
        vecf<VW> part0 = vzero<VW>(), part1 = vzero<VW>();
        for (int b = b0; b < b1; ++b) {
            const float u = us[b], t = them[b];
            const float* sv = saved + (size_t)b * 2 * L1;
            const vecf<VW> xw0 = ldv<VW>(sv + c), xw1 = ldv<VW>(sv + h + c);
            const vecf<VW> xb0 = ldv<VW>(sv + 2 * h + c), xb1 = ldv<VW>(sv + 3 * h + c);
            const vecf<VW> g0 = ldv<VW>(grad_l0 + (size_t)b * L1 + c);
            const vecf<VW> g1 = ldv<VW>(grad_l0 + (size_t)b * L1 + h + c);
            vecf<VW> gw0, gw1, gb0, gb1;
#pragma unroll
            for (int i = 0; i < VW; ++i) {
                const float cw0 = clamp_act(xw0.v[i], max_act), cw1 = clamp_act(xw1.v[i], max_act);
                const float cb0 = clamp_act(xb0.v[i], max_act), cb1 = clamp_act(xb1.v[i], max_act);
                const float dw0 = (xw0.v[i] >= 0.0f && xw0.v[i] <= max_act) ? g0.v[i] * cw1 : 0.0f;
                const float dw1 = (xw1.v[i] >= 0.0f && xw1.v[i] <= max_act) ? g0.v[i] * cw0 : 0.0f;
                const float db0 = (xb0.v[i] >= 0.0f && xb0.v[i] <= max_act) ? g1.v[i] * cb1 : 0.0f;
                const float db1 = (xb1.v[i] >= 0.0f && xb1.v[i] <= max_act) ? g1.v[i] * cb0 : 0.0f;
                gw0.v[i] = u * dw0 + t * db0;
                gw1.v[i] = u * dw1 + t * db1;
                gb0.v[i] = t * dw0 + u * db0;
                gb1.v[i] = t * dw1 + u * db1;
                part0.v[i] = part0.v[i] + (gw0.v[i] + gb0.v[i]);
                part1.v[i] = part1.v[i] + (gw1.v[i] + gb1.v[i]);
            }
            stv<VW>(Gw + (size_t)b * out_cols + c, gw0);
            stv<VW>(Gw + (size_t)b * out_cols + h + c, gw1);
            stv<VW>(Gb + (size_t)b * out_cols + c, gb0);
            stv<VW>(Gb + (size_t)b * out_cols + h + c, gb1);
        }
        stv<VW>(partial + (size_t)tile * out_cols + c, part0);
        stv<VW>(partial + (size_t)tile * out_cols + h + c, part1);
    }
    if (s == 0) {
        for (int j = lane; j < n_psqt; j += 64) {
            float part = 0.0f;
            for (int b = b0; b < b1; ++b) {
                const bool hit = psqt_idx[b] == (int64_t)j;
                const float gw = hit ? grad_wpsqt[b] : 0.0f;
                const float gb = hit ? grad_bpsqt[b] : 0.0f;
                Gw[(size_t)b * out_cols + L1 + j] = gw;
                Gb[(size_t)b * out_cols + L1 + j] = gb;
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
__global__ __launch_bounds__(64) void k_bias_final(const float* __restrict__ partial, float* __restrict__ gbias,
                                                   int ntiles, int out_cols) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c >= out_cols) return;
    constexpr int PF = 32;
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
                                                    int B, int K, int R, int cpp, int range) {
    extern __shared__ uint32_t lds_u32[];
    const int c = blockIdx.x;
    const int r0 = blockIdx.y * range;
    const int nr = min(range, R - r0);
    int pos0, npos, p;
    const int32_t* ix = chunk_indices(widx, bidx, c, cpp, B, K, &pos0, &npos, &p);
    for (int j = threadIdx.x; j < nr; j += 256) lds_u32[j] = 0;
    __syncthreads();
    const int nslots = npos * K;
    for (int i = threadIdx.x; i < nslots; i += 256) {
        const int r = ix[i] - r0;
        if (r >= 0 && r < nr) atomicAdd(&lds_u32[r], 1u);
    }
    __syncthreads();
    uint32_t* dst = cnt + (size_t)c * R + r0;
    for (int j = threadIdx.x; j < nr; j += 256) dst[j] = lds_u32[j];
}

// Per table row: chunk counts -> exclusive offsets; total and white share.
__global__ __launch_bounds__(64) void k_col_scan(uint32_t* __restrict__ cnt, uint32_t* __restrict__ wcount,
                                                 uint32_t* __restrict__ seg_off, int R, int cpp, int nchunks) {
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
    seg_off[r] = run;
}

// Single workgroup: seg_off (holding per-row totals) -> exclusive offsets, seg_off[R] = grand total;
// row_order = table rows by descending list length (length clipped to kLenBins-1 for the ordering),
// so the longest chains start first.
constexpr int kScanThreads = 1024;
constexpr int kLenBins = 1024;
constexpr int kScanPer = 32;   // rows a thread keeps in registers per pass
__global__ __launch_bounds__(kScanThreads) void k_row_scan(uint32_t* __restrict__ seg_off,
                                                           uint32_t* __restrict__ row_order, int R) {
    __shared__ uint32_t sums[kScanThreads];
    __shared__ uint32_t bins[kLenBins];
    __shared__ uint32_t carry_s;
    const int tid = threadIdx.x;
    if (tid < kLenBins) bins[tid] = 0;
    if (tid == 0) carry_s = 0;
    __syncthreads();
    // pass A: length histogram (for the longest-first order)
    for (int rb = tid; rb < R; rb += kScanThreads * 8) {
        uint32_t len[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) len[u] = (rb + u * kScanThreads < R) ? seg_off[rb + u * kScanThreads] : 0;
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (rb + u * kScanThreads < R) atomicAdd(&bins[min(len[u], (uint32_t)(kLenBins - 1))], 1u);
    }
    __syncthreads();
    // bins -> first slot of each length class, longest class first
    if (tid < kLenBins) sums[tid] = bins[kLenBins - 1 - tid];
    __syncthreads();
    for (int d = 1; d < kLenBins; d <<= 1) {
        uint32_t add = 0;
        if (tid < kLenBins && tid >= d) add = sums[tid - d];
        __syncthreads();
        if (tid < kLenBins) sums[tid] += add;
        __syncthreads();
    }
    if (tid < kLenBins) bins[kLenBins - 1 - tid] = sums[tid] - bins[kLenBins - 1 - tid];
    __syncthreads();
    // pass B: exclusive scan of the lengths, kScanThreads * kScanPer rows at a time
    for (int base = 0; base < R; base += kScanThreads * kScanPer) {
        const int r0 = base + tid * kScanPer;
        uint32_t len[kScanPer];
        uint32_t local = 0;
#pragma unroll
        for (int u = 0; u < kScanPer; ++u) {
            len[u] = (r0 + u < R) ? seg_off[r0 + u] : 0;
            local += len[u];
        }
        sums[tid] = local;
        __syncthreads();
        for (int d = 1; d < kScanThreads; d <<= 1) {
            const uint32_t add = tid >= d ? sums[tid - d] : 0;
            __syncthreads();
            sums[tid] += add;
            __syncthreads();
        }
        uint32_t run = carry_s + sums[tid] - local;
        const uint32_t block_total = sums[kScanThreads - 1];
#pragma unroll
        for (int u = 0; u < kScanPer; ++u) {
            if (r0 + u < R) {
                const uint32_t slot = atomicAdd(&bins[min(len[u], (uint32_t)(kLenBins - 1))], 1u);
                row_order[slot] = (uint32_t)(r0 + u);
                seg_off[r0 + u] = run;
                run += len[u];
            }
        }
        __syncthreads();
        if (tid == 0) carry_s += block_total;
        __syncthreads();
    }
    if (tid == 0) seg_off[R] = carry_s;
}

// Every slot of the chunk writes its position id.  Ranks inside the chunk are handed out position
// by position (one LDS atomic per position and slot group), so a row's list is in position order.
// LDS: `range` cursors, then (when they fit) the chunk's index lists staged by all four waves.
__global__ __launch_bounds__(256) void k_fill(const int32_t* __restrict__ widx, const int32_t* __restrict__ bidx,
                                              const uint32_t* __restrict__ cnt,
                                              const uint32_t* __restrict__ seg_off, uint32_t* __restrict__ list,
                                              int B, int K, int R, int cpp, int range, int stage) {
    extern __shared__ uint32_t lds_u32[];
    const int c = blockIdx.x;
    const int r0 = blockIdx.y * range;
    const int nr = min(range, R - r0);
    int pos0, npos, p;
    const int32_t* ix = chunk_indices(widx, bidx, c, cpp, B, K, &pos0, &npos, &p);
    const uint32_t* coff = cnt + (size_t)c * R + r0;
    {
        // cursors = segment offset + offset of this chunk inside the segment; loads batched 8 deep
        constexpr int PF = 8;
        for (int j0 = threadIdx.x; j0 < nr; j0 += 256 * PF) {
            uint32_t a[PF], b[PF];
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                const int j = j0 + u * 256;
                a[u] = j < nr ? seg_off[r0 + j] : 0;
                b[u] = j < nr ? coff[j] : 0;
            }
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                const int j = j0 + u * 256;
                if (j < nr) lds_u32[j] = a[u] + b[u];
            }
        }
    }
    int32_t* staged = reinterpret_cast<int32_t*>(lds_u32 + range);
    if (stage)
        for (int i = threadIdx.x; i < npos * K; i += 256) staged[i] = ix[i];
    __syncthreads();
    if (threadIdx.x >= 64) return;
    const int lane = threadIdx.x;
    const uint32_t id0 = (uint32_t)p * (uint32_t)B + (uint32_t)pos0;
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
// Segmented reduction.  One wave per (table row, column slice); rows are taken longest first.
// list[seg_off[r] .. +wcount[r]) are the white-perspective rows of G, the rest of the segment the
// black ones.  gW[r] = white chain (+ black chain when two perspectives).
template <int VW, int NQ>
__global__ __launch_bounds__(64) void k_seg_reduce(const float* __restrict__ G, const uint32_t* __restrict__ list,
                                                   const uint32_t* __restrict__ seg_off,
                                                   const uint32_t* __restrict__ wcount,
                                                   const uint32_t* __restrict__ row_order,
                                                   float* __restrict__ gW, int out_cols, int nslices,
                                                   int slice_v, int two_persp) {
    const int lane = threadIdx.x;
    const int ro = blockIdx.x / nslices;
    const int s = blockIdx.x - ro * nslices;
    const int r = (int)row_order[ro];
    const int nv = out_cols / VW;

    int col[NQ];
    bool act[NQ];
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        const int w = m * 64 + lane;
        const int q = s * slice_v + w;
        act[m] = w < slice_v && q < nv;
        col[m] = act[m] ? q * VW : 0;
    }
    const uint32_t beg = seg_off[r], end = seg_off[r + 1];
    const uint32_t mid = beg + wcount[r];

    vecf<VW> acc[2][NQ];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
        for (int m = 0; m < NQ; ++m) acc[p][m] = vzero<VW>();
        const uint32_t e_beg = p ? mid : beg, e_end = p ? end : mid;
        for (uint32_t e0 = e_beg; e0 < e_end; e0 += 64) {
            const uint32_t n = min(64u, e_end - e0);
            const int my = lane < (int)n ? (int)list[e0 + lane] : 0;
            const u64 mask = n >= 64 ? ~0ull : ((1ull << n) - 1ull);
            chain_rows<VW, NQ, kRowsUnroll>(acc[p], G, (size_t)out_cols, col, my, mask);
        }
    }
    float* dst = gW + (size_t)r * out_cols;
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        if (!act[m]) continue;
        if (two_persp) vadd<VW>(acc[0][m], acc[1][m]);
        stv<VW>(dst + col[m], acc[0][m]);
    }
}

// Table rows per sort pass and whether the chunk's index lists are staged in LDS by k_fill.
bool lds_plan(int R, int K, int* range_out, int* stage_out, size_t* hist_bytes, size_t* fill_bytes) {
    int dev = 0, max_lds = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    if (hipDeviceGetAttribute(&max_lds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) return false;
    if (max_lds < 16 * 1024) return false;
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

// Common tail of the two deterministic entry points.
int det_sort_reduce(const int32_t* widx, const int32_t* bidx, const float* G, float* gW, float* gbias, int B,
                    int K, int R, int out_cols, int n_persp, char* ws, const DetLayout& L, hipStream_t st) {
    uint32_t* cnt = (uint32_t*)(ws + L.cnt);
    uint32_t* wcount = (uint32_t*)(ws + L.wcount);
    uint32_t* seg_off = (uint32_t*)(ws + L.seg_off);
    uint32_t* row_order = (uint32_t*)(ws + L.row_order);
    uint32_t* list = (uint32_t*)(ws + L.list);
    float* partial = (float*)(ws + L.partial);

    int range = 0, stage = 0;
    size_t hist_bytes = 0, fill_bytes = 0;
    if (!lds_plan(R, K, &range, &stage, &hist_bytes, &fill_bytes)) return NNUEFT_E_UNSUPPORTED;
    const int nranges = (R + range - 1) / range;
    if (fill_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)k_chunk_hist, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)hist_bytes);
        if (e != hipSuccess) return (int)e;
        e = hipFuncSetAttribute((const void*)k_fill, hipFuncAttributeMaxDynamicSharedMemorySize, (int)fill_bytes);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(k_chunk_hist, dim3(L.nchunks, nranges), dim3(256), hist_bytes, st, widx, bidx, cnt, B, K, R,
                       L.cpp, range);
    NNUEFT_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_col_scan, dim3((R + 63) / 64), dim3(64), 0, st, cnt, wcount, seg_off, R, L.cpp,
                       L.nchunks);
    NNUEFT_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_row_scan, dim3(1), dim3(kScanThreads), 0, st, seg_off, row_order, R);
    NNUEFT_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_fill, dim3(L.nchunks, nranges), dim3(256), fill_bytes, st, widx, bidx, cnt, seg_off, list,
                       B, K, R, L.cpp, range, stage);
    NNUEFT_LAUNCH_CHECK();

    const bool vec = (out_cols % 4 == 0) && aligned16(G) && aligned16(gW);
    const int VWr = vec ? 4 : 1;
    const int nv = out_cols / VWr;
    const int NQ = nv > 64 ? 2 : 1;
    const int nslices = (nv + 64 * NQ - 1) / (64 * NQ);
    // equal slices, rounded up to whole 128-byte lines so no two waves share a cache line of a row
    const int line_v = 128 / (VWr * (int)sizeof(float));
    const int slice_v = ((nv + nslices - 1) / nslices + line_v - 1) / line_v * line_v;
    const long long grid = (long long)R * nslices;
    if (grid > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
    const int two = n_persp == 2;
#define SEG_LAUNCH(VW_, NQ_)                                                                                    \
    hipLaunchKernelGGL((k_seg_reduce<VW_, NQ_>), dim3((unsigned)grid), dim3(64), 0, st, G, list, seg_off, wcount, \
                       row_order, gW, out_cols, nslices, slice_v, two)
    if (vec && NQ == 2) SEG_LAUNCH(4, 2);
    else if (vec) SEG_LAUNCH(4, 1);
    else if (NQ == 2) SEG_LAUNCH(1, 2);
    else SEG_LAUNCH(1, 1);
#undef SEG_LAUNCH
    NNUEFT_LAUNCH_CHECK();

    hipLaunchKernelGGL(k_bias_final, dim3((out_cols + 63) / 64), dim3(64), 0, st, partial, gbias, L.ntiles,
                       out_cols);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

}  // namespace

extern "C" size_t nnueft_det_workspace_bytes(int B, int K, int R, int out_cols, int n_persp) {
    DetLayout L;
    if (!det_layout(B, K, R, out_cols, n_persp, &L)) return 0;
    return L.end;
}

extern "C" int nnueft_sparse_bwd_det(const int32_t* idx, const float* gout, float* gW, float* gbias, int B, int K,
                                     int R, int out_cols, void* workspace, size_t workspace_bytes, void* stream) {
    if (B <= 0 || K <= 0 || R <= 0 || out_cols <= 0) return NNUEFT_E_ARG;
    if (!idx || !gout || !gW || !gbias) return NNUEFT_E_ARG;
    if ((long long)B * K > 0x7fffffffLL || (long long)B > 0x3fffffffLL) return NNUEFT_E_UNSUPPORTED;
    DetLayout L;
    if (!det_layout(B, K, R, out_cols, 1, &L)) return NNUEFT_E_ARG;
    if (!workspace || !aligned256(workspace) || workspace_bytes < L.end) return NNUEFT_E_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    char* ws = (char*)workspace;
    hipLaunchKernelGGL(k_tile_colsum, dim3(L.ntiles, (out_cols + 255) / 256), dim3(256), 0, st, gout,
                       (float*)(ws + L.partial), B, out_cols);
    NNUEFT_LAUNCH_CHECK();
    return det_sort_reduce(idx, idx, gout, gW, gbias, B, K, R, out_cols, 1, ws, L, st);
}

extern "C" int nnueft_double_bwd_det(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                                     const int64_t* psqt_idx, float max_act, const float* grad_l0,
                                     const float* grad_wpsqt, const float* grad_bpsqt, const float* saved,
                                     float* gW, float* gbias, int B, int K, int R, int L1, int n_psqt,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    if (B <= 0 || K <= 0 || R <= 0 || L1 <= 0 || (L1 & 1) || n_psqt < 0) return NNUEFT_E_ARG;
    if (!us || !them || !widx || !bidx || !psqt_idx || !grad_l0 || !grad_wpsqt || !grad_bpsqt || !saved || !gW ||
        !gbias)
        return NNUEFT_E_ARG;
    if ((long long)B * K > 0x3fffffffLL || (long long)B > 0x3fffffffLL) return NNUEFT_E_UNSUPPORTED;
    const int out_cols = L1 + n_psqt;
    DetLayout L;
    if (!det_layout(B, K, R, out_cols, 2, &L)) return NNUEFT_E_ARG;
    if (!workspace || !aligned256(workspace) || workspace_bytes < L.end) return NNUEFT_E_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    char* ws = (char*)workspace;
    float* G = (float*)(ws + L.G);
    const bool vec = (L1 % 8 == 0) && (out_cols % 4 == 0) && aligned16(grad_l0) && aligned16(saved);
    const int hv = (L1 / 2) / (vec ? 4 : 1);
    const dim3 grid(L.ntiles, max(1, (hv + 63) / 64));
    if (vec)
        hipLaunchKernelGGL(k_bwd_rows<4>, grid, dim3(64), 0, st, us, them, psqt_idx, max_act, grad_l0, grad_wpsqt,
                           grad_bpsqt, saved, G, (float*)(ws + L.partial), B, L1, n_psqt);
    else
        hipLaunchKernelGGL(k_bwd_rows<1>, grid, dim3(64), 0, st, us, them, psqt_idx, max_act, grad_l0, grad_wpsqt,
                           grad_bpsqt, saved, G, (float*)(ws + L.partial), B, L1, n_psqt);
    NNUEFT_LAUNCH_CHECK();
    return det_sort_reduce(widx, bidx, G, gW, gbias, B, K, R, out_cols, 2, ws, L, st);
}
