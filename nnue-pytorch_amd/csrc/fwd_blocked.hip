// Forward, L2-blocked variant (used when the caller passes a workspace).
//
// The lists of one perspective of one position name rows of a single 768-row block of the table
// (one king bucket).  Sorting the (position, perspective) pairs of a batch by that block and
// giving each XCD a contiguous part of the sorted order, walked one column slice at a time, keeps
// the rows a XCD is gathering (768 rows x one slice = 0.75-1.5 MB) inside its own 4 MB L2, so the
// gather runs at L2 speed and the table crosses the fabric about once instead of ~24 times.
//
//   k_pair_order   counting sort of the 2B pairs by table block of their first valid index
//   k_acc_blocked  wave per (pair, column slice): chain from +0 over the list, result to saved[2, B, L1]
//   k_mix          per position: + bias, side-to-move mix, clamp, product, psqt chains; writes l0
//
// Workgroups are handed to the 8 XCDs round-robin by workgroup id, so id % 8 selects the XCD.
#include "gather.h"
#include "internal.h"

namespace nnueft_blocked {

// Tunables of the blocked gather (vectors of 4 floats per lane and row; rows fetched per group).
#ifndef NNUEFT_ACC_NQ
#define NNUEFT_ACC_NQ 3
#endif
#ifndef NNUEFT_ACC_U
#define NNUEFT_ACC_U 12
#endif

constexpr int kMaxBins = 512;   // table blocks the pair sort tells apart (17 x 512 x 4 bytes of LDS)

__device__ __forceinline__ const int32_t* pair_list(const int32_t* __restrict__ widx,
                                                    const int32_t* __restrict__ bidx, int pair, int B, int K) {
    const int p = pair >= B;
    return (p ? bidx : widx) + (size_t)(pair - p * B) * K;
}

// Table block of a list given its first slot (already loaded); scans on only when that slot is padding.
__device__ __forceinline__ int pair_key(const int32_t* __restrict__ ix, int first, int K, int R, int block_rows,
                                        int nbins) {
    if (first >= 0 && first < R) return first / block_rows;
    for (int k = 1; k < K; ++k) {
        const int r = ix[k];
        if (r >= 0 && r < R) return r / block_rows;
    }
    return nbins - 1;   // empty list
}

// Pair sort, three small launches.  order[] = pair ids (p * B + b) grouped by table block; the
// order inside a block is arbitrary (it only schedules work).
//   k_pair_hist     one pair per thread: key to keys[], per-workgroup histogram to hist[bin][wg]
//   k_pair_scan     exclusive scan of hist (flat, bin-major) in place -> first slot of every (bin, wg)
//   k_pair_scatter  pairs to their slots through LDS cursors
constexpr int kPairThreads = 256;

__global__ __launch_bounds__(kPairThreads) void k_pair_hist(const int32_t* __restrict__ widx,
                                                            const int32_t* __restrict__ bidx,
                                                            uint32_t* __restrict__ keys,
                                                            uint32_t* __restrict__ hist, int B, int K, int R,
                                                            int block_rows, int nbins) {
    __shared__ uint32_t bins[kMaxBins];
    const int tid = threadIdx.x;
    const int n = blockIdx.x * kPairThreads + tid;
    for (int i = tid; i < nbins; i += kPairThreads) bins[i] = 0;
    __syncthreads();
    if (n < 2 * B) {
        const int32_t* ix = pair_list(widx, bidx, n, B, K);
        const int key = pair_key(ix, ix[0], K, R, block_rows, nbins);
        keys[n] = (uint32_t)key;
        atomicAdd(&bins[key], 1u);
    }
    __syncthreads();
    for (int i = tid; i < nbins; i += kPairThreads) hist[(size_t)i * gridDim.x + blockIdx.x] = bins[i];
}

// In-place exclusive scan of data[0..n) by one workgroup of 1024 threads.
__global__ __launch_bounds__(1024) void k_pair_scan(uint32_t* __restrict__ data, int n) {
    __shared__ uint32_t wave_tot[16];
    __shared__ uint32_t carry_s;
    const int tid = threadIdx.x;
    constexpr int PER = 8;
    if (tid == 0) carry_s = 0;
    __syncthreads();
    for (int base = 0; base < n; base += 1024 * PER) {
        const int i0 = base + tid * PER;
        uint32_t v[PER];
        uint32_t local = 0;
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            v[u] = (i0 + u < n) ? data[i0 + u] : 0;
            local += v[u];
        }
        uint32_t incl = local;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t t = __shfl_up(incl, off);
            if ((tid & 63) >= off) incl += t;
        }
        if ((tid & 63) == 63) wave_tot[tid >> 6] = incl;
        __syncthreads();
        uint32_t run = carry_s;
        for (int w = 0; w < (tid >> 6); ++w) run += wave_tot[w];
        run += incl - local;
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            if (i0 + u < n) data[i0 + u] = run;
            run += v[u];
        }
        __syncthreads();
        if (tid == 1023) carry_s = run;
        __syncthreads();
    }
}

__global__ __launch_bounds__(kPairThreads) void k_pair_scatter(const uint32_t* __restrict__ keys,
                                                               const uint32_t* __restrict__ hist,
                                                               uint32_t* __restrict__ order, int npairs,
                                                               int nbins) {
    __shared__ uint32_t cursor[kMaxBins];
    const int tid = threadIdx.x;
    const int n = blockIdx.x * kPairThreads + tid;
    for (int i = tid; i < nbins; i += kPairThreads) cursor[i] = hist[(size_t)i * gridDim.x + blockIdx.x];
    __syncthreads();
    if (n < npairs) order[atomicAdd(&cursor[keys[n]], 1u)] = (uint32_t)n;
}

// saved[pair, slice] = chain from +0 over the pair's list (pair = perspective * B + position).
template <int VW, int NQ, int U>
__global__ __launch_bounds__(64) void k_acc_blocked(const int32_t* __restrict__ widx,
                                                    const int32_t* __restrict__ bidx,
                                                    const uint32_t* __restrict__ order,
                                                    const float* __restrict__ W, float* __restrict__ acc, int B,
                                                    int K, int R, int L1, int out_cols, int per_xcd) {
    const int lane = threadIdx.x;
    const int xcd = blockIdx.x % kXcd;
    const int j = blockIdx.x / kXcd;
    const int s = j / per_xcd;
    const int n = xcd * per_xcd + (j - s * per_xcd);
    if (n >= 2 * B) return;
    const int pair = (int)order[n];
    const int p = pair >= B;
    const int b = pair - p * B;
    const int nv = L1 / VW;

    int col[NQ];
    bool act[NQ];
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        const int q = (s * NQ + m) * 64 + lane;
        act[m] = q < nv;
        col[m] = act[m] ? q * VW : 0;
    }
    vecf<VW> a[NQ];
#pragma unroll
    for (int m = 0; m < NQ; ++m) a[m] = vzero<VW>();
    const int32_t* ix = (p ? bidx : widx) + (size_t)b * K;
    for (int k0 = 0; k0 < K; k0 += 64) {
        const int my = (k0 + lane < K) ? ix[k0 + lane] : -1;
        const u64 mask = __ballot(my >= 0 && my < R);
        chain_rows<VW, NQ, U>(a, W, (size_t)out_cols, col, my, mask);
    }
    float* dst = acc + (size_t)pair * L1;
#pragma unroll
    for (int m = 0; m < NQ; ++m)
        if (act[m]) stv_stream<VW>(dst + col[m], a[m]);
}

// One 64-lane slice of a position's output row: bias, mix, clamp, product (lane = threadIdx.x, s = the slice).
template <int VW>
__device__ __forceinline__ void mix_slice(int s, int b, int lane, const float* __restrict__ us,
                                          const float* __restrict__ them, const float* __restrict__ bias,
                                          const float* __restrict__ saved, float max_act, float* __restrict__ l0, int B,
                                          int L1, const ActGrid& act) {
    const int h = L1 >> 1;
    const int hv = h / VW;
    const int q = s * 64 + lane;
    if (q < hv) {
        const int c = q * VW;
        const float u = us[b], t = them[b];
        const float* sw = saved + (size_t)b * L1;
        const float* sb = saved + ((size_t)B + b) * L1;
        const vecf<VW> sw0 = ldv<VW>(sw + c), sw1 = ldv<VW>(sw + h + c);
        const vecf<VW> sb0 = ldv<VW>(sb + c), sb1 = ldv<VW>(sb + h + c);
        const vecf<VW> bias0 = ldv<VW>(bias + c), bias1 = ldv<VW>(bias + h + c);
        vecf<VW> o0, o1;
#pragma unroll
        for (int i = 0; i < VW; ++i) {
            float xw0, xw1, xb0, xb1;
            mix4(u, t, sw0.v[i], sw1.v[i], sb0.v[i], sb1.v[i], bias0.v[i], bias1.v[i], xw0, xw1, xb0, xb1);
            o0.v[i] = clamp_act(xw0, max_act) * clamp_act(xw1, max_act);
            o1.v[i] = clamp_act(xb0, max_act) * clamp_act(xb1, max_act);
            if (act.on) {   // the activation grid the caller would otherwise apply in a pass of its own
                o0.v[i] = (floorf(o0.v[i] * act.scale + act.eps) / act.scale) * act.post_mul;
                o1.v[i] = (floorf(o1.v[i] * act.scale + act.eps) / act.scale) * act.post_mul;
            }
        }
        float* o = l0 + (size_t)b * L1;
        stv<VW>(o + c, o0);
        stv<VW>(o + h + c, o1);
    }
}

// The two psqt chains of a position, one wave: wpsqt[b], bpsqt[b] = chain over the list's valid slots + bias.
__device__ __forceinline__ void psqt_chains(int b, int lane, const int32_t* __restrict__ widx,
                                            const int32_t* __restrict__ bidx, const int64_t* __restrict__ psqt_idx,
                                            const float* __restrict__ W, const float* __restrict__ bias,
                                            float* __restrict__ wpsqt, float* __restrict__ bpsqt, int K, int R, int L1,
                                            int n_psqt, const VirtualTable& vt) {
    const size_t out_cols = (size_t)L1 + n_psqt;
    const int64_t pi = psqt_idx[b];
    const bool do_psqt = pi >= 0 && pi < n_psqt;
    float ps[2] = {0.0f, 0.0f};
    if (do_psqt) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int32_t* ix = (p ? bidx : widx) + (size_t)b * K;
            for (int k0 = 0; k0 < K; k0 += 64) {
                const int my = (k0 + lane < K) ? ix[k0 + lane] : -1;
                const bool ok = my >= 0 && my < R;
                u64 mask = __ballot(ok);
                float myps = ok ? W[(size_t)my * out_cols + L1 + pi] : 0.0f;
                if (ok && vt.V) {
                    // the merged table's entry: W + V[row % 768], on the psqt grid when asked for
                    myps = myps + vt.V[(size_t)(my % nnueft_tile::kBlockRows) * out_cols + L1 + pi];
                    if (vt.quantize) myps = rintf(myps * vt.scale_psqt) / vt.scale_psqt;
                }
                while (mask) ps[p] = ps[p] + bcast_f(myps, pop_lane(mask));
            }
        }
    }
    if (lane == 0) {
        const float pb = do_psqt ? bias[L1 + pi] : 0.0f;
        wpsqt[b] = ps[0] + pb;
        bpsqt[b] = ps[1] + pb;
    }
}

// Per position: bias, mix, clamp, product; slice 0 also does the two psqt chains.
template <int VW>
__global__ __launch_bounds__(64) void k_mix(const float* __restrict__ us, const float* __restrict__ them,
                                            const int32_t* __restrict__ widx, const int32_t* __restrict__ bidx,
                                            const int64_t* __restrict__ psqt_idx, const float* __restrict__ W,
                                            const float* __restrict__ bias, const float* __restrict__ saved,
                                            float max_act, float* __restrict__ l0, float* __restrict__ wpsqt,
                                            float* __restrict__ bpsqt, int B, int K, int R, int L1, int n_psqt,
                                            int nslices, ActGrid act, VirtualTable vt) {
    const int lane = threadIdx.x;
    // 1-D launch, the slices of a position next to each other: its rows are then read and written
    // at about the same time (a few per cent faster than position-fastest)
    const int s = blockIdx.x % nslices;
    const int b = blockIdx.x / nslices;
    mix_slice<VW>(s, b, lane, us, them, bias, saved, max_act, l0, B, L1, act);
    // (no psqt outputs: the sort in front of the gather has summed the psqt chains already)
    if (s == 0 && wpsqt) psqt_chains(b, lane, widx, bidx, psqt_idx, W, bias, wpsqt, bpsqt, K, R, L1, n_psqt, vt);
}

// What is left when the gather has written the output rows itself (it does for a position whose (us, them) is
// (1, 0) or (0, 1): such a row is one perspective's sums on each half) and the sort in front of it the psqt chains:
// the whole row of a position with any other (us, them), which needs both perspectives' sums at once; every row
// when the gather met a sum that is not finite (*nonfinite != 0: 0 * inf of the other perspective's sum is NaN
// in the mix, which the gather's row does not show).  A lane looks at a position, the wave redoes the ones that
// need it one after the other.
constexpr int kRestThreads = 256;
template <int VW>
__global__ __launch_bounds__(kRestThreads) void k_mix_rest(const float* __restrict__ us, const float* __restrict__ them,
                                                           const float* __restrict__ bias,
                                                           const float* __restrict__ saved, float max_act,
                                                           float* __restrict__ l0, int B, int L1, int nslices,
                                                           ActGrid act, const uint32_t* __restrict__ nonfinite) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * (kRestThreads / 64) + (threadIdx.x >> 6);
    const int nwaves = gridDim.x * (kRestThreads / 64);
    const bool all = *nonfinite != 0u;
    for (int base = wave * 64; base < B; base += nwaves * 64) {
        const int p = base + lane;
        u64 todo = __ballot(p < B && (all || !one_sided(us[min(p, B - 1)], them[min(p, B - 1)])));
        while (todo) {
            const int b = base + pop_lane(todo);
            for (int s = 0; s < nslices; ++s) mix_slice<VW>(s, b, lane, us, them, bias, saved, max_act, l0, B, L1, act);
        }
    }
}

static inline size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

int table_block_rows(int R, int hint, int* nbins);

int launch_scan(uint32_t* data, int n, hipStream_t st) {
    hipLaunchKernelGGL(k_pair_scan, dim3(1), dim3(1024), 0, st, data, n);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

int launch_mix(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
               const int64_t* psqt_idx, const float* W, const float* bias, const float* saved, float max_act,
               float* l0, float* wpsqt, float* bpsqt, int B, int K, int R, int L1, int n_psqt, hipStream_t st,
               ActGrid act, VirtualTable vt, const uint32_t* nonfinite) {
    const int hv = (L1 / 2) / 4;
    const int mix_slices = (hv + 63) / 64;
    if ((long long)B * mix_slices > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
    if (nonfinite) {
        // the rows the gather left alone, nothing else: the psqt chains are the caller's
        if (wpsqt || bpsqt) return NNUEFT_E_ARG;
        const int waves = (B + 63) / 64;
        const int blocks = min((waves + kRestThreads / 64 - 1) / (kRestThreads / 64), 1024);
        hipLaunchKernelGGL(k_mix_rest<4>, dim3((unsigned)blocks), dim3(kRestThreads), 0, st, us, them, bias, saved, max_act,
                           l0, B, L1, mix_slices, act, nonfinite);
        NNUEFT_LAUNCH_CHECK();
        return 0;
    }
    const dim3 mix_grid((unsigned)B * mix_slices);
    hipLaunchKernelGGL(k_mix<4>, mix_grid, dim3(64), 0, st, us, them, widx, bidx, psqt_idx, W, bias, saved, max_act,
                       l0, wpsqt, bpsqt, B, K, R, L1, n_psqt, mix_slices, act, vt);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

struct PairSortLayout {
    size_t order, keys, hist, end;
    int ngroups, nbins, block_rows;
};

bool pair_sort_layout(int B, int R, int block_rows_hint, PairSortLayout* L) {
    if (B <= 0 || R <= 0) return false;
    L->block_rows = table_block_rows(R, block_rows_hint, &L->nbins);
    L->ngroups = (2 * B + kPairThreads - 1) / kPairThreads;
    size_t off = 0;
    L->order = off;
    off += up256((size_t)2 * B * sizeof(uint32_t));
    L->keys = off;
    off += up256((size_t)2 * B * sizeof(uint32_t));
    L->hist = off;
    off += up256((size_t)L->ngroups * L->nbins * sizeof(uint32_t));
    L->end = off;
    return true;
}

size_t pair_sort_workspace(int B, int R, int block_rows_hint) {
    PairSortLayout L;
    return pair_sort_layout(B, R, block_rows_hint, &L) ? L.end : 0;
}

int launch_pair_sort(const int32_t* widx, const int32_t* bidx, int B, int K, int R, int block_rows_hint, void* ws,
                     hipStream_t st, const uint32_t** order_out) {
    PairSortLayout L;
    if (!pair_sort_layout(B, R, block_rows_hint, &L)) return NNUEFT_E_ARG;
    char* base = (char*)ws;
    uint32_t* order = (uint32_t*)(base + L.order);
    uint32_t* keys = (uint32_t*)(base + L.keys);
    uint32_t* hist = (uint32_t*)(base + L.hist);
    hipLaunchKernelGGL(k_pair_hist, dim3(L.ngroups), dim3(kPairThreads), 0, st, widx, bidx, keys, hist, B, K, R,
                       L.block_rows, L.nbins);
    NNUEFT_LAUNCH_CHECK();
    const int rc_scan = launch_scan(hist, L.ngroups * L.nbins, st);
    if (rc_scan) return rc_scan;
    hipLaunchKernelGGL(k_pair_scatter, dim3(L.ngroups), dim3(kPairThreads), 0, st, keys, hist, order, 2 * B,
                       L.nbins);
    NNUEFT_LAUNCH_CHECK();
    *order_out = order;
    return 0;
}

// Rows per table block the pair sort tells apart: the hint (the caller's knowledge of the table's
// block structure) or 768, widened when the table would have more than kMaxBins - 1 blocks.
int table_block_rows(int R, int hint, int* nbins) {
    int block_rows = hint > 0 ? hint : 768;
    if ((R + block_rows - 1) / block_rows + 1 > kMaxBins) block_rows = (R + kMaxBins - 2) / (kMaxBins - 1);
    *nbins = (R + block_rows - 1) / block_rows + 1;
    return block_rows;
}

int double_fwd_blocked(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                       const int64_t* psqt_idx, const float* W, const float* bias, float max_act, float* l0,
                       float* wpsqt, float* bpsqt, float* saved, int B, int K, int R, int L1, int n_psqt,
                       void* ws, hipStream_t st, ActGrid act) {
    const uint32_t* order = nullptr;
    const int rc = launch_pair_sort(widx, bidx, B, K, R, 0, ws, st, &order);
    if (rc) return rc;
    const int out_cols = L1 + n_psqt;
    const int nv = L1 / 4;
    const int per_xcd = (2 * B + kXcd - 1) / kXcd;
    if (nv > 64) {
        constexpr int NQ = NNUEFT_ACC_NQ;
        const int nslices = (nv + 64 * NQ - 1) / (64 * NQ);
        const long long grid = (long long)kXcd * per_xcd * nslices;
        if (grid > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
        hipLaunchKernelGGL((k_acc_blocked<4, NQ, NNUEFT_ACC_U>), dim3((unsigned)grid), dim3(64), 0, st, widx, bidx,
                           order, W, saved, B, K, R, L1, out_cols, per_xcd);
    } else {
        const long long grid = (long long)kXcd * per_xcd;
        if (grid > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
        hipLaunchKernelGGL((k_acc_blocked<4, 1, 8>), dim3((unsigned)grid), dim3(64), 0, st, widx, bidx, order, W,
                           saved, B, K, R, L1, out_cols, per_xcd);
    }
    NNUEFT_LAUNCH_CHECK();
    return launch_mix(us, them, widx, bidx, psqt_idx, W, bias, saved, max_act, l0, wpsqt, bpsqt, B, K, R, L1, n_psqt,
                      st, act, VirtualTable{nullptr, 1.0f, 1.0f, 0, 0.0f}, nullptr);
}

}  // namespace nnueft_blocked
