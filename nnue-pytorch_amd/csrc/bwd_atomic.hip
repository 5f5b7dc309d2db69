// Atomic-mode backward: scatter the upstream rows into the weight gradient with fp32 atomics.
//
// One wave per (tile of kTile positions, column slice).  Lanes own single columns 64 apart, so one
// atomic instruction of the wave covers 256 contiguous bytes of a gradient row (a lane-per-float4
// layout would spread every instruction over 1 KiB).  Exact zeros are not sent: they change
// nothing and the clamp makes most upstream values zero.
//
// On this part the L2 forwards every fp32 atomic to the memory side (TCC_EA0_ATOMIC equals
// TCC_ATOMIC for these kernels), so their rate is set by the number of 64-byte segments touched,
// about 18 G requests/s, wherever the request comes from: grouping positions by table block (which
// speeds the gathers of the other kernels up severalfold) makes this kernel no faster.
#include "common.h"

namespace {

constexpr int kTile = 4;

__device__ __forceinline__ void add_nz(float* p, float v) {
    if (v != 0.0f) atomicAdd(p, v);
}

template <int NC>
__global__ __launch_bounds__(64) void k_sparse_bwd_atomic(const int32_t* __restrict__ idx,
                                                          const float* __restrict__ gout, float* __restrict__ gW,
                                                          float* __restrict__ gbias, int B, int K, int R,
                                                          int out_cols, int nslices) {
    const int lane = threadIdx.x;
    const int tile = blockIdx.x / nslices;
    const int s = blockIdx.x - tile * nslices;
    int col[NC];
    bool act[NC];
    float bsum[NC];
#pragma unroll
    for (int m = 0; m < NC; ++m) {
        col[m] = (s * NC + m) * 64 + lane;
        act[m] = col[m] < out_cols;
        bsum[m] = 0.0f;
    }
    const int b1 = min((tile + 1) * kTile, B);
    for (int b = tile * kTile; b < b1; ++b) {
        float g[NC];
#pragma unroll
        for (int m = 0; m < NC; ++m) {
            g[m] = act[m] ? gout[(size_t)b * out_cols + col[m]] : 0.0f;
            bsum[m] += g[m];
        }
        const int32_t* ix = idx + (size_t)b * K;
        for (int k0 = 0; k0 < K; k0 += 64) {
            const int my = (k0 + lane < K) ? ix[k0 + lane] : -1;
            u64 mask = __ballot(my >= 0 && my < R);
            while (mask) {
                float* row = gW + (size_t)bcast_i(my, pop_lane(mask)) * out_cols;
#pragma unroll
                for (int m = 0; m < NC; ++m)
                    if (act[m]) add_nz(row + col[m], g[m]);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < NC; ++m)
        if (act[m]) add_nz(gbias + col[m], bsum[m]);
}

template <int NC>
__global__ __launch_bounds__(64) void k_double_bwd_atomic(
    const float* __restrict__ us, const float* __restrict__ them, const int32_t* __restrict__ widx,
    const int32_t* __restrict__ bidx, const int64_t* __restrict__ psqt_idx, const float* __restrict__ bias,
    float max_act, const float* __restrict__ grad_l0, const float* __restrict__ grad_wpsqt, const float* __restrict__ grad_bpsqt,
    const float* __restrict__ saved, float* __restrict__ gW, float* __restrict__ gbias, int B, int K, int R,
    int L1, int n_psqt, int nslices) {
    const int lane = threadIdx.x;
    const int tile = blockIdx.x / nslices;
    const int s = blockIdx.x - tile * nslices;
    const int h = L1 >> 1;
    const size_t out_cols = (size_t)L1 + n_psqt;
    int col[NC];
    bool act[NC];
    float bs0[NC], bs1[NC];
#pragma unroll
    for (int m = 0; m < NC; ++m) {
        col[m] = (s * NC + m) * 64 + lane;
        act[m] = col[m] < h;
        bs0[m] = 0.0f;
        bs1[m] = 0.0f;
    }
    const int b1 = min((tile + 1) * kTile, B);
    for (int b = tile * kTile; b < b1; ++b) {
        const float u = us[b], t = them[b];
        const float* sw = saved + (size_t)b * L1;
        const float* sb = saved + ((size_t)B + b) * L1;
        const float* gl = grad_l0 + (size_t)b * L1;
        float g[2][2][NC];  // [perspective][half][m]
#pragma unroll
        for (int m = 0; m < NC; ++m) {
            float gw0 = 0.0f, gw1 = 0.0f, gb0 = 0.0f, gb1 = 0.0f;
            if (act[m]) {
                const int c = col[m];
                float xw0, xw1, xb0, xb1;
                mix4(u, t, sw[c], sw[h + c], sb[c], sb[h + c], bias[c], bias[h + c], xw0, xw1, xb0, xb1);
                grad4(u, t, xw0, xw1, xb0, xb1, gl[c], gl[h + c], max_act, gw0, gw1, gb0, gb1);
            }
            g[0][0][m] = gw0;
            g[0][1][m] = gw1;
            g[1][0][m] = gb0;
            g[1][1][m] = gb1;
            bs0[m] += gw0 + gb0;
            bs1[m] += gw1 + gb1;
        }
        const int64_t pi = psqt_idx[b];
        const bool do_psqt = (s == 0) && (lane == 0) && pi >= 0 && pi < n_psqt;
        const float gps[2] = {grad_wpsqt[b], grad_bpsqt[b]};
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int32_t* ix = (p ? bidx : widx) + (size_t)b * K;
            for (int k0 = 0; k0 < K; k0 += 64) {
                const int my = (k0 + lane < K) ? ix[k0 + lane] : -1;
                u64 mask = __ballot(my >= 0 && my < R);
                while (mask) {
                    float* row = gW + (size_t)bcast_i(my, pop_lane(mask)) * out_cols;
#pragma unroll
                    for (int m = 0; m < NC; ++m) {
                        if (act[m]) {
                            add_nz(row + col[m], g[p][0][m]);
                            add_nz(row + h + col[m], g[p][1][m]);
                        }
                    }
                    if (do_psqt) add_nz(row + L1 + pi, gps[p]);
                }
            }
        }
        if (do_psqt) add_nz(gbias + L1 + pi, gps[0] + gps[1]);
    }
#pragma unroll
    for (int m = 0; m < NC; ++m) {
        if (act[m]) {
            add_nz(gbias + col[m], bs0[m]);
            add_nz(gbias + h + col[m], bs1[m]);
        }
    }
}

}  // namespace

extern "C" int nnueft_sparse_bwd_atomic(const int32_t* idx, const float* gout, float* gW, float* gbias, int B,
                                        int K, int R, int out_cols, void* stream) {
    if (B < 0 || K <= 0 || R <= 0 || out_cols <= 0) return NNUEFT_E_ARG;
    if (B == 0) return 0;
    if (!idx || !gout || !gW || !gbias) return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int ntiles = (B + kTile - 1) / kTile;
    if (out_cols > 128) {
        const int nslices = (out_cols + 255) / 256;
        hipLaunchKernelGGL(k_sparse_bwd_atomic<4>, dim3(ntiles * nslices), dim3(64), 0, st, idx, gout, gW, gbias, B,
                           K, R, out_cols, nslices);
    } else {
        const int nslices = (out_cols + 63) / 64;
        hipLaunchKernelGGL(k_sparse_bwd_atomic<1>, dim3(ntiles * nslices), dim3(64), 0, st, idx, gout, gW, gbias, B,
                           K, R, out_cols, nslices);
    }
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

extern "C" int nnueft_double_bwd_atomic(const float* us, const float* them, const int32_t* widx,
                                        const int32_t* bidx, const int64_t* psqt_idx, const float* bias,
                                        float max_act, const float* grad_l0, const float* grad_wpsqt,
                                        const float* grad_bpsqt, const float* saved, float* gW, float* gbias, int B,
                                        int K, int R, int L1, int n_psqt, void* stream) {
    if (B < 0 || K <= 0 || R <= 0 || L1 <= 0 || (L1 & 1) || n_psqt < 0) return NNUEFT_E_ARG;
    if (B == 0) return 0;
    if (!us || !them || !widx || !bidx || !psqt_idx || !bias || !grad_l0 || !grad_wpsqt || !grad_bpsqt || !saved ||
        !gW || !gbias)
        return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int ntiles = (B + kTile - 1) / kTile;
    const int h = L1 / 2;
    if (h > 128) {
        const int nslices = (h + 255) / 256;
        hipLaunchKernelGGL(k_double_bwd_atomic<4>, dim3(ntiles * nslices), dim3(64), 0, st, us, them, widx, bidx,
                           psqt_idx, bias, max_act, grad_l0, grad_wpsqt, grad_bpsqt, saved, gW, gbias, B, K, R, L1,
                           n_psqt, nslices);
    } else {
        const int nslices = (h + 63) / 64;
        hipLaunchKernelGGL(k_double_bwd_atomic<1>, dim3(ntiles * nslices), dim3(64), 0, st, us, them, widx, bidx,
                           psqt_idx, bias, max_act, grad_l0, grad_wpsqt, grad_bpsqt, saved, gW, gbias, B, K, R, L1,
                           n_psqt, nslices);
    }
    NNUEFT_LAUNCH_CHECK();
    return 0;
}
