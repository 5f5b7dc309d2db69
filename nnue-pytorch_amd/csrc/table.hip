// Table-side passes of the feature transformer module, one read and one write of the table each
// instead of the reference's chain of elementwise torch ops:
//   k_table_merge         merged = fake_quantize(W + V[row % vrows])     (real + virtual weights)
//   k_table_virtual_grad  gV[v] = sum over the table blocks of gW[block * vrows + v]
#include "common.h"

namespace {

// round(x * scale) / scale with round-half-to-even, as torch's mul / round / div
__device__ __forceinline__ float fq(float x, float scale) { return rintf(x * scale) / scale; }

template <int VW>
__global__ __launch_bounds__(256) void k_table_merge(const float* __restrict__ W, const float* __restrict__ V,
                                                     float* __restrict__ out, int R, int cols, int L1, int vrows,
                                                     float scale_ft, float scale_psqt, int quantize) {
    const int nv = cols / VW;
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long long)R * nv) return;
    const int r = (int)(i / nv);
    const int c = (int)(i - (long long)r * nv) * VW;
    vecf<VW> w = ldv<VW>(W + (size_t)r * cols + c);
    if (V) {
        const vecf<VW> v = ldv<VW>(V + (size_t)(r % vrows) * cols + c);
        vadd<VW>(w, v);
    }
    if (quantize) {
#pragma unroll
        for (int k = 0; k < VW; ++k) w.v[k] = fq(w.v[k], (c + k) < L1 ? scale_ft : scale_psqt);
    }
    stv<VW>(out + (size_t)r * cols + c, w);
}

template <int VW>
__global__ __launch_bounds__(256) void k_table_virtual_grad(const float* __restrict__ gW, float* __restrict__ gV,
                                                            int R, int cols, int vrows) {
    const int nv = cols / VW;
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long long)vrows * nv) return;
    const int v = (int)(i / nv);
    const int c = (int)(i - (long long)v * nv) * VW;
    vecf<VW> acc = vzero<VW>();
    constexpr int PF = 8;
    int r = v;
    for (; r + (PF - 1) * vrows < R; r += PF * vrows) {
        vecf<VW> t[PF];
#pragma unroll
        for (int u = 0; u < PF; ++u) t[u] = ldv<VW>(gW + (size_t)(r + u * vrows) * cols + c);
#pragma unroll
        for (int u = 0; u < PF; ++u) vadd<VW>(acc, t[u]);
    }
    for (; r < R; r += vrows) vadd<VW>(acc, ldv<VW>(gW + (size_t)r * cols + c));
    stv<VW>(gV + (size_t)v * cols + c, acc);
}

}  // namespace

extern "C" int nnueft_table_merge(const float* W, const float* V, float* merged, int R, int cols, int L1, int vrows,
                                  float scale_ft, float scale_psqt, int fake_quantize, void* stream) {
    if (R <= 0 || cols <= 0 || L1 < 0 || L1 > cols) return NNUEFT_E_ARG;
    if (!W || !merged || (V && vrows <= 0)) return NNUEFT_E_ARG;
    if (fake_quantize && (!(scale_ft > 0.0f) || !(scale_psqt > 0.0f))) return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = (cols % 4 == 0) && aligned16(W) && aligned16(merged) && (!V || aligned16(V));
    const long long n = (long long)R * (cols / (vec ? 4 : 1));
    const long long blocks = (n + 255) / 256;
    if (blocks > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
    if (vec)
        hipLaunchKernelGGL(k_table_merge<4>, dim3((unsigned)blocks), dim3(256), 0, st, W, V, merged, R, cols, L1,
                           vrows, scale_ft, scale_psqt, fake_quantize);
    else
        hipLaunchKernelGGL(k_table_merge<1>, dim3((unsigned)blocks), dim3(256), 0, st, W, V, merged, R, cols, L1,
                           vrows, scale_ft, scale_psqt, fake_quantize);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

extern "C" int nnueft_table_virtual_grad(const float* gW, float* gV, int R, int cols, int vrows, void* stream) {
    if (R <= 0 || cols <= 0 || vrows <= 0 || !gW || !gV) return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = (cols % 4 == 0) && aligned16(gW) && aligned16(gV);
    const long long n = (long long)vrows * (cols / (vec ? 4 : 1));
    const long long blocks = (n + 255) / 256;
    if (blocks > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
    if (vec)
        hipLaunchKernelGGL(k_table_virtual_grad<4>, dim3((unsigned)blocks), dim3(256), 0, st, gW, gV, R, cols, vrows);
    else
        hipLaunchKernelGGL(k_table_virtual_grad<1>, dim3((unsigned)blocks), dim3(256), 0, st, gW, gV, R, cols, vrows);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}
