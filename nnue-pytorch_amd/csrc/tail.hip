// What runs per position after the bucketed linear layers, each a chain of a dozen or more
// elementwise torch ops on [B, 32]-sized tensors in the module code (model/modules/layer_stacks.py,
// model/nnue.py loss); on the GPU those are a few microseconds of launch each and no work.  One kernel
// per chain here, same arithmetic in the same order (every operation rounds on its own):
//
//   k_sqr_crelu_*     y = clamp(cat[fq(x^2) * c, fq(x)], 0, m)  (+ the skip value x[-2] - x[-1])
//   k_stack_output_*  net = fq_out(lin + skip) + (wpsqt - bpsqt) * (us - 0.5)
//   k_sf_loss_*       the win-rate-model loss: per-position terms, a fixed-order sum, the gradient
//
// fq(v) = floor(v * s + eps) / s and fq_out are straight-through in the backward pass.
#include "common.h"

namespace {

__device__ __forceinline__ float fq_act(float v, float s, float eps, int on) {
    return on ? floorf(v * s + eps) / s : v;
}

// one thread per element of x [B, n]; y [B, 2n]; skip [B] (may be null) = x[b, n-2] - x[b, n-1]
__global__ __launch_bounds__(256) void k_sqr_crelu_fwd(const float* __restrict__ x, float* __restrict__ y,
                                                       float* __restrict__ skip, long long total, int n, float s,
                                                       float eps, float c, float m, int fq) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const long long b = i / n;
    const int j = (int)(i - b * n);
    const float v = x[i];
    const float a = fq_act(v * v, s, eps, fq) * c;
    const float l = fq_act(v, s, eps, fq);
    y[b * 2 * n + j] = clamp_act(a, m);
    y[b * 2 * n + n + j] = clamp_act(l, m);
    if (skip && j == n - 1) skip[b] = x[i - 1] - v;
}

// gx = (gy_sqr * [0 <= a <= m] * c) * (2 x) + gy_lin * [0 <= l <= m]  (+- gskip on the last two columns)
__global__ __launch_bounds__(256) void k_sqr_crelu_bwd(const float* __restrict__ x, const float* __restrict__ gy,
                                                       const float* __restrict__ gskip, float* __restrict__ gx,
                                                       long long total, int n, float s, float eps, float c, float m,
                                                       int fq) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const long long b = i / n;
    const int j = (int)(i - b * n);
    const float v = x[i];
    const float a = fq_act(v * v, s, eps, fq) * c;
    const float l = fq_act(v, s, eps, fq);
    const float ga = (a >= 0.0f && a <= m) ? gy[b * 2 * n + j] : 0.0f;
    const float gl = (l >= 0.0f && l <= m) ? gy[b * 2 * n + n + j] : 0.0f;
    float g = (ga * c) * (2.0f * v) + gl;
    if (gskip) {
        if (j == n - 2) g = g + gskip[b];
        else if (j == n - 1) g = g - gskip[b];
    }
    gx[i] = g;
}

__global__ __launch_bounds__(256) void k_stack_output_fwd(const float* __restrict__ lin, const float* __restrict__ skip,
                                                          const float* __restrict__ wpsqt,
                                                          const float* __restrict__ bpsqt, const float* __restrict__ us,
                                                          float* __restrict__ net, int B, float den, long long den_i,
                                                          long long mult_i, float mult, int fq) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= B) return;
    float v = lin[i] + skip[i];
    if (fq) {
        const long long q = (llrintf(v * den) * mult_i) / den_i;   // integer division truncates
        v = (float)q / mult;
    }
    net[i] = v + (wpsqt[i] - bpsqt[i]) * (us[i] - 0.5f);
}

__global__ __launch_bounds__(256) void k_stack_output_bwd(const float* __restrict__ g, const float* __restrict__ us,
                                                          float* __restrict__ gw, float* __restrict__ gb, int B) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= B) return;
    const float t = g[i] * (us[i] - 0.5f);
    gw[i] = t;
    gb[i] = -t;
}

struct LossArgs {
    float in_offset, in_scaling, out_offset, out_scaling, pow_exp, qp_asymmetry, weight_factor, w2;
    float tb_base, tb_scale, tb_decay, lambda, one_minus_lambda;
};

__device__ __forceinline__ float sigmoidf(float z) { return 1.0f / (1.0f + expf(-z)); }

// terms [3, B]: loss_i * w_i, w_i, w_i * d loss_i / d scorenet_i
__global__ __launch_bounds__(256) void k_sf_loss_terms(const float* __restrict__ scorenet,
                                                       const float* __restrict__ score,
                                                       const float* __restrict__ outcome, float* __restrict__ terms,
                                                       int B, LossArgs p) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= B) return;
    float sc = score[i];
    const float mag = fabsf(sc);
    if (mag >= 32000.0f - 245.0f) {
        const float plies = fmaxf(32000.0f - mag, 0.0f);
        const float remapped = p.tb_base + powf(p.tb_decay, plies) * p.tb_scale;
        sc = sc < 0.0f ? -remapped : remapped;
    }
    const float x = scorenet[i];
    const float s1 = sigmoidf((x - p.in_offset) / p.in_scaling);
    const float s2 = sigmoidf((-x - p.in_offset) / p.in_scaling);
    const float qf = 0.5f * (1.0f + s1 - s2);
    const float pf = 0.5f * (1.0f + sigmoidf((sc - p.out_offset) / p.out_scaling) -
                             sigmoidf((-sc - p.out_offset) / p.out_scaling));
    const float pt = pf * p.lambda + outcome[i] * p.one_minus_lambda;
    const float d = pt - qf;
    const float a = fabsf(d);
    float l = powf(a, p.pow_exp);
    // d l / d qf = -sign(d) * e * a^(e-1)
    float dl = a > 0.0f ? p.pow_exp * powf(a, p.pow_exp - 1.0f) * (d > 0.0f ? -1.0f : 1.0f) : 0.0f;
    if (p.qp_asymmetry != 0.0f) {
        const float f = (qf > pt ? p.qp_asymmetry : 0.0f) + 1.0f;
        l = l * f;
        dl = dl * f;
    }
    const float dev = pf - 0.5f;
    const float w = 1.0f + p.weight_factor * powf(dev * dev * pf * (1.0f - pf), p.w2);
    const float dq = 0.5f * (s1 * (1.0f - s1) + s2 * (1.0f - s2)) / p.in_scaling;
    terms[i] = l * w;
    terms[(size_t)B + i] = w;
    terms[(size_t)2 * B + i] = w * dl * dq;
}

// One workgroup: sums [0] = sum of terms[0, :], [1] = sum of terms[1, :], loss = [0] / [1].  Thread t
// chains elements t, t + 1024, ...; the 1024 partial sums are added pairwise in a fixed tree.
constexpr int kLossThreads = 1024;
__global__ __launch_bounds__(kLossThreads) void k_sf_loss_reduce(const float* __restrict__ terms, float* __restrict__ sums,
                                                                 float* __restrict__ loss, int B) {
    __shared__ float part[2][kLossThreads];
    const int t = threadIdx.x;
    float a = 0.0f, w = 0.0f;
    for (int i = t; i < B; i += kLossThreads) {
        a = a + terms[i];
        w = w + terms[(size_t)B + i];
    }
    part[0][t] = a;
    part[1][t] = w;
    __syncthreads();
    for (int half = kLossThreads / 2; half > 0; half >>= 1) {
        if (t < half) {
            part[0][t] = part[0][t] + part[0][t + half];
            part[1][t] = part[1][t] + part[1][t + half];
        }
        __syncthreads();
    }
    if (t == 0) {
        sums[0] = part[0][0];
        sums[1] = part[1][0];
        loss[0] = part[0][0] / part[1][0];
    }
}

// d loss / d scorenet_i = terms[2, i] / sum of weights, times the incoming gradient (a device scalar)
__global__ __launch_bounds__(256) void k_sf_loss_bwd(const float* __restrict__ terms, const float* __restrict__ sums,
                                                     const float* __restrict__ gloss, float* __restrict__ gnet, int B) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= B) return;
    gnet[i] = terms[(size_t)2 * B + i] * (gloss[0] / sums[1]);
}

inline unsigned blocks_for(long long n) { return (unsigned)((n + 255) / 256); }

}  // namespace

extern "C" int nnueft_sqr_crelu_fwd(const float* x, float* y, float* skip, int B, int n, float scale, float eps,
                                    float sqr_factor, float max_act, int fake_quantize, void* stream) {
    if (B <= 0 || n <= 0 || !x || !y || (skip && n < 2)) return NNUEFT_E_ARG;
    if (fake_quantize && !(scale > 0.0f)) return NNUEFT_E_ARG;
    const long long total = (long long)B * n;
    if (total > 0x7fffffffLL * 256LL) return NNUEFT_E_UNSUPPORTED;
    hipLaunchKernelGGL(k_sqr_crelu_fwd, dim3(blocks_for(total)), dim3(256), 0, (hipStream_t)stream, x, y, skip, total, n,
                       scale, eps, sqr_factor, max_act, fake_quantize != 0);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

extern "C" int nnueft_sqr_crelu_bwd(const float* x, const float* gy, const float* gskip, float* gx, int B, int n,
                                    float scale, float eps, float sqr_factor, float max_act, int fake_quantize,
                                    void* stream) {
    if (B <= 0 || n <= 0 || !x || !gy || !gx || (gskip && n < 2)) return NNUEFT_E_ARG;
    if (fake_quantize && !(scale > 0.0f)) return NNUEFT_E_ARG;
    const long long total = (long long)B * n;
    if (total > 0x7fffffffLL * 256LL) return NNUEFT_E_UNSUPPORTED;
    hipLaunchKernelGGL(k_sqr_crelu_bwd, dim3(blocks_for(total)), dim3(256), 0, (hipStream_t)stream, x, gy, gskip, gx,
                       total, n, scale, eps, sqr_factor, max_act, fake_quantize != 0);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

extern "C" int nnueft_stack_output_fwd(const float* lin, const float* skip, const float* wpsqt, const float* bpsqt,
                                       const float* us, float* net, int B, long long den, long long mult,
                                       int fake_quantize, void* stream) {
    if (B <= 0 || !lin || !skip || !wpsqt || !bpsqt || !us || !net) return NNUEFT_E_ARG;
    if (fake_quantize && (den <= 0 || mult <= 0)) return NNUEFT_E_ARG;
    hipLaunchKernelGGL(k_stack_output_fwd, dim3(blocks_for(B)), dim3(256), 0, (hipStream_t)stream, lin, skip, wpsqt,
                       bpsqt, us, net, B, (float)den, den, mult, (float)mult, fake_quantize != 0);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

extern "C" int nnueft_stack_output_bwd(const float* gnet, const float* us, float* gwpsqt, float* gbpsqt, int B,
                                       void* stream) {
    if (B <= 0 || !gnet || !us || !gwpsqt || !gbpsqt) return NNUEFT_E_ARG;
    hipLaunchKernelGGL(k_stack_output_bwd, dim3(blocks_for(B)), dim3(256), 0, (hipStream_t)stream, gnet, us, gwpsqt,
                       gbpsqt, B);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

extern "C" int nnueft_sf_loss_fwd(const float* scorenet, const float* score, const float* outcome, float* terms,
                                  float* sums, float* loss, int B, float in_offset, float in_scaling, float out_offset,
                                  float out_scaling, float pow_exp, float qp_asymmetry, float w1, float w2,
                                  float tb_remap_base, float tb_remap_scale, float tb_remap_decay, double lambda,
                                  void* stream) {
    if (B <= 0 || !scorenet || !score || !outcome || !terms || !sums || !loss) return NNUEFT_E_ARG;
    if (!(in_scaling > 0.0f) || !(out_scaling > 0.0f)) return NNUEFT_E_ARG;
    LossArgs p;
    p.in_offset = in_offset; p.in_scaling = in_scaling; p.out_offset = out_offset; p.out_scaling = out_scaling;
    p.pow_exp = pow_exp; p.qp_asymmetry = qp_asymmetry; p.weight_factor = (float)(exp2((double)w1) - 1.0); p.w2 = w2;
    p.tb_base = tb_remap_base; p.tb_scale = tb_remap_scale; p.tb_decay = tb_remap_decay;
    p.lambda = (float)lambda; p.one_minus_lambda = (float)(1.0 - lambda);
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(k_sf_loss_terms, dim3(blocks_for(B)), dim3(256), 0, st, scorenet, score, outcome, terms, B, p);
    NNUEFT_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_sf_loss_reduce, dim3(1), dim3(kLossThreads), 0, st, terms, sums, loss, B);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

extern "C" int nnueft_sf_loss_bwd(const float* terms, const float* sums, const float* grad_loss, float* grad_scorenet,
                                  int B, void* stream) {
    if (B <= 0 || !terms || !sums || !grad_loss || !grad_scorenet) return NNUEFT_E_ARG;
    hipLaunchKernelGGL(k_sf_loss_bwd, dim3(blocks_for(B)), dim3(256), 0, (hipStream_t)stream, terms, sums, grad_loss,
                       grad_scorenet, B);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}
