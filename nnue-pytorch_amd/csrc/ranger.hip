// RangerLite parameter update, elementwise over one parameter tensor: second moment, first moment
// (plain, or the positive-negative pair that alternates between two buffers), optional decay,
// parameter step, and on merge steps the lookahead blend in the same pass.
// Each element is read and written once; every operation rounds on its own (no contraction), in
// the order written here, which is the order of the CPU checker.
#include "common.h"

namespace {

// One tensor's update; the layout is the public nnueft_ranger_args of the header.
typedef nnueft_ranger_args RangerArgs;

__device__ __forceinline__ void ranger_one(const RangerArgs& a, float& p, float g, float& gm, float& ngm, float& vm,
                                           float& slow) {
    if (a.update_variance) vm = vm * a.beta2 + (g * g) * a.one_minus_beta2;
    const float denom = sqrtf(vm / a.bias_correction2) + a.eps;
    float dir;
    if (a.neg_grad_ma) {
        const float pos = a.odd_step ? gm : ngm;
        const float neg = a.odd_step ? ngm : gm;
        const float new_pos = pos * a.beta1 + g * a.one_minus_beta1;
        dir = (new_pos * a.one_plus_pnm - neg * a.pnm_factor) / a.noise_norm;
        if (a.odd_step) gm = new_pos;
        else ngm = new_pos;
    } else {
        gm = gm * a.beta1 + g * a.one_minus_beta1;
        dir = gm;
    }
    float np = p;
    if (a.wd_factor != 0.0f) np = np * (1.0f - a.wd_factor);
    np = np - a.lr_div_bc1 * (dir / denom);
    if (a.lookahead_params) {
        np = np * a.lookahead_alpha + slow * a.one_minus_lookahead_alpha;
        slow = np;
    }
    p = np;
}

template <int VW>
__global__ __launch_bounds__(256) void k_ranger_update(RangerArgs a) {
    const long long nvec = a.n / VW;
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nvec; i += stride) {
        const size_t o = (size_t)i * VW;
        vecf<VW> p = ldv<VW>(a.p + o), g = ldv<VW>(a.grad + o), gm = ldv<VW>(a.grad_ma + o);
        vecf<VW> vm = ldv<VW>(a.variance_ma + o);
        vecf<VW> ngm = a.neg_grad_ma ? ldv<VW>(a.neg_grad_ma + o) : vzero<VW>();
        vecf<VW> slow = a.lookahead_params ? ldv<VW>(a.lookahead_params + o) : vzero<VW>();
#pragma unroll
        for (int k = 0; k < VW; ++k) ranger_one(a, p.v[k], g.v[k], gm.v[k], ngm.v[k], vm.v[k], slow.v[k]);
        stv<VW>(a.p + o, p);
        if (a.update_variance) stv<VW>(a.variance_ma + o, vm);
        if (a.neg_grad_ma) {
            // only the positive buffer of this step changed
            if (a.odd_step) stv<VW>(a.grad_ma + o, gm);
            else stv<VW>(a.neg_grad_ma + o, ngm);
        } else {
            stv<VW>(a.grad_ma + o, gm);
        }
        if (a.lookahead_params) stv<VW>(a.lookahead_params + o, slow);
    }
    if (VW > 1) {
        // tail of fewer than VW elements
        const long long i = nvec * VW + (long long)blockIdx.x * 256 + threadIdx.x;
        if (i < a.n) {
            float ngm = a.neg_grad_ma ? a.neg_grad_ma[i] : 0.0f, slow = a.lookahead_params ? a.lookahead_params[i] : 0.0f;
            float p = a.p[i], gm = a.grad_ma[i], vm = a.variance_ma[i];
            ranger_one(a, p, a.grad[i], gm, ngm, vm, slow);
            a.p[i] = p;
            if (a.update_variance) a.variance_ma[i] = vm;
            if (a.neg_grad_ma && !a.odd_step) a.neg_grad_ma[i] = ngm;
            else a.grad_ma[i] = gm;
            if (a.lookahead_params) a.lookahead_params[i] = slow;
        }
    }
}

// Several small tensors in one launch: workgroup -> tensor through the running count of workgroups,
// then one element per thread.  A launch costs a few microseconds whatever the tensor's size, and a
// model has many small tensors (biases, the layers of the stacks).
constexpr int kMultiMax = 16;
struct RangerMulti {
    RangerArgs t[kMultiMax];
    unsigned first[kMultiMax + 1];   // first workgroup of every tensor
    int count;
};

__global__ __launch_bounds__(256) void k_ranger_update_multi(RangerMulti m) {
    int k = 0;
    while (k + 1 < m.count && blockIdx.x >= m.first[k + 1]) ++k;
    const RangerArgs& a = m.t[k];
    const long long i = (long long)(blockIdx.x - m.first[k]) * 256 + threadIdx.x;
    if (i >= a.n) return;
    float ngm = a.neg_grad_ma ? a.neg_grad_ma[i] : 0.0f, slow = a.lookahead_params ? a.lookahead_params[i] : 0.0f;
    float p = a.p[i], gm = a.grad_ma[i], vm = a.variance_ma[i];
    ranger_one(a, p, a.grad[i], gm, ngm, vm, slow);
    a.p[i] = p;
    if (a.update_variance) a.variance_ma[i] = vm;
    if (a.neg_grad_ma && !a.odd_step) a.neg_grad_ma[i] = ngm;
    else a.grad_ma[i] = gm;
    if (a.lookahead_params) a.lookahead_params[i] = slow;
}

template <int VW>
__global__ __launch_bounds__(256) void k_ranger_variance(const float* __restrict__ grad, float* __restrict__ vm,
                                                         long long n, float beta2, float one_minus_beta2) {
    const long long nvec = n / VW;
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nvec; i += stride) {
        const size_t o = (size_t)i * VW;
        vecf<VW> g = ldv<VW>(grad + o), v = ldv<VW>(vm + o);
#pragma unroll
        for (int k = 0; k < VW; ++k) v.v[k] = v.v[k] * beta2 + (g.v[k] * g.v[k]) * one_minus_beta2;
        stv<VW>(vm + o, v);
    }
    if (VW > 1) {
        const long long i = nvec * VW + (long long)blockIdx.x * 256 + threadIdx.x;
        if (i < n) vm[i] = vm[i] * beta2 + (grad[i] * grad[i]) * one_minus_beta2;
    }
}

template <int VW>
__global__ __launch_bounds__(256) void k_lookahead_merge(float* __restrict__ p, float* __restrict__ slow, long long n,
                                                         float alpha, float one_minus_alpha) {
    const long long nvec = n / VW;
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nvec; i += stride) {
        const size_t o = (size_t)i * VW;
        vecf<VW> a = ldv<VW>(p + o), s = ldv<VW>(slow + o);
#pragma unroll
        for (int k = 0; k < VW; ++k) a.v[k] = a.v[k] * alpha + s.v[k] * one_minus_alpha;
        stv<VW>(p + o, a);
        stv<VW>(slow + o, a);
    }
    if (VW > 1) {
        const long long i = nvec * VW + (long long)blockIdx.x * 256 + threadIdx.x;
        if (i < n) {
            const float a = p[i] * alpha + slow[i] * one_minus_alpha;
            p[i] = a;
            slow[i] = a;
        }
    }
}

// one vector per thread (measured 12 % faster on the 75 M-element table than a grid-stride loop over
// a few thousand workgroups); the loops only matter beyond 2^31 workgroups
inline unsigned grid_for(long long nvec) {
    const long long want = (nvec + 255) / 256;
    return (unsigned)max(1LL, min(want, 0x7fffffffLL));
}

int launch_update(RangerArgs a, hipStream_t st) {
    if (a.n <= 0) return NNUEFT_E_ARG;
    if (!a.p || !a.grad || !a.grad_ma || !a.variance_ma) return NNUEFT_E_ARG;
    const bool vec = aligned16(a.p) && aligned16(a.grad) && aligned16(a.grad_ma) && aligned16(a.variance_ma) &&
                     (!a.neg_grad_ma || aligned16(a.neg_grad_ma)) && (!a.lookahead_params || aligned16(a.lookahead_params)) && a.n >= 4;
    if (vec) hipLaunchKernelGGL(k_ranger_update<4>, dim3(grid_for(a.n / 4)), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(k_ranger_update<1>, dim3(grid_for(a.n)), dim3(256), 0, st, a);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

}  // namespace

extern "C" int nnueft_ranger_lite_update_pnm(float* p, const float* grad, float* grad_ma, float* neg_grad_ma,
                                             float* variance_ma, long long n, float beta2, float one_minus_beta2,
                                             float bias_correction2, float beta1_sq, float one_minus_beta1_sq,
                                             float one_plus_pnm, float pnm_factor, float noise_norm,
                                             float lr_div_bc1, float eps, long long step, float wd_factor,
                                             int update_variance, float* lookahead_params, float lookahead_alpha,
                                             void* stream) {
    if (!neg_grad_ma) return NNUEFT_E_ARG;
    RangerArgs a{};
    a.p = p; a.grad = grad; a.grad_ma = grad_ma; a.neg_grad_ma = neg_grad_ma; a.variance_ma = variance_ma;
    a.lookahead_params = lookahead_params; a.n = n;
    a.beta2 = beta2; a.one_minus_beta2 = one_minus_beta2; a.bias_correction2 = bias_correction2;
    a.beta1 = beta1_sq; a.one_minus_beta1 = one_minus_beta1_sq;
    a.one_plus_pnm = one_plus_pnm; a.pnm_factor = pnm_factor; a.noise_norm = noise_norm;
    a.lr_div_bc1 = lr_div_bc1; a.eps = eps; a.wd_factor = wd_factor;
    a.lookahead_alpha = lookahead_alpha; a.one_minus_lookahead_alpha = 1.0f - lookahead_alpha;
    a.odd_step = (int)(step & 1LL); a.update_variance = update_variance != 0;
    return launch_update(a, (hipStream_t)stream);
}

extern "C" int nnueft_ranger_lite_update_adam(float* p, const float* grad, float* grad_ma, float* variance_ma,
                                              long long n, float beta2, float one_minus_beta2, float bias_correction2,
                                              float beta1, float one_minus_beta1, float lr_div_bc1, float eps,
                                              float wd_factor, int update_variance, float* lookahead_params,
                                              float lookahead_alpha, void* stream) {
    RangerArgs a{};
    a.p = p; a.grad = grad; a.grad_ma = grad_ma; a.neg_grad_ma = nullptr; a.variance_ma = variance_ma;
    a.lookahead_params = lookahead_params; a.n = n;
    a.beta2 = beta2; a.one_minus_beta2 = one_minus_beta2; a.bias_correction2 = bias_correction2;
    a.beta1 = beta1; a.one_minus_beta1 = one_minus_beta1;
    a.lr_div_bc1 = lr_div_bc1; a.eps = eps; a.wd_factor = wd_factor;
    a.lookahead_alpha = lookahead_alpha; a.one_minus_lookahead_alpha = 1.0f - lookahead_alpha;
    a.update_variance = update_variance != 0;
    return launch_update(a, (hipStream_t)stream);
}

extern "C" int nnueft_ranger_lite_update_multi(const nnueft_ranger_args* tensors, int count, void* stream) {
    if (count <= 0 || !tensors) return NNUEFT_E_ARG;
    for (int i = 0; i < count; ++i) {
        const nnueft_ranger_args& a = tensors[i];
        if (a.n <= 0 || !a.p || !a.grad || !a.grad_ma || !a.variance_ma) return NNUEFT_E_ARG;
        if ((a.n + 255) / 256 > 0x0fffffffLL) return NNUEFT_E_UNSUPPORTED;
    }
    for (int i0 = 0; i0 < count; i0 += kMultiMax) {
        RangerMulti m{};
        m.count = min(kMultiMax, count - i0);
        unsigned blocks = 0;
        for (int k = 0; k < m.count; ++k) {
            m.t[k] = tensors[i0 + k];
            m.first[k] = blocks;
            blocks += (unsigned)((m.t[k].n + 255) / 256);
        }
        m.first[m.count] = blocks;
        hipLaunchKernelGGL(k_ranger_update_multi, dim3(blocks), dim3(256), 0, (hipStream_t)stream, m);
        NNUEFT_LAUNCH_CHECK();
    }
    return 0;
}

extern "C" int nnueft_ranger_lite_update_variance(const float* grad, float* variance_ma, long long n, float beta2,
                                                  float one_minus_beta2, void* stream) {
    if (n <= 0 || !grad || !variance_ma) return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (aligned16(grad) && aligned16(variance_ma) && n >= 4)
        hipLaunchKernelGGL(k_ranger_variance<4>, dim3(grid_for(n / 4)), dim3(256), 0, st, grad, variance_ma, n, beta2,
                           one_minus_beta2);
    else
        hipLaunchKernelGGL(k_ranger_variance<1>, dim3(grid_for(n)), dim3(256), 0, st, grad, variance_ma, n, beta2,
                           one_minus_beta2);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

extern "C" int nnueft_ranger_lite_lookahead_merge(float* p, float* lookahead_params, long long n, float alpha,
                                                  void* stream) {
    if (n <= 0 || !p || !lookahead_params) return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (aligned16(p) && aligned16(lookahead_params) && n >= 4)
        hipLaunchKernelGGL(k_lookahead_merge<4>, dim3(grid_for(n / 4)), dim3(256), 0, st, p, lookahead_params, n, alpha,
                           1.0f - alpha);
    else
        hipLaunchKernelGGL(k_lookahead_merge<1>, dim3(grid_for(n)), dim3(256), 0, st, p, lookahead_params, n, alpha,
                           1.0f - alpha);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}
