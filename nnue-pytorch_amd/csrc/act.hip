// Activation fake quantization of the feature transformer's output, one pass instead of the
// module's chain of elementwise torch ops:  out = (floor(x * scale + eps) / scale) * post_mul,
// every operation rounding on its own, as torch's mul / add / floor / div / mul do.
#include "common.h"

namespace {

template <int VW>
__global__ __launch_bounds__(256) void k_act_fake_quantize(const float* __restrict__ x, float* __restrict__ out,
                                                           long long n, float scale, float eps, float post_mul) {
    const long long nvec = n / VW;
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nvec; i += stride) {
        vecf<VW> v = ldv<VW>(x + (size_t)i * VW);
#pragma unroll
        for (int k = 0; k < VW; ++k) v.v[k] = (floorf(v.v[k] * scale + eps) / scale) * post_mul;
        stv<VW>(out + (size_t)i * VW, v);
    }
    if (VW > 1) {
        const long long i = nvec * VW + (long long)blockIdx.x * 256 + threadIdx.x;
        if (i < n) out[i] = (floorf(x[i] * scale + eps) / scale) * post_mul;
    }
}

}  // namespace

extern "C" int nnueft_act_fake_quantize(const float* x, float* out, long long n, float scale, float eps,
                                        float post_mul, void* stream) {
    if (n <= 0 || !x || !out || !(scale > 0.0f)) return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (aligned16(x) && aligned16(out) && n >= 4) {
        const long long wg = (n / 4 + 255) / 256;
        hipLaunchKernelGGL(k_act_fake_quantize<4>, dim3((unsigned)max(1LL, min(wg, 0x7fffffffLL))), dim3(256), 0, st, x,
                           out, n, scale, eps, post_mul);
    } else {
        const long long wg = (n + 255) / 256;
        hipLaunchKernelGGL(k_act_fake_quantize<1>, dim3((unsigned)max(1LL, min(wg, 0x7fffffffLL))), dim3(256), 0, st, x,
                           out, n, scale, eps, post_mul);
    }
    NNUEFT_LAUNCH_CHECK();
    return 0;
}
