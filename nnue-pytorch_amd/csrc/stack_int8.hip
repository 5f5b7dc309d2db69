// Quantized layer stacks: the integer evaluation of one position's bucketed stack
//   a1 = b1 + W1 . x                     x u8 [L1] (the int16 feature transformer's output), W1 int8
//   y1 = clip([ (a1*a1) >> sqr1 , a1 >> lin1 ])          2*L2 values in 0..act_max
//   a2 = b2 + W2 . y1 ;  y2 = clip([ (a2*a2) >> sqr2 , a2 >> lin2 ])      2*L3 values
//   a3 = bo + Wo . [y1, y2]
//   out = trunc( 2 * (a3 + a1[L2-2] - a1[L2-1]) * out_mult / out_den )
// One wave per position.  The first layer dominates (L1 x L2 multiply-adds): lanes take dwords of x
// 64 apart (coalesced 256-byte loads of x and of every weight row) and feed v_dot4_i32_i8; x is
// at most 127, so it is a valid signed byte.
#include "common.h"

namespace {

constexpr int kMaxHidden = 32;   // L2 and L3 are at most this (their doubled width fits the wave)

__device__ __forceinline__ int wave_sum(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

__device__ __forceinline__ int clip_act(long long v, int act_max) {
    return (int)(v < 0 ? 0 : (v > act_max ? act_max : v));
}

template <int MAXD>   // dwords of x per lane
__global__ __launch_bounds__(64) void k_stack_int8(const uint8_t* __restrict__ x, const int64_t* __restrict__ bucket,
                                                   const int8_t* __restrict__ W1, const int32_t* __restrict__ b1,
                                                   const int8_t* __restrict__ W2, const int32_t* __restrict__ b2,
                                                   const int8_t* __restrict__ Wo, const int32_t* __restrict__ bo,
                                                   int32_t* __restrict__ out, int L1, int L2, int L3, int count,
                                                   int lin1, int sqr1, int lin2, int sqr2, int act_max, int out_mult,
                                                   int out_den) {
    const int lane = threadIdx.x;
    const int pos = blockIdx.x;
    long long bk = bucket[pos];
    if (bk < 0) bk = 0;
    if (bk >= count) bk = count - 1;
    const int nd = L1 >> 2;

    int xv[MAXD];
    const int* xrow = reinterpret_cast<const int*>(x + (size_t)pos * L1);
#pragma unroll
    for (int m = 0; m < MAXD; ++m) {
        const int d = lane + 64 * m;
        xv[m] = d < nd ? xrow[d] : 0;
    }
    // layer 1: every lane ends up with all L2 sums
    int a1[kMaxHidden];
    int skip = 0;
#pragma unroll
    for (int o = 0; o < kMaxHidden; ++o) {
        a1[o] = 0;
        if (o < L2) {
            const int* wrow = reinterpret_cast<const int*>(W1 + ((size_t)bk * L2 + o) * L1);
            int part = 0;
#pragma unroll
            for (int m = 0; m < MAXD; ++m) {
                const int d = lane + 64 * m;
                const int w = d < nd ? wrow[d] : 0;
                part = __builtin_amdgcn_sdot4(w, xv[m], part, false);
            }
            a1[o] = wave_sum(part) + b1[bk * L2 + o];
            if (o == L2 - 2) skip += a1[o];
            if (o == L2 - 1) skip -= a1[o];
        }
    }
    // y1: lane l < L2 holds the squared branch of sum l, lane L2 + l the linear branch
    int mine1 = 0;
#pragma unroll
    for (int o = 0; o < kMaxHidden; ++o)
        if (o < L2 && (lane == o || lane == L2 + o)) mine1 = a1[o];
    int y1 = 0;
    if (lane < L2) y1 = clip_act(((long long)mine1 * mine1) >> sqr1, act_max);
    else if (lane < 2 * L2) y1 = clip_act((long long)(mine1 >> lin1), act_max);

    // layer 2: lane j < L3 computes sum j over the 2*L2 values of y1
    int a2 = 0;
    if (lane < L3) a2 = b2[bk * L3 + lane];
    const int8_t* w2row = W2 + ((size_t)bk * L3 + (lane < L3 ? lane : 0)) * (2 * L2);
    for (int i = 0; i < 2 * L2; ++i) {
        const int yi = __shfl(y1, i);
        if (lane < L3) a2 += (int)w2row[i] * yi;
    }
    const int src2 = __shfl(a2, lane < L3 ? lane : (lane - L3 < L3 ? lane - L3 : 0));
    int y2 = 0;
    if (lane < L3) y2 = clip_act(((long long)src2 * src2) >> sqr2, act_max);
    else if (lane < 2 * L3) y2 = clip_act((long long)(src2 >> lin2), act_max);

    // output layer over [y1 (2*L2), y2 (2*L3)]
    const int8_t* worow = Wo + (size_t)bk * (2 * L2 + 2 * L3);
    int part = 0;
    if (lane < 2 * L2) part += (int)worow[lane] * y1;
    if (lane < 2 * L3) part += (int)worow[2 * L2 + lane] * y2;
    const int a3 = wave_sum(part) + bo[bk];
    if (lane == 0) {
        const long long num = 2ll * ((long long)a3 + skip) * out_mult;
        out[pos] = (int32_t)(num / out_den);   // C division: toward zero
    }
}

}  // namespace

extern "C" int nnueft_stack_int8_fwd(const uint8_t* x, const int64_t* bucket, const int8_t* W1, const int32_t* b1,
                                     const int8_t* W2, const int32_t* b2, const int8_t* Wo, const int32_t* bo,
                                     int32_t* out, int B, int L1, int L2, int L3, int count, int lin_shift1,
                                     int sqr_shift1, int lin_shift2, int sqr_shift2, int act_max, int out_mult,
                                     int out_den, void* stream) {
    if (B < 0 || L1 <= 0 || L2 < 2 || L3 < 1 || count <= 0) return NNUEFT_E_ARG;
    if (L2 > kMaxHidden || L3 > kMaxHidden || (L1 & 3)) return NNUEFT_E_UNSUPPORTED;
    if (lin_shift1 < 0 || lin_shift1 > 31 || lin_shift2 < 0 || lin_shift2 > 31 || sqr_shift1 < 0 || sqr_shift1 > 62 ||
        sqr_shift2 < 0 || sqr_shift2 > 62 || act_max < 0 || act_max > 127 || out_den <= 0)
        return NNUEFT_E_ARG;
    if (B == 0) return 0;
    if (!x || !bucket || !W1 || !b1 || !W2 || !b2 || !Wo || !bo || !out) return NNUEFT_E_ARG;
    if ((reinterpret_cast<uintptr_t>(x) & 3u) || (reinterpret_cast<uintptr_t>(W1) & 3u)) return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int nd = L1 / 4;
    const int per_lane = (nd + 63) / 64;
#define STACK_LAUNCH(MAXD)                                                                                          \
    hipLaunchKernelGGL(k_stack_int8<MAXD>, dim3(B), dim3(64), 0, st, x, bucket, W1, b1, W2, b2, Wo, bo, out, L1, L2, \
                       L3, count, lin_shift1, sqr_shift1, lin_shift2, sqr_shift2, act_max, out_mult, out_den)
    if (per_lane <= 1) STACK_LAUNCH(1);
    else if (per_lane <= 4) STACK_LAUNCH(4);
    else if (per_lane <= 8) STACK_LAUNCH(8);
    else if (per_lane <= 12) STACK_LAUNCH(12);
    else if (per_lane <= 16) STACK_LAUNCH(16);
    else return NNUEFT_E_UNSUPPORTED;   // L1 > 4096
#undef STACK_LAUNCH
    NNUEFT_LAUNCH_CHECK();
    return 0;
}
