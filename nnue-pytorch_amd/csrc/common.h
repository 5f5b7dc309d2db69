// Shared device helpers for the feature-transformer kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nnueft.h"

#define NNUEFT_WAVE 64
// Positions per tile of the deterministic bias-gradient order (part of the ABI contract).
#define NNUEFT_BIAS_TILE 32
// Deterministic weight gradient: a table row named by more slots than NNUEFT_ROW_SPLIT (both
// perspectives together) is summed window by window, a window being nnueft_window_positions(B)
// consecutive positions: as few windows as keep each at NNUEFT_ROW_WINDOW_MIN positions or fewer, at
// most NNUEFT_ROW_WINDOWS of them, a multiple of 128.  (A window's upstream rows, one 1 KB slice of
// each, are what a XCD's L2 has to hold while the split rows are reduced: 1 MB at 1024 positions.)
#ifndef NNUEFT_ROW_SPLIT
#define NNUEFT_ROW_SPLIT 512
#endif
#ifndef NNUEFT_ROW_WINDOWS
#define NNUEFT_ROW_WINDOWS 16
#endif
#ifndef NNUEFT_ROW_WINDOW_MIN
#define NNUEFT_ROW_WINDOW_MIN 1024
#endif
static inline int nnueft_window_positions(int B) {
    int nwin = (B + NNUEFT_ROW_WINDOW_MIN - 1) / NNUEFT_ROW_WINDOW_MIN;
    if (nwin < 1) nwin = 1;
    if (nwin > NNUEFT_ROW_WINDOWS) nwin = NNUEFT_ROW_WINDOWS;
    const int w = (B + nwin - 1) / nwin;
    return (w + 127) / 128 * 128;
}

typedef unsigned long long u64;

// A lane's slice of a row: VW consecutive floats, moved with one 4- or 16-byte access.
template <int VW>
struct vecf {
    float v[VW];
};

template <int VW>
__device__ __forceinline__ vecf<VW> ldv(const float* p);
template <>
__device__ __forceinline__ vecf<4> ldv<4>(const float* p) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    vecf<4> r;
    r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
    return r;
}
template <>
__device__ __forceinline__ vecf<1> ldv<1>(const float* p) {
    vecf<1> r;
    r.v[0] = *p;
    return r;
}

template <int VW>
__device__ __forceinline__ void stv(float* p, const vecf<VW>& x);
template <>
__device__ __forceinline__ void stv<4>(float* p, const vecf<4>& x) {
    *reinterpret_cast<float4*>(p) = make_float4(x.v[0], x.v[1], x.v[2], x.v[3]);
}
template <>
__device__ __forceinline__ void stv<1>(float* p, const vecf<1>& x) {
    *p = x.v[0];
}

// Streaming store: the line is marked for early eviction, so write-once outputs do not push the
// rows being gathered out of L2.
template <int VW>
__device__ __forceinline__ void stv_stream(float* p, const vecf<VW>& x);
template <>
__device__ __forceinline__ void stv_stream<4>(float* p, const vecf<4>& x) {
#ifdef NNUEFT_NO_NT
    stv<4>(p, x);
#else
    typedef float f4 __attribute__((ext_vector_type(4)));
    f4 v = {x.v[0], x.v[1], x.v[2], x.v[3]};
    __builtin_nontemporal_store(v, reinterpret_cast<f4*>(p));
#endif
}
template <>
__device__ __forceinline__ void stv_stream<1>(float* p, const vecf<1>& x) {
#ifdef NNUEFT_NO_NT
    *p = x.v[0];
#else
    __builtin_nontemporal_store(x.v[0], p);
#endif
}

// Streaming load of 4 floats: data read once, not to displace what the kernel keeps in L2.
__device__ __forceinline__ vecf<4> ldv4_stream(const float* p) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const f4 v = __builtin_nontemporal_load(reinterpret_cast<const f4*>(p));
    vecf<4> r;
    r.v[0] = v.x; r.v[1] = v.y; r.v[2] = v.z; r.v[3] = v.w;
    return r;
}

template <int VW>
__device__ __forceinline__ vecf<VW> vzero() {
    vecf<VW> r;
#pragma unroll
    for (int i = 0; i < VW; ++i) r.v[i] = 0.0f;
    return r;
}

template <int VW>
__device__ __forceinline__ void vadd(vecf<VW>& a, const vecf<VW>& b) {
#pragma unroll
    for (int i = 0; i < VW; ++i) a.v[i] = a.v[i] + b.v[i];
}

__device__ __forceinline__ float clamp_act(float x, float hi) { return x < 0.0f ? 0.0f : (x > hi ? hi : x); }

// The four mixed pre-clamp values of a column pair (i, i + L1/2) from the two perspectives' row sums
// (sw*, sb*: white / black sums of the two columns; b0, b1: bias of the two columns).  Forward and
// backward both go through this function, so the backward sees exactly the forward's values.
__device__ __forceinline__ void mix4(float u, float t, float sw0, float sw1, float sb0, float sb1, float b0,
                                     float b1, float& xw0, float& xw1, float& xb0, float& xb1) {
    const float w0 = sw0 + b0, w1 = sw1 + b1;
    const float k0 = sb0 + b0, k1 = sb1 + b1;
    xw0 = u * w0 + t * k0;
    xw1 = u * w1 + t * k1;
    xb0 = u * k0 + t * w0;
    xb1 = u * k1 + t * w1;
}

// Whether a position's output row is one perspective's sums on each half: with (us, them) = (1, 0) the mixed
// values are w and k themselves, with (0, 1) they change places (u * w + t * k = w bit for bit when u = 1, t = 0
// and k is finite: a sum of a chain from +0 plus a bias is never -0).
__device__ __forceinline__ bool one_sided(float u, float t) {
    return (u == 1.0f && t == 0.0f) || (u == 0.0f && t == 1.0f);
}

// The four upstream values of that column pair for the two perspectives' sparse-linear outputs.
__device__ __forceinline__ void grad4(float u, float t, float xw0, float xw1, float xb0, float xb1, float g0,
                                      float g1, float max_act, float& gw0, float& gw1, float& gb0, float& gb1) {
    const float cw0 = clamp_act(xw0, max_act), cw1 = clamp_act(xw1, max_act);
    const float cb0 = clamp_act(xb0, max_act), cb1 = clamp_act(xb1, max_act);
    const float dw0 = (xw0 >= 0.0f && xw0 <= max_act) ? g0 * cw1 : 0.0f;
    const float dw1 = (xw1 >= 0.0f && xw1 <= max_act) ? g0 * cw0 : 0.0f;
    const float db0 = (xb0 >= 0.0f && xb0 <= max_act) ? g1 * cb1 : 0.0f;
    const float db1 = (xb1 >= 0.0f && xb1 <= max_act) ? g1 * cb0 : 0.0f;
    gw0 = u * dw0 + t * db0;
    gw1 = u * dw1 + t * db1;
    gb0 = t * dw0 + u * db0;
    gb1 = t * dw1 + u * db1;
}

// Lowest set bit of a wave mask, removed from the mask.  The mask comes from __ballot, so the
// result is wave-uniform and can drive scalar control flow and v_readlane.
__device__ __forceinline__ int pop_lane(u64& mask) {
    const int k = __ffsll((long long)mask) - 1;
    mask &= mask - 1;
    return k;
}

__device__ __forceinline__ int bcast_i(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }
__device__ __forceinline__ float bcast_f(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline bool aligned256(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 255u) == 0; }

#define NNUEFT_LAUNCH_CHECK()                         \
    do {                                              \
        hipError_t e__ = hipGetLastError();           \
        if (e__ != hipSuccess) return (int)e__;       \
    } while (0)
