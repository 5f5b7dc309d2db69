// The one inner loop every fp32 kernel here shares: a wave walks a list of row numbers held one
// per lane and adds a slice of each named row into per-lane accumulators, strictly in list
// order (the order is part of the result: fp32 addition does not associate).
#pragma once

#include "common.h"

// Fetch U rows, then add them one after the other.  U*NV loads are in flight per lane.
template <int VW, int NV, int U>
__device__ __forceinline__ void chain_group(vecf<VW> (&acc)[NV], const float* __restrict__ base, size_t stride,
                                            const int (&col)[NV], int myrow, u64& mask) {
    const float* rp[U];
#pragma unroll
    for (int u = 0; u < U; ++u) rp[u] = base + (size_t)bcast_i(myrow, pop_lane(mask)) * stride;
    vecf<VW> v[U][NV];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int j = 0; j < NV; ++j) v[u][j] = ldv<VW>(rp[u] + col[j]);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int j = 0; j < NV; ++j) vadd<VW>(acc[j], v[u][j]);
}

// acc[j] += base[row * stride + col[j] ...]  for every lane of `mask` in ascending lane order,
// where `row` is that lane's `myrow`.  Groups of U rows (U <= 64), then one group per set bit of
// the remaining count, so a short list still keeps several rows in flight.
template <int VW, int NV, int U>
__device__ __forceinline__ void chain_rows(vecf<VW> (&acc)[NV], const float* __restrict__ base, size_t stride,
                                           const int (&col)[NV], int myrow, u64 mask) {
    int cnt = __popcll(mask);
    while (cnt >= U) {
        chain_group<VW, NV, U>(acc, base, stride, col, myrow, mask);
        cnt -= U;
    }
    // what is left is below U: one group per set bit of the count, largest first
    if constexpr (U > 32) {
        if (cnt & 32) chain_group<VW, NV, 32>(acc, base, stride, col, myrow, mask);
    }
    if constexpr (U > 16) {
        if (cnt & 16) chain_group<VW, NV, 16>(acc, base, stride, col, myrow, mask);
    }
    if constexpr (U > 8) {
        if (cnt & 8) chain_group<VW, NV, 8>(acc, base, stride, col, myrow, mask);
    }
    if constexpr (U > 4) {
        if (cnt & 4) chain_group<VW, NV, 4>(acc, base, stride, col, myrow, mask);
    }
    if constexpr (U > 2) {
        if (cnt & 2) chain_group<VW, NV, 2>(acc, base, stride, col, myrow, mask);
    }
    if constexpr (U > 1) {
        if (cnt & 1) chain_group<VW, NV, 1>(acc, base, stride, col, myrow, mask);
    }
}
