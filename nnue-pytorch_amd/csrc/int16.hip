// Quantized feature transformer: int16 gather-accumulate, clip, pairwise product >> shift -> u8.
//
// One wave per (position, column slice); a lane owns NQ vectors of VW int16 in each half of the
// accumulator, 64 lanes apart, so each load instruction of the wave reads 1 KiB of a gathered row
// (VW = 8).  Adds are unsigned 16-bit, i.e. they wrap like the engine's SIMD adds.
#include "common.h"

namespace {

typedef unsigned short us8 __attribute__((ext_vector_type(8)));

template <int VW>
struct veci {
    unsigned short v[VW];
};

template <int VW>
__device__ __forceinline__ veci<VW> ldi(const int16_t* p);
template <>
__device__ __forceinline__ veci<8> ldi<8>(const int16_t* p) {
    const us8 t = *reinterpret_cast<const us8*>(p);
    veci<8> r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r.v[i] = t[i];
    return r;
}
template <>
__device__ __forceinline__ veci<1> ldi<1>(const int16_t* p) {
    veci<1> r;
    r.v[0] = (unsigned short)*p;
    return r;
}

template <int VW>
__device__ __forceinline__ void iadd(veci<VW>& a, const veci<VW>& b) {
#pragma unroll
    for (int i = 0; i < VW; ++i) a.v[i] = (unsigned short)(a.v[i] + b.v[i]);
}

template <int VW>
__device__ __forceinline__ void store_u8(uint8_t* p, const uint8_t (&o)[VW]);
template <>
__device__ __forceinline__ void store_u8<8>(uint8_t* p, const uint8_t (&o)[8]) {
    uint2 w;
    w.x = (uint32_t)o[0] | ((uint32_t)o[1] << 8) | ((uint32_t)o[2] << 16) | ((uint32_t)o[3] << 24);
    w.y = (uint32_t)o[4] | ((uint32_t)o[5] << 8) | ((uint32_t)o[6] << 16) | ((uint32_t)o[7] << 24);
    *reinterpret_cast<uint2*>(p) = w;
}
template <>
__device__ __forceinline__ void store_u8<1>(uint8_t* p, const uint8_t (&o)[1]) {
    *p = o[0];
}

constexpr int kU = 4;

template <int VW, int NQ>
__global__ __launch_bounds__(64) void k_ft_int16_fwd(const int32_t* __restrict__ widx,
                                                     const int32_t* __restrict__ bidx,
                                                     const uint8_t* __restrict__ stm,
                                                     const int16_t* __restrict__ W16,
                                                     const int16_t* __restrict__ b16,
                                                     const int32_t* __restrict__ psqt32,
                                                     const int64_t* __restrict__ psqt_idx,
                                                     uint8_t* __restrict__ out_u8, int32_t* __restrict__ psqt_out,
                                                     int K, int R, int L1, int n_psqt, int clip_max, int shift,
                                                     int nslices) {
    const int lane = threadIdx.x;
    const int b = blockIdx.x / nslices;
    const int s = blockIdx.x - b * nslices;
    const int h = L1 >> 1;
    const int hv = h / VW;

    int col[2 * NQ];
    bool act[NQ];
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        const int q = (s * NQ + m) * 64 + lane;
        act[m] = q < hv;
        col[2 * m] = act[m] ? q * VW : 0;
        col[2 * m + 1] = col[2 * m] + h;
    }
    const int64_t pi = psqt_idx[b];
    const bool do_psqt = (s == 0) && pi >= 0 && pi < n_psqt;

    veci<VW> acc[2][2 * NQ];
    uint32_t ps[2] = {0u, 0u};
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
        for (int j = 0; j < 2 * NQ; ++j) acc[p][j] = ldi<VW>(b16 + col[j]);
        const int32_t* ix = (p ? bidx : widx) + (size_t)b * K;
        for (int k0 = 0; k0 < K; k0 += 64) {
            const int my = (k0 + lane < K) ? ix[k0 + lane] : -1;
            const bool ok = my >= 0 && my < R;
            u64 mask = __ballot(ok);
            if (do_psqt && ok) ps[p] += (uint32_t)psqt32[(size_t)my * n_psqt + pi];
            int cnt = __popcll(mask);
            while (cnt >= kU) {
                const int16_t* rp[kU];
#pragma unroll
                for (int u = 0; u < kU; ++u) rp[u] = W16 + (size_t)bcast_i(my, pop_lane(mask)) * L1;
                veci<VW> v[kU][2 * NQ];
#pragma unroll
                for (int u = 0; u < kU; ++u)
#pragma unroll
                    for (int j = 0; j < 2 * NQ; ++j) v[u][j] = ldi<VW>(rp[u] + col[j]);
#pragma unroll
                for (int u = 0; u < kU; ++u)
#pragma unroll
                    for (int j = 0; j < 2 * NQ; ++j) iadd<VW>(acc[p][j], v[u][j]);
                cnt -= kU;
            }
            while (cnt > 0) {
                const int16_t* rp = W16 + (size_t)bcast_i(my, pop_lane(mask)) * L1;
#pragma unroll
                for (int j = 0; j < 2 * NQ; ++j) iadd<VW>(acc[p][j], ldi<VW>(rp + col[j]));
                --cnt;
            }
        }
    }

    const int first = stm[b] ? 1 : 0;
    uint8_t* dst = out_u8 + (size_t)b * L1;
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        if (!act[m]) continue;
#pragma unroll
        for (int o = 0; o < 2; ++o) {
            // perspective shown in output half o: `first` for o = 0, the other one for o = 1
            const bool take_black = (o == 0) ? (first == 1) : (first == 0);
            uint8_t res[VW];
#pragma unroll
            for (int i = 0; i < VW; ++i) {
                const int a0 = (int)(int16_t)(take_black ? acc[1][2 * m].v[i] : acc[0][2 * m].v[i]);
                const int a1 = (int)(int16_t)(take_black ? acc[1][2 * m + 1].v[i] : acc[0][2 * m + 1].v[i]);
                const int c0 = min(max(a0, 0), clip_max);
                const int c1 = min(max(a1, 0), clip_max);
                res[i] = (uint8_t)((c0 * c1) >> shift);
            }
            store_u8<VW>(dst + (size_t)o * h + col[2 * m], res);
        }
    }
    if (s == 0) {
        int32_t d = (int32_t)(first ? ps[1] - ps[0] : ps[0] - ps[1]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) d += __shfl_xor(d, off);
        if (lane == 0) psqt_out[b] = d / 2;
    }
}

template <int VW, int NQ>
int launch_int16(const int32_t* widx, const int32_t* bidx, const uint8_t* stm, const int16_t* W16,
                 const int16_t* b16, const int32_t* psqt32, const int64_t* psqt_idx, uint8_t* out_u8,
                 int32_t* psqt_out, int B, int K, int R, int L1, int n_psqt, int clip_max, int shift,
                 hipStream_t st) {
    const int hv = (L1 / 2) / VW;
    const int nslices = max(1, (hv + 64 * NQ - 1) / (64 * NQ));
    const long long grid = (long long)B * nslices;
    if (grid > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
    hipLaunchKernelGGL((k_ft_int16_fwd<VW, NQ>), dim3((unsigned)grid), dim3(64), 0, st, widx, bidx, stm, W16, b16,
                       psqt32, psqt_idx, out_u8, psqt_out, K, R, L1, n_psqt, clip_max, shift, nslices);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

}  // namespace

extern "C" int nnueft_ft_int16_fwd(const int32_t* widx, const int32_t* bidx, const uint8_t* stm,
                                   const int16_t* W16, const int16_t* b16, const int32_t* psqt32,
                                   const int64_t* psqt_idx, uint8_t* out_u8, int32_t* psqt_out, int B, int K, int R,
                                   int L1, int n_psqt, int clip_max, int shift, void* stream) {
    if (B < 0 || K <= 0 || R <= 0 || L1 <= 0 || (L1 & 1) || n_psqt < 0) return NNUEFT_E_ARG;
    if (clip_max < 0 || clip_max > 32767 || shift < 0 || shift > 30) return NNUEFT_E_ARG;
    if (B == 0) return 0;
    if (!widx || !bidx || !stm || !W16 || !b16 || !psqt_idx || !out_u8 || !psqt_out) return NNUEFT_E_ARG;
    if (n_psqt > 0 && !psqt32) return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    // The per-slot psqt sum is a wave reduction over one 64-slot group at a time; order is free (integers).
    const bool vec = (L1 % 16 == 0) && aligned16(W16) && aligned16(b16) && ((reinterpret_cast<uintptr_t>(out_u8) & 7u) == 0);
#define ARGS widx, bidx, stm, W16, b16, psqt32, psqt_idx, out_u8, psqt_out, B, K, R, L1, n_psqt, clip_max, shift, st
    if (vec) {
        const int hv = L1 / 16;
        if (hv > 128) return launch_int16<8, 3>(ARGS);
        if (hv > 64) return launch_int16<8, 2>(ARGS);
        return launch_int16<8, 1>(ARGS);
    }
    if (L1 / 2 > 64) return launch_int16<1, 2>(ARGS);
    return launch_int16<1, 1>(ARGS);
#undef ARGS
}
