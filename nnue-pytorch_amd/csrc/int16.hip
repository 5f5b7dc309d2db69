// Quantized feature transformer: int16 gather-accumulate, clip, pairwise product >> shift -> u8.
//
// Adds are unsigned 16-bit (they wrap like the engine's SIMD adds); a lane moves 8 int16 (16 bytes)
// per load and adds them with packed 16-bit instructions.
//
// Two paths:
//   k_ft_int16_fwd        one wave per (position, column slice), both perspectives; no scratch memory
//   L2-blocked (workspace) positions' lists grouped by table block, XCD = workgroup id % 8, one column
//                         slice at a time (see fwd_blocked.hip for the idea):
//       k_acc16_white     wave per (white list, slice): b16 + sum of rows -> accW[B, L1] int16
//       k_black_mix16     wave per (black list, paired slice): black sums in registers, the white ones
//                         read back, side-to-move order, clip, product, u8 store; psqt sums
//   LDS-tiled (workspace, table blocks of 768 rows, L1 a multiple of 64, lists of 32 slots at most): the
//                         forward's gather out of LDS tiles (fwd_tile.hip) over the int16 table
//       k_acc_tile        a tile is 32 column pairs (j, j + L1/2): the sums of a pair and tile stay in registers and
//                         leave as 32 output bytes (+ b16, clip, product >> shift) in the half the side to move selects
//       k_tl_lists        (the sort in front of it) the psqt difference of every position, while it has the lists
#include "internal.h"

namespace {

typedef unsigned short us8 __attribute__((ext_vector_type(8)));

template <int VW>
struct vecs;   // VW int16 lanes as one value
template <>
struct vecs<8> {
    us8 v;
};
template <>
struct vecs<1> {
    unsigned short v;
};

template <int VW>
__device__ __forceinline__ vecs<VW> ldi(const int16_t* p);
template <>
__device__ __forceinline__ vecs<8> ldi<8>(const int16_t* p) {
    vecs<8> r;
    r.v = *reinterpret_cast<const us8*>(p);
    return r;
}
template <>
__device__ __forceinline__ vecs<1> ldi<1>(const int16_t* p) {
    vecs<1> r;
    r.v = (unsigned short)*p;
    return r;
}

template <int VW>
__device__ __forceinline__ void iadd(vecs<VW>& a, const vecs<VW>& b) {
    a.v = a.v + b.v;   // unsigned: wraps
}

__device__ __forceinline__ int lane16(const vecs<8>& a, int i) { return (int)(short)a.v[i]; }
__device__ __forceinline__ int lane16(const vecs<1>& a, int) { return (int)(short)a.v; }

// streaming store of 8 int16 (written once, read once by the next kernel)
__device__ __forceinline__ void sti8(int16_t* p, const vecs<8>& x) {
    __builtin_nontemporal_store(x.v, reinterpret_cast<us8*>(p));
}

// out bytes = (clip(a0) * clip(a1)) >> shift for the VW column pairs held in a0 / a1
template <int VW>
__device__ __forceinline__ void pair_product_store(uint8_t* p, const vecs<VW>& a0, const vecs<VW>& a1, int clip_max,
                                                   int shift) {
    uint8_t o[VW];
#pragma unroll
    for (int i = 0; i < VW; ++i) {
        const int c0 = min(max(lane16(a0, i), 0), clip_max);
        const int c1 = min(max(lane16(a1, i), 0), clip_max);
        o[i] = (uint8_t)((c0 * c1) >> shift);
    }
    if constexpr (VW == 8) {
        uint2 w;
        w.x = (uint32_t)o[0] | ((uint32_t)o[1] << 8) | ((uint32_t)o[2] << 16) | ((uint32_t)o[3] << 24);
        w.y = (uint32_t)o[4] | ((uint32_t)o[5] << 8) | ((uint32_t)o[6] << 16) | ((uint32_t)o[7] << 24);
        *reinterpret_cast<uint2*>(p) = w;
    } else {
        *p = o[0];
    }
}

// acc[j] += W16[row, col[j] ...] for the lanes of `mask` (any order: integer adds), U rows at a time
template <int VW, int NV, int U>
__device__ __forceinline__ void gather16(vecs<VW> (&acc)[NV], const int16_t* __restrict__ W16, int L1,
                                         const int (&col)[NV], int myrow, u64 mask) {
    int cnt = __popcll(mask);
    while (cnt >= U) {
        const int16_t* rp[U];
#pragma unroll
        for (int u = 0; u < U; ++u) rp[u] = W16 + (size_t)bcast_i(myrow, pop_lane(mask)) * L1;
        vecs<VW> v[U][NV];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < NV; ++j) v[u][j] = ldi<VW>(rp[u] + col[j]);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < NV; ++j) iadd<VW>(acc[j], v[u][j]);
        cnt -= U;
    }
    while (cnt > 0) {
        const int16_t* rp = W16 + (size_t)bcast_i(myrow, pop_lane(mask)) * L1;
#pragma unroll
        for (int j = 0; j < NV; ++j) iadd<VW>(acc[j], ldi<VW>(rp + col[j]));
        --cnt;
    }
}

__device__ __forceinline__ int wave_sum_i(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// psqt_out[b] = (sum over the mover's list - sum over the other list) / 2 of psqt32[., bucket]
__device__ __forceinline__ void psqt_diff(const int32_t* __restrict__ widx, const int32_t* __restrict__ bidx,
                                          const int32_t* __restrict__ psqt32, int64_t pi, int first, int b, int K,
                                          int R, int n_psqt, int lane, int32_t* __restrict__ psqt_out) {
    uint32_t ps[2] = {0u, 0u};
    if (pi >= 0 && pi < n_psqt) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int32_t* ix = (p ? bidx : widx) + (size_t)b * K;
            for (int k = lane; k < K; k += 64) {
                const int r = ix[k];
                if (r >= 0 && r < R) ps[p] += (uint32_t)psqt32[(size_t)r * n_psqt + pi];
            }
        }
    }
    const int d = wave_sum_i((int32_t)(first ? ps[1] - ps[0] : ps[0] - ps[1]));
    if (lane == 0) psqt_out[b] = d / 2;
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
    vecs<VW> acc[2][2 * NQ];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
        for (int j = 0; j < 2 * NQ; ++j) acc[p][j] = ldi<VW>(b16 + col[j]);
        const int32_t* ix = (p ? bidx : widx) + (size_t)b * K;
        for (int k0 = 0; k0 < K; k0 += 64) {
            const int my = (k0 + lane < K) ? ix[k0 + lane] : -1;
            gather16<VW, 2 * NQ, kU>(acc[p], W16, L1, col, my, __ballot(my >= 0 && my < R));
        }
    }
    const int first = stm[b] ? 1 : 0;
    uint8_t* dst = out_u8 + (size_t)b * L1;
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        if (!act[m]) continue;
        // output half 0 shows the side to move, half 1 the other side
        if (first) {
            pair_product_store<VW>(dst + col[2 * m], acc[1][2 * m], acc[1][2 * m + 1], clip_max, shift);
            pair_product_store<VW>(dst + h + col[2 * m], acc[0][2 * m], acc[0][2 * m + 1], clip_max, shift);
        } else {
            pair_product_store<VW>(dst + col[2 * m], acc[0][2 * m], acc[0][2 * m + 1], clip_max, shift);
            pair_product_store<VW>(dst + h + col[2 * m], acc[1][2 * m], acc[1][2 * m + 1], clip_max, shift);
        }
    }
    if (s == 0) psqt_diff(widx, bidx, psqt32, psqt_idx[b], first, b, K, R, n_psqt, lane, psqt_out);
}

// ---- L2-blocked path ----------------------------------------------------------------------------

// accW[b, slice] = b16 + rows of the white list.  Tasks walk the jointly sorted pair order; black
// pairs are left to k_black_mix16.
template <int NQ, int U>
__global__ __launch_bounds__(64) void k_acc16_white(const int32_t* __restrict__ widx,
                                                    const uint32_t* __restrict__ order,
                                                    const int16_t* __restrict__ W16, const int16_t* __restrict__ b16,
                                                    int16_t* __restrict__ accW, int B, int K, int R, int L1,
                                                    int per_xcd) {
    const int lane = threadIdx.x;
    const int xcd = blockIdx.x % nnueft_blocked::kXcd;
    const int j = blockIdx.x / nnueft_blocked::kXcd;
    const int s = j / per_xcd;
    const int n = xcd * per_xcd + (j - s * per_xcd);
    if (n >= 2 * B) return;
    const int pair = (int)order[n];
    if (pair >= B) return;
    const int b = pair;
    const int nv = L1 / 8;
    int col[NQ];
    bool act[NQ];
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        const int q = (s * NQ + m) * 64 + lane;
        act[m] = q < nv;
        col[m] = act[m] ? q * 8 : 0;
    }
    vecs<8> acc[NQ];
#pragma unroll
    for (int m = 0; m < NQ; ++m) acc[m] = ldi<8>(b16 + col[m]);
    const int32_t* ix = widx + (size_t)b * K;
    for (int k0 = 0; k0 < K; k0 += 64) {
        const int my = (k0 + lane < K) ? ix[k0 + lane] : -1;
        gather16<8, NQ, U>(acc, W16, L1, col, my, __ballot(my >= 0 && my < R));
    }
#pragma unroll
    for (int m = 0; m < NQ; ++m)
        if (act[m]) sti8(accW + (size_t)b * L1 + col[m], acc[m]);
}

// Black list of a position: sums of column pairs (j, j + h) in registers, white sums from accW,
// then the output bytes of both halves for these columns.
template <int U>
__global__ __launch_bounds__(64) void k_black_mix16(const int32_t* __restrict__ widx,
                                                    const int32_t* __restrict__ bidx,
                                                    const uint32_t* __restrict__ order,
                                                    const uint8_t* __restrict__ stm,
                                                    const int16_t* __restrict__ W16, const int16_t* __restrict__ b16,
                                                    const int16_t* __restrict__ accW,
                                                    const int32_t* __restrict__ psqt32,
                                                    const int64_t* __restrict__ psqt_idx,
                                                    uint8_t* __restrict__ out_u8, int32_t* __restrict__ psqt_out,
                                                    int B, int K, int R, int L1, int n_psqt, int clip_max, int shift,
                                                    int per_xcd) {
    const int lane = threadIdx.x;
    const int xcd = blockIdx.x % nnueft_blocked::kXcd;
    const int j = blockIdx.x / nnueft_blocked::kXcd;
    const int s = j / per_xcd;
    const int n = xcd * per_xcd + (j - s * per_xcd);
    if (n >= 2 * B) return;
    const int pair = (int)order[n];
    if (pair < B) return;
    const int b = pair - B;
    const int h = L1 >> 1;
    const int hv = h / 8;
    const int q = s * 64 + lane;
    const int first = stm[b] ? 1 : 0;
    if (s == 0) psqt_diff(widx, bidx, psqt32, psqt_idx[b], first, b, K, R, n_psqt, lane, psqt_out);
    const bool act = q < hv;
    int col[2];
    col[0] = act ? q * 8 : 0;
    col[1] = col[0] + h;
    vecs<8> acc[2];
    acc[0] = ldi<8>(b16 + col[0]);
    acc[1] = ldi<8>(b16 + col[1]);
    const int32_t* ix = bidx + (size_t)b * K;
    for (int k0 = 0; k0 < K; k0 += 64) {
        const int my = (k0 + lane < K) ? ix[k0 + lane] : -1;
        gather16<8, 2, U>(acc, W16, L1, col, my, __ballot(my >= 0 && my < R));
    }
    if (!act) return;
    const vecs<8> w0 = ldi<8>(accW + (size_t)b * L1 + col[0]);
    const vecs<8> w1 = ldi<8>(accW + (size_t)b * L1 + col[1]);
    uint8_t* dst = out_u8 + (size_t)b * L1;
    if (first) {
        pair_product_store<8>(dst + col[0], acc[0], acc[1], clip_max, shift);
        pair_product_store<8>(dst + h + col[0], w0, w1, clip_max, shift);
    } else {
        pair_product_store<8>(dst + col[0], w0, w1, clip_max, shift);
        pair_product_store<8>(dst + h + col[0], acc[0], acc[1], clip_max, shift);
    }
}

struct Int16Layout {
    size_t accW, sort, end;
    size_t tile_sort;              // the LDS-tiled path's view of the same bytes: its sort scratch
    bool tile_ok;                  // the table's blocks fit its tiles
};

inline size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

bool int16_layout(int B, int R, int L1, int block_rows, Int16Layout* L) {
    if (B <= 0 || R <= 0 || L1 <= 0) return false;
    size_t off = 0;
    L->accW = off;
    off += up256((size_t)B * L1 * sizeof(int16_t));
    L->sort = off;
    off += up256(nnueft_blocked::pair_sort_workspace(B, R, block_rows));
    L->end = off;
    // the LDS-tiled path needs its sort scratch only: the sums never leave the gather
    L->tile_sort = 0;
    const int br = block_rows > 0 ? block_rows : nnueft_tile::kBlockRows;
    const size_t tile_ws = br <= nnueft_tile::kBlockRows ? nnueft_tile::workspace_int16(B, R, br) : 0;
    L->tile_ok = tile_ws > 0;
    const size_t tile_end = L->tile_sort + up256(tile_ws);
    if (L->tile_ok && tile_end > L->end) L->end = tile_end;
    return true;
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

extern "C" size_t nnueft_int16_workspace_bytes(int B, int K, int R, int L1, int table_block_rows) {
    if (K <= 0) return 0;
    Int16Layout L;
    return int16_layout(B, R, L1, table_block_rows, &L) ? L.end : 0;
}

extern "C" int nnueft_ft_int16_fwd(const int32_t* widx, const int32_t* bidx, const uint8_t* stm,
                                   const int16_t* W16, const int16_t* b16, const int32_t* psqt32,
                                   const int64_t* psqt_idx, uint8_t* out_u8, int32_t* psqt_out, int B, int K, int R,
                                   int L1, int n_psqt, int clip_max, int shift, int table_block_rows, void* workspace,
                                   size_t workspace_bytes, void* stream) {
    if (B < 0 || K <= 0 || R <= 0 || L1 <= 0 || (L1 & 1) || n_psqt < 0 || table_block_rows < 0) return NNUEFT_E_ARG;
    if (clip_max < 0 || clip_max > 32767 || shift < 0 || shift > 30) return NNUEFT_E_ARG;
    if (B == 0) return 0;
    if (!widx || !bidx || !stm || !W16 || !b16 || !psqt_idx || !out_u8 || !psqt_out) return NNUEFT_E_ARG;
    if (n_psqt > 0 && !psqt32) return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = (L1 % 16 == 0) && aligned16(W16) && aligned16(b16) &&
                     ((reinterpret_cast<uintptr_t>(out_u8) & 7u) == 0);
    if (workspace) {
        Int16Layout L;
        if (!int16_layout(B, R, L1, table_block_rows, &L)) return NNUEFT_E_ARG;
        if (!aligned256(workspace) || workspace_bytes < L.end) return NNUEFT_E_WORKSPACE;
        const nnueft_dev::DeviceInfo* info = nullptr;
        const int rc_dev = nnueft_dev::device_info(nullptr, &info);
        if (rc_dev) return rc_dev;
        const int br = table_block_rows > 0 ? table_block_rows : nnueft_tile::kBlockRows;
        if (vec && L.tile_ok && nnueft_tile::fits_int16(*info, B, K, R, L1, br)) {
            char* ws = (char*)workspace;
            // an output half depends on one list's sums only, so the gather finishes the bytes itself (32 column
            // pairs a tile) and no sums pass through memory; the psqt difference comes out of the sort of the lists
            return nnueft_tile::int16_fused_tile(widx, bidx, stm, W16, b16, psqt32, psqt_idx, out_u8, psqt_out, B, K, R, L1,
                                                 n_psqt, clip_max, shift, br, ws + L.tile_sort, st);
        }
        if (vec && (long long)B <= 0x3fffffffLL && nnueft_blocked::blocked_layout_fits(*info)) {
            char* ws = (char*)workspace;
            int16_t* accW = (int16_t*)(ws + L.accW);
            const uint32_t* order = nullptr;
            int rc = nnueft_blocked::launch_pair_sort(widx, bidx, B, K, R, table_block_rows, ws + L.sort, st, &order);
            if (rc) return rc;
            const int per_xcd = (2 * B + nnueft_blocked::kXcd - 1) / nnueft_blocked::kXcd;
            constexpr int NQA = 3;
            const int nv = L1 / 8;
            const int sl_a = (nv + 64 * NQA - 1) / (64 * NQA);
            const int sl_b = max(1, (nv / 2 + 63) / 64);
            if ((long long)nnueft_blocked::kXcd * per_xcd * max(sl_a, sl_b) > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
            hipLaunchKernelGGL((k_acc16_white<NQA, 8>), dim3(nnueft_blocked::kXcd * per_xcd * sl_a), dim3(64), 0, st,
                               widx, order, W16, b16, accW, B, K, R, L1, per_xcd);
            NNUEFT_LAUNCH_CHECK();
            hipLaunchKernelGGL(k_black_mix16<8>, dim3(nnueft_blocked::kXcd * per_xcd * sl_b), dim3(64), 0, st, widx,
                               bidx, order, stm, W16, b16, accW, psqt32, psqt_idx, out_u8, psqt_out, B, K, R, L1,
                               n_psqt, clip_max, shift, per_xcd);
            NNUEFT_LAUNCH_CHECK();
            return 0;
        }
    }
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
