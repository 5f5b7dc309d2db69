// Forward gather-sum kernels.
//
// Work decomposition: one wave (= one workgroup of 64 lanes) per (position, column slice).  A lane
// owns NQ vectors of VW floats per half-row, 64 lanes apart, so every load instruction of the wave
// reads 64*VW*4 contiguous bytes of a gathered row (1 KiB with VW = 4).  The index list of the
// position sits one slot per lane; the valid slots are walked through a ballot mask, so padding
// costs nothing and no LDS is needed.
#include <cmath>

#include "gather.h"
#include "internal.h"

namespace {

constexpr int kUnroll = 4;

// out[b, :] = (sum_k W[idx[b,k], :]) + bias
template <int VW, int NQ>
__global__ __launch_bounds__(64) void k_sparse_fwd(const int32_t* __restrict__ idx, const float* __restrict__ W,
                                                   const float* __restrict__ bias, float* __restrict__ out,
                                                   int K, int R, int out_cols, int nslices) {
    const int lane = threadIdx.x;
    const int b = blockIdx.x / nslices;
    const int s = blockIdx.x - b * nslices;
    const int nv = out_cols / VW;

    int col[NQ];
    bool act[NQ];
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        const int q = (s * NQ + m) * 64 + lane;
        act[m] = q < nv;
        col[m] = act[m] ? q * VW : 0;
    }
    vecf<VW> acc[NQ];
#pragma unroll
    for (int m = 0; m < NQ; ++m) acc[m] = vzero<VW>();

    const int32_t* ix = idx + (size_t)b * K;
    for (int k0 = 0; k0 < K; k0 += 64) {
        const int my = (k0 + lane < K) ? ix[k0 + lane] : -1;
        const u64 mask = __ballot(my >= 0 && my < R);
        chain_rows<VW, NQ, kUnroll>(acc, W, (size_t)out_cols, col, my, mask);
    }
    float* o = out + (size_t)b * out_cols;
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        if (act[m]) {
            vadd<VW>(acc[m], ldv<VW>(bias + col[m]));
            stv<VW>(o + col[m], acc[m]);
        }
    }
}

// Both perspectives of one position, mix, clamp, pairwise product.
template <int VW, int NQ>
__global__ __launch_bounds__(64) void k_double_fwd(const float* __restrict__ us, const float* __restrict__ them,
                                                   const int32_t* __restrict__ widx,
                                                   const int32_t* __restrict__ bidx,
                                                   const int64_t* __restrict__ psqt_idx,
                                                   const float* __restrict__ W, const float* __restrict__ bias,
                                                   float max_act, float* __restrict__ l0,
                                                   float* __restrict__ wpsqt, float* __restrict__ bpsqt,
                                                   float* __restrict__ saved, int B, int K, int R, int L1,
                                                   int n_psqt, int nslices) {
    const int lane = threadIdx.x;
    // slice-major task order: at any time the whole GPU gathers the same 1/nslices of the table's
    // columns, which keeps the live part of the table inside the memory-side cache
    const int s = blockIdx.x / B;
    const int b = blockIdx.x - s * B;
    const int h = L1 >> 1;
    const int hv = h / VW;
    const size_t out_cols = (size_t)L1 + n_psqt;

    // col[2m] is the lane's m-th vector in the first half, col[2m+1] its partner h columns on.
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

    vecf<VW> acc[2][2 * NQ];
    float ps[2] = {0.0f, 0.0f};
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
        for (int j = 0; j < 2 * NQ; ++j) acc[p][j] = vzero<VW>();
        const int32_t* ix = (p ? bidx : widx) + (size_t)b * K;
        for (int k0 = 0; k0 < K; k0 += 64) {
            const int my = (k0 + lane < K) ? ix[k0 + lane] : -1;
            const bool ok = my >= 0 && my < R;
            const u64 mask = __ballot(ok);
            float myps = 0.0f;
            if (do_psqt && ok) myps = W[(size_t)my * out_cols + L1 + pi];
            chain_rows<VW, 2 * NQ, kUnroll>(acc[p], W, out_cols, col, my, mask);
            if (do_psqt) {
                u64 m2 = mask;
                while (m2) ps[p] = ps[p] + bcast_f(myps, pop_lane(m2));
            }
        }
    }

    const float u = us[b], t = them[b];
    float* sw = saved + (size_t)b * L1;
    float* sb = saved + ((size_t)B + b) * L1;
    float* o = l0 + (size_t)b * L1;
#pragma unroll
    for (int m = 0; m < NQ; ++m) {
        if (!act[m]) continue;
        const int c = col[2 * m];
        const vecf<VW> bias0 = ldv<VW>(bias + c), bias1 = ldv<VW>(bias + c + h);
        vecf<VW> o0, o1;
#pragma unroll
        for (int i = 0; i < VW; ++i) {
            float xw0, xw1, xb0, xb1;
            mix4(u, t, acc[0][2 * m].v[i], acc[0][2 * m + 1].v[i], acc[1][2 * m].v[i], acc[1][2 * m + 1].v[i],
                 bias0.v[i], bias1.v[i], xw0, xw1, xb0, xb1);
            o0.v[i] = clamp_act(xw0, max_act) * clamp_act(xw1, max_act);
            o1.v[i] = clamp_act(xb0, max_act) * clamp_act(xb1, max_act);
        }
        stv<VW>(sw + c, acc[0][2 * m]);
        stv<VW>(sw + h + c, acc[0][2 * m + 1]);
        stv<VW>(sb + c, acc[1][2 * m]);
        stv<VW>(sb + h + c, acc[1][2 * m + 1]);
        stv<VW>(o + c, o0);
        stv<VW>(o + h + c, o1);
    }
    if (s == 0 && lane == 0) {
        const float pb = do_psqt ? bias[L1 + pi] : 0.0f;
        wpsqt[b] = ps[0] + pb;
        bpsqt[b] = ps[1] + pb;
    }
}

template <int VW, int NQ>
int launch_sparse_fwd(const int32_t* idx, const float* W, const float* bias, float* out, int B, int K, int R,
                      int out_cols, hipStream_t st) {
    const int nv = out_cols / VW;
    const int nslices = (nv + 64 * NQ - 1) / (64 * NQ);
    const long long grid = (long long)B * nslices;
    if (grid > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
    hipLaunchKernelGGL((k_sparse_fwd<VW, NQ>), dim3((unsigned)grid), dim3(64), 0, st, idx, W, bias, out, K, R,
                       out_cols, nslices);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

template <int VW, int NQ>
int launch_double_fwd(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                      const int64_t* psqt_idx, const float* W, const float* bias, float max_act, float* l0,
                      float* wpsqt, float* bpsqt, float* saved, int B, int K, int R, int L1, int n_psqt,
                      hipStream_t st) {
    const int hv = (L1 / 2) / VW;
    const int nslices = hv > 0 ? (hv + 64 * NQ - 1) / (64 * NQ) : 1;
    const long long grid = (long long)B * nslices;
    if (grid > 0x7fffffffLL) return NNUEFT_E_UNSUPPORTED;
    hipLaunchKernelGGL((k_double_fwd<VW, NQ>), dim3((unsigned)grid), dim3(64), 0, st, us, them, widx, bidx,
                       psqt_idx, W, bias, max_act, l0, wpsqt, bpsqt, saved, B, K, R, L1, n_psqt, nslices);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

}  // namespace

extern "C" int nnueft_sparse_fwd(const int32_t* idx, const float* W, const float* bias, float* out, int B, int K,
                                 int R, int out_cols, void* stream) {
    if (B < 0 || K <= 0 || R <= 0 || out_cols <= 0) return NNUEFT_E_ARG;
    if (B == 0) return 0;
    if (!idx || !W || !bias || !out) return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = (out_cols % 4 == 0) && aligned16(W) && aligned16(bias) && aligned16(out);
    if (vec) {
        if (out_cols / 4 > 64) return launch_sparse_fwd<4, 2>(idx, W, bias, out, B, K, R, out_cols, st);
        return launch_sparse_fwd<4, 1>(idx, W, bias, out, B, K, R, out_cols, st);
    }
    if (out_cols > 64) return launch_sparse_fwd<1, 2>(idx, W, bias, out, B, K, R, out_cols, st);
    return launch_sparse_fwd<1, 1>(idx, W, bias, out, B, K, R, out_cols, st);
}

extern "C" size_t nnueft_fwd_workspace_bytes(int B, int K, int R, int L1, int n_psqt) {
    if (B <= 0 || K <= 0 || R <= 0 || L1 <= 0 || n_psqt < 0) return 0;
    return nnueft_tile::workspace(B, R);
}

extern "C" int nnueft_act_fake_quantize(const float* x, float* out, long long n, float scale, float eps,
                                        float post_mul, void* stream);

namespace {

int double_fwd(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
               const int64_t* psqt_idx, const float* W, const float* bias, float max_act, float* l0, float* wpsqt,
               float* bpsqt, float* saved, int B, int K, int R, int L1, int n_psqt, void* workspace,
               size_t workspace_bytes, void* stream, ActGrid act, VirtualTable vt = VirtualTable{nullptr, 1.0f, 1.0f, 0, 0.0f}) {
    if (B < 0 || K <= 0 || R <= 0 || L1 <= 0 || (L1 & 1) || n_psqt < 0) return NNUEFT_E_ARG;
    if (B == 0) return 0;
    if (!us || !them || !widx || !bidx || !psqt_idx || !W || !bias || !l0 || !wpsqt || !bpsqt || !saved)
        return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = (L1 % 8 == 0) && ((L1 + n_psqt) % 4 == 0) && aligned16(W) && aligned16(bias) &&
                     aligned16(l0) && aligned16(saved);
    if (workspace) {
        if (!aligned256(workspace) || workspace_bytes < nnueft_blocked::pair_sort_workspace(B, R, 0))
            return NNUEFT_E_WORKSPACE;
        // the L2-blocked path needs 16-byte rows and the XCD layout it is made for; other shapes and
        // devices take the plain kernel below
        const nnueft_dev::DeviceInfo* info = nullptr;
        const int rc_dev = nnueft_dev::device_info(nullptr, &info);
        if (rc_dev) return rc_dev;
        // wide rows gather out of LDS tiles when the caller's workspace has room for that path's lists
        if (vec && nnueft_tile::fits(*info, B, K, R, L1) && workspace_bytes >= nnueft_tile::workspace(B, R))
            return nnueft_tile::double_fwd_tile(us, them, widx, bidx, psqt_idx, W, bias, max_act, l0, wpsqt, bpsqt,
                                                saved, B, K, R, L1, n_psqt, workspace, st, act, vt);
        if (vt.V) return NNUEFT_E_UNSUPPORTED;   // only the LDS-tiled gather merges on the fly
        if (vec && (long long)B <= 0x3fffffffLL && nnueft_blocked::blocked_layout_fits(*info))
            return nnueft_blocked::double_fwd_blocked(us, them, widx, bidx, psqt_idx, W, bias, max_act, l0, wpsqt,
                                                      bpsqt, saved, B, K, R, L1, n_psqt, workspace, st, act);
    }
    if (vt.V) return NNUEFT_E_UNSUPPORTED;
    if (act.on) {
        // the plain kernels know nothing of the grid: run them, then the grid in place
        ActGrid off{};
        const int rc = double_fwd(us, them, widx, bidx, psqt_idx, W, bias, max_act, l0, wpsqt, bpsqt, saved, B, K, R,
                                  L1, n_psqt, nullptr, 0, stream, off);
        if (rc) return rc;
        return nnueft_act_fake_quantize(l0, l0, (long long)B * L1, act.scale, act.eps, act.post_mul, stream);
    }
    if (vec) {
        if (L1 / 8 > 64)
            return launch_double_fwd<4, 2>(us, them, widx, bidx, psqt_idx, W, bias, max_act, l0, wpsqt, bpsqt,
                                           saved, B, K, R, L1, n_psqt, st);
        return launch_double_fwd<4, 1>(us, them, widx, bidx, psqt_idx, W, bias, max_act, l0, wpsqt, bpsqt, saved,
                                       B, K, R, L1, n_psqt, st);
    }
    if (L1 / 2 > 64)
        return launch_double_fwd<1, 2>(us, them, widx, bidx, psqt_idx, W, bias, max_act, l0, wpsqt, bpsqt, saved,
                                       B, K, R, L1, n_psqt, st);
    return launch_double_fwd<1, 1>(us, them, widx, bidx, psqt_idx, W, bias, max_act, l0, wpsqt, bpsqt, saved, B,
                                   K, R, L1, n_psqt, st);
}

}  // namespace

extern "C" int nnueft_double_fwd(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                                 const int64_t* psqt_idx, const float* W, const float* bias, float max_act,
                                 float* l0, float* wpsqt, float* bpsqt, float* saved, int B, int K, int R,
                                 int L1, int n_psqt, void* workspace, size_t workspace_bytes, void* stream) {
    ActGrid off{};
    return double_fwd(us, them, widx, bidx, psqt_idx, W, bias, max_act, l0, wpsqt, bpsqt, saved, B, K, R, L1, n_psqt,
                      workspace, workspace_bytes, stream, off);
}

extern "C" int nnueft_double_fwd_act(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                                     const int64_t* psqt_idx, const float* W, const float* bias, float max_act,
                                     float* l0, float* wpsqt, float* bpsqt, float* saved, int B, int K, int R,
                                     int L1, int n_psqt, void* workspace, size_t workspace_bytes, float act_scale,
                                     float act_eps, float act_post_mul, void* stream) {
    if (!(act_scale > 0.0f)) return NNUEFT_E_ARG;
    ActGrid act{act_scale, act_eps, act_post_mul, 1};
    return double_fwd(us, them, widx, bidx, psqt_idx, W, bias, max_act, l0, wpsqt, bpsqt, saved, B, K, R, L1, n_psqt,
                      workspace, workspace_bytes, stream, act);
}

// Whether nnueft_double_fwd_virtual can run these sizes on the current device (1) or not (0; negative: error).
extern "C" int nnueft_double_fwd_virtual_fits(int B, int K, int R, int L1, int n_psqt, int virtual_rows) {
    if (B <= 0 || K <= 0 || R <= 0 || L1 <= 0 || (L1 & 1) || n_psqt < 0) return 0;
    const nnueft_dev::DeviceInfo* info = nullptr;
    const int rc = nnueft_dev::device_info(nullptr, &info);
    if (rc) return rc > 0 ? -rc - 1000 : rc;
    const bool vec = (L1 % 8 == 0) && ((L1 + n_psqt) % 4 == 0);
    return vec && virtual_rows == nnueft_tile::kBlockRows && nnueft_tile::fits(*info, B, K, R, L1) ? 1 : 0;
}

extern "C" int nnueft_double_fwd_virtual(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                                         const int64_t* psqt_idx, const float* W, const float* V, const float* bias,
                                         float max_act, float* l0, float* wpsqt, float* bpsqt, float* saved, int B,
                                         int K, int R, int L1, int n_psqt, int virtual_rows, float scale_ft,
                                         float scale_psqt, int fake_quantize, void* workspace, size_t workspace_bytes,
                                         int act_on, float act_scale, float act_eps, float act_post_mul, void* stream) {
    if (!V || virtual_rows != nnueft_tile::kBlockRows) return V ? NNUEFT_E_UNSUPPORTED : NNUEFT_E_ARG;
    if (fake_quantize && (!(scale_ft > 0.0f) || !(scale_psqt > 0.0f))) return NNUEFT_E_ARG;
    if (act_on && !(act_scale > 0.0f)) return NNUEFT_E_ARG;
    if (!workspace) return NNUEFT_E_WORKSPACE;
    if (!aligned16(V)) return NNUEFT_E_UNSUPPORTED;
    ActGrid act{act_scale, act_eps, act_post_mul, act_on ? 1 : 0};
    if (!act_on) act = ActGrid{};
    // a power of two divides exactly as its reciprocal multiplies (1 / 2^k is exact and so is every product with it
    // short of underflow, which a multiple of 2^-k of this size never meets)
    int exp2 = 0;
    const bool pow2 = fake_quantize && std::frexp(scale_ft, &exp2) == 0.5f && exp2 > -100 && exp2 < 100;
    VirtualTable vt{V, scale_ft, scale_psqt, fake_quantize ? 1 : 0, pow2 ? 1.0f / scale_ft : 0.0f};
    return double_fwd(us, them, widx, bidx, psqt_idx, W, bias, max_act, l0, wpsqt, bpsqt, saved, B, K, R, L1, n_psqt,
                      workspace, workspace_bytes, stream, act, vt);
}
