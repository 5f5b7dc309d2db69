/*
 * CPU restatement of the nnue-pytorch sparse feature transformer.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared against and the "port" CPU baseline timed next to them; nothing in
 * the shipped library links, loads or calls it.
 *
 * What each function follows in the reference (paths relative to the
 * reference checkout):
 *
 *   nnueft_oracle_sparse_fwd      model/modules/feature_transformer/sparse_linear_functions.py:16-50
 *                                 (_torch_sparse_linear: embedding_bag(sum) over the index list with
 *                                 negative slots masked, then "+ bias")
 *   nnueft_oracle_sparse_bwd      autograd of the same function; same maths as
 *                                 sparse_linear_kernel.py:237-288 (gW[idx,:] += g, gb += g)
 *   nnueft_oracle_double_fwd      double_ft_functions.py:62-80 (the torch composition) ==
 *                                 fused_ft_kernel.py:27-117 (the fused kernel)
 *   nnueft_oracle_double_bwd      autograd of double_ft_functions.py:62-80 ==
 *                                 fused_ft_kernel.py:147-272, except that the clamp mask is torch's
 *                                 (gradient passes where 0 <= x <= max, x taken before the clamp).
 *                                 The activations kept between forward and backward are the two
 *                                 perspectives' row sums (before the bias); the mixed values are
 *                                 recomputed from them with the forward's own operations.
 *   nnueft_oracle_ranger_lite_*   model/optimizers/ranger_lite.py:46-201 (fused update kernels),
 *                                 :737-760 (lookahead merge)
 *   nnueft_oracle_ft_int16_fwd    no code in the reference (the accumulate runs in the engine);
 *                                 spec docs/nnue.md:1014-1069 (int16 accumulate) and :2097-2134
 *                                 (pairwise product, shift), constants model/quantize.py:58-73
 *
 * Summation order (this is what "bit-exact" means for the fp32 paths):
 *   forward   s = +0; s += W[idx_k] for k ascending over the valid slots; out = s + bias.
 *             torch's CPU embedding_bag produces exactly this (checked in the tests).
 *   weight    per perspective, one chain per table row starting at +0 and adding the
 *   gradient  upstream row of every slot that names the table row, slots visited in ascending
 *             (position, slot) order; the two perspectives' chains are then added
 *             (white + black).  torch's CPU embedding_bag backward followed by autograd's
 *             accumulation of the two uses of `weight` produces exactly this.
 *             That is the order for every row when row_split = 0 (the strict order).
 *             With row_split > 0 (this build's own order; NNUEFT_ORACLE_ROW_SPLIT is the default the
 *             kernels are tuned for): a table row named by more than
 *             row_split slots of the batch, both perspectives together, is summed
 *             window by window: window w = positions [w*W, (w+1)*W), W = nnueft_oracle_row_window(B);
 *             per perspective each window's slots are chained from +0, the window sums are
 *             chained from +0 in ascending w, then white + black.  torch agrees with such a row
 *             to rounding only (exactly when all addends are small integers).
 *   bias      positions are cut into tiles of NNUEFT_ORACLE_BIAS_TILE; per column a chain
 *   gradient  over the positions of a tile (starting at +0, ascending), then a chain over the
 *             tile sums (starting at +0, ascending).  This order is this build's own; torch
 *             reduces in a different, unspecified order, so torch agrees to rounding only.
 *
 * Indices outside [0, R) (negative padding included) contribute nothing.
 *
 * Build:  gcc -O2 -fopenmp -ffp-contract=off -shared -fPIC nnueft_oracle.c -o libnnueft_oracle.so
 * -ffp-contract=off matters: a*b+c must round twice, like the separate torch ops it restates.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define NNUEFT_ORACLE_BIAS_TILE 32
#define COLBLK 64

int nnueft_oracle_bias_tile(void) { return NNUEFT_ORACLE_BIAS_TILE; }

#define NNUEFT_ORACLE_ROW_SPLIT 512
int nnueft_oracle_row_split(void) { return NNUEFT_ORACLE_ROW_SPLIT; }

/* Window length: as few windows as keep every window at 1024 positions or fewer, at most 16 of them,
 * equal lengths rounded up to a multiple of 128. */
int nnueft_oracle_row_window(int B)
{
    int nwin = (B + 1023) / 1024;
    if (nwin < 1) nwin = 1;
    if (nwin > 16) nwin = 16;
    int w = (B + nwin - 1) / nwin;
    return (w + 127) / 128 * 128;
}

static inline int valid(int32_t r, int R) { return r >= 0 && r < R; }

/* out[b,:] = (sum_k W[idx[b,k],:]) + bias */
int nnueft_oracle_sparse_fwd(const int32_t* idx, const float* W, const float* bias, float* out,
                             int B, int K, int R, int out_cols)
{
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b) {
        float* o = out + (size_t)b * out_cols;
        for (int c = 0; c < out_cols; ++c) o[c] = 0.0f;
        for (int k = 0; k < K; ++k) {
            int32_t r = idx[(size_t)b * K + k];
            if (!valid(r, R)) continue;
            const float* w = W + (size_t)r * out_cols;
            for (int c = 0; c < out_cols; ++c) o[c] = o[c] + w[c];
        }
        for (int c = 0; c < out_cols; ++c) o[c] = o[c] + bias[c];
    }
    return 0;
}

/* split_id[r] = ordinal of row r among the rows named by more than row_split slots of idx_a and
 * idx_b together (idx_b may be NULL), -1 for the others; row_split = 0: no row.  Returns how many. */
static int find_split_rows(const int32_t* idx_a, const int32_t* idx_b, int B, int K, int R, int row_split,
                           int32_t* split_id)
{
    int64_t* count = (int64_t*)calloc((size_t)R, sizeof(int64_t));
    if (!count) return -1;
    for (int pass = 0; pass < 2; ++pass) {
        const int32_t* idx = pass ? idx_b : idx_a;
        if (!idx) continue;
        for (size_t i = 0; i < (size_t)B * K; ++i)
            if (valid(idx[i], R)) count[idx[i]]++;
    }
    int n = 0;
    for (int r = 0; r < R; ++r) split_id[r] = (row_split > 0 && count[r] > row_split) ? n++ : -1;
    free(count);
    return n;
}

/* One perspective's chains, columns [c0,c1): acc[r] += G[b] for slots in ascending (b,k).  A split
 * row instead collects each window in `cur`, and at every window boundary adds it to the row's
 * running sum of windows in `tot` (both [nsplit, c1-c0], zeroed here); acc[r] += nothing until
 * the end, where acc[r] = tot. */
static void scatter_chain(const int32_t* idx, const float* G, size_t g_stride, float* acc,
                          int B, int K, int R, int out_cols, int c0, int c1,
                          const int32_t* split_id, int nsplit, int window, float* cur, float* tot)
{
    const int w = c1 - c0;
    if (nsplit > 0) {
        memset(cur, 0, sizeof(float) * (size_t)nsplit * w);
        memset(tot, 0, sizeof(float) * (size_t)nsplit * w);
    }
    for (int b = 0; b < B; ++b) {
        if (nsplit > 0 && b > 0 && b % window == 0)
            for (size_t i = 0; i < (size_t)nsplit * w; ++i) { tot[i] = tot[i] + cur[i]; cur[i] = 0.0f; }
        const float* g = G + (size_t)b * g_stride;
        for (int k = 0; k < K; ++k) {
            int32_t r = idx[(size_t)b * K + k];
            if (!valid(r, R)) continue;
            if (split_id[r] >= 0) {
                float* a = cur + (size_t)split_id[r] * w;
                for (int c = c0; c < c1; ++c) a[c - c0] = a[c - c0] + g[c];
            } else {
                float* a = acc + (size_t)r * out_cols;
                for (int c = c0; c < c1; ++c) a[c] = a[c] + g[c];
            }
        }
    }
    if (nsplit > 0) {
        for (size_t i = 0; i < (size_t)nsplit * w; ++i) tot[i] = tot[i] + cur[i];
        for (int r = 0; r < R; ++r)
            if (split_id[r] >= 0)
                for (int c = c0; c < c1; ++c) acc[(size_t)r * out_cols + c] = tot[(size_t)split_id[r] * w + (c - c0)];
    }
}

/* Tiled column sum: gbias[c] = chain over tiles of (chain over the tile's positions of v[b,c]). */
static void bias_tiled(const float* V1, const float* V2, size_t stride, float* gbias, int B, int out_cols)
{
#pragma omp parallel for schedule(static)
    for (int c = 0; c < out_cols; ++c) {
        float total = 0.0f;
        for (int t0 = 0; t0 < B; t0 += NNUEFT_ORACLE_BIAS_TILE) {
            int t1 = t0 + NNUEFT_ORACLE_BIAS_TILE < B ? t0 + NNUEFT_ORACLE_BIAS_TILE : B;
            float part = 0.0f;
            for (int b = t0; b < t1; ++b) {
                float v = V1[(size_t)b * stride + c];
                if (V2) v = v + V2[(size_t)b * stride + c];
                part = part + v;
            }
            total = total + part;
        }
        gbias[c] = total;
    }
}

/* gW[r,:] = chain over slots naming r of gout[b,:]; gbias = tiled column sum of gout. */
int nnueft_oracle_sparse_bwd(const int32_t* idx, const float* gout, float* gW, float* gbias,
                             int B, int K, int R, int out_cols, int row_split)
{
    if (row_split < 0) return -1;
    memset(gW, 0, (size_t)R * out_cols * sizeof(float));
    int32_t* split_id = (int32_t*)malloc(sizeof(int32_t) * (size_t)R);
    if (!split_id) return -2;
    const int nsplit = find_split_rows(idx, NULL, B, K, R, row_split, split_id);
    if (nsplit < 0) { free(split_id); return -2; }
    const int window = nnueft_oracle_row_window(B);
    int nblk = (out_cols + COLBLK - 1) / COLBLK;
    int failed = 0;
#pragma omp parallel for schedule(dynamic)
    for (int j = 0; j < nblk; ++j) {
        int c0 = j * COLBLK, c1 = c0 + COLBLK < out_cols ? c0 + COLBLK : out_cols;
        float* tmp = (float*)malloc(sizeof(float) * 2 * (size_t)(nsplit ? nsplit : 1) * COLBLK);
        if (!tmp) { failed = 1; continue; }
        scatter_chain(idx, gout, (size_t)out_cols, gW, B, K, R, out_cols, c0, c1, split_id, nsplit, window, tmp,
                      tmp + (size_t)(nsplit ? nsplit : 1) * COLBLK);
        free(tmp);
    }
    free(split_id);
    if (failed) return -2;
    bias_tiled(gout, NULL, (size_t)out_cols, gbias, B, out_cols);
    return 0;
}

static inline float clampf(float x, float lo, float hi) { return x < lo ? lo : (x > hi ? hi : x); }

/* The four mixed pre-clamp values of column pair (i, i+h) from the two perspectives' row sums. */
static inline void mix4(float u, float t, const float* sw, const float* sb, const float* bias, int i, int h,
                        float* xw0, float* xw1, float* xb0, float* xb1)
{
    const float w0 = sw[i] + bias[i], w1 = sw[i + h] + bias[i + h];
    const float b0 = sb[i] + bias[i], b1 = sb[i + h] + bias[i + h];
    *xw0 = u * w0 + t * b0;
    *xw1 = u * w1 + t * b1;
    *xb0 = u * b0 + t * w0;
    *xb1 = u * b1 + t * w1;
}

/*
 * Both perspectives, side-to-move mix, clamp, pairwise product.
 * saved[p, b, 0:L1] receives the row sums of perspective p (0 white, 1 black) BEFORE the bias:
 * the chain from +0 over the valid slots.  Everything downstream is a function of them.
 */
int nnueft_oracle_double_fwd(const float* us, const float* them,
                             const int32_t* widx, const int32_t* bidx, const int64_t* psqt_idx,
                             const float* W, const float* bias, float max_act,
                             float* l0, float* wpsqt, float* bpsqt, float* saved,
                             int B, int K, int R, int L1, int n_psqt)
{
    const int out_cols = L1 + n_psqt;
    const int h = L1 / 2;
    if (L1 % 2) return -1;
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b) {
        const int64_t pi = psqt_idx[b];
        const int psqt_ok = pi >= 0 && pi < n_psqt;
        float ps[2] = {0.0f, 0.0f};
        for (int p = 0; p < 2; ++p) {
            const int32_t* ix = (p == 0 ? widx : bidx) + (size_t)b * K;
            float* a = saved + ((size_t)p * B + b) * L1;
            for (int c = 0; c < L1; ++c) a[c] = 0.0f;
            for (int k = 0; k < K; ++k) {
                int32_t r = ix[k];
                if (!valid(r, R)) continue;
                const float* w = W + (size_t)r * out_cols;
                for (int c = 0; c < L1; ++c) a[c] = a[c] + w[c];
                if (psqt_ok) ps[p] = ps[p] + w[L1 + pi];
            }
            if (psqt_ok) ps[p] = ps[p] + bias[L1 + pi];
        }
        wpsqt[b] = ps[0];
        bpsqt[b] = ps[1];
        const float u = us[b], t = them[b];
        const float* sw = saved + (size_t)b * L1;
        const float* sb = saved + ((size_t)B + b) * L1;
        float* o = l0 + (size_t)b * L1;
        for (int i = 0; i < h; ++i) {
            float xw0, xw1, xb0, xb1;
            mix4(u, t, sw, sb, bias, i, h, &xw0, &xw1, &xb0, &xb1);
            o[i] = clampf(xw0, 0.0f, max_act) * clampf(xw1, 0.0f, max_act);
            o[h + i] = clampf(xb0, 0.0f, max_act) * clampf(xb1, 0.0f, max_act);
        }
    }
    return 0;
}

/*
 * Per-position upstream rows of the two sparse-linear outputs:
 * G[p, b, 0:L1] per the product/clamp/mix chain rule, G[p, b, L1+j] = grad_psqt_p[b] if j == psqt_idx[b] else 0.
 * Layout [2, B, out_cols].
 */
int nnueft_oracle_double_bwd_rows(const float* us, const float* them, const int64_t* psqt_idx,
                                  const float* bias, float max_act,
                                  const float* grad_l0, const float* grad_wpsqt, const float* grad_bpsqt,
                                  const float* saved, float* G, int B, int L1, int n_psqt)
{
    const int out_cols = L1 + n_psqt;
    const int h = L1 / 2;
    if (L1 % 2) return -1;
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b) {
        const float u = us[b], t = them[b];
        const float* sw = saved + (size_t)b * L1;
        const float* sb = saved + ((size_t)B + b) * L1;
        const float* g = grad_l0 + (size_t)b * L1;
        float* gw = G + (size_t)b * out_cols;
        float* gb = G + ((size_t)B + b) * out_cols;
        for (int i = 0; i < h; ++i) {
            float xw0, xw1, xb0, xb1;
            mix4(u, t, sw, sb, bias, i, h, &xw0, &xw1, &xb0, &xb1);
            float cw0 = clampf(xw0, 0.0f, max_act), cw1 = clampf(xw1, 0.0f, max_act);
            float cb0 = clampf(xb0, 0.0f, max_act), cb1 = clampf(xb1, 0.0f, max_act);
            float dw0 = (xw0 >= 0.0f && xw0 <= max_act) ? g[i] * cw1 : 0.0f;
            float dw1 = (xw1 >= 0.0f && xw1 <= max_act) ? g[i] * cw0 : 0.0f;
            float db0 = (xb0 >= 0.0f && xb0 <= max_act) ? g[h + i] * cb1 : 0.0f;
            float db1 = (xb1 >= 0.0f && xb1 <= max_act) ? g[h + i] * cb0 : 0.0f;
            gw[i] = u * dw0 + t * db0;
            gw[h + i] = u * dw1 + t * db1;
            gb[i] = t * dw0 + u * db0;
            gb[h + i] = t * dw1 + u * db1;
        }
        const int64_t pi = psqt_idx[b];
        for (int j = 0; j < n_psqt; ++j) {
            gw[L1 + j] = (j == pi) ? grad_wpsqt[b] : 0.0f;
            gb[L1 + j] = (j == pi) ? grad_bpsqt[b] : 0.0f;
        }
    }
    return 0;
}

/* gW = (white chains) + (black chains); gbias = tiled column sum of (G_w + G_b). */
int nnueft_oracle_double_bwd(const float* us, const float* them,
                             const int32_t* widx, const int32_t* bidx, const int64_t* psqt_idx,
                             const float* bias, float max_act,
                             const float* grad_l0, const float* grad_wpsqt, const float* grad_bpsqt,
                             const float* saved, float* gW, float* gbias,
                             int B, int K, int R, int L1, int n_psqt, int row_split)
{
    const int out_cols = L1 + n_psqt;
    if (row_split < 0) return -1;
    float* G = (float*)malloc(sizeof(float) * 2 * (size_t)B * out_cols);
    float* accb = (float*)calloc((size_t)R * out_cols, sizeof(float));
    if (!G || !accb) { free(G); free(accb); return -2; }
    int rc = nnueft_oracle_double_bwd_rows(us, them, psqt_idx, bias, max_act, grad_l0, grad_wpsqt, grad_bpsqt,
                                           saved, G, B, L1, n_psqt);
    if (rc) { free(G); free(accb); return rc; }
    memset(gW, 0, (size_t)R * out_cols * sizeof(float));
    int32_t* split_id = (int32_t*)malloc(sizeof(int32_t) * (size_t)R);
    const int nsplit = split_id ? find_split_rows(widx, bidx, B, K, R, row_split, split_id) : -1;
    if (nsplit < 0) { free(G); free(accb); free(split_id); return -2; }
    const int window = nnueft_oracle_row_window(B);
    int nblk = (out_cols + COLBLK - 1) / COLBLK;
    int failed = 0;
#pragma omp parallel for schedule(dynamic)
    for (int j = 0; j < nblk; ++j) {
        int c0 = j * COLBLK, c1 = c0 + COLBLK < out_cols ? c0 + COLBLK : out_cols;
        const size_t half = (size_t)(nsplit ? nsplit : 1) * COLBLK;
        float* tmp = (float*)malloc(sizeof(float) * 2 * half);
        if (!tmp) { failed = 1; continue; }
        scatter_chain(widx, G, (size_t)out_cols, gW, B, K, R, out_cols, c0, c1, split_id, nsplit, window, tmp,
                      tmp + half);
        scatter_chain(bidx, G + (size_t)B * out_cols, (size_t)out_cols, accb, B, K, R, out_cols, c0, c1, split_id,
                      nsplit, window, tmp, tmp + half);
        free(tmp);
        for (int r = 0; r < R; ++r)
            for (int c = c0; c < c1; ++c)
                gW[(size_t)r * out_cols + c] = gW[(size_t)r * out_cols + c] + accb[(size_t)r * out_cols + c];
    }
    bias_tiled(G, G + (size_t)B * out_cols, (size_t)out_cols, gbias, B, out_cols);
    free(G);
    free(accb);
    free(split_id);
    return failed ? -2 : 0;
}

/*
 * Quantized feature transformer, as the engine evaluates an exported net.
 *   acc_p[c]  = b16[c] + sum_k W16[idx_p[k], c]          int16, wrapping
 *   c_p[c]    = min(max(acc_p[c], 0), clip_max)
 *   out[b, o*h + j] = (c_{P(o)}[j] * c_{P(o)}[j + h]) >> shift     o = 0: side to move, 1: the other side
 *   psqt_out[b] = (sum_k psqt32[idx_{P(0)}[k], bucket] - sum_k psqt32[idx_{P(1)}[k], bucket]) / 2   (C division)
 * stm[b] = 0 when white is to move (P(0) = white), 1 when black is.
 */
int nnueft_oracle_ft_int16_fwd(const int32_t* widx, const int32_t* bidx, const uint8_t* stm,
                               const int16_t* W16, const int16_t* b16, const int32_t* psqt32,
                               const int64_t* psqt_idx, uint8_t* out_u8, int32_t* psqt_out,
                               int B, int K, int R, int L1, int n_psqt, int clip_max, int shift)
{
    const int h = L1 / 2;
    if (L1 % 2) return -1;
#pragma omp parallel
    {
        int16_t* acc = (int16_t*)malloc(sizeof(int16_t) * 2 * (size_t)L1);
#pragma omp for schedule(static)
        for (int b = 0; b < B; ++b) {
            const int64_t pi = psqt_idx[b];
            const int psqt_ok = pi >= 0 && pi < n_psqt;
            int32_t ps[2] = {0, 0};
            for (int p = 0; p < 2; ++p) {
                const int32_t* ix = (p == 0 ? widx : bidx) + (size_t)b * K;
                int16_t* a = acc + (size_t)p * L1;
                for (int c = 0; c < L1; ++c) a[c] = b16[c];
                for (int k = 0; k < K; ++k) {
                    int32_t r = ix[k];
                    if (!valid(r, R)) continue;
                    const int16_t* w = W16 + (size_t)r * L1;
                    for (int c = 0; c < L1; ++c) a[c] = (int16_t)(uint16_t)((uint16_t)a[c] + (uint16_t)w[c]);
                    if (psqt_ok) ps[p] = (int32_t)((uint32_t)ps[p] + (uint32_t)psqt32[(size_t)r * n_psqt + pi]);
                }
            }
            const int first = stm[b] ? 1 : 0;
            for (int o = 0; o < 2; ++o) {
                const int16_t* a = acc + (size_t)(o == 0 ? first : 1 - first) * L1;
                uint8_t* dst = out_u8 + (size_t)b * L1 + (size_t)o * h;
                for (int j = 0; j < h; ++j) {
                    int32_t c0 = a[j] < 0 ? 0 : (a[j] > clip_max ? clip_max : a[j]);
                    int32_t c1 = a[j + h] < 0 ? 0 : (a[j + h] > clip_max ? clip_max : a[j + h]);
                    dst[j] = (uint8_t)((c0 * c1) >> shift);
                }
            }
            psqt_out[b] = (ps[first] - ps[1 - first]) / 2;
        }
        free(acc);
    }
    return 0;
}

/*
 * merged = q(W + V[row % vrows]) -- HalfKav2Hm.merged_weight (model/modules/features/halfka_v2_hm.py:68-69)
 * followed by the weight fake quantization of ComposedFeatureTransformer.merged_weight_and_bias
 * (composed_feature_transformer.py:61-76): q(x) = round(x * s) / s, half to even (model/quantize.py:48-58),
 * s = scale_ft for the first L1 columns, scale_psqt for the others.
 */
#include <math.h>
int nnueft_oracle_table_merge(const float* W, const float* V, float* merged, int R, int cols, int L1, int vrows,
                              float scale_ft, float scale_psqt, int fake_quantize)
{
#pragma omp parallel for schedule(static)
    for (int r = 0; r < R; ++r) {
        for (int c = 0; c < cols; ++c) {
            float x = W[(size_t)r * cols + c];
            if (V) x = x + V[(size_t)(r % vrows) * cols + c];
            if (fake_quantize) {
                const float s = c < L1 ? scale_ft : scale_psqt;
                x = nearbyintf(x * s) / s;
            }
            merged[(size_t)r * cols + c] = x;
        }
    }
    return 0;
}

/* gV[v] = chain from +0 over the table blocks k (ascending) of gW[k * vrows + v]. */
int nnueft_oracle_table_virtual_grad(const float* gW, float* gV, int R, int cols, int vrows)
{
#pragma omp parallel for schedule(static)
    for (int v = 0; v < vrows; ++v) {
        for (int c = 0; c < cols; ++c) {
            float acc = 0.0f;
            for (int r = v; r < R; r += vrows) acc = acc + gW[(size_t)r * cols + c];
            gV[(size_t)v * cols + c] = acc;
        }
    }
    return 0;
}

/*
 * Quantized layer stacks: integer image of the fake-quantized forward of
 * model/modules/layer_stacks.py:33-84 on the tensors of quantize_fc_layer (model/quantize.py:218-236).
 * No code in the reference.  See include/nnueft.h for the formula.
 */
static inline int clip_act(long long v, int act_max) { return (int)(v < 0 ? 0 : (v > act_max ? act_max : v)); }

int nnueft_oracle_stack_int8_fwd(const uint8_t* x, const int64_t* bucket, const int8_t* W1, const int32_t* b1,
                                 const int8_t* W2, const int32_t* b2, const int8_t* Wo, const int32_t* bo,
                                 int32_t* out, int B, int L1, int L2, int L3, int count,
                                 int lin1, int sqr1, int lin2, int sqr2, int act_max, int out_mult, int out_den)
{
    if (L2 > 64 || L3 > 64 || L2 < 2) return -1;
#pragma omp parallel for schedule(static)
    for (int p = 0; p < B; ++p) {
        long long bk = bucket[p];
        if (bk < 0) bk = 0;
        if (bk >= count) bk = count - 1;
        int a1[64], y1[128], a2[64], y2[128];
        for (int o = 0; o < L2; ++o) {
            int acc = b1[bk * L2 + o];
            const int8_t* w = W1 + ((size_t)bk * L2 + o) * L1;
            for (int i = 0; i < L1; ++i) acc += (int)w[i] * (int)x[(size_t)p * L1 + i];
            a1[o] = acc;
        }
        for (int o = 0; o < L2; ++o) {
            y1[o] = clip_act(((long long)a1[o] * a1[o]) >> sqr1, act_max);
            y1[L2 + o] = clip_act((long long)(a1[o] >> lin1), act_max);
        }
        for (int j = 0; j < L3; ++j) {
            int acc = b2[bk * L3 + j];
            const int8_t* w = W2 + ((size_t)bk * L3 + j) * (2 * L2);
            for (int i = 0; i < 2 * L2; ++i) acc += (int)w[i] * y1[i];
            a2[j] = acc;
        }
        for (int j = 0; j < L3; ++j) {
            y2[j] = clip_act(((long long)a2[j] * a2[j]) >> sqr2, act_max);
            y2[L3 + j] = clip_act((long long)(a2[j] >> lin2), act_max);
        }
        const int8_t* w = Wo + (size_t)bk * (2 * L2 + 2 * L3);
        int a3 = bo[bk];
        for (int i = 0; i < 2 * L2; ++i) a3 += (int)w[i] * y1[i];
        for (int i = 0; i < 2 * L3; ++i) a3 += (int)w[2 * L2 + i] * y2[i];
        const long long num = 2ll * ((long long)a3 + a1[L2 - 2] - a1[L2 - 1]) * out_mult;
        out[p] = (int32_t)(num / out_den);
    }
    return 0;
}

/*
 * RangerLite update of one parameter tensor; follows the reference's fused kernels
 * (model/optimizers/ranger_lite.py:46-201) and, where lookahead is given, lookahead_process_step
 * (:737-760).  neg_grad_ma NULL: plain first moment (the *_adam kernels; beta1 / one_minus_beta1 are
 * then beta1 itself), else the positive-negative pair (beta1 = beta1^2).  update_variance 0: the
 * *_phase2 kernels.  lookahead NULL: no merge.  Every operation rounds on its own.
 */
#include <math.h>
int nnueft_oracle_ranger_lite_update(float* p, const float* grad, float* grad_ma, float* neg_grad_ma,
                                     float* variance_ma, float* lookahead, long long n,
                                     float beta2, float one_minus_beta2, float bias_correction2,
                                     float beta1, float one_minus_beta1, float one_plus_pnm, float pnm_factor,
                                     float noise_norm, float lr_div_bc1, float eps, long long step, float wd_factor,
                                     int update_variance, float alpha)
{
    const int odd = (int)(step & 1);
    const float one_minus_alpha = 1.0f - alpha;
    for (long long i = 0; i < n; ++i) {
        const float g = grad[i];
        float vm = variance_ma[i];
        if (update_variance) {
            vm = vm * beta2 + (g * g) * one_minus_beta2;
            variance_ma[i] = vm;
        }
        const float denom = sqrtf(vm / bias_correction2) + eps;
        float dir;
        if (neg_grad_ma) {
            float* pos = odd ? grad_ma : neg_grad_ma;
            const float* neg = odd ? neg_grad_ma : grad_ma;
            const float np_ = pos[i] * beta1 + g * one_minus_beta1;
            dir = (np_ * one_plus_pnm - neg[i] * pnm_factor) / noise_norm;
            pos[i] = np_;
        } else {
            const float gm = grad_ma[i] * beta1 + g * one_minus_beta1;
            grad_ma[i] = gm;
            dir = gm;
        }
        float q = p[i];
        if (wd_factor != 0.0f) q = q * (1.0f - wd_factor);
        q = q - lr_div_bc1 * (dir / denom);
        if (lookahead) {
            q = q * alpha + lookahead[i] * one_minus_alpha;
            lookahead[i] = q;
        }
        p[i] = q;
    }
    return 0;
}

int nnueft_oracle_ranger_lite_update_variance(const float* grad, float* variance_ma, long long n, float beta2,
                                              float one_minus_beta2)
{
    for (long long i = 0; i < n; ++i) variance_ma[i] = variance_ma[i] * beta2 + (grad[i] * grad[i]) * one_minus_beta2;
    return 0;
}

/* out = (floor(x * scale + eps) / scale) * post_mul: _fake_quantize_acts (model/quantize.py:36-45) and the
 * correction factor applied after it (composed_feature_transformer.py:143-149). */
int nnueft_oracle_act_fake_quantize(const float* x, float* out, long long n, float scale, float eps, float post_mul)
{
    for (long long i = 0; i < n; ++i) out[i] = (floorf(x[i] * scale + eps) / scale) * post_mul;
    return 0;
}

/*
 * Bucketed linear layer and its gradients: StackedLinear.forward (model/modules/stacked_linear.py:38-66;
 * F.linear over all blocks, then select_output) and what autograd derives from it, written for the
 * one block a position selects.  Sums run over ascending input index / ascending position; the
 * GPU kernels associate differently, so they are compared to a tolerance.
 */
int nnueft_oracle_bucket_linear_fwd(const float* x, const int64_t* bucket, const float* W, const float* bias,
                                    float* y, int B, int in, int out, int count)
{
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b) {
        const int64_t k = bucket[b];
        if (k < 0 || k >= count) continue;
        for (int o = 0; o < out; ++o) {
            const float* w = W + ((size_t)k * out + o) * in;
            double acc = bias[k * out + o];
            for (int i = 0; i < in; ++i) acc += (double)x[(size_t)b * in + i] * (double)w[i];
            y[(size_t)b * out + o] = (float)acc;
        }
    }
    return 0;
}

int nnueft_oracle_bucket_linear_bwd(const float* x, const int64_t* bucket, const float* W, const float* gy,
                                    float* gx, float* gW, float* gbias, int B, int in, int out, int count)
{
    double* aw = (double*)calloc((size_t)count * out * in, sizeof(double));
    double* ab = (double*)calloc((size_t)count * out, sizeof(double));
    if (!aw || !ab) { free(aw); free(ab); return -2; }
    for (int b = 0; b < B; ++b) {
        const int64_t k = bucket[b];
        if (k < 0 || k >= count) continue;
        for (int i = 0; i < in; ++i) {
            double acc = 0.0;
            for (int o = 0; o < out; ++o) acc += (double)gy[(size_t)b * out + o] * (double)W[((size_t)k * out + o) * in + i];
            if (gx) gx[(size_t)b * in + i] = (float)acc;
        }
        for (int o = 0; o < out; ++o) {
            const double g = gy[(size_t)b * out + o];
            ab[k * out + o] += g;
            double* row = aw + ((size_t)k * out + o) * in;
            for (int i = 0; i < in; ++i) row[i] += g * (double)x[(size_t)b * in + i];
        }
    }
    for (size_t i = 0; i < (size_t)count * out * in; ++i) gW[i] = (float)aw[i];
    for (int i = 0; i < count * out; ++i) gbias[i] = (float)ab[i];
    free(aw);
    free(ab);
    return 0;
}
