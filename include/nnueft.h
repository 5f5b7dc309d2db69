/*
 * libnnueft — sparse feature transformer of nnue-pytorch for AMD Instinct MI355X (gfx950).
 *
 * C ABI.  Every pointer is a DEVICE pointer owned by the caller unless stated otherwise; the
 * library never allocates, frees or retains memory.  `stream` is a hipStream_t passed as void*
 * (NULL = the default stream); all work is enqueued on it and the call returns without waiting.
 * The library may be called from several host threads.  What it keeps between calls: per device,
 * a few facts queried once (LDS size, number of XCDs) and the fixed scratch array of
 * nnueft_double_fwd_noalloc; per host thread and device, two events for the two-stream backward.
 * After the first call on a device an entry point makes no calls but kernel launches and event
 * record / wait, so it can be recorded by a stream capture (make that first call before capturing).
 *
 * Return value: 0 on success, a negative NNUEFT_E_* code for a rejected argument, or a positive
 * hipError_t when a launch failed.  nnueft_error_string() describes either.
 *
 * Shapes and names follow the reference (paths relative to the nnue-pytorch checkout):
 *   B  batch size (positions)          K  slots per index list (max_active_features)
 *   R  rows of the weight table        out_cols = L1 + n_psqt (row width of the table)
 * Index lists are int32[B,K], row-major; any entry outside [0,R) (the loader pads with -1,
 * data_loader/cpp/training_data_loader.cpp:516-519) contributes nothing.
 *
 * Summation order of the fp32 paths (what "deterministic" and "bit-exact" refer to):
 *   forward        s = +0; s += W[idx[k]] for k ascending over the valid slots; result = s + bias
 *   weight grad    (deterministic entry points) per perspective and table row one chain starting at
 *                  +0 over the slots naming that row in ascending (position, slot) order; then
 *                  white chain + black chain.  This is the order of torch's CPU embedding_bag
 *                  backward, i.e. of the reference's CPU path.
 *                  With row_split = 0 that holds for every row (the strict order: bit for bit the
 *                  reference's CPU path).  With row_split > 0, for speed on batches where a few rows are
 *                  named by a large part of the positions, a table row named by more than row_split
 *                  slots of the batch (both perspectives together) is summed window by window
 *                  (nnueft_row_split() is the value this build is tuned for).  Window w holds
 *                  positions [w * nnueft_row_window(B), (w + 1) * nnueft_row_window(B)); per
 *                  perspective, each window's slots are chained from +0 as above, the window sums
 *                  are chained from +0 in ascending w, and the two perspectives are added.  Such
 *                  a row agrees with the CPU path to rounding, not bit for bit.
 *   bias grad      (deterministic entry points) positions are cut into tiles of nnueft_bias_tile();
 *                  per column a chain over a tile's positions, then a chain over the tile sums.
 *   The atomic entry points add in an unspecified order.
 */
#ifndef NNUEFT_H
#define NNUEFT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NNUEFT_VERSION 2

#define NNUEFT_E_ARG (-1)         /* null pointer, non-positive or inconsistent dimension, odd L1 */
#define NNUEFT_E_WORKSPACE (-2)   /* workspace missing, misaligned (256 B) or smaller than nnueft_det_workspace_bytes() */
#define NNUEFT_E_UNSUPPORTED (-3) /* a dimension beyond what the kernels index (see each entry point) */
#define NNUEFT_E_SCRATCH (-4)     /* sizes beyond what the library's own fixed scratch memory holds (nnueft_double_fwd_noalloc) */

int nnueft_version(void);
const char* nnueft_error_string(int code);

/* Positions per tile of the deterministic bias-gradient order. */
int nnueft_bias_tile(void);

/* Deterministic weight-gradient order: the `row_split` argument of the deterministic entry points.
 * 0: every row in the strict order.  n > 0: rows named by more than n slots are summed in windows of
 * nnueft_row_window(B) positions (see "Summation order" above).  nnueft_row_split() returns the
 * threshold the kernels are tuned for (512); any non-negative value is accepted. */
int nnueft_row_split(void);
int nnueft_row_window(int B);

/* Accelerator dies (XCDs, each with an L2 of its own) of the current device, 0 if the runtime does
 * not say; negative on error.  The L2-blocked kernels are laid out for 8: on a device that presents
 * another number, nnueft_double_fwd and nnueft_ft_int16_fwd take their unblocked kernels (same
 * results), and the deterministic backward keeps its results but loses its cache blocking. */
int nnueft_device_xcds(void);

/*
 * out[b,:] = (sum_k W[idx[b,k],:]) + bias.
 * Replaces the `sparse_input_linear_forward` CuPy kernel launched from
 * model/modules/feature_transformer/sparse_linear_functions.py:85-99
 * (kernel: sparse_linear_kernel.py:114-157); same result as _torch_sparse_linear, :16-50.
 * idx int32[B,K]; W f32[R,out_cols] row-major contiguous; bias f32[out_cols]; out f32[B,out_cols].
 */
int nnueft_sparse_fwd(const int32_t* idx, const float* W, const float* bias, float* out,
                      int B, int K, int R, int out_cols, void* stream);

/*
 * gW[idx[b,k],:] += gout[b,:] and gbias += gout[b,:] with floating-point atomics.
 * gW f32[R,out_cols] and gbias f32[out_cols] must be zero (or hold a value to accumulate onto).
 * Replaces `sparse_input_linear_backward`, sparse_linear_functions.py:118-134
 * (kernel: sparse_linear_kernel.py:237-288).
 */
int nnueft_sparse_bwd_atomic(const int32_t* idx, const float* gout, float* gW, float* gbias,
                             int B, int K, int R, int out_cols, void* stream);

/*
 * Bytes of scratch the deterministic backward entry points need (256-B aligned device memory,
 * contents irrelevant on entry, garbage on exit).  n_persp = 1 for nnueft_sparse_bwd_det,
 * 2 for nnueft_double_bwd_det; row_split as passed to them (the window sums of split rows are
 * sized for the worst case, so row_split = 0 needs the least).  Returns 0 for invalid dimensions.
 */
size_t nnueft_det_workspace_bytes(int B, int K, int R, int out_cols, int n_persp, int row_split);

/*
 * Same gradient as nnueft_sparse_bwd_atomic in the fixed order stated at the top: a stable
 * counting sort of the (row, position) pairs followed by a segmented reduction.  Every element
 * of gW and gbias is written exactly once, so neither needs to be cleared.
 * No counterpart in the reference (its GPU backward is atomic only); the order is that of the
 * reference's CPU path (torch embedding_bag backward, sparse_linear_functions.py:43-50).
 */
int nnueft_sparse_bwd_det(const int32_t* idx, const float* gout, float* gW, float* gbias,
                          int B, int K, int R, int out_cols, int row_split,
                          void* workspace, size_t workspace_bytes, void* stream);

/*
 * Bytes of scratch nnueft_double_fwd can use (256-B aligned device memory, contents irrelevant on
 * entry and on exit).  Returns 0 for invalid dimensions.
 */
size_t nnueft_fwd_workspace_bytes(int B, int K, int R, int L1, int n_psqt);

/*
 * Both perspectives, then the side-to-move mix, clamp and pairwise product:
 *   w = sum W[widx] + bias, b = sum W[bidx] + bias              (first L1 columns)
 *   x_w = us*w + them*b,  x_b = us*b + them*w
 *   l0[:, :h] = clamp(x_w[:h]) * clamp(x_w[h:]),  l0[:, h:] = clamp(x_b[:h]) * clamp(x_b[h:]),  h = L1/2
 *   wpsqt = sum W[widx, L1+psqt_idx] + bias[L1+psqt_idx],  bpsqt likewise
 * Replaces `fused_double_ft_forward`, fused_ft_functions.py:51-75 (kernel: fused_ft_kernel.py:27-117);
 * same result as the torch composition double_ft_functions.py:62-80.
 * us, them f32[B]; widx, bidx int32[B,K]; psqt_idx int64[B]; W f32[R,L1+n_psqt]; bias f32[L1+n_psqt];
 * l0 f32[B,L1]; wpsqt, bpsqt f32[B]; saved f32[2,B,L1].
 * `saved` receives the two perspectives' row sums before the bias (saved[0] white, saved[1] black);
 * the backward recomputes the mixed values from them with the forward's own operations.  (The
 * reference stores the clamped mixed values instead, fused_ft_kernel.py:95-99, and thereby loses
 * torch's clamp gradient at exactly 0 and exactly max.)  L1 must be even.
 * workspace: NULL, or nnueft_fwd_workspace_bytes() bytes.  With a workspace (and 16-byte aligned rows:
 * L1 % 8 == 0, (L1+n_psqt) % 4 == 0) the positions are grouped by the 768-row table block their lists
 * name.  Rows of 512 columns and more (L1 % 32 == 0, K <= 32, a table of at most 62 blocks) are then
 * gathered out of LDS: a workgroup holds a tile of one block, 768 rows x 32 columns, and sums it for
 * every list of the block.  From 2048 columns on (L1 % 64 == 0) the same kernel also writes l0 for every
 * position whose (us, them) is (1, 0) or (0, 1), what the loaders produce; other values of us and them are
 * allowed as everywhere and take a pass over `saved`, as does a batch in which a sum is not finite (0 * inf
 * of the mix is NaN, here as in the reference).  Other shapes are blocked for the per-XCD L2 caches: each
 * XCD works through its share of the grouped lists one column slice at a time.  Results are bit-identical
 * with and without the workspace.
 */
int nnueft_double_fwd(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                      const int64_t* psqt_idx, const float* W, const float* bias, float max_act,
                      float* l0, float* wpsqt, float* bpsqt, float* saved,
                      int B, int K, int R, int L1, int n_psqt,
                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * nnueft_double_fwd whose l0 already carries the activation grid its caller applies next:
 *   l0 = (floor(l0 * act_scale + act_eps) / act_scale) * act_post_mul,
 * i.e. `fake_quantize_ft_act(l0_) * l0_correction_factor` of ComposedFeatureTransformer.forward
 * (composed_feature_transformer.py:143-149) inside the kernel that produces l0, instead of one more
 * pass over [B, L1].  Every operation rounds on its own: the same bits as the separate pass
 * (nnueft_act_fake_quantize).  `saved`, wpsqt and bpsqt are those of nnueft_double_fwd, so the
 * backward entry points serve both (the grid is straight-through; the caller scales grad_l0 by
 * act_post_mul).
 */
int nnueft_double_fwd_act(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                          const int64_t* psqt_idx, const float* W, const float* bias, float max_act,
                          float* l0, float* wpsqt, float* bpsqt, float* saved,
                          int B, int K, int R, int L1, int n_psqt,
                          void* workspace, size_t workspace_bytes,
                          float act_scale, float act_eps, float act_post_mul, void* stream);

/*
 * The fused forward over a table that is never written to memory: W + V[row % virtual_rows], rounded to
 * multiples of 1 / scale_ft (first L1 columns) and 1 / scale_psqt (the others) when fake_quantize is set.
 * Replaces the table passes in front of the operator in ComposedFeatureTransformer.forward: the merge of
 * real and virtual weights (features/halfka_v2_hm.py:68-69, `weight + virtual_weight.repeat(32, 1)`) and
 * their fake quantization (composed_feature_transformer.py:61-76, model/quantize.py:47-56), each a pass over
 * the whole table in the reference.  The merge happens where a tile of the table goes into LDS, with the
 * operations of nnueft_table_merge in their order, so the outputs have the bits of nnueft_table_merge followed
 * by nnueft_double_fwd / nnueft_double_fwd_act (act_on != 0: the activation grid as there).
 * V f32[virtual_rows, L1 + n_psqt].  Only the LDS-tiled gather can do this: virtual_rows must be 768 and
 * nnueft_double_fwd_virtual_fits() must return 1 for the sizes on the current device (rows of 512 columns and
 * more, L1 % 32 == 0, K <= 32, 8 XCDs), else NNUEFT_E_UNSUPPORTED; the workspace is required
 * (nnueft_fwd_workspace_bytes).  The backward entry points serve it unchanged: they never read the table;
 * their weight gradient is that of the merged table (the gradient of W as it is, of V after
 * nnueft_table_virtual_grad).
 */
int nnueft_double_fwd_virtual_fits(int B, int K, int R, int L1, int n_psqt, int virtual_rows);
int nnueft_double_fwd_virtual(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                              const int64_t* psqt_idx, const float* W, const float* V, const float* bias,
                              float max_act, float* l0, float* wpsqt, float* bpsqt, float* saved,
                              int B, int K, int R, int L1, int n_psqt, int virtual_rows,
                              float scale_ft, float scale_psqt, int fake_quantize,
                              void* workspace, size_t workspace_bytes,
                              int act_on, float act_scale, float act_eps, float act_post_mul, void* stream);

/*
 * nnueft_double_fwd for callers that cannot allocate device memory or size a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the scratch memory of the
 * L2-blocked gather (pair order, keys, per-workgroup histograms) is a fixed array inside the library,
 * one copy per GPU, 2 MiB, held until the process ends.  Same arguments and results as
 * nnueft_double_fwd minus the workspace; no counterpart in the reference.  The call allocates and
 * frees nothing.  Limit: the scratch of the L2-blocked gather, 2 * B * 8 bytes plus 4 bytes per
 * (256 lists, table block), must fit 2 MiB (B = 65536 with a 24576-row table fits), beyond it
 * NNUEFT_E_SCRATCH; the LDS-tiled gather is taken where its larger scratch fits as well.  All calls on one GPU share that GPU's array:
 * calls that overlap in time on one GPU (two streams, two threads) race on it; calls on one stream
 * are ordered and safe.  The first call on a device looks up the array's address (not a stream
 * operation: make one call on each device before capturing a graph there).
 */
int nnueft_double_fwd_noalloc(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                              const int64_t* psqt_idx, const float* W, const float* bias, float max_act,
                              float* l0, float* wpsqt, float* bpsqt, float* saved,
                              int B, int K, int R, int L1, int n_psqt, void* stream);

/*
 * Gradient of nnueft_double_fwd with respect to W and bias, floating-point atomics.
 * `saved` is the forward's; `bias` the forward's bias.  gW f32[R,L1+n_psqt] and gbias f32[L1+n_psqt]
 * must be zero on entry.
 * Replaces `fused_double_ft_backward`, fused_ft_functions.py:94-120 (kernel: fused_ft_kernel.py:147-272).
 */
int nnueft_double_bwd_atomic(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                             const int64_t* psqt_idx, const float* bias, float max_act,
                             const float* grad_l0, const float* grad_wpsqt, const float* grad_bpsqt,
                             const float* saved, float* gW, float* gbias,
                             int B, int K, int R, int L1, int n_psqt, void* stream);

/*
 * The same gradient as nnueft_double_bwd_atomic (sums in no fixed order, so their last bits vary from run
 * to run), with the atomic adds made in LDS: a workgroup keeps a tile of one 768-row table block of gW
 * (768 rows x 16 columns, as doubles) in LDS, adds the upstream rows of every position whose list names rows of
 * that block, and writes the tile out once, rounded to float.  gW and gbias are fully written and need not be zero on entry.
 * workspace: nnueft_atomic_lds_workspace_bytes(B, K, R, L1 + n_psqt, 2) bytes of device memory, 256-byte
 * aligned; a return of 0 from that function, or NNUEFT_E_UNSUPPORTED from this one, says that the
 * shape or the device cannot take this path (K > 32, a row that is not whole 16-byte vectors, more than
 * 62 table blocks, a device that does not present 8 XCDs): call nnueft_double_bwd_atomic then.
 * The bias gradient is the deterministic one (tiles of nnueft_bias_tile() positions).  B >= 1.
 * Replaces `fused_double_ft_backward`, fused_ft_functions.py:94-120 (kernel: fused_ft_kernel.py:147-272,
 * whose shared-memory partial sums, :172-176, are what the LDS tile generalises).
 */
size_t nnueft_atomic_lds_workspace_bytes(int B, int K, int R, int out_cols, int n_persp);
/* The one-list form (n_persp = 1 for the workspace): gradient of nnueft_sparse_fwd, as nnueft_sparse_bwd_atomic.
 * Replaces `sparse_input_linear_backward`, sparse_linear_functions.py:118-134 (kernel: sparse_linear_kernel.py:237-288). */
int nnueft_sparse_bwd_atomic_lds(const int32_t* idx, const float* gout, float* gW, float* gbias,
                                 int B, int K, int R, int out_cols,
                                 void* workspace, size_t workspace_bytes, void* stream);
int nnueft_double_bwd_atomic_lds(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                                 const int64_t* psqt_idx, const float* bias, float max_act,
                                 const float* grad_l0, const float* grad_wpsqt, const float* grad_bpsqt,
                                 const float* saved, float* gW, float* gbias,
                                 int B, int K, int R, int L1, int n_psqt,
                                 void* workspace, size_t workspace_bytes, void* stream);

/*
 * Same gradient in the fixed order stated at the top; gW and gbias are fully written.
 * No counterpart in the reference's GPU code; the order is that of autograd through the
 * reference's CPU composition (double_ft_functions.py:62-80).
 * sorted_lists: NULL, or the block nnueft_det_sort wrote for these index lists, sizes and row_split
 * (typically while the forward pass ran: the sort reads nothing but the lists); the call then skips
 * its own sort.  The block stays valid for further calls, one at a time: it holds the task counters
 * of the reduction, which the call's last kernel rewinds, so two reductions that overlap on one
 * block (two streams, two threads) race on them.
 * row_split = 0 (the strict order) with rows of 256 columns and more, lists of up to 32 slots and a
 * device of 8 XCDs: the chains of the table rows are summed out of LDS tiles of the upstream rows
 * (a second set of tables in the sorted block).  A batch in which a list names rows of two 768-row
 * table blocks, or one row twice, is noticed on the device and summed by the segmented reduction
 * in the same call; the bits are the same either way.
 * aux_stream: NULL, or a second stream of the same device.
 *   With sorted_lists NULL: sorting the index lists and computing the upstream rows are independent;
 *   given a second stream the call runs the sort there, beside the other work on `stream`, and
 *   joins the two before the reduction (events, no host wait).
 *   With sorted_lists given: the stream nnueft_det_sort was enqueued on, if the caller has not
 *   ordered `stream` after that sort itself; the reduction then waits for all work enqueued on
 *   aux_stream so far, the upstream rows do not.
 *   Either way, on return all later work enqueued on `stream` is ordered after the whole call, and
 *   nothing is left pending on aux_stream that the caller has to wait for.
 */
int nnueft_double_bwd_det(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                          const int64_t* psqt_idx, const float* bias, float max_act,
                          const float* grad_l0, const float* grad_wpsqt, const float* grad_bpsqt,
                          const float* saved, float* gW, float* gbias,
                          int B, int K, int R, int L1, int n_psqt, int row_split,
                          void* workspace, size_t workspace_bytes, void* sorted_lists, void* stream,
                          void* aux_stream);

/*
 * The part of the deterministic backward that depends on the index lists only: the stable sort of
 * the (table row, position) pairs and the work split of the reduction.  sorted_lists: device
 * memory of nnueft_det_sort_bytes(...) bytes, 256-byte aligned; pass it to nnueft_double_bwd_det
 * with the same lists, sizes and row_split.  n_persp = 2: both lists; 1: widx only (bidx ignored).
 */
size_t nnueft_det_sort_bytes(int B, int K, int R, int out_cols, int n_persp);
int nnueft_det_sort(const int32_t* widx, const int32_t* bidx, int B, int K, int R, int out_cols, int n_persp,
                    int row_split, void* sorted_lists, size_t sorted_bytes, void* stream);

/*
 * The reduction stage of the deterministic backward on its own: gW[r, :] = the chains stated at the
 * top over the upstream rows G f32[n_persp, B, out_cols] (G[p, b] is what position b contributes to
 * every table row its list p names), given the block nnueft_det_sort wrote for the lists.  For
 * callers that make the upstream rows themselves and for timing the stage; nnueft_sparse_bwd_det is
 * nnueft_det_sort + this with G = gout, nnueft_double_bwd_det computes G first.  gW fully written.
 * workspace: nnueft_det_workspace_bytes(...) bytes (only the window sums of split rows are used).
 * No counterpart in the reference.
 */
int nnueft_det_reduce_rows(const float* G, float* gW, int B, int K, int R, int out_cols, int n_persp,
                           int row_split, void* workspace, size_t workspace_bytes, void* sorted_lists,
                           void* stream);
/*
 * The same with g_pitch >= out_cols floats from one row of G to the next (G f32[n_persp, B, g_pitch]).
 * nnueft_det_upstream_pitch(out_cols) is the pitch nnueft_double_bwd_det gives its own upstream rows: whole
 * 128-byte lines, so that the 1 KB a wave gathers of a row lies in 8 cache lines and not in 9 (3080 -> 3104
 * floats: the reduction 452 -> 438 us and the kernel that writes the rows 182 -> 170 us at L1 = 3072,
 * B = 16384).  Results do not depend on the pitch.  No counterpart in the reference.
 */
int nnueft_det_upstream_pitch(int out_cols);
int nnueft_det_reduce_rows_pitched(const float* G, int g_pitch, float* gW, int B, int K, int R, int out_cols,
                                   int n_persp, int row_split, void* workspace, size_t workspace_bytes,
                                   void* sorted_lists, void* stream);

/*
 * merged[r, c] = q(W[r, c] + V[r % vrows, c]): the table the gather reads, from the real weights
 * W f32[R, cols] and the virtual (factorised) weights V f32[vrows, cols] shared by all table blocks
 * (V may be NULL).  With fake_quantize != 0, q(x) = round(x * s) / s (round half to even) with
 * s = scale_ft for the first L1 columns and scale_psqt for the rest; otherwise q is the identity.
 * One pass in place of HalfKav2Hm.merged_weight (model/modules/features/halfka_v2_hm.py:68-69),
 * the two fake_quantize_weights calls and the torch.cat of
 * ComposedFeatureTransformer.merged_weight_and_bias (composed_feature_transformer.py:61-76;
 * formula model/quantize.py:48-58).  Bit-identical to those torch ops.
 */
int nnueft_table_merge(const float* W, const float* V, float* merged, int R, int cols, int L1, int vrows,
                       float scale_ft, float scale_psqt, int fake_quantize, void* stream);

/*
 * gV[v, c] = sum_k gW[k * vrows + v, c], k ascending from +0: the gradient of the virtual weights
 * given the gradient of the merged table (the backward of `virtual_weight.repeat(NUM_BUCKETS, 1)`,
 * halfka_v2_hm.py:68-69).  The straight-through estimator makes the gradient of the real weights
 * gW itself.  gW f32[R, cols]; gV f32[vrows, cols], fully written.
 */
int nnueft_table_virtual_grad(const float* gW, float* gV, int R, int cols, int vrows, void* stream);

/*
 * Quantized feature transformer as the engine evaluates an exported net (no code in the
 * reference; spec docs/nnue.md:1014-1069 and :2097-2134, constants model/quantize.py:58-73,
 * tensors produced by QuantizationManager.quantize_feature_transformer_*, model/quantize.py:175-204):
 *   acc_p[c] = b16[c] + sum_k W16[idx_p[k], c]                      int16, wrapping
 *   c_p[c]   = min(max(acc_p[c], 0), clip_max)
 *   out[b, o*h + j] = (c_P(o)[j] * c_P(o)[j+h]) >> shift            o = 0 side to move, 1 the other
 *   psqt_out[b] = (sum psqt32[idx_P(0), bucket] - sum psqt32[idx_P(1), bucket]) / 2     (C division)
 * stm u8[B]: 0 white to move, 1 black; W16 int16[R,L1]; b16 int16[L1]; psqt32 int32[R,n_psqt];
 * psqt_idx int64[B]; out_u8 u8[B,L1]; psqt_out int32[B].  clip_max*clip_max >> shift must fit 8 bits.
 * workspace: NULL, or nnueft_int16_workspace_bytes() bytes (two int16 per position and column plus the list
 * sort's scratch); with it the sums are gathered out of LDS tiles of the table like nnueft_double_fwd's
 * (L1 % 64 == 0, at least 512 columns, lists of 32 slots at most, table blocks of 768 rows at most), or
 * else (L1 % 16 == 0) blocked for the per-XCD L2 caches.  table_block_rows: rows of one block of
 * the table whose rows a list stays inside (704 for an exported HalfKAv2_hm net, 0 = 768); only a
 * scheduling hint: a list that leaves its block is summed all the same.  Results do not depend on either.
 */
size_t nnueft_int16_workspace_bytes(int B, int K, int R, int L1, int table_block_rows);
int nnueft_ft_int16_fwd(const int32_t* widx, const int32_t* bidx, const uint8_t* stm,
                        const int16_t* W16, const int16_t* b16, const int32_t* psqt32,
                        const int64_t* psqt_idx, uint8_t* out_u8, int32_t* psqt_out,
                        int B, int K, int R, int L1, int n_psqt, int clip_max, int shift,
                        int table_block_rows, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Quantized layer stacks on the output of nnueft_ft_int16_fwd: the integer evaluation of the
 * bucketed stack of model/modules/layer_stacks.py:33-84 with the tensors of
 * QuantizationManager.quantize_fc_layer (model/quantize.py:218-236; int8 weights, int32 biases).
 * No code in the reference (the engine runs it); each step is the integer image of the
 * fake-quantized float forward, with a1, a2, a3 the int32 accumulators of the three layers:
 *   a1 = b1 + W1 . x                                     x u8 [L1], 0..127
 *   y1 = clip([ (a1*a1) >> sqr_shift1, a1 >> lin_shift1 ], 0, act_max)        2*L2 values
 *   a2 = b2 + W2 . y1 ;  y2 = clip([ (a2*a2) >> sqr_shift2, a2 >> lin_shift2 ], 0, act_max)
 *   a3 = bo + Wo . [y1, y2]
 *   out = 2 * (a3 + a1[L2-2] - a1[L2-1]) * out_mult / out_den         (64-bit, C division)
 * With the default scales (weights x128 / x64 / x128, activations x128): lin_shift1 = 7,
 * sqr_shift1 = 21, lin_shift2 = 6, sqr_shift2 = 19, act_max = 127, out_mult = 9600, out_den = 32768;
 * out is then the stack's output at scale 9600 (the scale of nnueft_ft_int16_fwd's psqt_out).
 * x u8[B,L1]; bucket int64[B] in [0,count); W1 int8[count*L2, L1]; b1 int32[count*L2];
 * W2 int8[count*L3, 2*L2]; b2 int32[count*L3]; Wo int8[count, 2*L2+2*L3]; bo int32[count]; out int32[B].
 * Limits: L1 % 4 == 0, L1 <= 4096, 2 <= L2 <= 32, L3 <= 32.
 */
int nnueft_stack_int8_fwd(const uint8_t* x, const int64_t* bucket, const int8_t* W1, const int32_t* b1,
                          const int8_t* W2, const int32_t* b2, const int8_t* Wo, const int32_t* bo,
                          int32_t* out, int B, int L1, int L2, int L3, int count,
                          int lin_shift1, int sqr_shift1, int lin_shift2, int sqr_shift2, int act_max,
                          int out_mult, int out_den, void* stream);

/*
 * Bucketed linear layer: y[b, :] = bias[bucket[b]] + W[bucket[b]] x[b], where W holds `count` blocks
 * of [out, in] one after the other (the layout of nn.Linear(in, out * count)).  Same values, up to
 * the order of the floating-point sums, as StackedLinear.forward of the reference
 * (model/modules/stacked_linear.py:38-66): F.linear over all blocks followed by select_output; the
 * backward is what autograd derives from that: gx[b] = W[bucket[b]]^T gy[b]; gW and gbias of a
 * block sum gy[b] (x) x[b] and gy[b] over the positions of that bucket (ascending position order,
 * so the result does not change from run to run), blocks no position uses get zeros.
 * x f32[B, in]; bucket int64[B], every entry in [0, count) (a position outside is skipped: its row
 * of y and gx is left unwritten); W f32[count * out, in]; bias f32[count * out]; y, gy f32[B, out];
 * gx f32[B, in] or NULL; gW, gbias fully written.  Limits: out <= 32, count <= 64, in % 32 == 0,
 * x and W 16-byte aligned.  workspace: nnueft_bucket_linear_workspace_bytes(B, count) bytes.  A call
 * first groups the positions by bucket into the workspace; nnueft_bucket_linear_group does only
 * that, and a call given a workspace that already holds the grouping of the same bucket tensor
 * (from it or from an earlier call, untouched since) says so with workspace_grouped = 1 and skips it:
 * the three layers of a stack and their backward passes share one grouping.
 * Tolerance against the reference: 1e-5 relative to the largest magnitude of the result.
 */
size_t nnueft_bucket_linear_workspace_bytes(int B, int count);
int nnueft_bucket_linear_group(const int64_t* bucket, int B, int count, void* workspace, size_t workspace_bytes,
                               void* stream);
int nnueft_bucket_linear_fwd(const float* x, const int64_t* bucket, const float* W, const float* bias, float* y,
                             int B, int in, int out, int count, void* workspace, size_t workspace_bytes,
                             int workspace_grouped, void* stream);
int nnueft_bucket_linear_bwd(const float* x, const int64_t* bucket, const float* W, const float* gy, float* gx,
                             float* gW, float* gbias, int B, int in, int out, int count, void* workspace,
                             size_t workspace_bytes, int workspace_grouped, void* stream);

/*
 * out[i] = (floor(x[i] * scale + eps) / scale) * post_mul, each operation rounding on its own: the
 * activation fake quantization of the feature transformer's output (_fake_quantize_acts,
 * model/quantize.py:36-45, called from composed_feature_transformer.py:143-144) together with the
 * l0 correction factor that follows it (:149), in one pass over [B, L1] instead of six.  The
 * straight-through estimator makes the gradient of x the incoming gradient times post_mul.
 * x, out f32[n]; out may be x.
 */
int nnueft_act_fake_quantize(const float* x, float* out, long long n, float scale, float eps, float post_mul,
                             void* stream);

/*
 * RangerLite parameter update, one call per parameter tensor (n contiguous f32 elements each of
 * p, grad and the state tensors).  They replace the reference's CuPy kernels of the same names,
 * model/optimizers/ranger_lite.py:46-201 (launched from :325-477 and :563-583), element for element:
 *   vm   = vm * beta2 + (g * g) * one_minus_beta2              (skipped when update_variance == 0:
 *                                                                the *_phase2 kernels, after
 *                                                                nnueft_ranger_lite_update_variance)
 *   den  = sqrt(vm / bias_correction2) + eps
 *   pnm:  pos = (step odd ? grad_ma : neg_grad_ma), neg = the other one
 *         pos = pos * beta1_sq + g * one_minus_beta1_sq          (written back to its buffer)
 *         dir = (pos * one_plus_pnm - neg * pnm_factor) / noise_norm
 *   adam: grad_ma = grad_ma * beta1 + g * one_minus_beta1 ;  dir = grad_ma
 *   p    = (wd_factor != 0 ? p * (1 - wd_factor) : p) - lr_div_bc1 * (dir / den)
 * Every operation rounds on its own, in this order.  wd_factor and update_variance fold the
 * reference's "full" and "phase2" variants into one entry point each.
 * lookahead_params: NULL, or the slow weights on a merge step; then, in the same pass,
 *   p = p * lookahead_alpha + lookahead_params * (1 - lookahead_alpha) ;  lookahead_params = p
 * which is lookahead_process_step (ranger_lite.py:737-760) without a second sweep over the
 * tensors.  nnueft_ranger_lite_lookahead_merge is that blend alone.
 */
int nnueft_ranger_lite_update_pnm(float* p, const float* grad, float* grad_ma, float* neg_grad_ma,
                                  float* variance_ma, long long n, float beta2, float one_minus_beta2,
                                  float bias_correction2, float beta1_sq, float one_minus_beta1_sq,
                                  float one_plus_pnm, float pnm_factor, float noise_norm, float lr_div_bc1,
                                  float eps, long long step, float wd_factor, int update_variance,
                                  float* lookahead_params, float lookahead_alpha, void* stream);
int nnueft_ranger_lite_update_adam(float* p, const float* grad, float* grad_ma, float* variance_ma,
                                   long long n, float beta2, float one_minus_beta2, float bias_correction2,
                                   float beta1, float one_minus_beta1, float lr_div_bc1, float eps,
                                   float wd_factor, int update_variance, float* lookahead_params,
                                   float lookahead_alpha, void* stream);
/*
 * The same update for several tensors in one launch (a launch costs a few microseconds whatever the
 * tensor's size, and a model has many small ones).  `tensors` is a host array of `count` records,
 * copied into the kernel's arguments 16 at a time; every record carries its own hyperparameters, since
 * parameter groups may differ.  neg_grad_ma == NULL selects the plain first moment (beta1,
 * one_minus_beta1 as in nnueft_ranger_lite_update_adam), otherwise the pair (beta1 = beta1^2,
 * one_minus_beta1 = 1 - beta1^2; odd_step = step & 1).  Element for element the arithmetic of the
 * single-tensor entry points.
 */
typedef struct nnueft_ranger_args {
    float* p;
    const float* grad;
    float* grad_ma;
    float* neg_grad_ma;
    float* variance_ma;
    float* lookahead_params;   /* NULL: no lookahead merge in this call */
    long long n;
    float beta2, one_minus_beta2, bias_correction2;
    float beta1, one_minus_beta1;
    float one_plus_pnm, pnm_factor, noise_norm;
    float lr_div_bc1, eps, wd_factor, lookahead_alpha, one_minus_lookahead_alpha;
    int odd_step;
    int update_variance;
} nnueft_ranger_args;
int nnueft_ranger_lite_update_multi(const nnueft_ranger_args* tensors, int count, void* stream);

int nnueft_ranger_lite_update_variance(const float* grad, float* variance_ma, long long n, float beta2,
                                       float one_minus_beta2, void* stream);
int nnueft_ranger_lite_lookahead_merge(float* p, float* lookahead_params, long long n, float alpha,
                                       void* stream);

/*
 * The per-position chains after the bucketed layers, one launch each instead of a dozen or more
 * elementwise torch ops (every operation still rounds on its own, in the order of those ops).
 *
 * nnueft_sqr_crelu_*: y f32[B, 2n] = clamp(cat[fq(x * x) * sqr_factor, fq(x)], 0, max_act) for x f32[B, n],
 * fq(v) = floor(v * scale + eps) / scale when fake_quantize, else v; skip (NULL or f32[B]) receives
 * x[:, n-2] - x[:, n-1].  LayerStacks.forward's two `_sqr_crelu`-style blocks and the skip connection
 * (model/modules/layer_stacks.py:39-70).  Backward: fq is straight-through, the clamp passes the
 * gradient where 0 <= value <= max_act; gskip (NULL or f32[B]) is added to / subtracted from the
 * last two columns of gx.
 */
int nnueft_sqr_crelu_fwd(const float* x, float* y, float* skip, int B, int n, float scale, float eps,
                         float sqr_factor, float max_act, int fake_quantize, void* stream);
int nnueft_sqr_crelu_bwd(const float* x, const float* gy, const float* gskip, float* gx, int B, int n, float scale,
                         float eps, float sqr_factor, float max_act, int fake_quantize, void* stream);

/*
 * net[i] = fq_out(lin[i] + skip[i]) + (wpsqt[i] - bpsqt[i]) * (us[i] - 0.5), all f32[B];
 * fq_out(v) = trunc(round(v * den) * mult / den) / mult in 64-bit integers when fake_quantize
 * (fake_quantize_output of model/quantize.py; model/modules/layer_stacks.py:76-80, model/model.py:131).  Backward: lin and skip
 * receive gnet itself; gwpsqt = gnet * (us - 0.5), gbpsqt = -gwpsqt.
 */
int nnueft_stack_output_fwd(const float* lin, const float* skip, const float* wpsqt, const float* bpsqt,
                            const float* us, float* net, int B, long long den, long long mult, int fake_quantize,
                            void* stream);
int nnueft_stack_output_bwd(const float* gnet, const float* us, float* gwpsqt, float* gbpsqt, int B, void* stream);

/*
 * The training loss of model/nnue.py:39-70 (win-rate model, tablebase score remap, lambda blend,
 * |pt - qf|^pow_exp with optional asymmetry, position weights) for scorenet/score/outcome f32[B].
 * terms f32[3, B] receives loss_i * w_i, w_i and w_i * dloss_i/dscorenet_i; sums f32[2] the sums of the
 * first two rows (each thread of one 1024-thread workgroup chains every 1024th element, then a fixed
 * pairwise tree: the same bits on every run); loss[0] = sums[0] / sums[1].
 * Backward: grad_scorenet[i] = terms[2, i] * (grad_loss[0] / sums[1]); grad_loss is a device scalar.
 */
int nnueft_sf_loss_fwd(const float* scorenet, const float* score, const float* outcome, float* terms, float* sums,
                       float* loss, int B, float in_offset, float in_scaling, float out_offset, float out_scaling,
                       float pow_exp, float qp_asymmetry, float w1, float w2, float tb_remap_base,
                       float tb_remap_scale, float tb_remap_decay, double lambda, void* stream);
int nnueft_sf_loss_bwd(const float* terms, const float* sums, const float* grad_loss, float* grad_scorenet, int B,
                       void* stream);

/*
 * Loader hand-off: from the words of a batch already on the device, them[i] = 1 - us[i] and
 * piece_count[i] = (int64) piece_count32[i], i < B, in one launch.  Replaces the `1.0 - us` and
 * `.to(dtype=torch.int64)` ops at the end of SparseBatch.get_tensors (data_loader/_native.py:76-86).
 */
int nnueft_batch_unpack(const float* us, const int32_t* piece_count32, float* them, int64_t* piece_count,
                        int B, void* stream);

/*
 * Measurement aids (no counterpart in the reference; nothing in the library's own paths calls them): what the
 * memory paths of the gathers deliver on the device at hand, for the roofline figures of a benchmark.
 * nnueft_probe_l2_gather: every CU gathers pieces of `span` (128 or 1024) contiguous bytes at random places of a
 * set of set_bytes that is resident in its XCD's L2 (src: 8 * set_bytes of device memory, one set per XCD),
 * `depth` (4, 8 or 16) loads of 16 bytes in flight per lane, `iters` rounds; *bytes_read (host) = bytes the launch
 * reads.  nnueft_probe_lds_read: every CU reads 16 bytes per lane out of a 96 KB LDS tile, pattern 0 a wave
 * 1 KB in a row, pattern 1 each 8-lane group a whole 128-byte row at a random row.  sink: 4 bytes of device
 * memory (never written in practice).  Time the launches with events on `stream`.
 */
int nnueft_probe_l2_gather(const void* src, size_t src_bytes, float* sink, int set_bytes, int span, int depth,
                           int iters, long long* bytes_read, void* stream);
int nnueft_probe_lds_read(float* sink, int pattern, int iters, long long* bytes_read, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NNUEFT_H */
