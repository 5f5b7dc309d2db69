// Functions shared between the translation units of libnnueft (not part of the ABI).
#pragma once

#include "common.h"

// The activation grid of the feature transformer's output, (floor(x * scale + eps) / scale) * post_mul,
// when the forward applies it itself (on == 0: it does not).
struct ActGrid {
    float scale, eps, post_mul;
    int on;
};

// The virtual weights a forward may merge into the table on the fly: the table it sums is
// W + V[row % 768] (V: f32 [768, L1 + n_psqt]), rounded to multiples of 1 / scale_ft (first L1 columns) and
// 1 / scale_psqt (the rest) when `quantize` is set.  V == nullptr: the table is W as it is.
struct VirtualTable {
    const float* V;
    float scale_ft, scale_psqt;
    int quantize;
    float inv_scale_ft;   // 1 / scale_ft when scale_ft is a power of two (dividing by it is then the same as
                          // multiplying by this, bit for bit, at a fraction of the instructions), else 0
};

namespace nnueft_dev {

// What the launchers need to know about a device; queried once per device and process.
struct DeviceInfo {
    int max_lds;   // most LDS a workgroup can ask for, bytes
    int xcds;      // accelerator dies (each with an L2 of its own) the device presents; 0 = unknown
    int cus;       // compute units
};
// The current device and its facts.  Returns 0, a negative NNUEFT_E_* or a positive hipError_t.
int device_info(int* device, const DeviceInfo** info);
// Two events without timing that belong to the calling thread and `device`, created on first use and
// kept, for ordering a second stream against the caller's (record / wait only on the launch path).
int thread_events(int device, hipEvent_t* fork, hipEvent_t* join);

}  // namespace nnueft_dev

namespace nnueft_blocked {

// XCDs the blocked kernels are laid out for; workgroup id % kXcd is the XCD a workgroup lands on
// (workgroups are dealt to the XCDs round-robin).  Results never depend on it; on a device that
// presents another number of XCDs the entry points take the unblocked kernels where they have them.
constexpr int kXcd = 8;
inline bool blocked_layout_fits(const nnueft_dev::DeviceInfo& d) { return d.xcds == kXcd || d.xcds == 0; }

// Pair sort: order[] = ids (perspective * B + position) of the 2B index lists of a batch grouped by
// the table block they name (block_rows_hint rows per block, 0 = 768).  `ws` needs pair_sort_workspace() bytes; returns the order array
// (inside ws) through *order.
size_t pair_sort_workspace(int B, int R, int block_rows_hint);
int launch_pair_sort(const int32_t* widx, const int32_t* bidx, int B, int K, int R, int block_rows_hint, void* ws,
                     hipStream_t st, const uint32_t** order);

// In-place exclusive scan of data[0..n) (one workgroup); the second half of the forward (bias, mix, clamp,
// product, psqt chains) over row sums saved[2, B, L1]; wpsqt == nullptr (with bpsqt): without the psqt chains (the
// caller has them from elsewhere).  nonfinite != nullptr: the gather has already written the
// output row of every position whose (us, them) is (1, 0) or (0, 1), and the psqt chains are done (wpsqt and bpsqt
// must be nullptr); only the other positions' rows are left, unless *nonfinite (device memory) says that some sum was
// not finite: then every row is redone.
int launch_scan(uint32_t* data, int n, hipStream_t st);
int launch_mix(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
               const int64_t* psqt_idx, const float* W, const float* bias, const float* saved, float max_act,
               float* l0, float* wpsqt, float* bpsqt, int B, int K, int R, int L1, int n_psqt, hipStream_t st,
               ActGrid act, VirtualTable vt, const uint32_t* nonfinite);

int double_fwd_blocked(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                       const int64_t* psqt_idx, const float* W, const float* bias, float max_act, float* l0,
                       float* wpsqt, float* bpsqt, float* saved, int B, int K, int R, int L1, int n_psqt, void* ws,
                       hipStream_t st, ActGrid act);

}  // namespace nnueft_blocked

namespace nnueft_tile {

// Forward gather out of LDS-resident tiles of the table (one 768-row block x 32 columns).  fits(): whether
// the shape and the device can take it; workspace(): bytes it needs (at least the L2-blocked path's).
constexpr int kBlockRows = 768;   // rows of a table block (a king bucket of HalfKAv2_hm); also the virtual rows
bool fits(const nnueft_dev::DeviceInfo& d, int B, int K, int R, int L1);
size_t workspace(int B, int R);
int double_fwd_tile(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                    const int64_t* psqt_idx, const float* W, const float* bias, float max_act, float* l0,
                    float* wpsqt, float* bpsqt, float* saved, int B, int K, int R, int L1, int n_psqt, void* ws,
                    hipStream_t st, ActGrid act, VirtualTable vt);
// The same gather over the quantized table W16 [R, L1] int16 (wrapping 16-bit sums), finishing the quantized forward
// itself: a tile is 32 column pairs (j, j + L1/2), and a pair's sums leave the kernel as
// out_u8[b, half * L1/2 + j] = (clip(sum_j + b16_j) * clip(sum_{j+L1/2} + b16_{j+L1/2})) >> shift, half 0 for the list of the
// side to move (stm[b] != 0: the black list).  No sums pass through memory.  The sort in front of the gather also
// writes psqt_out[b] = (sum of psqt32[row, psqt_idx[b]] over the mover's list - the same over the other list) / 2.
// block_rows <= 768: the rows of a table block (704 for an exported net).  workspace_int16(): bytes of its scratch (0: the shape cannot take it).
bool fits_int16(const nnueft_dev::DeviceInfo& d, int B, int K, int R, int L1, int block_rows);
size_t workspace_int16(int B, int R, int block_rows);
int int16_fused_tile(const int32_t* widx, const int32_t* bidx, const uint8_t* stm, const int16_t* W16, const int16_t* b16,
                     const int32_t* psqt32, const int64_t* psqt_idx, uint8_t* out_u8, int32_t* psqt_out, int B, int K, int R,
                     int L1, int n_psqt, int clip_max, int shift, int block_rows, void* ws, hipStream_t st);
}  // namespace nnueft_tile

namespace nnueft_chain {

// The strict-order backward out of LDS tiles (bwd_chain.hip).  shape_workspace(): bytes of its tables, 0 where the
// shape cannot take it; device_ok(): whether the device can; sort(): the tables of a batch's index lists; reduce():
// the weight gradient from the upstream rows G[n_persp * B, g_pitch] (every element of gW written).  A batch whose
// lists it cannot take (rows of two blocks, or a row twice, in one list) sets *fallback_flag(): reduce() then does
// nothing, and the caller's other path has to run; the flag is valid once sort() has run on the stream.
size_t shape_workspace(int B, int K, int R, int out_cols, int n_persp);
bool device_ok(const nnueft_dev::DeviceInfo& d);
const uint32_t* fallback_flag(const void* ws, int B, int R, int n_persp);
// split_word / tag_word: two words outside `ws` that every sort of these lists writes (the threshold the lists were
// sorted for, and what the tables in `ws` were made for): sort() sets them, reduce() does nothing unless the tag is
// the one of its own arguments, so that it never reads tables that were not made (lists sorted for another
// threshold, whose block may not even hold room for `ws`).
int sort(const int32_t* widx, const int32_t* bidx, int B, int K, int R, int n_persp, void* ws, uint32_t* split_word,
         uint32_t* tag_word, hipStream_t st);
int reduce(const float* G, int g_pitch, float* gW, int B, int R, int out_cols, int n_persp, void* ws,
           const uint32_t* tag_word, hipStream_t st);

}  // namespace nnueft_chain

namespace nnueft_det {

// Upstream rows G[2, B, g_pitch] (L1 + n_psqt floats of a row used) of the two sparse-linear outputs and the
// bias partial sums partial[ceil(B / NNUEFT_BIAS_TILE), L1 + n_psqt]; then the chain over the partial sums.
int launch_bwd_rows(const float* us, const float* them, const int64_t* psqt_idx, const float* bias, float max_act,
                    const float* grad_l0, const float* grad_wpsqt, const float* grad_bpsqt, const float* saved,
                    float* G, int g_pitch, float* partial, int B, int L1, int n_psqt, hipStream_t st);
// partial[tile, c] = chain over the tile's positions of gout[b, c] (the bias partial sums of the one-list backward)
int launch_tile_colsum(const float* gout, float* partial, int B, int out_cols, hipStream_t st);
int launch_bias_final(const float* partial, float* gbias, int B, int out_cols, uint32_t* sched, hipStream_t st);

}  // namespace nnueft_det
