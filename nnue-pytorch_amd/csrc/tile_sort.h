// What the LDS-tiled kernels share: the sort of the (position, perspective) pairs by table block and list
// length, its workspace layout and its tables (fwd_tile.hip makes them; the forward gather there and the
// backward scatter in bwd_tile.hip read them).
#pragma once

#include "internal.h"

namespace nnueft_tile {

using nnueft_blocked::kXcd;

constexpr int kRows = 768;                         // rows of a table block = rows of a tile
constexpr int kTileCols = 32;                      // floats per tile row
constexpr int kRowBytes = kTileCols * 4;
constexpr int kTileBytes = (kRows + 1) * kRowBytes;   // + one row of zeros for the padding slots
constexpr int kSlots = 32;                         // list slots the 16-bit lists hold
constexpr int kLenBins = kSlots + 1;
constexpr int kLenBins8 = kLenBins * kSlots;       // entries a chunk can get beyond its even share of a block
constexpr int kChunk = 1536;                       // most pairs whose lists a workgroup holds
constexpr int kListCap = 27648;                    // most list entries (padded, 16 bits each) it holds
constexpr int kListSlack = kLenBins8;              // see chunks_of()
constexpr int kMaxBlocks = 62;
constexpr int kMaxChunks = 1024;                   // chunks whose places a workgroup of the sort keeps in LDS
constexpr int kBins = 2048;                        // LDS counters of the sort (kMaxBlocks * kLenBins + 1 used at most)
static_assert(kMaxBlocks * kLenBins + 1 <= kBins, "sort bins");
static_assert(kRows == kBlockRows, "rows of a table block");
constexpr uint32_t kForeign = 63;                  // count field of a list that leaves its block
// loff[]: a list's place among its chunk's lists in units of 8 entries (12 bits), and, when the sort was given the
// sides to move, two facts about the pair for the forward that writes the output rows itself
constexpr uint32_t kLoffMask = 0xfffu;
constexpr uint32_t kLoffSecondHalf = 0x4000u;      // the pair's sums make the second half of the position's output row
constexpr uint32_t kLoffOwnRow = 0x8000u;          // (us, them) is (1, 0) or (0, 1): the pair's sums alone make that half
static_assert(kListCap / 8 <= (int)kLoffMask, "list offsets");
constexpr int kSchedNonFinite = kXcd * 32 + 1;     // word of Sorted::sched: a gather met a sum that is not finite
#ifndef NNUEFT_TILE_NT
#define NNUEFT_TILE_NT 1024
#endif
constexpr int kAccThreads = NNUEFT_TILE_NT;
constexpr int kAccThreadsVirtual = 768;
constexpr int kSortThreads = 256;
// tile, lists, pair ids, list offsets, two counters, the bias of two tiles
constexpr int kLdsBytes = kTileBytes + (kListCap + 32) * 2 + kChunk * 4 + kChunk * 2 + 16 + 2 * kRowBytes;
static_assert(kLdsBytes <= 160 * 1024, "LDS of a CU");

typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

// A chunk of a block's pairs: pairs [start, start + count) of pidcnt / loff, their lists in
// lists[pool8 * 8 .. + n8 * 8) (every list padded to a multiple of 8 entries).
struct Chunk {
    int block, start, count, pool8, n8, pad0, pad1, pad2;
};

// entries of a list of `cnt` slots in the pool
__host__ __device__ __forceinline__ int padded(int cnt) { return (cnt + 7) & ~7; }

// A table block as the backward scatter walks it: its pairs are slots [base, base + nc * len) of pidcnt / loff,
// nc chunks of len slots of which chunk j holds ranks_of_chunk(nb, j, nc) pairs; the lists of chunk j begin at
// cpool8[chunk0 + j] (units of 8 entries).
struct BlockRec {
    int base, nb, nc, len, chunk0, pad0, pad1, pad2;
};

// how many of the ranks 0 .. x - 1 go to chunk j of nc
__host__ __device__ __forceinline__ int ranks_of_chunk(int x, int j, int nc) { return (x - j + nc - 1) / nc; }

// What the sort and the kernels that read its tables share in the workspace.
struct Layout {
    size_t hist, total, lists, pidcnt, loff, chunks, sched, brec, cpool8, border, end;
    int npairs;       // index lists sorted: 2 B (both perspectives) or B (one)
    int ngroups, nblocks, nbins, max_chunks, nslots;
    int block_rows;   // rows of a table block (kRows, or fewer: the tile then keeps rows to spare)
};

// npairs index lists: pair p < B is widx[p], pair p >= B is bidx[p - B].
bool layout(int npairs, int R, Layout* L, int block_rows = kRows);

// The tables of the sort inside a workspace laid out by layout().
struct Sorted {
    const uint16_t* lists;
    const uint32_t* pidcnt;
    const uint16_t* loff;
    const Chunk* chunks;
    const BlockRec* brec;
    const uint32_t* cpool8;
    const uint32_t* border;   // table blocks, most pairs first
    uint32_t* sched;          // kXcd unit counters 32 words apart (zero after the sort), [kXcd * 32] = chunks in all,
                              // [kSchedNonFinite] = 0 after the sort
};

// What the sort can do on its way for the forward that calls it (all of it optional; L.npairs == 2 B):
//   us, them (both or neither; f32 [B]): the sides to move, for the kLoff* bits of loff[]; without them those bits are 0;
//   wpsqt, bpsqt (f32 [B], with psqt_idx, W [R, L1 + n_psqt], bias): every list's psqt chain, W[row, L1 + psqt_idx] over
//   the list's valid rows in slot order + bias[L1 + psqt_idx] (0 for a psqt_idx outside [0, n_psqt)).
//   psqt_out (int32 [B], with psqt_idx, psqt32 [R, n_psqt] int32, stm u8 [B]): the quantized forward's psqt difference,
//   (sum of psqt32[row, psqt_idx] over the mover's list - the same over the other list) / 2 with wrapping sums (the
//   thread that has a position's white list fetches its black list too).
struct SortExtras {
    const float* us;
    const float* them;
    const int64_t* psqt_idx;
    const float* W;
    const float* bias;
    float* wpsqt;
    float* bpsqt;
    int L1, n_psqt;
    const int32_t* psqt32;
    const uint8_t* stm;
    int32_t* psqt_out;
};

// k_tl_hist, k_tl_binscan, k_tl_lists on `st`.
int launch_sort(const int32_t* widx, const int32_t* bidx, int B, int K, int R, const Layout& L, void* ws, hipStream_t st,
                Sorted* out, SortExtras ex = SortExtras{});

// One wave per bin: hist[bin][0 .. ngroups) becomes its exclusive prefix, total[bin] the sum.
int launch_binscan(uint32_t* hist, uint32_t* total, int nbins, int ngroups, hipStream_t st);

static inline size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace nnueft_tile


