// Backward, strict summation order, LDS-tiled: the forward's gather out of LDS tiles turned around.
//
// All indices of one list name rows of one 768-row block of the table.  A workgroup keeps, for a chunk of a
// block's pairs of one perspective (up to 624 pairs in ascending position order), a tile of their upstream rows in
// LDS (624 rows x 16 columns, 40 KB) together with the inverted lists of the chunk (for every table row of the
// block, the pairs of the chunk that name it, in ascending position order, as 16-bit places inside the chunk),
// and sums every row's chain out of LDS, the adds in list order.  The weight gradient of a row is its white chain
// plus its black chain, each from +0 in ascending position order: the order of the reference's CPU path
// (sparse_linear_functions.py:43-50 run once per perspective, the two gradients added).  The white sums wait in
// LDS (768 rows x 16 columns) for the black ones.  The upstream rows are read once from memory, the gradient is
// written once.
//
// The chains of a chunk are sorted by length and dealt to tasks:
//   a chain that every pair of the chunk is part of (the own king's row)  the tile's rows from first to last, no
//                                                                        list, 16 lanes, a lane a column
//   4 long chains (more than 64 slots)                                   16 lanes each, a lane a column
//   16 chains                                                            4 lanes each, a lane four columns
// Every list of a task is padded to the task's longest (the padding names a row of zeros), so the loops over a
// task's slots have no per-lane condition, and every LDS read is issued unconditionally, so that the waits count
// instructions and never drain the queue.
//
//   k_cs_hist     one pair per thread: key (block, perspective) counted per workgroup; lists that leave their block
//                 are counted apart
//   k_tl_binscan  per key, the counts of the workgroups become their exclusive prefix (fwd_tile.hip)
//   k_cs_place    pairs to their places, a key's pairs in ascending pair order; the chunk table, the blocks by
//                 pairs, the counters
//   k_cs_expand   one workgroup per chunk: a bit per (row, pair) set with LDS atomics (ascending order for free),
//                 rows ranked by chain length (by counting), tasks formed, lists written
//   k_chain_tile  persistent workgroups, one per CU: units of (table block, column tile) dealt to the workgroups of
//                 an XCD round by round; a step is one chunk of a unit; while a step runs, the tile, the lists and
//                 the facts of the next step are on their way into registers, the pair ids of the one after it and
//                 the chunk record of the one after that are being read.  A step lasts as long as its longest
//                 chain (the own king's row: as many dependent adds as the chunk has pairs), so the waves that sum
//                 the long chains are fixed (wave i takes long task i), ask for the next step's data first, while
//                 the address units are idle, and run at raised priority; the other waves do a task before they ask
//
// A batch with a list that names rows of more than one block, or the same row twice (the interface allows both),
// is left to the sort and the segmented reduction of bwd_det.hip: the kernels here then do nothing, and a flag in
// the workspace tells those to run.
#include <atomic>
#include <type_traits>

#include "tile_sort.h"

namespace nnueft_chain {

using nnueft_tile::f4;
using nnueft_tile::u4;
using nnueft_tile::kXcd;
using nnueft_tile::up256;

constexpr int kRows = 768;                 // rows of a table block = chains of a chunk
constexpr int kCols = 16;                  // columns of a tile
constexpr int kRowB = kCols * 4;           // bytes of a tile row
constexpr int kCP = 624;                   // most pairs of a chunk (a multiple of 16)
constexpr int kSlots = 32;
constexpr int kTaskChains = 16;            // chains of a short task: 4 lanes each
constexpr int kLongTasks = 8;              // most tasks of long chains (a lane a column): dense ones and 4-chain ones
constexpr int kDenseMax = 4;               // most dense chains (each a task of its own)
constexpr int kLongMin = 64;               // a chain of more slots than this is long
constexpr int kMinCols = 256;              // narrower rows are left to the segmented reduction
constexpr int kMaskWords = (kCP + 31) / 32;
// Padded list entries of a chunk at most: chains sorted by length, so what the tasks' longest chains have more
// than their shortest adds up to no more than the longest chain of all (<= kCP) per lane group; + rounding to
// blocks of 4 (short tasks) or 8 (long ones).
constexpr int kEntCap = kCP * kSlots + kTaskChains * kCP + kRows * 3 + kLongTasks * 4 * 8;
constexpr int kTileB = (kCP + 1) * kRowB;  // + the row of zeros the padding names
// A chunk's facts: word 0 = long tasks | all tasks << 16; words 1 .. 63 one per task (place of its lists in 8-byte
// units | blocks << 20, bit 31: dense); from byte 256 the row of every chain in task order (a long task has 4 chains,
// the others 16; chains that fill up a task name row 768, which exists in LDS and nowhere else).
constexpr int kMaxTasks = 63;
constexpr int kSortWaves = kRows / 64;             // the list maker sorts a block's rows, a row a thread
constexpr int kCntBins = 640;                      // chain lengths 0 .. kCP
static_assert(kCntBins > kCP && kCntBins % 2 == 0, "a counter per chain length");

constexpr int kRowSlots = 832;
constexpr int kMdB = 256 + kRowSlots * 2;
constexpr int kMdWords = kMdB / 4;
constexpr int kEntGuard = 1024;            // bytes behind the lists that always name the row of zeros
constexpr int kLdsSum = kTileB;
constexpr int kLdsEnt = kLdsSum + (kRows + 1) * kRowB;
constexpr int kLdsMd = kLdsEnt + kEntCap * 2 + kEntGuard;
constexpr int kLdsCtr = kLdsMd + kMdB;
constexpr int kLdsUb = kLdsCtr + 32;
constexpr int kLds = kLdsUb + nnueft_tile::kMaxBlocks * 16;
constexpr int kThreads = 1024;
constexpr int kSortThreads = 256;
constexpr int kMaxKeys = 2 * nnueft_tile::kMaxBlocks;
static_assert(kCP % 16 == 0, "a dense chain is read in blocks of 16 rows");
static_assert(kMdB % 16 == 0 && kEntCap % 8 == 0, "16-byte copies");
static_assert(kEntCap * 2 / 16 <= 4 * kThreads, "lists: four 16-byte pieces a thread");
static_assert(kLds <= 160 * 1024, "LDS of a CU");
static_assert(kLongTasks + (kRows + kTaskChains - 1) / kTaskChains <= kMaxTasks, "tasks of a chunk");

// Words of the block the sort leaves for the kernels behind it.
constexpr int kFlagWord = 0;               // not zero: the batch is left to the sort and reduction of bwd_det.hip
constexpr int kChunksWord = 1;             // chunks in all
constexpr int kSchedWords = 32;

// A chunk of a block's pairs of one perspective: pairs bpairs[start .. start + count), its lists
// ent[ent4 * 4 .. + n4 * 4), its facts md[chunk].
struct RChunk {
    int block, start, count, ent4, n4, flags, persp, pad1;   // flags: 1 = first chunk of its perspective, 2 = last
};

// The chunks of a block: chunk0 .. + nw - 1 white, then nb black.  The kernel reads the table in the order it walks
// the blocks: most pairs first.
struct BlockChunks {
    int chunk0, nw, nb, blk;
};

struct ChainLayout {
    size_t hist, total, bpairs, chunks, ublocks, md, ent, sched, end;
    int npairs, n_persp, ngroups, nblocks, nkeys, max_chunks;
};

bool chain_layout(int B, int n_persp, int R, ChainLayout* L) {
    if (B <= 0 || R <= 0 || (n_persp != 1 && n_persp != 2) || (long long)n_persp * B >= (1ll << 26)) return false;
    L->npairs = n_persp * B;
    L->n_persp = n_persp;
    L->nblocks = (R + kRows - 1) / kRows;
    if (L->nblocks > nnueft_tile::kMaxBlocks) return false;
    L->nkeys = 2 * L->nblocks;
    L->ngroups = (L->npairs + kSortThreads - 1) / kSortThreads;
    L->max_chunks = L->nkeys + (L->npairs + kCP - 1) / kCP;
    size_t off = 0;
    L->hist = off;
    off += up256((size_t)(L->nkeys + 1) * L->ngroups * sizeof(uint32_t));
    L->total = off;
    off += up256((size_t)(L->nkeys + 1) * sizeof(uint32_t));
    L->bpairs = off;
    off += up256((size_t)(L->npairs + 64) * sizeof(uint32_t));
    L->chunks = off;
    off += up256((size_t)L->max_chunks * sizeof(RChunk));
    L->ublocks = off;
    off += up256((size_t)nnueft_tile::kMaxBlocks * sizeof(BlockChunks));
    L->md = off;
    off += up256((size_t)L->max_chunks * kMdB);
    L->ent = off;
    off += up256((size_t)L->max_chunks * kEntCap * sizeof(uint16_t) + 256);
    L->sched = off;
    off += up256((size_t)kSchedWords * sizeof(uint32_t));
    L->end = off;
    return true;
}

// What tables were made for: the sizes that lay them out (never 0).
static inline uint32_t table_tag(int B, int R, int n_persp) {
    uint32_t h = 0x9e3779b9u;
    for (uint32_t v : {(uint32_t)B, (uint32_t)R, (uint32_t)n_persp}) h = (h ^ v) * 0x85ebca6bu + 0xc2b2ae35u;
    return h | 1u;
}

// a value every lane holds alike, moved to a scalar register
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }

// A pair's list in registers: kSlots entries, -1 beyond K; 16-byte loads when `vec` (K a multiple of 4, the lists at
// 16-byte boundaries), so that the list is one or two trips to memory and not K.
struct ListRegs {
    int v[kSlots];
};

__device__ __forceinline__ ListRegs load_list(const int32_t* __restrict__ ix, int K, bool vec) {
    ListRegs l;
    if (vec) {
        const int4* p = reinterpret_cast<const int4*>(ix);
#pragma unroll
        for (int q = 0; q < kSlots / 4; ++q) {
            const int4 t = 4 * q < K ? p[q] : make_int4(-1, -1, -1, -1);
            l.v[4 * q] = t.x; l.v[4 * q + 1] = t.y; l.v[4 * q + 2] = t.z; l.v[4 * q + 3] = t.w;
        }
    } else {
#pragma unroll
        for (int k = 0; k < kSlots; ++k) l.v[k] = k < K ? ix[k] : -1;
    }
    return l;
}

// The key of a pair's list: (block of its first valid entry) * 2 + perspective; nkeys for a list that names rows of
// more than one block.  A list without a valid entry belongs to block 0 (it adds nothing anywhere).
__device__ __forceinline__ int list_key(const ListRegs& l, int R, int persp, int nkeys) {
    int block = -1;
    bool foreign = false;
#pragma unroll
    for (int k = 0; k < kSlots; ++k) {
        const int r = l.v[k];
        if (r >= 0 && r < R) {
            // r / 768 for r below 2^32 / 768, without the division
            const int b = (int)__umulhi((uint32_t)r, 0xffffffffu / (uint32_t)kRows + 1u);
            if (block < 0) block = b;
            foreign |= b != block;
        }
    }
    if (foreign) return nkeys;
    return (block < 0 ? 0 : block) * 2 + persp;
}

__device__ __forceinline__ const int32_t* pair_list(const int32_t* __restrict__ widx, const int32_t* __restrict__ bidx,
                                                    int pair, int B, int K, int* persp) {
    const int p = pair >= B;
    *persp = p;
    return (p ? bidx : widx) + (size_t)(pair - p * B) * K;
}

__global__ __launch_bounds__(kSortThreads) void k_cs_hist(const int32_t* __restrict__ widx,
                                                          const int32_t* __restrict__ bidx,
                                                          uint32_t* __restrict__ hist, int npairs, int B, int K, int R,
                                                          int nkeys, int vec) {
    __shared__ uint32_t bins[kMaxKeys + 1];
    const int tid = threadIdx.x;
    const int n = blockIdx.x * kSortThreads + tid;
    for (int i = tid; i <= nkeys; i += kSortThreads) bins[i] = 0;
    __syncthreads();
    if (n < npairs) {
        int persp;
        const int32_t* ix = pair_list(widx, bidx, n, B, K, &persp);
        atomicAdd(&bins[list_key(load_list(ix, K, vec), R, persp, nkeys)], 1u);
    }
    __syncthreads();
    for (int i = tid; i <= nkeys; i += kSortThreads) hist[(size_t)i * gridDim.x + blockIdx.x] = bins[i];
}

// chunks of a key with n pairs, and the pairs of each but the last
__device__ __forceinline__ int chunks_of(int n) { return max(1, (n + kCP - 1) / kCP); }

__global__ __launch_bounds__(kSortThreads) void k_cs_place(const int32_t* __restrict__ widx,
                                                           const int32_t* __restrict__ bidx,
                                                           const uint32_t* __restrict__ hist,
                                                           const uint32_t* __restrict__ total,
                                                           uint32_t* __restrict__ bpairs, RChunk* __restrict__ chunks,
                                                           BlockChunks* __restrict__ ublocks,
                                                           uint32_t* __restrict__ sched, uint32_t* __restrict__ split_word,
                                                           uint32_t* __restrict__ tag_word, uint32_t tag, int npairs,
                                                           int n_persp, int B, int K, int R, int nkeys, int nblocks,
                                                           int vec) {
    __shared__ uint32_t keybase[kMaxKeys + 1];
    __shared__ uint32_t wcnt[kSortThreads / 64][kMaxKeys];
    __shared__ uint32_t chunk0[kMaxKeys + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = blockIdx.x * kSortThreads + tid;
    const int ngroups = gridDim.x;
    for (int i = tid; i < (kSortThreads / 64) * kMaxKeys; i += kSortThreads) (&wcnt[0][0])[i] = 0;
    if (blockIdx.x == 0 && tid < 64) bpairs[npairs + tid] = 0;   // a chunk without pairs reads one id at its start
    __shared__ uint32_t tot[kMaxKeys + 1];
    for (int i = tid; i <= nkeys; i += kSortThreads) tot[i] = total[i];
    __syncthreads();
    if (tid < 64) {
        // where a key's pairs and chunks begin: two keys a lane, a scan over the wave
        static_assert(kMaxKeys <= 128, "two keys a lane");
        uint32_t np[2], nc[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = 2 * tid + h;
            np[h] = k < nkeys ? tot[k] : 0u;
            // a single list of the batch (n_persp == 1) has no black chunks at all
            nc[h] = k < nkeys && !(n_persp == 1 && (k & 1)) ? (uint32_t)chunks_of((int)tot[k]) : 0u;
        }
        uint32_t ip = np[0] + np[1], ic = nc[0] + nc[1];
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t tp = __shfl_up(ip, off), tc = __shfl_up(ic, off);
            if (lane >= off) {
                ip += tp;
                ic += tc;
            }
        }
        uint32_t run = ip - np[0] - np[1], cr = ic - nc[0] - nc[1];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = 2 * tid + h;
            if (k <= nkeys) {
                keybase[k] = run;
                chunk0[k] = cr;
            }
            run += np[h];
            cr += nc[h];
        }
    }
    __syncthreads();
    int key = nkeys;
    if (n < npairs) {
        int persp;
        const int32_t* ix = pair_list(widx, bidx, n, B, K, &persp);
        key = list_key(load_list(ix, K, vec), R, persp, nkeys);
    }
    // a pair's place among the pairs of its key in this workgroup: those of the waves in front, then those of the
    // lanes in front
    const bool act = key < nkeys;
    uint32_t rank = 0;
    unsigned long long todo = __ballot(act);
    while (todo) {
        const int leader = __ffsll((long long)todo) - 1;
        const int k = __builtin_amdgcn_readlane(key, leader);
        const unsigned long long m = __ballot(act && key == k);
        if (act && key == k) rank = (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
        if (lane == leader) wcnt[wave][k] = (uint32_t)__popcll(m);
        todo &= ~m;
    }
    __syncthreads();
    if (act) {
        uint32_t before = 0;
        for (int w = 0; w < wave; ++w) before += wcnt[w][key];
        bpairs[keybase[key] + hist[(size_t)key * ngroups + blockIdx.x] + before + rank] = (uint32_t)n;
    }
    if (blockIdx.x != 0) return;
    // the first workgroup also writes the tables of the batch, and what they were made for
    if (tid == 0) {
        *split_word = 0;   // the strict order
        *tag_word = tag;
    }
    for (int i = tid; i < kSchedWords; i += kSortThreads)
        sched[i] = i == kFlagWord ? (tot[nkeys] != 0 ? 1u : 0u) : i == kChunksWord ? chunk0[nkeys] : 0u;
    for (int k = tid; k < nkeys; k += kSortThreads) {
        if (n_persp == 1 && (k & 1)) continue;
        const int nk = (int)tot[k];
        const int nc = chunks_of(nk);
        const int ln = (nk + nc - 1) / nc;
        for (int j = 0; j < nc; ++j) {
            const int c = (int)chunk0[k] + j;
            RChunk rc;
            rc.block = k >> 1;
            rc.start = (int)keybase[k] + j * ln;
            rc.count = max(0, min(ln, nk - j * ln));
            rc.ent4 = c * (kEntCap / 4);
            rc.n4 = 0;
            rc.flags = (j == 0 ? 1 : 0) | (j == nc - 1 ? 2 : 0);
            rc.persp = k & 1;
            rc.pad1 = 0;
            chunks[c] = rc;
        }
    }
    for (int b = tid; b < nblocks; b += kSortThreads) {
        const uint32_t mine = tot[2 * b] + tot[2 * b + 1];
        int r = 0;
        for (int o = 0; o < nblocks; ++o) {
            const uint32_t other = tot[2 * o] + tot[2 * o + 1];
            r += other > mine || (other == mine && o < b);
        }
        ublocks[r] = BlockChunks{(int)chunk0[2 * b], chunks_of((int)tot[2 * b]),
                                 n_persp == 1 ? 0 : chunks_of((int)tot[2 * b + 1]), b};
    }
}

// One workgroup per chunk: the inverted lists of the chunk, sorted into tasks.
__global__ __launch_bounds__(kThreads) void k_cs_expand(const int32_t* __restrict__ widx,
                                                        const int32_t* __restrict__ bidx,
                                                        const uint32_t* __restrict__ bpairs, RChunk* __restrict__ chunks,
                                                        uint32_t* __restrict__ md, uint16_t* __restrict__ ent,
                                                        uint32_t* __restrict__ sched, int B, int K, int R, int vec) {
    extern __shared__ float4 lds_raw[];
    uint32_t* mask = reinterpret_cast<uint32_t*>(lds_raw);             // [kRows][kMaskWords]
    uint32_t* keys = mask + kRows * kMaskWords;                        // [1024] sort keys, then the rows in slot order
    uint32_t* mdw = keys + 1024;                                       // [kMdWords]
    uint32_t* small = mdw + kMdWords;                                  // [8] counters
    uint16_t* lent = reinterpret_cast<uint16_t*>(small + 8);           // [kEntCap]
    uint16_t* whist = lent + kEntCap;   // [kSortWaves][kCntBins] rows of a wave by chain length (the sort)
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int c = blockIdx.x;
    if (sched[kFlagWord] != 0 || c >= (int)sched[kChunksWord]) return;
    const RChunk C = chunks[c];
    for (int i = tid; i < kRows * kMaskWords; i += kThreads) mask[i] = 0;
    if (tid < 8) small[tid] = 0;
    __syncthreads();
    // a bit per (row, pair): the pairs of a row in ascending order are its set bits from the lowest
    if (tid < C.count) {
        const int pair = (int)bpairs[C.start + tid];
        int persp;
        const ListRegs l = load_list(pair_list(widx, bidx, pair, B, K, &persp), K, vec);
        const int row0 = C.block * kRows;
        bool twice = false;
#pragma unroll
        for (int k = 0; k < kSlots; ++k) {
            const int r = l.v[k];
            if (r >= 0 && r < R) {
                const uint32_t bit = 1u << (tid & 31);
                twice |= (atomicOr(&mask[(r - row0) * kMaskWords + (tid >> 5)], bit) & bit) != 0;
            }
        }
        if (twice) atomicOr(&sched[kFlagWord], 2u);   // a row twice in one list: not for the bit map
    }
    __syncthreads();
    // Rows by chain length, longest first (ties: lower row first), by counting: a row's place = the rows with longer
    // chains + the rows of its length in the waves in front + those in front of it in its own wave.  (A bitonic sort
    // of the 1024 keys, 55 steps with a barrier each, took 10 of the kernel's 33 microseconds.)
    uint32_t cnt = 0;
    if (tid < kRows)
        for (int w = 0; w < kMaskWords; ++w) cnt += (uint32_t)__popc(mask[tid * kMaskWords + w]);
    for (int i = tid; i < kSortWaves * kCntBins / 2; i += kThreads) reinterpret_cast<uint32_t*>(whist)[i] = 0;
    __syncthreads();
    int before = 0;   // rows of the same length in front, in this wave
    if (tid < kRows) {
        static_assert(kRows % 64 == 0, "the waves that hold rows are full");
        u64 todo = ~(u64)0;
        const u64 lt = ((u64)1 << lane) - 1;
        while (todo) {
            const int l = __ffsll((long long)todo) - 1;
            const uint32_t k = (uint32_t)__builtin_amdgcn_readlane((int)cnt, l);
            const u64 m = __ballot(cnt == k);
            if (cnt == k) before = __popcll(m & lt);
            if (lane == l) whist[(tid >> 6) * kCntBins + k] = (uint16_t)__popcll(m);
            todo &= ~m;
        }
    }
    __syncthreads();
    {
        // thread i has length kCP - i: the rows longer than that (an exclusive scan over the threads), then the place
        // of every wave's rows of that length
        const int k = kCP - tid;
        uint32_t tot = 0;
        if (k >= 0)
            for (int w = 0; w < kSortWaves; ++w) tot += whist[w * kCntBins + k];
        uint32_t incl = tot;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t t = __shfl_up(incl, off);
            if (lane >= off) incl += t;
        }
        if (lane == 63) keys[tid >> 6] = incl;
        __syncthreads();
        uint32_t run = incl - tot;
        for (int w = 0; w < (tid >> 6); ++w) run += keys[w];
        __syncthreads();   // keys gets the sorted rows next
        if (k >= 0)
            for (int w = 0; w < kSortWaves; ++w) {
                const uint32_t h = whist[w * kCntBins + k];
                whist[w * kCntBins + k] = (uint16_t)run;
                run += h;
            }
    }
    __syncthreads();
    if (tid < kRows) keys[whist[(tid >> 6) * kCntBins + cnt] + before] = (cnt << 10) | (uint32_t)(1023 - tid);
    __syncthreads();
    uint32_t my_cnt = 0;
    int my_row = kRows;
    if (tid < kRows) {
        const uint32_t key = keys[tid];
        my_cnt = key >> 10;
        my_row = 1023 - (int)(key & 1023u);
        if ((int)my_cnt == C.count && (int)my_cnt > kLongMin) atomicAdd(&small[0], 1u);   // dense
        if ((int)my_cnt > kLongMin) atomicAdd(&small[1], 1u);                             // long, dense ones included
    }
    __syncthreads();
    const int nd = min((int)small[0], kDenseMax);
    const int nlt = min(kLongTasks - nd, ((int)small[1] - nd + 3) / 4);
    const int nl = nlt * 4;
    const int nshort = (kRows - nd - nl + kTaskChains - 1) / kTaskChains;
    const int ntasks = nd + nlt + nshort;
    // slot s of the sorted rows: dense (s < nd), else place s - nd among the long and short chains
    for (int i = tid; i < kMdWords; i += kThreads) mdw[i] = 0;
    __syncthreads();
    {
        uint16_t* rows = reinterpret_cast<uint16_t*>(mdw + 64);
        for (int i = tid; i < kRowSlots; i += kThreads) rows[i] = (uint16_t)kRows;
    }
    __syncthreads();
    if (tid < kRows) {
        uint16_t* rows = reinterpret_cast<uint16_t*>(mdw + 64);
        rows[tid < nd ? tid * 4 : nd * 4 + (tid - nd)] = (uint16_t)my_row;
        // the first chain of a task is its longest
        const int s = tid - nd;
        if (tid < nd) mdw[1 + tid] = 0x80000000u | ((uint32_t)((C.count + 15) / 16) << 20);
        else if (s < nl && (s & 3) == 0) mdw[1 + nd + (s >> 2)] = ((my_cnt + 7) / 8) << 20;
        else if (s >= nl && ((s - nl) & 15) == 0) mdw[1 + nd + nlt + ((s - nl) >> 4)] = ((my_cnt + 3) / 4) << 20;
    }
    __syncthreads();
    if (tid < 64) {
        // places of the tasks' lists, in 8-byte units: a long task's block is 4 chains x 8 entries, a short task's
        // 16 chains x 4 entries; lane t has task t (there are fewer than 64), and the last lane the total
        static_assert(kMaxTasks < 64, "a lane a task, and one to spare");
        const bool has_list = tid >= nd && tid < ntasks;
        uint32_t sz = 0;
        if (has_list) sz = ((mdw[1 + tid] >> 20) & 0x7ffu) * (tid < nd + nlt ? 8u : 16u);
        uint32_t incl = sz;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t t = __shfl_up(incl, off);
            if (lane >= off) incl += t;
        }
        if (has_list) mdw[1 + tid] |= incl - sz;
        if (tid == 63) {
            const uint32_t run = incl + (incl & 1u);
            small[2] = run;
            if (run * 4 > (uint32_t)kEntCap) atomicOr(&sched[kFlagWord], 4u);
        }
        if (tid == 0) mdw[0] = (uint32_t)(nd + nlt) | ((uint32_t)ntasks << 16);
    }
    __syncthreads();
    const int n4 = (int)small[2];
    if (n4 * 4 > kEntCap) return;
    for (int i = tid; i < n4 * 4; i += kThreads) lent[i] = (uint16_t)kCP;
    __syncthreads();
    // A thread a chain: its row's bit map word by word, the set bits to the row's list in order.  The slots are in
    // order of chain length, so the lanes of a wave have about as much to do.  (A thread per (row, word), which has
    // to find the set bits in front of its word and a third of whose words are empty, took 8.7 of the kernel's 19
    // microseconds.)
    if (tid < kRows && tid >= nd && my_cnt > 0) {
        const int s = tid - nd;
        const bool is_long = s < nl;
        const int task = is_long ? nd + (s >> 2) : nd + nlt + ((s - nl) >> 4);
        const uint32_t base = (mdw[1 + task] & 0xfffffu) * 4;
        // entry `pos` of the chain: a long task's block is 4 chains x 8 entries, a short task's 16 chains x 4 entries
        const uint32_t first = is_long ? base + (uint32_t)(s & 3) * 8 : base + (uint32_t)((s - nl) & 15) * 4;
        const int sh = is_long ? 3 : 2;
        const uint32_t stride = is_long ? 32u : 64u, in_block = is_long ? 7u : 3u;
        uint32_t pos = 0;
        for (int w = 0; w < kMaskWords; ++w) {
            uint32_t bits = mask[my_row * kMaskWords + w];
            while (bits) {
                const int bit = __ffs((int)bits) - 1;
                bits &= bits - 1;
                lent[first + (pos >> sh) * stride + (pos & in_block)] = (uint16_t)(w * 32 + bit);
                ++pos;
            }
        }
    }
    __syncthreads();
    {
        const u4* src = reinterpret_cast<const u4*>(lent);
        u4* dst = reinterpret_cast<u4*>(ent + (size_t)C.ent4 * 4);
        for (int i = tid; i < n4 / 2; i += kThreads) dst[i] = src[i];
        const u4* ms = reinterpret_cast<const u4*>(mdw);
        u4* md4 = reinterpret_cast<u4*>(md + (size_t)c * kMdWords);
        for (int i = tid; i < kMdB / 16; i += kThreads) md4[i] = ms[i];
        if (tid == 0) chunks[c].n4 = n4;
    }
}
constexpr int kExpandLds = (kRows * kMaskWords + 1024) * 4 + kMdB + 32 + kEntCap * 2 + kSortWaves * kCntBins * 2;
static_assert(kExpandLds <= 160 * 1024, "LDS of the list maker");

typedef __attribute__((address_space(3))) const f4 lds_f4;
typedef __attribute__((address_space(3))) const float lds_f;
__device__ __forceinline__ f4 lds_read16(uint32_t addr) { return *reinterpret_cast<lds_f4*>(addr); }

template <int HI>
__device__ __forceinline__ uint32_t row_addr(uint32_t w, uint32_t off) {
    uint32_t r;
    const uint32_t stride = kRowB;
    if (HI)
        asm("v_mad_u32_u16 %0, %1, %2, %3 op_sel:[1,0,0,0]" : "=v"(r) : "v"(w), "s"(stride), "v"(off));
    else
        asm("v_mad_u32_u16 %0, %1, %2, %3 op_sel:[0,0,0,0]" : "=v"(r) : "v"(w), "s"(stride), "v"(off));
    return r;
}

__device__ __forceinline__ RChunk uni_chunk(const RChunk& c) {
    return RChunk{uni(c.block), uni(c.start), uni(c.count), uni(c.ent4), uni(c.n4), uni(c.flags), uni(c.persp), 0};
}

// A step of a workgroup's walk: one chunk of one unit (table block x column tile).
struct Step {
    int unit, blk, c, cols, chunk0, nw, nb, ci, round;
};

// What a task does with its chains' sums.
constexpr int kKeep = 0;     // to LDS: the chain goes on in the next chunk, or waits for the other perspective
constexpr int kOutAdd = 1;   // the only black chunk of its block: gradient = white sum from LDS + the chain
constexpr int kOut = 2;      // the last chunk of a block without black chunks: gradient = the chain

__global__ __launch_bounds__(kThreads) void k_chain_tile(const float* __restrict__ G, int g_pitch,
                                                         const uint32_t* __restrict__ bpairs,
                                                         const RChunk* __restrict__ chunks,
                                                         const BlockChunks* __restrict__ ublocks,
                                                         const uint32_t* __restrict__ md,
                                                         const uint16_t* __restrict__ ent,
                                                         uint32_t* __restrict__ sched, float* __restrict__ gW,
                                                         int R, int out_cols, int main_tiles, int tpx, int tail_cols,
                                                         int nblocks, int gw_vec, const uint32_t* __restrict__ tag_word,
                                                         uint32_t tag) {
    extern __shared__ float4 lds_raw[];
    char* tb = reinterpret_cast<char*>(lds_raw);
    f4* lsum = reinterpret_cast<f4*>(tb + kLdsSum);
    uint2* lent = reinterpret_cast<uint2*>(tb + kLdsEnt);
    uint32_t* ltask = reinterpret_cast<uint32_t*>(tb + kLdsMd);
    uint16_t* lrows = reinterpret_cast<uint16_t*>(tb + kLdsMd + 256);
    uint32_t* ctr = reinterpret_cast<uint32_t*>(tb + kLdsCtr);   // [0] task counter
    int4* lub = reinterpret_cast<int4*>(tb + kLdsUb);
    // tables that were not made for these lists (sorted for another threshold) are not even there: nothing is read
    // before the tag says they are
    if (*tag_word != tag || sched[kFlagWord] != 0) return;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    constexpr int NT = kThreads;
    constexpr int NP = (kCP + 1) * (kRowB / 16);
    constexpr int IT = (NP + NT - 1) / NT;
    constexpr int LI = (kEntCap * 2 / 16 + NT - 1) / NT;
    constexpr int MD16 = kMdB / 16;
    const int x = blockIdx.x % kXcd;
    // the column tiles of this XCD; the tile of the last out_cols % 16 columns is dealt to the XCDs block by block
    const int my_tiles = max(0, min(tpx, main_tiles - x * tpx));
    const int nmain = nblocks * my_tiles;
    const int ntail = tail_cols && nblocks > x ? (nblocks - x + kXcd - 1) / kXcd : 0;
    const int nunits = nmain + ntail;
    const int g = lane >> 2, li = lane & 3;
    const uint32_t lane_off = (uint32_t)(uintptr_t)tb + li * 16;

    auto decode = [&](int u) {
        Step S{u, 0, 0, 0, 0, 1, 1, 0, 0};
        if (u >= nunits) return S;
        int r;
        if (u < nmain) {
            r = u / my_tiles;
            S.c = x * tpx + (u - r * my_tiles);
            S.cols = kCols;
        } else {
            r = (u - nmain) * kXcd + x;
            S.c = main_tiles;
            S.cols = tail_cols;
        }
        const int4 ub = lub[r];
        S.chunk0 = uni(ub.x);
        S.nw = uni(ub.y);
        S.nb = uni(ub.z);
        S.blk = uni(ub.w);
        return S;
    };

    // What a step asks for, for the step after it, at one place in the code (the registers are then the same ones
    // all the way round): the tile, the lists, the facts.  Every lane loads: a lane beyond the chunk's pairs or the
    // tile's columns reads a place that exists (dropped when the tile is written to LDS), so that no branch splits
    // the loads.
    f4 v[IT];
    u4 t[LI];
    u4 tm = u4{0u, 0u, 0u, 0u};
    uint32_t pr[IT];   // the pair ids of the rows a thread loads, read a step earlier
#pragma unroll
    for (int i = 0; i < IT; ++i) {
        v[i] = f4{0.f, 0.f, 0.f, 0.f};
        pr[i] = 0;
    }
#pragma unroll
    for (int i = 0; i < LI; ++i) t[i] = u4{0u, 0u, 0u, 0u};
    const int wave0 = uni(tid & ~63);   // the wave's first thread
#define NNUEFT_PREFETCH(C_, ci_, c_, cols_)                                                               \
    {                                                                                                     \
        const int col0_ = (c_) * kCols;                                                                   \
        const u4* src_ = reinterpret_cast<const u4*>(ent + (size_t)(C_).ent4 * 4);                        \
        const int n16_ = (C_).n4 >> 1;                                                                    \
        _Pragma("unroll") for (int i_ = 0; i_ < IT; ++i_) {                                               \
            const int p4_ = (tid + i_ * NT) & 3;                                                          \
            /* a wave whose rows all lie beyond the chunk's pairs loads nothing */                         \
            if ((wave0 + i_ * NT) >> 2 < (C_).count)                                                      \
                v[i_] = *reinterpret_cast<const f4*>(G + (size_t)pr[i_] * g_pitch + col0_ +               \
                                                     (p4_ * 4 < (cols_) ? p4_ * 4 : 0));                  \
        }                                                                                                 \
        _Pragma("unroll") for (int i_ = 0; i_ < LI; ++i_)                                                 \
            if (wave0 + i_ * NT < n16_) t[i_] = src_[min(tid + i_ * NT, n16_ - 1)];                       \
        if (wave0 < MD16) tm = reinterpret_cast<const u4*>(md + (size_t)(ci_) * kMdWords)[min(tid, MD16 - 1)]; \
    }
#define NNUEFT_PAIR_IDS(C_)                                                                               \
    {                                                                                                     \
        _Pragma("unroll") for (int i_ = 0; i_ < IT; ++i_) {                                               \
            const int row_ = (tid + i_ * NT) >> 2;                                                        \
            if ((wave0 + i_ * NT) >> 2 < (C_).count) pr[i_] = bpairs[(C_).start + min(row_, (C_).count - 1)]; \
        }                                                                                                 \
    }

    // One task: the chains of `task` summed, their sums kept or written out (MODE).  Returns the task to do next
    // (drawn at the start, so that the counter's answer is there at the end).
    auto do_task = [&](const int task, const int nlong, const int MODE, int c, bool first, int row0, int rows_here, int cols) {
        int nxt = 0;
        if (lane == 0) nxt = (int)atomicAdd(ctr, 1u);
        {
            const uint32_t tmd = ltask[1 + task];
            const int nb = uni((int)((tmd >> 20) & 0x7ffu));
            if (task < nlong) {
                // long chains: 16 lanes each, a lane a column
                const int g16 = lane >> 4, col = lane & 15;
                const int row = lrows[task * 4 + g16];
                const uint32_t off = (uint32_t)(uintptr_t)tb + col * 4;
                float* sp = reinterpret_cast<float*>(lsum) + row * kCols + col;
                float a = 0.f;
                if (!first) asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(a) : "v"((uint32_t)(uintptr_t)sp));
                // a long chain is what the step waits for: its wave goes first on its SIMD
                __builtin_amdgcn_s_setprio(3);
                if (tmd & 0x80000000u) {
                    // a chain that every pair of the chunk is part of: the tile's rows from the first to the last, no
                    // list; nb blocks of 16 rows (rows past the chunk's pairs are zero)
                    // Written instruction by instruction: two blocks of 16 rows are in flight, and a wait lets the
                    // older one land while the younger one stays out (the compiler's own placement of the waits
                    // drains the queue once per block, which is what this chain, the longest of the step, waits for).
                    // The waits are tied to the registers they make valid, so that no add moves in front of them.
                    typedef float f2 __attribute__((ext_vector_type(2)));
                    f2 qa[8], qb[8];
#define NNUEFT_RD2(dst_, addr_, o0_, o1_) \
    asm volatile("ds_read2_b32 %0, %1 offset0:" #o0_ " offset1:" #o1_ : "=v"(dst_) : "v"(addr_))
#define NNUEFT_ISSUE16(q_, addr_)                                                                          \
    NNUEFT_RD2(q_[0], addr_, 0, 16); NNUEFT_RD2(q_[1], addr_, 32, 48); NNUEFT_RD2(q_[2], addr_, 64, 80);    \
    NNUEFT_RD2(q_[3], addr_, 96, 112); NNUEFT_RD2(q_[4], addr_, 128, 144); NNUEFT_RD2(q_[5], addr_, 160, 176); \
    NNUEFT_RD2(q_[6], addr_, 192, 208); NNUEFT_RD2(q_[7], addr_, 224, 240);
#define NNUEFT_LANDED(n_, q_)                                                                              \
    asm volatile("s_waitcnt lgkmcnt(" #n_ ")"                                                             \
                 : "+v"(q_[0]), "+v"(q_[1]), "+v"(q_[2]), "+v"(q_[3]), "+v"(q_[4]), "+v"(q_[5]), "+v"(q_[6]), "+v"(q_[7]))
#define NNUEFT_ADD16(q_)                                                                                   \
    _Pragma("unroll") for (int h = 0; h < 8; ++h) {                                                        \
        a += q_[h].x;                                                                                      \
        a += q_[h].y;                                                                                      \
    }
                    static_assert(kRowB == 64, "offsets of the reads: 16 dwords a row");
                    uint32_t pa = off;
                    NNUEFT_ISSUE16(qa, pa)
                    for (int k = 0; k < nb; k += 2) {
                        const uint32_t pb = pa + 16 * kRowB;
                        NNUEFT_ISSUE16(qb, pb)
                        NNUEFT_LANDED(8, qa);
                        NNUEFT_ADD16(qa)
                        pa += 32 * kRowB;
                        NNUEFT_ISSUE16(qa, pa)   // past the last block: inside LDS, never added
                        NNUEFT_LANDED(8, qb);
                        if (k + 1 < nb) { NNUEFT_ADD16(qb) }
                    }
                    NNUEFT_LANDED(0, qa);
#undef NNUEFT_RD2
#undef NNUEFT_ISSUE16
#undef NNUEFT_LANDED
#undef NNUEFT_ADD16
                } else {
                    // 4 chains: block j of the task's lists is 4 chains x 8 entries
                    const u4* lp = reinterpret_cast<const u4*>(lent + (tmd & 0xfffffu)) + g16;
                    float ra[4], rb[4];
#define NNUEFT_ISSUE4(r_, w0_, w1_)                                \
    r_[0] = *reinterpret_cast<lds_f*>(row_addr<0>((w0_), off));    \
    r_[1] = *reinterpret_cast<lds_f*>(row_addr<1>((w0_), off));    \
    r_[2] = *reinterpret_cast<lds_f*>(row_addr<0>((w1_), off));    \
    r_[3] = *reinterpret_cast<lds_f*>(row_addr<1>((w1_), off));
                    u4 e = lp[0], en = lp[4];
                    NNUEFT_ISSUE4(ra, e.x, e.y)
                    for (int k = 0; k < nb; ++k) {
                        const u4 en2 = lp[(k + 2) * 4];
                        NNUEFT_ISSUE4(rb, e.z, e.w)
#pragma unroll
                        for (int h = 0; h < 4; ++h) a += ra[h];
                        NNUEFT_ISSUE4(ra, en.x, en.y)
#pragma unroll
                        for (int h = 0; h < 4; ++h) a += rb[h];
                        e = en;
                        en = en2;
                    }
#undef NNUEFT_ISSUE4
                }
                __builtin_amdgcn_s_setprio(0);
                if (MODE == kKeep) {
                    *sp = a;
                } else {
                    const float o = MODE == kOutAdd ? *sp + a : a;
                    if (row < rows_here && col < cols) gW[(size_t)(row0 + row) * out_cols + c * kCols + col] = o;
                }
            } else {
                // 16 chains, 4 lanes each: block j of the task's lists is 16 chains x 4 entries
                const int row = lrows[nlong * 4 + (task - nlong) * kTaskChains + g];
                // (left to the compiler: it issues the four reads of a block and adds as they land, which keeps
                // fewer reads of these chains in the queue in front of the long chain's; hand-written loops with
                // two and with four reads ahead made the step slower, 0.380 -> 0.394 and 0.427 ms)
                const uint2* lp = lent + (tmd & 0xfffffu) + g;
                f4* sp = lsum + row * (kRowB / 16) + li;
                f4 a = {0.f, 0.f, 0.f, 0.f};
                if (!first) a = *sp;
                f4 ra[2], rb[2];
#define NNUEFT_ISSUE(r_, w_)                               \
    r_[0] = lds_read16(row_addr<0>((w_), lane_off));       \
    r_[1] = lds_read16(row_addr<1>((w_), lane_off));
                uint2 e = lp[0], en = lp[kTaskChains];
                NNUEFT_ISSUE(ra, e.x)
                for (int k = 0; k < nb; ++k) {
                    const uint2 en2 = lp[(k + 2) * kTaskChains];
                    NNUEFT_ISSUE(rb, e.y)
                    a += ra[0];
                    a += ra[1];
                    NNUEFT_ISSUE(ra, en.x)
                    a += rb[0];
                    a += rb[1];
                    e = en;
                    en = en2;
                }
#undef NNUEFT_ISSUE
                if (MODE == kKeep) {
                    *sp = a;
                } else {
                    const f4 o = MODE == kOutAdd ? *sp + a : a;
                    if (row < rows_here && li * 4 < cols) {
                        float* dst = gW + (size_t)(row0 + row) * out_cols + c * kCols + li * 4;
                        if (gw_vec) {
                            __builtin_nontemporal_store(o, reinterpret_cast<f4*>(dst));
                        } else {
                            dst[0] = o.x;
                            if (li * 4 + 1 < cols) dst[1] = o.y;
                            if (li * 4 + 2 < cols) dst[2] = o.z;
                            if (li * 4 + 3 < cols) dst[3] = o.w;
                        }
                    }
                }
            }
        }
        return uni(nxt);
    };
    auto draw = [&]() {
        int t = 0;
        if (lane == 0) t = (int)atomicAdd(ctr, 1u);
        return uni(t);
    };

    // The step after S.  The units of an XCD are dealt to its workgroups round by round, forth and back (blocks with
    // the most pairs come first, so every workgroup gets about the same mix and the cheapest units come last): no
    // counter in memory, whose answer a wave has to wait for behind the loads it has just issued (with one, and with
    // a ticket drawn ahead and read a step later, the reduction at L1 = 3072, B = 16384 took 0.353 and 0.332 ms
    // against 0.321; on game-like lists 0.550 and 0.559 against 0.526; only at L1 = 1024, B = 8192 on game-like
    // lists, where a workgroup gets 8 units of very unequal blocks, the counter was ahead: 0.159 against 0.186 ms).
    const int wg = blockIdx.x / kXcd, nwg = gridDim.x / kXcd;
    auto unit_of = [&](int round) { return round * nwg + ((round & 1) ? nwg - 1 - wg : wg); };
    auto next_step = [&](const Step& S) {
        if (S.unit >= nunits) return S;
        Step N = S;
        N.ci = S.ci + 1;
        if (N.ci == S.nw + S.nb) {
            N = decode(unit_of(S.round + 1));
            N.round = S.round + 1;
        }
        return N;
    };
    for (int i = tid; i < nblocks; i += NT) lub[i] = reinterpret_cast<const int4*>(ublocks)[i];
    {
        // list entries are read a little past a task's last block and used as row numbers: whatever lies there
        // must name a row of the tile
        constexpr uint32_t zz = (uint32_t)kCP | ((uint32_t)kCP << 16);
        for (int i = tid; i < (kEntCap * 2 + kEntGuard) / 16; i += NT) reinterpret_cast<u4*>(lent)[i] = u4{zz, zz, zz, zz};
    }
    __syncthreads();
    // D1: the step whose data is in (or on its way into) the registers; D2: its successor, whose pair ids are being
    // read; D3: the one after, whose chunk record is being read
    Step D1 = decode(unit_of(0));
    RChunk C1{}, C2{}, c3raw{};
    Step D2 = next_step(D1);
    Step D3 = next_step(D2);
    if (D1.unit < nunits) {
        C1 = uni_chunk(chunks[D1.chunk0 + D1.ci]);
        NNUEFT_PAIR_IDS(C1)
        NNUEFT_PREFETCH(C1, D1.chunk0 + D1.ci, D1.c, D1.cols)
    }
    if (D2.unit < nunits) {
        C2 = uni_chunk(chunks[D2.chunk0 + D2.ci]);
        NNUEFT_PAIR_IDS(C2)
    }
    if (D3.unit < nunits) c3raw = chunks[D3.chunk0 + D3.ci];
    while (D1.unit < nunits) {
        const Step cur = D1;
        const RChunk C = C1;
        const int row0 = cur.blk * kRows;
        const int rows_here = min(kRows, R - row0);
        __syncthreads();   // the tasks of the step in front are done with LDS
        if (cur.ci == cur.nw && cur.nb > 1) {
            // the white sums make room for the black chain's: they wait in the gradient itself
            for (int f = tid; f < rows_here * kCols; f += NT) {
                const int col = f & (kCols - 1);
                if (col < cur.cols)
                    gW[(size_t)(row0 + (f >> 4)) * out_cols + cur.c * kCols + col] = reinterpret_cast<float*>(lsum)[f];
            }
        }
        {
            const int n16 = C.n4 >> 1;
#pragma unroll
            for (int i = 0; i < LI; ++i)
                if (tid + i * NT < n16) reinterpret_cast<u4*>(lent)[tid + i * NT] = t[i];
            if (tid < MD16) reinterpret_cast<u4*>(ltask)[tid] = tm;
#pragma unroll
            for (int i = 0; i < IT; ++i) {
                const int f = tid + i * NT;
                const bool live = (f >> 2) < C.count && (f & 3) * 4 < cur.cols;
                if (f < NP) reinterpret_cast<f4*>(tb)[f] = live ? v[i] : f4{0.f, 0.f, 0.f, 0.f};
            }
        }
        if (tid == 0) ctr[0] = tm.x & 0xffffu;   // the tasks the counter hands out begin behind the long ones
        __syncthreads();
        // everything one step on
        auto advance = [&]() {
            D1 = D2;
            C1 = C2;
            if (D1.unit < nunits) NNUEFT_PREFETCH(C1, D1.chunk0 + D1.ci, D1.c, D1.cols)
            D2 = D3;
            if (D2.unit < nunits) {
                C2 = uni_chunk(c3raw);
                NNUEFT_PAIR_IDS(C2)
            }
            D3 = next_step(D2);
            if (D3.unit < nunits) c3raw = chunks[D3.chunk0 + D3.ci];
        };
        const bool first = C.flags & 1;
        const bool last_of_unit = cur.ci + 1 == cur.nw + cur.nb;
        const int mode = last_of_unit && cur.nb == 1 ? kOutAdd : last_of_unit && cur.nb == 0 ? kOut : kKeep;
        const uint32_t head = ltask[0];
        const int nlong = uni((int)(head & 0xffffu)), ntasks = uni((int)(head >> 16));
        // The step waits for its long chains.  Long task i belongs to wave i (the counter hands out the others): that
        // wave asks for the data of the steps to come at once, while the address units are idle, and starts on its
        // chain; every other wave does a task first and asks then (one place in the code for the asking, see above),
        // so that the long chain's wave neither queues behind their loads nor waits for its own at the next step.
        const int wave = wave0 >> 6;
        int task = ntasks;
        if (wave >= nlong) {
            task = draw();
            if (task < ntasks) task = do_task(task, nlong, mode, cur.c, first, row0, rows_here, cur.cols);
        }
        advance();
        if (wave < nlong) task = do_task(wave, nlong, mode, cur.c, first, row0, rows_here, cur.cols);
        while (task < ntasks) task = do_task(task, nlong, mode, cur.c, first, row0, rows_here, cur.cols);
        if (last_of_unit && cur.nb > 1) {
            // several black chunks: the gradient holds the white sums, LDS the black ones
            __syncthreads();
            for (int f = tid; f < rows_here * kCols; f += NT) {
                const int col = f & (kCols - 1);
                if (col < cur.cols) {
                    float* dst = gW + (size_t)(row0 + (f >> 4)) * out_cols + cur.c * kCols + col;
                    *dst = *dst + reinterpret_cast<float*>(lsum)[f];
                }
            }
        }
    }
#undef NNUEFT_PREFETCH
#undef NNUEFT_PAIR_IDS
}

constexpr int kMaxDevices = 64;
std::atomic<int> g_chain_lds_allowed[kMaxDevices];

int allow_chain_lds(int device) {
    if (device < 0 || device >= kMaxDevices) return NNUEFT_E_UNSUPPORTED;
    if (g_chain_lds_allowed[device].load(std::memory_order_acquire)) return 0;
    hipError_t e = hipFuncSetAttribute((const void*)k_chain_tile, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute((const void*)k_cs_expand, hipFuncAttributeMaxDynamicSharedMemorySize, kExpandLds);
    if (e != hipSuccess) return (int)e;
    g_chain_lds_allowed[device].store(1, std::memory_order_release);
    return 0;
}

size_t shape_workspace(int B, int K, int R, int out_cols, int n_persp) {
    ChainLayout L;
    if (K > kSlots || out_cols < kMinCols || out_cols % 4 || !chain_layout(B, n_persp, R, &L)) return 0;
    return L.end;
}

bool device_ok(const nnueft_dev::DeviceInfo& d) {
    return d.xcds == kXcd && d.cus >= kXcd && d.max_lds >= kLds && d.max_lds >= kExpandLds;
}

const uint32_t* fallback_flag(const void* ws, int B, int R, int n_persp) {
    ChainLayout L;
    if (!chain_layout(B, n_persp, R, &L)) return nullptr;
    return (const uint32_t*)((const char*)ws + L.sched) + kFlagWord;
}

int sort(const int32_t* widx, const int32_t* bidx, int B, int K, int R, int n_persp, void* ws, uint32_t* split_word,
         uint32_t* tag_word, hipStream_t st) {
    ChainLayout L;
    if (!chain_layout(B, n_persp, R, &L)) return NNUEFT_E_UNSUPPORTED;
    int device = 0;
    const nnueft_dev::DeviceInfo* info = nullptr;
    int rc = nnueft_dev::device_info(&device, &info);
    if (rc) return rc;
    rc = allow_chain_lds(device);
    if (rc) return rc;
    char* base = (char*)ws;
    uint32_t* hist = (uint32_t*)(base + L.hist);
    uint32_t* total = (uint32_t*)(base + L.total);
    uint32_t* bpairs = (uint32_t*)(base + L.bpairs);
    RChunk* chunks = (RChunk*)(base + L.chunks);
    BlockChunks* ublocks = (BlockChunks*)(base + L.ublocks);
    uint32_t* md = (uint32_t*)(base + L.md);
    uint16_t* ent = (uint16_t*)(base + L.ent);
    uint32_t* sched = (uint32_t*)(base + L.sched);
    const int vec = (K % 4 == 0) && aligned16(widx) && aligned16(bidx);
    hipLaunchKernelGGL(k_cs_hist, dim3(L.ngroups), dim3(kSortThreads), 0, st, widx, bidx, hist, L.npairs, B, K, R, L.nkeys, vec);
    NNUEFT_LAUNCH_CHECK();
    rc = nnueft_tile::launch_binscan(hist, total, L.nkeys + 1, L.ngroups, st);
    if (rc) return rc;
    hipLaunchKernelGGL(k_cs_place, dim3(L.ngroups), dim3(kSortThreads), 0, st, widx, bidx, hist, total, bpairs, chunks,
                       ublocks, sched, split_word, tag_word, table_tag(B, R, n_persp), L.npairs, n_persp, B, K, R, L.nkeys,
                       L.nblocks, vec);
    NNUEFT_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_cs_expand, dim3(L.max_chunks), dim3(kThreads), kExpandLds, st, widx, bidx, bpairs, chunks, md,
                       ent, sched, B, K, R, vec);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

int reduce(const float* G, int g_pitch, float* gW, int B, int R, int out_cols, int n_persp, void* ws,
           const uint32_t* tag_word, hipStream_t st) {
    ChainLayout L;
    if (!chain_layout(B, n_persp, R, &L)) return NNUEFT_E_UNSUPPORTED;
    if (!aligned16(G) || g_pitch % 4) return NNUEFT_E_UNSUPPORTED;
    int device = 0;
    const nnueft_dev::DeviceInfo* info = nullptr;
    int rc = nnueft_dev::device_info(&device, &info);
    if (rc) return rc;
    rc = allow_chain_lds(device);
    if (rc) return rc;
    char* base = (char*)ws;
    const int main_tiles = out_cols / kCols;
    const int tail_cols = out_cols % kCols;
    const int tpx = (main_tiles + kXcd - 1) / kXcd;
    const int grid = info->cus / kXcd * kXcd;
    hipLaunchKernelGGL(k_chain_tile, dim3(grid), dim3(kThreads), kLds, st, G, g_pitch, (const uint32_t*)(base + L.bpairs),
                       (const RChunk*)(base + L.chunks), (const BlockChunks*)(base + L.ublocks),
                       (const uint32_t*)(base + L.md), (const uint16_t*)(base + L.ent), (uint32_t*)(base + L.sched), gW, R,
                       out_cols, main_tiles, tpx, tail_cols, L.nblocks, aligned16(gW) ? 1 : 0, tag_word, table_tag(B, R, n_persp));
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

}  // namespace nnueft_chain
