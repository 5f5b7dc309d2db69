// Forward, LDS-tiled variant: the gather reads the table out of LDS instead of through L2.
//
// All indices of one list name rows of a single 768-row block of the table (one king bucket).  A
// workgroup keeps one tile of the table in LDS, 768 rows x 32 columns (96 KB), and the lists of a chunk
// of that block's (position, perspective) pairs (up to 1536 pairs and 27 648 list entries, 55 KB, as
// 16-bit row numbers inside the block, every list at its own length rounded up to 8 entries), and
// sums the tile's columns for every pair: 8 lanes a pair, one 16-byte LDS read per row and lane, the
// adds in slot order.  Every row of the table then crosses the CU's L1 once per chunk of pairs (a whole
// block at B = 16384) instead of once per pair naming it (about 24 times there), which is what bounds
// the gather through L2: a CU can only keep so many L1 misses pending.
//
//   k_tl_hist     one pair per thread: key (block, list length) counted per workgroup
//   k_tl_binscan  per key, the counts of the workgroups become their exclusive prefix
//   k_tl_lists    pairs to their slots, longest lists first inside a block and dealt to the block's
//                 chunks in turn; writes the packed 16-bit lists, pair ids, list places and the chunk
//                 table (longest chunks first)
//   k_acc_tile    persistent workgroups, one per CU: units of (chunk, group of column tiles) handed out
//                 per XCD; the next tile (also the first one of the next unit) is fetched into registers
//                 while the current one is summed; waves take tasks of 8 pairs from a counter in LDS
//   k_mix         as in the L2-blocked path
//
// Rows of 2048 columns and more: the gather visits the column tiles in pairs (columns j and j + L1/2) and writes
// the output rows of the positions whose (us, them) is (1, 0) or (0, 1) itself (see FuseF); k_mix_rest then does
// the psqt chains and the other positions.
//
// A list that names rows of more than one block (the interface allows it) is summed from global
// memory by the same wave; results are bit-identical to the other forward kernels.
#include <atomic>
#include <cstdlib>

#include "gather.h"
#include "tile_sort.h"

namespace nnueft_tile {

bool layout(int npairs, int R, Layout* L, int block_rows) {
    if (npairs <= 0 || R <= 0 || block_rows <= 0 || block_rows > kRows) return false;
    L->npairs = npairs;
    L->block_rows = block_rows;
    L->nblocks = (R + block_rows - 1) / block_rows;
    if (L->nblocks > kMaxBlocks) return false;
    L->nbins = L->nblocks * kLenBins + 1;   // + one empty bin: its offset is the end of the last block
    L->ngroups = (npairs + kSortThreads - 1) / kSortThreads;
    L->max_chunks = (npairs + 511) / 512 + 2 * L->nblocks + 2;
    L->nslots = npairs + L->max_chunks;     // a block's chunks are equally long, the last ones one pair short
    size_t off = 0;
    L->hist = off;
    off += up256((size_t)L->ngroups * L->nbins * sizeof(uint32_t));
    L->total = off;
    off += up256((size_t)kBins * sizeof(uint32_t));
    L->lists = off;
    off += up256(((size_t)npairs * kSlots + 64) * sizeof(uint16_t));
    L->pidcnt = off;
    off += up256((size_t)L->nslots * sizeof(uint32_t));
    L->loff = off;
    off += up256((size_t)L->nslots * sizeof(uint16_t));
    L->chunks = off;
    off += up256((size_t)L->max_chunks * sizeof(Chunk));
    L->sched = off;
    off += up256((size_t)(kXcd + 1) * 32 * sizeof(uint32_t));
    L->brec = off;
    off += up256((size_t)kMaxBlocks * sizeof(BlockRec));
    L->cpool8 = off;
    off += up256((size_t)kMaxChunks * sizeof(uint32_t));
    L->border = off;
    off += up256((size_t)kMaxBlocks * sizeof(uint32_t));
    L->end = off;
    return true;
}

size_t workspace(int B, int R) {
    Layout L;
    const size_t blocked = nnueft_blocked::pair_sort_workspace(B, R, 0);
    if (B >= (1 << 25) || !layout(2 * B, R, &L)) return blocked;
    return L.end > blocked ? L.end : blocked;
}

bool fits(const nnueft_dev::DeviceInfo& d, int B, int K, int R, int L1) {
    Layout L;
    return K <= kSlots && L1 % kTileCols == 0 && L1 >= 512 && (long long)2 * B < (1ll << 26) &&
           d.max_lds >= kLdsBytes && d.xcds == kXcd && d.cus >= kXcd && layout(2 * B, R, &L) &&
           L.max_chunks <= kMaxChunks;
}

__device__ __forceinline__ const int32_t* pair_list(const int32_t* __restrict__ widx,
                                                    const int32_t* __restrict__ bidx, int pair, int B, int K) {
    const int p = pair >= B;
    return (p ? bidx : widx) + (size_t)(pair - p * B) * K;
}

// A thread's view of one list: valid entries counted, the block of the first, whether all stay in it.
struct ListFacts {
    int cnt, block;
    bool foreign;
};

// The list of a thread in registers: kSlots entries, -1 beyond K (16-byte loads when `vec`).
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

__device__ __forceinline__ ListFacts list_facts(const ListRegs& l, int R, int block_rows) {
    ListFacts f{0, 0, false};
    int first = -1, base = 0;
#pragma unroll
    for (int k = 0; k < kSlots; ++k) {
        const int r = l.v[k];
        if (r >= 0 && r < R) {
            if (first < 0) {
                // r / block_rows for r below 2^32 / block_rows, without the division
                first = (int)__umulhi((uint32_t)r, 0xffffffffu / (uint32_t)block_rows + 1u);
                base = first * block_rows;
            }
            f.foreign |= r < base || r >= base + block_rows;
            ++f.cnt;
        }
    }
    f.block = first < 0 ? 0 : first;
    return f;
}

__device__ __forceinline__ int sort_key(const ListFacts& f) { return f.block * kLenBins + (kSlots - f.cnt); }

__global__ __launch_bounds__(kSortThreads) void k_tl_hist(const int32_t* __restrict__ widx,
                                                          const int32_t* __restrict__ bidx,
                                                          uint32_t* __restrict__ hist, int npairs, int B, int K,
                                                          int R, int nbins, int vec, int block_rows) {
    __shared__ uint32_t bins[kBins];
    const int tid = threadIdx.x;
    const int n = blockIdx.x * kSortThreads + tid;
    for (int i = tid; i < nbins; i += kSortThreads) bins[i] = 0;
    __syncthreads();
    if (n < npairs) atomicAdd(&bins[sort_key(list_facts(load_list(pair_list(widx, bidx, n, B, K), K, vec), R, block_rows))], 1u);
    __syncthreads();
    for (int i = tid; i < nbins; i += kSortThreads) hist[(size_t)i * gridDim.x + blockIdx.x] = bins[i];
}

// Chunks of a block with n pairs whose lists take e entries (each list padded to a multiple of 8): as few as
// keep each at kChunk pairs and kListCap entries.  Pair i of the block (longest list first) goes to chunk
// i % nc, so every chunk gets the same mix of list lengths; of the pairs of one length a chunk can get one more
// than its even share, kListSlack entries in all, which the entry limit leaves free.
__device__ __forceinline__ int chunks_of(int n, int e) {
    if (n == 0) return 0;
    const int by_pairs = (n + kChunk - 1) / kChunk;
    const int by_entries = (e + (kListCap - kListSlack) - 1) / (kListCap - kListSlack);
    return max(1, max(by_pairs, by_entries));
}

// One wave per bin: the counts of the workgroups become their exclusive prefix, the sum goes to total[bin].
__global__ __launch_bounds__(kSortThreads) void k_tl_binscan(uint32_t* __restrict__ hist, uint32_t* __restrict__ total,
                                                             int nbins, int ngroups) {
    const int lane = threadIdx.x & 63;
    const int bin = blockIdx.x * (kSortThreads / 64) + (threadIdx.x >> 6);
    if (bin >= nbins) return;
    uint32_t* h = hist + (size_t)bin * ngroups;
    uint32_t run = 0;
    for (int g0 = 0; g0 < ngroups; g0 += 64) {
        const int g = g0 + lane;
        const uint32_t v = g < ngroups ? h[g] : 0;
        uint32_t incl = v;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t t = __shfl_up(incl, off);
            if (lane >= off) incl += t;
        }
        if (g < ngroups) h[g] = run + incl - v;
        run += __shfl(incl, 63);
    }
    if (lane == 0) total[bin] = run;
}

__global__ __launch_bounds__(kSortThreads) void k_tl_lists(const int32_t* __restrict__ widx,
                                                           const int32_t* __restrict__ bidx,
                                                           const uint32_t* __restrict__ hist,
                                                           const uint32_t* __restrict__ total,
                                                           uint16_t* __restrict__ lists,
                                                           uint32_t* __restrict__ pidcnt, uint16_t* __restrict__ loff,
                                                           Chunk* __restrict__ chunks,
                                                           uint32_t* __restrict__ sched,
                                                           BlockRec* __restrict__ brec, uint32_t* __restrict__ cpool8,
                                                           uint32_t* __restrict__ border, int npairs, int B, int K,
                                                           int R, int nblocks, int nbins, int vec, int block_rows,
                                                           SortExtras ex) {
    const float* __restrict__ us = ex.us;
    const float* __restrict__ them = ex.them;
    __shared__ uint32_t cursor[kBins];      // next slot of this workgroup in every bin
    __shared__ uint32_t bin_base[kBins];    // first slot of every bin
    __shared__ uint32_t bin_eoff[kBins];    // list entries of its block before the bin's lists
    __shared__ uint32_t chunk_pool8[kMaxChunks];   // where a chunk's lists begin, in units of 8 entries
    __shared__ uint32_t ck_start[kMaxChunks];      // the chunk table before it is put in order (first workgroup)
    __shared__ uint16_t ck_block[kMaxChunks], ck_count[kMaxChunks], ck_n8[kMaxChunks];
    __shared__ uint32_t wave_tot[kSortThreads / 64];
    __shared__ uint32_t blk_nc[kMaxBlocks], blk_e8[kMaxBlocks];
    __shared__ uint32_t blk_chunk0[kMaxBlocks + 1];   // chunks before the block; [nblocks] = chunks in all
    __shared__ uint32_t blk_pool8[kMaxBlocks + 1];    // list entries / 8 before the block
    const int tid = threadIdx.x;
    const int n = blockIdx.x * kSortThreads + tid;
    const int ngroups = gridDim.x;
    // first slot of every bin: exclusive scan of the bin totals, kBins / kSortThreads consecutive bins a thread
    {
        constexpr int PER = kBins / kSortThreads;
        static_assert(kBins % kSortThreads == 0, "bins per thread");
        uint32_t v[PER];
        uint32_t local = 0;
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int i = tid * PER + u;
            v[u] = i < nbins ? total[i] : 0;
            local += v[u];
        }
        uint32_t incl = local;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t t = __shfl_up(incl, off);
            if ((tid & 63) >= off) incl += t;
        }
        if ((tid & 63) == 63) wave_tot[tid >> 6] = incl;
        __syncthreads();
        uint32_t run = incl - local;
        for (int w = 0; w < (tid >> 6); ++w) run += wave_tot[w];
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int i = tid * PER + u;
            if (i < nbins) {
                bin_base[i] = run;
                cursor[i] = run + hist[(size_t)i * ngroups + blockIdx.x];
            }
            run += v[u];
        }
    }
    __syncthreads();
    // bin (b, k) holds the lists of block b with kSlots - k entries; bin_base[nbins - 1] is the end of the last block
    if (tid < nblocks) {
        const uint32_t* bb = bin_base + tid * kLenBins;
        int e = 0;
        for (int k = 0; k < kLenBins; ++k) {
            bin_eoff[tid * kLenBins + k] = (uint32_t)e;   // entries of the block's longer lists
            e += (int)(bb[k + 1] - bb[k]) * padded(kSlots - k);
        }
        blk_e8[tid] = (uint32_t)(e >> 3);
        blk_nc[tid] = (uint32_t)chunks_of((int)(bb[kLenBins] - bb[0]), e);
    }
    __syncthreads();
    if (tid == 0) {
        uint32_t c = 0, p8 = 0;
        for (int b = 0; b < nblocks; ++b) {
            blk_chunk0[b] = c;
            blk_pool8[b] = p8;
            c += blk_nc[b];
            p8 += blk_e8[b];
        }
        blk_chunk0[nblocks] = c;
        blk_pool8[nblocks] = p8;
    }
    __syncthreads();
    // where the lists of every chunk begin (and, by the first workgroup, the chunk table)
    if (tid < nblocks) {
        const uint32_t* bb = bin_base + tid * kLenBins;
        const int nb = (int)(bb[kLenBins] - bb[0]);
        const int nc = (int)blk_nc[tid];
        const int len = nc ? (nb + nc - 1) / nc : 0;
        uint32_t p8 = blk_pool8[tid];
        for (int j = 0; j < nc; ++j) {
            int e = 0;
            for (int k = 0; k < kLenBins; ++k) {
                const int r0 = (int)(bb[k] - bb[0]), r1 = (int)(bb[k + 1] - bb[0]);
                e += (ranks_of_chunk(r1, j, nc) - ranks_of_chunk(r0, j, nc)) * padded(kSlots - k);
            }
            const uint32_t ci = blk_chunk0[tid] + (uint32_t)j;
            if (ci < (uint32_t)kMaxChunks) chunk_pool8[ci] = p8;
            if (blockIdx.x == 0 && ci < (uint32_t)kMaxChunks) {
                cpool8[ci] = p8;
                ck_block[ci] = (uint16_t)tid;
                ck_start[ci] = (bb[0] + blk_chunk0[tid]) + (uint32_t)(j * len);
                ck_count[ci] = (uint16_t)ranks_of_chunk(nb, j, nc);
                ck_n8[ci] = (uint16_t)(e >> 3);
            }
            p8 += (uint32_t)(e >> 3);
        }
    }
    if (blockIdx.x == 0 && tid <= kXcd) sched[tid * 32] = tid == kXcd ? blk_chunk0[nblocks] : 0u;
    if (blockIdx.x == 0 && tid == 0) sched[kSchedNonFinite] = 0u;
    // the blocks as the backward scatter walks them, and their order by population (most pairs first)
    if (blockIdx.x == 0 && tid < nblocks) {
        const uint32_t* bb = bin_base + tid * kLenBins;
        const int nb = (int)(bb[kLenBins] - bb[0]);
        const int nc = (int)blk_nc[tid];
        brec[tid] = BlockRec{(int)(bb[0] + blk_chunk0[tid]), nb, nc, nc ? (nb + nc - 1) / nc : 0, (int)blk_chunk0[tid], 0, 0, 0};
        int rank = 0;
        for (int k = 0; k < nblocks; ++k) {
            const int other = (int)(bin_base[(k + 1) * kLenBins] - bin_base[k * kLenBins]);
            rank += other > nb || (other == nb && k < tid);
        }
        border[rank] = (uint32_t)tid;
    }
    __syncthreads();
    // The chunk table, longest lists first: the gather hands units out in table order, and the CUs of an XCD
    // finish closer together when the small units come last.
    if (blockIdx.x == 0) {
        const int nch = min((int)blk_chunk0[nblocks], kMaxChunks);
        for (int ci = tid; ci < nch; ci += kSortThreads) {
            const uint32_t mine = ck_n8[ci];
            int rank = 0;
            for (int k = 0; k < nch; ++k) {
                const uint32_t other = ck_n8[k];
                rank += other > mine || (other == mine && k < ci);
            }
            chunks[rank] = Chunk{(int)ck_block[ci], (int)ck_start[ci], (int)ck_count[ci], (int)chunk_pool8[ci],
                                 (int)ck_n8[ci], 0, 0, 0};
        }
    }
    if (n >= npairs) return;
    const ListRegs l = load_list(pair_list(widx, bidx, n, B, K), K, vec);
    // The pair's psqt chain, while its list is in registers: the entries of the list's valid rows are asked for here
    // and summed at the end of the kernel, so that they are on their way during the rest.
    float psv[kSlots];
    int64_t psqt_col = -1;
    if (ex.wpsqt) {
        const int64_t pi = ex.psqt_idx[n >= B ? n - B : n];
        if (pi >= 0 && pi < ex.n_psqt) psqt_col = pi;
    }
#pragma unroll
    for (int k = 0; k < kSlots; ++k) {
        const int r = l.v[k];
        psv[k] = psqt_col >= 0 && r >= 0 && r < R ? ex.W[(size_t)r * ((size_t)ex.L1 + ex.n_psqt) + ex.L1 + psqt_col] : 0.0f;
    }
    // The quantized forward's psqt difference of the position whose white list this is: both lists' entries asked
    // for here, summed at the end of the kernel.
    uint32_t qw[kSlots], qb[kSlots];
    const bool q_psqt = ex.psqt_out != nullptr && n < B;
    if (q_psqt) {
        const int64_t pi = ex.psqt_idx[n];
        const bool ok = pi >= 0 && pi < ex.n_psqt;
        const ListRegs lb = load_list(pair_list(widx, bidx, n + B, B, K), K, vec);
#pragma unroll
        for (int k = 0; k < kSlots; ++k) {
            const int rw = l.v[k], rb = lb.v[k];
            qw[k] = ok && rw >= 0 && rw < R ? (uint32_t)ex.psqt32[(size_t)rw * ex.n_psqt + pi] : 0u;
            qb[k] = ok && rb >= 0 && rb < R ? (uint32_t)ex.psqt32[(size_t)rb * ex.n_psqt + pi] : 0u;
        }
    }
    const ListFacts f = list_facts(l, R, block_rows);
    const int bin = sort_key(f);
    const uint32_t slot = atomicAdd(&cursor[bin], 1u);
    const uint32_t* bb = bin_base + f.block * kLenBins;
    const int nb = (int)(bb[kLenBins] - bb[0]);
    const int nc = (int)blk_nc[f.block];
    const int len = (nb + nc - 1) / nc;
    const int i = (int)(slot - bb[0]);       // rank inside the block, longest lists first
    const int j = i % nc;
    const size_t dst = (size_t)(bb[0] + blk_chunk0[f.block]) + (size_t)j * len + i / nc;
    pidcnt[dst] = (uint32_t)n | ((f.foreign ? kForeign : (uint32_t)f.cnt) << 26);
    // the list's place among its chunk's lists: behind the chunk's longer lists and its earlier ones of this length
    int off = 0;
    const int kbin = bin - f.block * kLenBins;
    const int pad = padded(f.cnt);
    if (nc == 1) {
        off = (int)bin_eoff[bin] + (i - (int)(bb[kbin] - bb[0])) * pad;
    } else {
        for (int k = 0; k < kbin; ++k) {
            const int r0 = (int)(bb[k] - bb[0]), r1 = (int)(bb[k + 1] - bb[0]);
            off += (ranks_of_chunk(r1, j, nc) - ranks_of_chunk(r0, j, nc)) * padded(kSlots - k);
        }
        off += (i / nc - ranks_of_chunk((int)(bb[kbin] - bb[0]), j, nc)) * pad;
    }
    // with the sides to move at hand (both perspectives' lists, n = perspective * B + position): whether the pair's
    // sums alone make a half of the position's output row, and which half
    uint32_t side = 0;
    if (us) {
        const int p = n >= B;
        const float u = us[n - p * B], t = them[n - p * B];
        side = (one_sided(u, t) ? kLoffOwnRow : 0u) | ((p == 0) == (u == 1.0f) ? 0u : kLoffSecondHalf);
    }
    loff[dst] = (uint16_t)((uint32_t)(off >> 3) | side);
    const uint32_t ci = blk_chunk0[f.block] + (uint32_t)j;
    // row numbers inside the block, valid entries first in slot order, the rest name the row of zeros
    uint32_t w[kSlots / 2];
    const int base = f.block * block_rows;
    bool prefix = true;   // the valid entries are the first cnt slots (what a loader writes)
#pragma unroll
    for (int k = 0; k < kSlots; ++k) prefix &= (k < f.cnt) == (l.v[k] >= 0 && l.v[k] < R);
    if (f.foreign) {
#pragma unroll
        for (int q = 0; q < kSlots / 2; ++q) w[q] = (uint32_t)kRows | ((uint32_t)kRows << 16);
    } else if (prefix) {
#pragma unroll
        for (int q = 0; q < kSlots / 2; ++q) {
            const uint32_t lo = 2 * q < f.cnt ? (uint32_t)(l.v[2 * q] - base) : (uint32_t)kRows;
            const uint32_t hi = 2 * q + 1 < f.cnt ? (uint32_t)(l.v[2 * q + 1] - base) : (uint32_t)kRows;
            w[q] = lo | (hi << 16);
        }
    } else {
#pragma unroll
        for (int q = 0; q < kSlots / 2; ++q) w[q] = (uint32_t)kRows | ((uint32_t)kRows << 16);
        int m = 0;
#pragma unroll
        for (int k = 0; k < kSlots; ++k) {
            const int r = l.v[k];
            if (r >= 0 && r < R) {
                const uint32_t v = (uint32_t)(r - base);
#pragma unroll
                for (int q = 0; q <= k / 2; ++q)
                    if (q == (m >> 1)) w[q] = (m & 1) ? ((w[q] & 0xffffu) | (v << 16)) : ((w[q] & 0xffff0000u) | v);
                ++m;
            }
        }
    }
    if (ex.wpsqt) {
        // in slot order; a slot without a row adds +0, which leaves a sum that began at +0 as it is
        float ps = 0.0f;
#pragma unroll
        for (int k = 0; k < kSlots; ++k) ps = ps + psv[k];
        if (psqt_col >= 0) ps = ps + ex.bias[ex.L1 + psqt_col];
        (n >= B ? ex.bpsqt : ex.wpsqt)[n >= B ? n - B : n] = ps;
    }
    if (q_psqt) {
        uint32_t white = 0u, black = 0u;
#pragma unroll
        for (int k = 0; k < kSlots; ++k) {
            white += qw[k];
            black += qb[k];
        }
        // (sum over the mover's list - sum over the other list) / 2
        ex.psqt_out[n] = (int32_t)(ex.stm[n] ? black - white : white - black) / 2;
    }
    if (ci >= (uint32_t)kMaxChunks) return;   // (the launcher takes this path only when the table is long enough)
    u4* out = reinterpret_cast<u4*>(lists + ((size_t)chunk_pool8[ci] << 3) + off);
#pragma unroll
    for (int q = 0; q < kSlots / 8; ++q)
        if (q * 8 < pad) out[q] = u4{w[4 * q], w[4 * q + 1], w[4 * q + 2], w[4 * q + 3]};
}

// (16-bit half of w) * bytes per tile row + off: the LDS address of a lane's piece of a row, one instruction.
template <int HI>
__device__ __forceinline__ uint32_t row_addr(uint32_t w, uint32_t off) {
    uint32_t r;
    const uint32_t stride = kRowBytes;
    if (HI)
        asm("v_mad_u32_u16 %0, %1, %2, %3 op_sel:[1,0,0,0]" : "=v"(r) : "v"(w), "s"(stride), "v"(off));
    else
        asm("v_mad_u32_u16 %0, %1, %2, %3 op_sel:[0,0,0,0]" : "=v"(r) : "v"(w), "s"(stride), "v"(off));
    return r;
}

// 16 bytes of LDS at a byte address that already holds the tile's place in LDS (no add of the base per read).
typedef __attribute__((address_space(3))) const f4 lds_f4;
__device__ __forceinline__ f4 lds_read16(uint32_t addr) { return *reinterpret_cast<lds_f4*>(addr); }

// round(x * scale) / scale with round-half-to-even, as torch's mul / round / div (the table merge's grid)
__device__ __forceinline__ float fq(float x, float scale) { return rintf(x * scale) / scale; }

// One element of the table the gather sums: W[row] alone, or merged with the virtual weights of the row's place
// in its block, W + V[row % virtual rows], on the fake-quantization grid when asked for; the same operations, in
// the same order, as the separate merge pass (k_table_merge), so a forward over either gives the same bits.
__device__ __forceinline__ f4 merged4(f4 w, f4 v, const VirtualTable& vt) {
    w += v;
    if (vt.quantize) {
        if (vt.inv_scale_ft != 0.0f) {
            w.x = rintf(w.x * vt.scale_ft) * vt.inv_scale_ft;
            w.y = rintf(w.y * vt.scale_ft) * vt.inv_scale_ft;
            w.z = rintf(w.z * vt.scale_ft) * vt.inv_scale_ft;
            w.w = rintf(w.w * vt.scale_ft) * vt.inv_scale_ft;
        } else {
            w.x = fq(w.x, vt.scale_ft);
            w.y = fq(w.y, vt.scale_ft);
            w.z = fq(w.z, vt.scale_ft);
            w.w = fq(w.w, vt.scale_ft);
        }
    }
    return w;
}

// a += r: four floats, or (I16) eight 16-bit integers that wrap
typedef unsigned short us8 __attribute__((ext_vector_type(8)));
template <bool I16>
__device__ __forceinline__ void acc_add(f4& a, const f4& r) {
    if constexpr (I16) a = __builtin_bit_cast(f4, (us8)(__builtin_bit_cast(us8, a) + __builtin_bit_cast(us8, r)));
    else a += r;
}

// saved[pair, columns of the tile] = chain from +0 over the pair's list, for every pair of the chunk.
// VIRT: the table is W + V[row % kRows] (see merged4); the tile is merged on its way into LDS.  That variant
// runs with 768 threads: the tile of V waits in registers beside the tile of W.
// What the quantized forward does with a pair's sums when the gather finishes them itself (FUSE == kFuse16): + bias, clip,
// product of column j with column j + L1/2, >> shift, one byte per column pair, written to the half of the
// position's output row that the side to move selects.
struct Fuse16 {
    const uint8_t* stm;
    const int16_t* b16;
    uint8_t* out;
    int clip_max, shift;
    // what the sort needs for the psqt difference (it has every list in registers anyway)
    const int32_t* psqt32;
    const int64_t* psqt_idx;
    int32_t* psqt_out;
    int n_psqt;
};

// What the float forward does with a pair's sums when the gather finishes them itself (FUSE == kFuseF).  A unit then
// visits the column tiles two by two, tile c and its partner c + ntiles / 2 (columns j and j + L1/2): after the
// second the wave that holds a pair's sums of the partner tile reads the pair's sums of the first back (they went to
// `saved` a moment ago, from the same CU) and has both factors of the product.  For a position whose (us, them) is
// (1, 0) or (0, 1) the pair's half of the output row is + bias, clamp, product, the activation grid when asked for:
// exactly what the mix of both perspectives gives there, as long as the other perspective's sums are finite (0 * inf
// is NaN in the mix).  A sum that is not finite therefore raises sched[kSchedNonFinite], and the pass that follows
// (k_mix_rest) then redoes every row from the saved sums; it always does the rows of positions with any other
// (us, them), which this kernel leaves alone.
struct FuseF {
    const float* us;
    const float* them;
    const float* bias;
    float* l0;
    float max_act;
    ActGrid act;
    // what the sort needs to sum the psqt chains on its way (it has every list in registers anyway)
    const int64_t* psqt_idx;
    float* wpsqt;
    float* bpsqt;
};
constexpr int kFuse16 = 1, kFuseF = 2;

__device__ __forceinline__ bool finite4(const f4& x) {
    return fabsf(x.x) <= 3.402823466e+38f && fabsf(x.y) <= 3.402823466e+38f && fabsf(x.z) <= 3.402823466e+38f &&
           fabsf(x.w) <= 3.402823466e+38f;
}

typedef unsigned int u2 __attribute__((ext_vector_type(2)));

// 16 bytes of a row in the kFuse16 layout: four 16-bit columns at `lo` and the four that pair with them, L1/2 further on
__device__ __forceinline__ f4 load_pair8(const char* lo, size_t half_bytes) {
    const u2 a = *reinterpret_cast<const u2*>(lo);
    const u2 b = *reinterpret_cast<const u2*>(lo + half_bytes);
    return __builtin_bit_cast(f4, u4{a.x, a.y, b.x, b.y});
}

template <int NT, bool VIRT, bool I16, int FUSE = 0>
__global__ __launch_bounds__(NT) void k_acc_tile(const int32_t* __restrict__ widx,
                                                          const int32_t* __restrict__ bidx,
                                                          const uint16_t* __restrict__ lists,
                                                          const uint32_t* __restrict__ pidcnt,
                                                          const uint16_t* __restrict__ loff,
                                                          const Chunk* __restrict__ chunks,
                                                          uint32_t* __restrict__ sched, const float* __restrict__ W,
                                                          float* __restrict__ acc, int B, int K, int R, int L1,
                                                          int out_cols, int tiles_per_xcd, int tile_group,
                                                          VirtualTable vt, int block_rows, Fuse16 fz, FuseF ff) {
    static_assert((FUSE == kFuse16) == I16, "the quantized table is gathered with its own epilogue, and only it");
    static_assert(FUSE == 0 || FUSE == kFuse16 || FUSE == kFuseF, "epilogue");
    constexpr bool F16 = FUSE == kFuse16;   // the tile's rows are column pairs (j, j + L1/2) of the quantized table
    constexpr bool FF = FUSE == kFuseF;     // the tiles come in pairs (c, c + ntiles / 2) of the float table
    extern __shared__ float4 lds_raw[];
    char* tb = reinterpret_cast<char*>(lds_raw);
    u4* lst = reinterpret_cast<u4*>(tb + kTileBytes);                                         // (kListCap + 32) * 2 bytes
    uint32_t* mpid = reinterpret_cast<uint32_t*>(tb + kTileBytes + (kListCap + 32) * 2);      // kChunk
    uint16_t* moff = reinterpret_cast<uint16_t*>(mpid + kChunk);                              // kChunk
    uint32_t* ctr = reinterpret_cast<uint32_t*>(moff + kChunk);   // [0] task counter, [1] the unit this workgroup works on next
    f4* lbias = reinterpret_cast<f4*>(ctr + 4);                   // FF: the bias of the pair of tiles at work, 2 x 32 floats
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    constexpr int N4 = kRows * (kRowBytes / 16);
    static_assert(N4 % NT == 0, "tile load");
    constexpr int IT = N4 / NT;
    const int x = blockIdx.x % kXcd;
    // a tile row is 128 bytes: 32 floats, or 64 of the 16-bit weights of the quantized table (I16: a row of W is
    // then L1 int16, a row of acc too, the sums wrap like 16-bit adds and their order does not matter)
    // FF: what the XCDs share out and the units visit are the pairs of tiles, ntiles / 2 of them
    const int ntiles = I16 ? L1 / (2 * kTileCols) : (FF ? L1 / (2 * kTileCols) : L1 / kTileCols);
    const int partner = ntiles;   // FF: tile c + partner holds the columns L1/2 beyond tile c's
    const size_t w_pitch = I16 ? (size_t)L1 * 2 : (size_t)out_cols * 4;
    const size_t a_pitch = I16 ? (size_t)L1 * 2 : (size_t)L1 * 4;
    const char* Wb = reinterpret_cast<const char*>(W);
    // F16: a tile row is 32 column pairs (j, j + L1/2): lane piece q holds columns 4q .. 4q+3 of the tile's 32 and
    // their four partners, so the product needs no other lane
    const size_t half_bytes = (size_t)L1;   // L1/2 columns of 2 bytes
    // the column tiles of this XCD, in groups of tile_group; a unit = (chunk, group)
    const int my_tiles = max(0, min(tiles_per_xcd, ntiles - x * tiles_per_xcd));
    const int groups = (my_tiles + tile_group - 1) / tile_group;
    // A unit's tiles are `groups` apart, so that the units (chunk, g), (chunk, g + 1), handed to two CUs one after
    // the other, fetch neighbouring tiles at about the same time: a 128-byte tile row straddles two cache lines of
    // a 12 320-byte table row (F16: it is two half lines whose other halves the neighbour tile holds), and the
    // second fetch of a shared line then hits the XCD's L2 (forward at L1 = 3072: 0.318 -> 0.306 ms; the
    // quantized table: fetched 0.43 -> 0.26 GB)
    const int qs = groups;
    const int nunits = (int)sched[kXcd * 32] * groups;
    uint32_t* unit_ctr = sched + x * 32;
    const int g = lane >> 3, j = lane & 7;
    // low half of a flat LDS address = the byte address inside LDS
    const uint32_t lane_off = (uint32_t)(uintptr_t)tb + j * 16;
    if (tid < kRowBytes / 16) reinterpret_cast<f4*>(tb)[kRows * (kRowBytes / 16) + tid] = f4{0.f, 0.f, 0.f, 0.f};
    if (tid == 0) ctr[1] = atomicAdd(unit_ctr, 1u);

    f4 v[IT];
    f4 vv[VIRT ? IT : 1];
#define NNUEFT_UNIT(u_, C_, q0_, q1_)                       \
    {                                                       \
        const int ch_ = (u_) / groups;                      \
        C_ = chunks[ch_];                                   \
        q0_ = (u_) - ch_ * groups;                          \
        q1_ = my_tiles;                                     \
    }
#define NNUEFT_LOAD_TILE(blk_, c_)                                                                       \
    {                                                                                                    \
        const int row0_ = (blk_) * block_rows;                                                           \
        const int rows_here_ = min(block_rows, R - row0_);                                               \
        const char* src = Wb + (size_t)row0_ * w_pitch + (c_) * kRowBytes;                               \
        _Pragma("unroll") for (int i = 0; i < IT; ++i) {                                                 \
            const int f = tid + i * NT;                                                                  \
            const int row = f >> 3;                                                                      \
            if (F16)                                                                                     \
                v[i] = row < rows_here_ ? load_pair8(Wb + (size_t)(row0_ + row) * w_pitch + (c_) * 64 +  \
                                                     (f & 7) * 8, half_bytes)                            \
                                        : f4{0.f, 0.f, 0.f, 0.f};                                        \
            else                                                                                         \
            v[i] = row < rows_here_                                                                      \
                       ? *reinterpret_cast<const f4*>(src + (size_t)row * w_pitch + (f & 7) * 16)        \
                       : f4{0.f, 0.f, 0.f, 0.f};                                                         \
            if (VIRT)                                                                                    \
                vv[i] = row < rows_here_ ? *reinterpret_cast<const f4*>(vt.V + (size_t)row * out_cols +  \
                                                                        (c_) * kTileCols + (f & 7) * 4)  \
                                         : f4{0.f, 0.f, 0.f, 0.f};                                       \
        }                                                                                                \
    }
    __syncthreads();
    int unit = __builtin_amdgcn_readfirstlane((int)ctr[1]);
    Chunk C{};
    int q0 = 0, q1 = 0;
    if (unit < nunits) {
        NNUEFT_UNIT(unit, C, q0, q1)
        NNUEFT_LOAD_TILE(C.block, x * tiles_per_xcd + q0)
    }
    // Entering an iteration the first tile of the unit is on its way into v: the last tile of a unit fetches
    // the first one of the next.
    while (unit < nunits) {
        __syncthreads();   // the previous unit is done with the lists and the tile, and everyone has read ctr[1]
        if (tid == 0) ctr[1] = atomicAdd(unit_ctr, 1u);
        {
            constexpr int LI = ((kListCap + 32) / 8 + NT - 1) / NT;
            constexpr int PI = (kChunk + NT - 1) / NT;
            const u4* ms = reinterpret_cast<const u4*>(lists + ((size_t)C.pool8 << 3));
            u4 t[LI];
            uint32_t tp[PI];
            uint16_t to[PI];
#pragma unroll
            for (int i = 0; i < LI; ++i) t[i] = tid + i * NT < C.n8 ? ms[tid + i * NT] : u4{0u, 0u, 0u, 0u};
#pragma unroll
            for (int i = 0; i < PI; ++i) {
                tp[i] = tid + i * NT < C.count ? pidcnt[C.start + tid + i * NT] : 0u;
                to[i] = tid + i * NT < C.count ? loff[C.start + tid + i * NT] : (uint16_t)0;
            }
#pragma unroll
            for (int i = 0; i < LI; ++i)
                if (tid + i * NT < C.n8) lst[tid + i * NT] = t[i];
#pragma unroll
            for (int i = 0; i < PI; ++i)
                if (tid + i * NT < C.count) {
                    mpid[tid + i * NT] = tp[i];
                    moff[tid + i * NT] = to[i];
                }
        }
        const int ntasks = (C.count + 7) >> 3;
        int nunit = nunits;
        Chunk Cn{};
        int qn0 = 0, qn1 = 0;
        // FF: a visit is two tiles, c and then its partner (second == 1)
        for (int qq = FF ? 2 * q0 : q0; qq < (FF ? 2 * q1 : q1); qq += FF ? (qq & 1 ? 2 * qs - 1 : 1) : qs) {
            const int q = FF ? qq >> 1 : qq;
            const int second = FF ? qq & 1 : 0;
            const int c = x * tiles_per_xcd + q + second * partner;
            // everyone is done reading the previous tile.  (FF: the sums of the first tile of the visit are on their
            // way to memory, and the waves that read them back after the second are others than those that wrote them,
            // but of this workgroup: the barrier orders the two, and a fence of wider scope would write the XCD's L2
            // back, 0.7 ms a forward.)
            // (The wait for this wave's stores to be acknowledged is not something the barrier asks for on this
            // device, whose waves of a workgroup share an L1 that keeps their accesses in order; it costs nothing
            // measurable and leaves nothing to that order.)
            if (FF && second) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (q != q0 || second) __syncthreads();
#pragma unroll
            for (int i = 0; i < IT; ++i) {
                const int f = tid + i * NT;
                reinterpret_cast<f4*>(tb)[f] = VIRT ? merged4(v[i], vv[i], vt) : v[i];
            }
            if (tid == 0) ctr[0] = 0;
            f4 bias8 = {0.f, 0.f, 0.f, 0.f};
            if (F16) bias8 = load_pair8(reinterpret_cast<const char*>(fz.b16) + c * 64 + j * 8, half_bytes);
            if (FF && tid < kTileCols / 4)
                lbias[second * (kTileCols / 4) + tid] = *reinterpret_cast<const f4*>(ff.bias + c * kTileCols + tid * 4);
            __syncthreads();
            if (q == q0 && !second) {
                nunit = __builtin_amdgcn_readfirstlane((int)ctr[1]);
                if (nunit < nunits) NNUEFT_UNIT(nunit, Cn, qn0, qn1)
            }
            if (FF && !second) {
                NNUEFT_LOAD_TILE(C.block, c + partner)
            } else if (q + qs < q1) {
                NNUEFT_LOAD_TILE(C.block, x * tiles_per_xcd + q + qs)
            } else if (nunit < nunits) {
                NNUEFT_LOAD_TILE(Cn.block, x * tiles_per_xcd + qn0)
            }
            int task = 0;
            if (lane == 0) task = (int)atomicAdd(ctr, 1u);
            task = __builtin_amdgcn_readfirstlane(task);
            while (task < ntasks) {
                int nxt = 0;
                if (lane == 0) nxt = (int)atomicAdd(ctr, 1u);
                int s = task * 8 + g;
                const bool valid = s < C.count;
                if (!valid) s = task * 8;
                const uint32_t pc = mpid[s];
                const uint32_t field = pc >> 26;
                const int pair = (int)(pc & 0x3ffffffu);
                const int mx = __builtin_amdgcn_readfirstlane((int)field);   // lists are sorted longest first
                // F16: which half of the output row the pair's bytes go to (asked for here, used after the sums)
                int half = 0;
                if (F16) {
                    const int persp = pair >= B;
                    half = persp == (fz.stm[pair - persp * B] ? 1 : 0) ? 0 : 1;   // half 0 shows the side to move
                }
                // FF, second tile of a visit: the pair's sums of the first tile, back from `saved`, and whether the
                // pair's half of the output row is written here (asked for now, used after the sums)
                bool own_row = false;
                f4 first = {0.f, 0.f, 0.f, 0.f};
                if (FF && second) {
                    const uint32_t mo = moff[s];
                    own_row = (mo & kLoffOwnRow) != 0;
                    half = (mo & kLoffSecondHalf) ? 1 : 0;
                    first = *reinterpret_cast<const f4*>(reinterpret_cast<const char*>(acc) + (size_t)pair * a_pitch +
                                                         (c - partner) * kRowBytes + j * 16);
                }
                f4 a = {0.f, 0.f, 0.f, 0.f};
                if (__ballot(field == kForeign) != 0) {
                    // some list of the task leaves its block: the wave's 8 pairs from global memory
                    const int32_t* ix = pair_list(widx, bidx, pair, B, K);
                    for (int k = 0; k < K; ++k) {
                        const int r = ix[k];
                        if (r >= 0 && r < R) {
                            f4 w = F16 ? load_pair8(Wb + (size_t)r * w_pitch + c * 64 + j * 8, half_bytes)
                                        : *reinterpret_cast<const f4*>(Wb + (size_t)r * w_pitch + c * kRowBytes + j * 16);
                            if (VIRT)
                                w = merged4(w, *reinterpret_cast<const f4*>(vt.V + (size_t)(r % kRows) * out_cols +
                                                                            c * kTileCols + j * 4), vt);
                            acc_add<I16>(a, w);
                        }
                    }
                } else {
                    // the pair's own list is padded to a multiple of 8 entries; what the longest list of the
                    // task has beyond that names the row of zeros
                    uint32_t oo[kSlots / 2];
                    const int own = padded((int)field);
                    const u4* lp = lst + (moff[s] & kLoffMask);
                    constexpr uint32_t zz = (uint32_t)kRows | ((uint32_t)kRows << 16);
#pragma unroll
                    for (int i = 0; i < kSlots / 8; ++i) {
                        const u4 t = i * 8 < own ? lp[i] : u4{zz, zz, zz, zz};
                        oo[4 * i] = t.x; oo[4 * i + 1] = t.y; oo[4 * i + 2] = t.z; oo[4 * i + 3] = t.w;
                    }
                    // blocks of four slots, the next block's reads issued before the current block's adds
                    f4 r[2][4];
#define NNUEFT_ISSUE(buf_, i_)                                                                   \
    r[buf_][0] = lds_read16(row_addr<0>(oo[2 * (i_)], lane_off));          \
    r[buf_][1] = lds_read16(row_addr<1>(oo[2 * (i_)], lane_off));          \
    r[buf_][2] = lds_read16(row_addr<0>(oo[2 * (i_) + 1], lane_off));      \
    r[buf_][3] = lds_read16(row_addr<1>(oo[2 * (i_) + 1], lane_off));
                    NNUEFT_ISSUE(0, 0)
#pragma unroll
                    for (int i = 0; i < kSlots / 4; ++i) {
                        if (i * 4 < mx) {
                            if ((i + 1) * 4 < mx) { NNUEFT_ISSUE((i + 1) & 1, (i + 1) & 7) }
#pragma unroll
                            for (int h = 0; h < 4; ++h) acc_add<I16>(a, r[i & 1][h]);
                        }
                    }
                }
                if (FF && second) {
                    const f4 x0 = first + lbias[j], x1 = a + lbias[kTileCols / 4 + j];
                    if (!finite4(x0) || !finite4(x1)) sched[kSchedNonFinite] = 1u;
                    f4 o;
                    o.x = clamp_act(x0.x, ff.max_act) * clamp_act(x1.x, ff.max_act);
                    o.y = clamp_act(x0.y, ff.max_act) * clamp_act(x1.y, ff.max_act);
                    o.z = clamp_act(x0.z, ff.max_act) * clamp_act(x1.z, ff.max_act);
                    o.w = clamp_act(x0.w, ff.max_act) * clamp_act(x1.w, ff.max_act);
                    if (ff.act.on) {
                        o.x = (floorf(o.x * ff.act.scale + ff.act.eps) / ff.act.scale) * ff.act.post_mul;
                        o.y = (floorf(o.y * ff.act.scale + ff.act.eps) / ff.act.scale) * ff.act.post_mul;
                        o.z = (floorf(o.z * ff.act.scale + ff.act.eps) / ff.act.scale) * ff.act.post_mul;
                        o.w = (floorf(o.w * ff.act.scale + ff.act.eps) / ff.act.scale) * ff.act.post_mul;
                    }
                    if (valid) {
                        const int pos = pair >= B ? pair - B : pair;
                        __builtin_nontemporal_store(a, reinterpret_cast<f4*>(reinterpret_cast<char*>(acc) + (size_t)pair * a_pitch +
                                                                             c * kRowBytes + j * 16));
                        if (own_row)
                            __builtin_nontemporal_store(o, reinterpret_cast<f4*>(reinterpret_cast<char*>(ff.l0) + (size_t)pos * a_pitch +
                                                                                 (size_t)half * (a_pitch >> 1) +
                                                                                 (c - partner) * kRowBytes + j * 16));
                    }
                } else if (FF) {
                    // first tile of a visit: a plain store, the sums are read back after the second
                    if (valid)
                        *reinterpret_cast<f4*>(reinterpret_cast<char*>(acc) + (size_t)pair * a_pitch + c * kRowBytes + j * 16) = a;
                } else if (F16) {
                    acc_add<true>(a, bias8);
                    const us8 s8 = __builtin_bit_cast(us8, a);
                    uint32_t o4 = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int c0 = min(max((int)(short)s8[e], 0), fz.clip_max);
                        const int c1 = min(max((int)(short)s8[e + 4], 0), fz.clip_max);
                        o4 |= ((uint32_t)((c0 * c1) >> fz.shift) & 0xffu) << (8 * e);
                    }
                    if (valid) {
                        const int pos = pair >= B ? pair - B : pair;
                        // streaming store: 32 bytes a pair and tile, written once (measured 0.43 against 0.455 ms
                        // for the whole forward at B = 65536 with a plain store)
                        __builtin_nontemporal_store(o4, reinterpret_cast<uint32_t*>(fz.out + (size_t)pos * L1 + (size_t)half * (L1 >> 1) +
                                                                                 c * 32 + j * 4));
                    }
                } else if (valid)
                    __builtin_nontemporal_store(a, reinterpret_cast<f4*>(reinterpret_cast<char*>(acc) + (size_t)pair * a_pitch +
                                                                         c * kRowBytes + j * 16));
                task = __builtin_amdgcn_readfirstlane(nxt);
            }
        }
        unit = nunit;
        C = Cn;
        q0 = qn0;
        q1 = qn1;
    }
#undef NNUEFT_UNIT
#undef NNUEFT_LOAD_TILE
}

// The gather may ask for most of a CU's LDS; that permission belongs to the loaded kernel on a device
// and is given once per device.
constexpr int kMaxDevices = 64;
std::atomic<int> g_lds_allowed[kMaxDevices];

int allow_lds(int device) {
    if (device < 0 || device >= kMaxDevices) return NNUEFT_E_UNSUPPORTED;
    if (g_lds_allowed[device].load(std::memory_order_acquire)) return 0;
    hipError_t e = hipFuncSetAttribute((const void*)k_acc_tile<kAccThreads, false, false>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e == hipSuccess)
        e = hipFuncSetAttribute((const void*)k_acc_tile<kAccThreadsVirtual, true, false>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e == hipSuccess)
        e = hipFuncSetAttribute((const void*)k_acc_tile<kAccThreads, false, true, kFuse16>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e == hipSuccess)
        e = hipFuncSetAttribute((const void*)k_acc_tile<kAccThreads, false, false, kFuseF>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e != hipSuccess) return (int)e;
    g_lds_allowed[device].store(1, std::memory_order_release);
    return 0;
}

int launch_binscan(uint32_t* hist, uint32_t* total, int nbins, int ngroups, hipStream_t st) {
    hipLaunchKernelGGL(k_tl_binscan, dim3((nbins + kSortThreads / 64 - 1) / (kSortThreads / 64)), dim3(kSortThreads), 0, st, hist,
                       total, nbins, ngroups);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

int launch_sort(const int32_t* widx, const int32_t* bidx, int B, int K, int R, const Layout& L, void* ws, hipStream_t st,
                Sorted* out, SortExtras ex) {
    if ((ex.us != nullptr) != (ex.them != nullptr) || ((ex.us || ex.wpsqt) && L.npairs != 2 * B)) return NNUEFT_E_ARG;
    if (ex.wpsqt && !(ex.bpsqt && ex.psqt_idx && ex.W && ex.bias)) return NNUEFT_E_ARG;
    if (ex.psqt_out && (L.npairs != 2 * B || !ex.psqt_idx || !ex.stm || (ex.n_psqt > 0 && !ex.psqt32))) return NNUEFT_E_ARG;
    char* base = (char*)ws;
    uint32_t* hist = (uint32_t*)(base + L.hist);
    uint16_t* lists = (uint16_t*)(base + L.lists);
    uint32_t* pidcnt = (uint32_t*)(base + L.pidcnt);
    uint16_t* loff = (uint16_t*)(base + L.loff);
    Chunk* chunks = (Chunk*)(base + L.chunks);
    uint32_t* sched = (uint32_t*)(base + L.sched);
    uint32_t* total = (uint32_t*)(base + L.total);
    BlockRec* brec = (BlockRec*)(base + L.brec);
    uint32_t* cpool8 = (uint32_t*)(base + L.cpool8);
    uint32_t* border = (uint32_t*)(base + L.border);
    const int vec = (K % 4 == 0) && aligned16(widx) && aligned16(bidx);
    hipLaunchKernelGGL(k_tl_hist, dim3(L.ngroups), dim3(kSortThreads), 0, st, widx, bidx, hist, L.npairs, B, K, R, L.nbins, vec,
                       L.block_rows);
    NNUEFT_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_tl_binscan, dim3((L.nbins + kSortThreads / 64 - 1) / (kSortThreads / 64)), dim3(kSortThreads), 0, st, hist,
                       total, L.nbins, L.ngroups);
    NNUEFT_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_tl_lists, dim3(L.ngroups), dim3(kSortThreads), 0, st, widx, bidx, hist, total, lists, pidcnt,
                       loff, chunks, sched, brec, cpool8, border, L.npairs, B, K, R, L.nblocks, L.nbins, vec, L.block_rows,
                       ex);
    NNUEFT_LAUNCH_CHECK();
    *out = Sorted{lists, pidcnt, loff, chunks, brec, cpool8, border, sched};
    return 0;
}

// Sort of the lists and the gather of every pair's row sums into `sums` ([2, B, L1] floats, or with `i16` 16-bit
// integers over a table W of [R, L1] int16).
static int gather_tile(const int32_t* widx, const int32_t* bidx, const void* W, void* sums, int B, int K, int R, int L1,
                       int out_cols, void* ws, hipStream_t st, VirtualTable vt, bool i16, int block_rows = kRows,
                       Fuse16 fz = Fuse16{nullptr, nullptr, nullptr, 0, 0, nullptr, nullptr, nullptr, 0},
                       FuseF ff = FuseF{nullptr, nullptr, nullptr, nullptr, 0.0f, ActGrid{1.0f, 0.0f, 1.0f, 0}, nullptr, nullptr,
                                        nullptr},
                       const uint32_t** nonfinite = nullptr) {
    if (ff.l0 && (i16 || vt.V || L1 % (2 * kTileCols) != 0)) return NNUEFT_E_ARG;   // the tiles must come in pairs
    Layout L;
    if (!layout(2 * B, R, &L, block_rows)) return NNUEFT_E_UNSUPPORTED;
    int device = 0;
    const nnueft_dev::DeviceInfo* info = nullptr;
    int rc = nnueft_dev::device_info(&device, &info);
    if (rc) return rc;
    rc = allow_lds(device);
    if (rc) return rc;
    Sorted S;
    SortExtras ex{};
    ex.us = ff.us;
    ex.them = ff.them;
    if (ff.wpsqt) {
        // the sort sums the psqt chains on its way
        ex.psqt_idx = ff.psqt_idx;
        ex.W = (const float*)W;
        ex.bias = ff.bias;
        ex.wpsqt = ff.wpsqt;
        ex.bpsqt = ff.bpsqt;
        ex.L1 = L1;
        ex.n_psqt = out_cols - L1;
    }
    if (fz.psqt_out) {
        ex.psqt_idx = fz.psqt_idx;
        ex.n_psqt = fz.n_psqt;
        ex.psqt32 = fz.psqt32;
        ex.stm = fz.stm;
        ex.psqt_out = fz.psqt_out;
    }
    rc = launch_sort(widx, bidx, B, K, R, L, ws, st, &S, ex);
    if (rc) return rc;
    const uint16_t* lists = S.lists;
    const uint32_t* pidcnt = S.pidcnt;
    const uint16_t* loff = S.loff;
    const Chunk* chunks = S.chunks;
    uint32_t* sched = S.sched;
    // what the XCDs share out: tiles, or (ff) pairs of a tile and the one L1/2 columns further on
    const int ntiles = i16 || ff.l0 ? L1 / (2 * kTileCols) : L1 / kTileCols;
    const int tiles_per_xcd = (ntiles + kXcd - 1) / kXcd;
    // about three tiles (two pairs) per visit of a chunk: its lists are copied into LDS once per visit, and a batch
    // is cut into enough units for the CUs of an XCD to finish together
    const int per_visit = ff.l0 ? 2 : 3;
    int tile_group = (tiles_per_xcd + (tiles_per_xcd + per_visit - 1) / per_visit - 1) / ((tiles_per_xcd + per_visit - 1) / per_visit);
#ifdef NNUEFT_TUNE_ENV
    if (const char* e = getenv("NNUEFT_TILE_GROUP")) tile_group = atoi(e) > 0 ? atoi(e) : tile_group;
#endif
    const int grid = info->cus / kXcd * kXcd;
    const float* Wf = (const float*)W;
    float* sf = (float*)sums;
    if (i16 && fz.out)
        hipLaunchKernelGGL((k_acc_tile<kAccThreads, false, true, kFuse16>), dim3(grid), dim3(kAccThreads), kLdsBytes, st, widx,
                           bidx, lists, pidcnt, loff, chunks, sched, Wf, sf, B, K, R, L1, out_cols, tiles_per_xcd,
                           tile_group, vt, L.block_rows, fz, ff);
    else if (i16)
        return NNUEFT_E_ARG;   // the quantized table is only gathered with the fused epilogue
    else if (ff.l0)
        hipLaunchKernelGGL((k_acc_tile<kAccThreads, false, false, kFuseF>), dim3(grid), dim3(kAccThreads), kLdsBytes, st,
                           widx, bidx, lists, pidcnt, loff, chunks, sched, Wf, sf, B, K, R, L1, out_cols, tiles_per_xcd,
                           tile_group, vt, L.block_rows, fz, ff);
    else if (vt.V)
        hipLaunchKernelGGL((k_acc_tile<kAccThreadsVirtual, true, false>), dim3(grid), dim3(kAccThreadsVirtual), kLdsBytes, st,
                           widx, bidx, lists, pidcnt, loff, chunks, sched, Wf, sf, B, K, R, L1, out_cols, tiles_per_xcd,
                           tile_group, vt, L.block_rows, fz, ff);
    else
        hipLaunchKernelGGL((k_acc_tile<kAccThreads, false, false>), dim3(grid), dim3(kAccThreads), kLdsBytes, st, widx, bidx,
                           lists, pidcnt, loff, chunks, sched, Wf, sf, B, K, R, L1, out_cols, tiles_per_xcd,
                           tile_group, vt, L.block_rows, fz, ff);
    NNUEFT_LAUNCH_CHECK();
    if (nonfinite) *nonfinite = sched + kSchedNonFinite;
    return 0;
}

int double_fwd_tile(const float* us, const float* them, const int32_t* widx, const int32_t* bidx,
                    const int64_t* psqt_idx, const float* W, const float* bias, float max_act, float* l0,
                    float* wpsqt, float* bpsqt, float* saved, int B, int K, int R, int L1, int n_psqt, void* ws,
                    hipStream_t st, ActGrid act, VirtualTable vt) {
    // The gather finishes the output rows itself where that pays: tiles that come in pairs, four pairs or more for
    // every XCD (L1 >= 2048: forward 0.25 -> 0.22 ms at L1 = 2048, 0.34 -> 0.31 ms at L1 = 3072, B = 16384; narrower
    // rows leave the XCD's CUs too few units to share, 0.086 -> 0.092 ms at L1 = 1024, B = 8192), a table that is not
    // merged on the fly (that variant has no registers to spare).  Else the sums first, then the pass over them.
    bool pairs = !vt.V && L1 % (2 * kTileCols) == 0 && L1 / (2 * kTileCols) >= 4 * kXcd;
#ifdef NNUEFT_NO_FWD_FUSE
    pairs = false;
#endif
    if (!pairs) {
        // (the psqt chains out of the sort here too, unless the table is merged on the fly: the sort does not merge)
        const bool sort_psqt = !vt.V;
        FuseF none{};
        if (sort_psqt) {
            none.bias = bias;
            none.psqt_idx = psqt_idx;
            none.wpsqt = wpsqt;
            none.bpsqt = bpsqt;
        }
        const int rc = gather_tile(widx, bidx, W, saved, B, K, R, L1, L1 + n_psqt, ws, st, vt, false, kRows,
                                   Fuse16{nullptr, nullptr, nullptr, 0, 0, nullptr, nullptr, nullptr, 0}, none);
        if (rc) return rc;
        return nnueft_blocked::launch_mix(us, them, widx, bidx, psqt_idx, W, bias, saved, max_act, l0,
                                          sort_psqt ? nullptr : wpsqt, sort_psqt ? nullptr : bpsqt, B, K, R, L1, n_psqt, st,
                                          act, vt, nullptr);
    }
    // the gather writes the sums and, where one perspective's sums are all a half row needs, the output row too
    const uint32_t* nonfinite = nullptr;
    const int rc = gather_tile(widx, bidx, W, saved, B, K, R, L1, L1 + n_psqt, ws, st, vt, false, kRows,
                               Fuse16{nullptr, nullptr, nullptr, 0, 0, nullptr, nullptr, nullptr, 0},
                               FuseF{us, them, bias, l0, max_act, act, psqt_idx, wpsqt, bpsqt}, &nonfinite);
    if (rc) return rc;
    // (the psqt chains are done: no psqt outputs for the pass)
    return nnueft_blocked::launch_mix(us, them, widx, bidx, psqt_idx, W, bias, saved, max_act, l0, nullptr, nullptr, B,
                                      K, R, L1, n_psqt, st, act, vt, nonfinite);
}

bool fits_int16(const nnueft_dev::DeviceInfo& d, int B, int K, int R, int L1, int block_rows) {
    Layout L;
    return L1 % (2 * kTileCols) == 0 && fits(d, B, K, R, L1) && layout(2 * B, R, &L, block_rows) &&
           L.max_chunks <= kMaxChunks;
}

size_t workspace_int16(int B, int R, int block_rows) {
    Layout L;
    return B < (1 << 25) && layout(2 * B, R, &L, block_rows) ? L.end : 0;
}

int int16_fused_tile(const int32_t* widx, const int32_t* bidx, const uint8_t* stm, const int16_t* W16, const int16_t* b16,
                     const int32_t* psqt32, const int64_t* psqt_idx, uint8_t* out_u8, int32_t* psqt_out, int B, int K, int R,
                     int L1, int n_psqt, int clip_max, int shift, int block_rows, void* ws, hipStream_t st) {
    return gather_tile(widx, bidx, W16, nullptr, B, K, R, L1, L1, ws, st, VirtualTable{nullptr, 1.0f, 1.0f, 0, 0.0f}, true,
                       block_rows, Fuse16{stm, b16, out_u8, clip_max, shift, psqt32, psqt_idx, psqt_out, n_psqt});
}

}  // namespace nnueft_tile
