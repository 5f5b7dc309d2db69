// Backward, atomic mode, LDS-tiled: the scatter adds into a tile of the weight gradient that lives in LDS.
//
// The mirror image of the forward's gather out of LDS tiles (fwd_tile.hip).  All indices of one list name rows of
// one 768-row block of the table, so a workgroup can keep a tile of the gradient of that block in LDS, walk every
// (position, perspective) pair of the block, and add the pair's upstream values with LDS atomics into every row
// the pair's list names.  The tile is then written out once: the dense gradient is fully written (no zero-fill
// before, no global atomic), and the upstream rows are read once.
//
// The tile holds doubles, 768 rows x 16 columns (96 KB): on this part an LDS atomic add of 32-bit floats is
// carried out lane by lane (about 190 clocks per wave instruction, measured), one of 64-bit floats takes about 8.
// 4 lanes a pair, each lane with 16 bytes of the pair's upstream row; the sums are rounded to float once, on the
// way out, so they are closer to the exact sum than any float chain.  The order in which the waves of a
// workgroup reach a row is not fixed: a sum can differ in its last float bit from run to run where the double
// sums straddle a rounding boundary.
//
//   k_bwd_rows       upstream rows G[2, B, pitch] and the bias partial sums (bwd_det.hip)
//   k_tl_*           the forward's sort of the pairs by (table block, list length) (fwd_tile.hip)
//   k_scatter_tile   persistent workgroups, one per CU: units of (table block, column tile) handed out per XCD,
//                    blocks with the most pairs first; waves take batches of 64 pairs from a counter in LDS; the
//                    loads of a task (16 pairs) are issued before the adds of the task in front of it, those of a
//                    unit's first tasks before the tile of the unit in front of it is written out
//   k_scatter_foreign  lists that name rows of more than one block (the interface allows them): global atomics
//                    on the written gradient
//   k_bias_final     chain over the bias partial sums (bwd_det.hip)
#include <atomic>

#include "tile_sort.h"

namespace nnueft_tile {

namespace {

#ifndef NNUEFT_SCATTER_NT
#define NNUEFT_SCATTER_NT 1024
#endif
constexpr int kScThreads = NNUEFT_SCATTER_NT;
constexpr int kScCols = 16;                            // columns of a gradient tile (doubles in LDS)
constexpr int kScTile = (kRows + 1) * kRowBytes;       // + one row that takes the adds of the padding slots and is never written out
constexpr int kScLds = kScTile + 64;
static_assert(kScCols * 8 == kRowBytes, "a tile row of doubles is as long as the forward's row of floats");

typedef __attribute__((address_space(3))) double lds_double;
typedef double d2 __attribute__((ext_vector_type(2)));

// The atomic add the scatter is built on.  LDS adds of 64-bit floats run at about 8 clocks per wave instruction
// on this part; those of 32-bit floats are carried out lane by lane (about 190 clocks per wave instruction).
__device__ __forceinline__ void lds_add(uint32_t addr, double v) {
    __hip_atomic_fetch_add(reinterpret_cast<lds_double*>(addr), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

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

// What a lane knows of one pair of a batch.
struct Meta {
    uint32_t pc;   // pair id | count << 26 (0: no pair)
    uint32_t la;   // where its list begins, in units of 8 entries
};

constexpr int kTaskPairs = 16;   // pairs a wave adds side by side: 4 lanes a pair
#ifndef NNUEFT_SCATTER_BATCH
#define NNUEFT_SCATTER_BATCH 1
#endif
constexpr int kBatchTasks = NNUEFT_SCATTER_BATCH;   // tasks a wave takes per ticket (their pairs' facts are loaded a lane each)
static_assert(kBatchTasks * kTaskPairs <= 64, "a lane per pair of a batch");

__device__ __forceinline__ Meta load_meta(const BlockRec& rec, int tpc, int ntasks, int batch, int lane,
                                          const uint32_t* __restrict__ pidcnt, const uint16_t* __restrict__ loff,
                                          const uint32_t* __restrict__ cpool8) {
    Meta m{0u, 0u};
    const int t = batch * kBatchTasks + lane / kTaskPairs;
    if (t < ntasks && lane < kBatchTasks * kTaskPairs) {
        const int jc = t / tpc;
        const int local = (t - jc * tpc) * kTaskPairs + lane % kTaskPairs;
        if (local < ranks_of_chunk(rec.nb, jc, rec.nc)) {
            const int s = rec.base + jc * rec.len + local;
            m.pc = pidcnt[s];
            m.la = cpool8[rec.chunk0 + jc] + (uint32_t)loff[s];
        }
    }
    return m;
}

// A unit of work: one table block x one column tile.
struct Unit {
    int blk, c, cols;
    BlockRec rec;
    int tpc, ntasks, nbatch;
};

// A task on its way into registers: the lists of 16 pairs (every lane of a pair holds the pair's list) and the
// lane's four upstream values.
struct Task {
    u4 l[kSlots / 8];
    f4 gv;
    int mx;   // the longest list of the task (0: nothing to do)
};

// gW[rows of a block, 16 columns] = sum over the block's pairs of the pair's upstream values, added to every row
// its list names; double precision in LDS, rounded once on the way out.
template <int NT>
__global__ __launch_bounds__(NT) void k_scatter_tile(const uint16_t* __restrict__ lists,
                                                     const uint32_t* __restrict__ pidcnt,
                                                     const uint16_t* __restrict__ loff,
                                                     const BlockRec* __restrict__ brec,
                                                     const uint32_t* __restrict__ cpool8,
                                                     const uint32_t* __restrict__ border,
                                                     uint32_t* __restrict__ sched, const float* __restrict__ G,
                                                     int g_pitch, float* __restrict__ gW, int R, int out_cols,
                                                     int main_tiles, int tpx, int tail_cols, int nblocks,
                                                     int block_rows) {
    extern __shared__ float4 lds_raw[];
    char* tb = reinterpret_cast<char*>(lds_raw);
    // [0] batch counter, [1], [2] the units this workgroup works on next (written one iteration ahead, in turns)
    uint32_t* ctr = reinterpret_cast<uint32_t*>(tb + kScTile);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    constexpr int NW = NT / 64;
    constexpr int NP = kRows * (kScCols / 4);   // pieces of four columns in a tile
    static_assert(NP % NT == 0, "tile write-out");
    constexpr int IT = NP / NT;
    const int x = blockIdx.x % kXcd;
    // the column tiles of this XCD: a run of whole tiles, and of the tile of the last out_cols % 16 columns the
    // blocks ranked x, x + 8, ...
    const int my_tiles = max(0, min(tpx, main_tiles - x * tpx));
    const int nmain = nblocks * my_tiles;
    const int ntail = tail_cols && nblocks > x ? (nblocks - x + kXcd - 1) / kXcd : 0;
    const int nunits = nmain + ntail;
    uint32_t* unit_ctr = sched + x * 32;
    const int g = lane >> 2, li = lane & 3;
    const uint32_t tile_base = (uint32_t)(uintptr_t)tb;   // low half of a flat LDS address = the byte address inside LDS
    // a lane adds its four values in an order rotated by its pair's place in the task, so that the 16 pairs of
    // an instruction spread evenly over the LDS banks whatever rows they add to
    uint32_t off[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) off[d] = tile_base + li * 32 + ((d + g) & 3) * 8;

    auto decode = [&](int u) {
        Unit U{};
        if (u >= nunits) return U;
        int r;
        if (u < nmain) {
            r = u / my_tiles;
            U.c = x * tpx + (u - r * my_tiles);
            U.cols = kScCols;
        } else {
            r = (u - nmain) * kXcd + x;
            U.c = main_tiles;
            U.cols = tail_cols;
        }
        U.blk = (int)border[r];
        U.rec = brec[U.blk];
        U.tpc = (U.rec.len + kTaskPairs - 1) / kTaskPairs;   // tasks per chunk
        U.ntasks = U.rec.nc * U.tpc;
        U.nbatch = (U.ntasks + kBatchTasks - 1) / kBatchTasks;
        return U;
    };
    // the longest list of each task of a batch, in every lane of the task
    auto task_max = [&](const Meta& m) {
        const uint32_t field = m.pc >> 26;
        int cm = field == kForeign ? 0 : (int)field;
        cm = max(cm, __shfl_xor(cm, 1));
        cm = max(cm, __shfl_xor(cm, 2));
        cm = max(cm, __shfl_xor(cm, 4));
        cm = max(cm, __shfl_xor(cm, 8));
        return cm;
    };
    // entries beyond a pair's own count (its padding, and what the longest list of the task has more) name the spare row
    constexpr uint32_t zz = (uint32_t)kRows | ((uint32_t)kRows << 16);
    auto issue = [&](const Unit& U, const Meta& m, int cm, int k) {
        Task T;
        T.mx = __builtin_amdgcn_readlane(cm, k * kTaskPairs);
        const uint32_t pck = (uint32_t)__shfl((int)m.pc, k * kTaskPairs + g);
        const uint32_t lak = (uint32_t)__shfl((int)m.la, k * kTaskPairs + g);
        const uint32_t fk = pck >> 26;
        const int ck = fk == kForeign ? 0 : (int)fk;
        const size_t pair = pck & 0x3ffffffu;
        const u4* lp = reinterpret_cast<const u4*>(lists) + lak;
#pragma unroll
        for (int i = 0; i < kSlots / 8; ++i) T.l[i] = i * 8 < ck ? lp[i] : u4{zz, zz, zz, zz};
        T.gv = f4{0.f, 0.f, 0.f, 0.f};
        if (ck > 0 && U.c * kScCols + li * 4 < out_cols)
            T.gv = *reinterpret_cast<const f4*>(G + pair * (size_t)g_pitch + U.c * kScCols + li * 4);
        return T;
    };
    auto no_task = [&]() {
        Task T;
#pragma unroll
        for (int i = 0; i < kSlots / 8; ++i) T.l[i] = u4{zz, zz, zz, zz};
        T.gv = f4{0.f, 0.f, 0.f, 0.f};
        T.mx = 0;
        return T;
    };
    // every lane adds at every slot up to the task's longest list: zeros change nothing, and a branch around
    // them costs more than the add
    auto process = [&](const Task& T) {
        if (T.mx == 0) return;
        // val[d] = gv[(d + g) & 3]
        const int rot = g & 3;
        const float a0 = (rot & 1) ? T.gv.y : T.gv.x, a1 = (rot & 1) ? T.gv.z : T.gv.y;
        const float a2 = (rot & 1) ? T.gv.w : T.gv.z, a3 = (rot & 1) ? T.gv.x : T.gv.w;
        double val[4];
        val[0] = (double)((rot & 2) ? a2 : a0);
        val[1] = (double)((rot & 2) ? a3 : a1);
        val[2] = (double)((rot & 2) ? a0 : a2);
        val[3] = (double)((rot & 2) ? a1 : a3);
#pragma unroll
        for (int i = 0; i < kSlots; ++i) {
            if ((i & 3) == 0 && i >= T.mx) break;
            const u4 q = T.l[i >> 3];
            const uint32_t w = ((i >> 1) & 3) == 0 ? q.x : ((i >> 1) & 3) == 1 ? q.y : ((i >> 1) & 3) == 2 ? q.z : q.w;
#pragma unroll
            for (int d = 0; d < 4; ++d) lds_add((i & 1) ? row_addr<1>(w, off[d]) : row_addr<0>(w, off[d]), val[d]);
        }
    };

    for (int i = tid; i < kScTile / 16; i += NT) reinterpret_cast<f4*>(tb)[i] = f4{0.f, 0.f, 0.f, 0.f};
    if (tid == 0) {
        ctr[0] = NW;
        ctr[1] = atomicAdd(unit_ctr, 1u);
    }
    __syncthreads();
    int unit = __builtin_amdgcn_readfirstlane((int)ctr[1]);
    Unit U = decode(unit);
    Meta mt = load_meta(U.rec, U.tpc, U.ntasks, wave, lane, pidcnt, loff, cpool8);
    int cm = task_max(mt);
    Task cur = wave < U.nbatch ? issue(U, mt, cm, 0) : no_task();
    for (int it = 0; unit < nunits; ++it) {
        uint32_t* next_slot = ctr + 1 + ((it + 1) & 1);
        if (tid == 0) *next_slot = atomicAdd(unit_ctr, 1u);
        __syncthreads();   // the tile is zero, the batch counter is set, the next unit is known
        const int nunit = __builtin_amdgcn_readfirstlane((int)*next_slot);
        // the next unit's first batch of this wave: on its way while the current unit is added
        const Unit Un = decode(nunit);
        const Meta mtn = load_meta(Un.rec, Un.tpc, Un.ntasks, wave, lane, pidcnt, loff, cpool8);
        int batch = wave;
        while (batch < U.nbatch) {
            int nxt = 0;
            if (lane == 0) nxt = (int)atomicAdd(ctr, 1u);
            nxt = __builtin_amdgcn_readfirstlane(nxt);
            const Meta mn = load_meta(U.rec, U.tpc, U.ntasks, nxt, lane, pidcnt, loff, cpool8);
            int cmn = 0;
            // the loads of a task are issued before the adds of the task in front of it
#pragma unroll
            for (int k = 0; k < kBatchTasks; ++k) {
                Task nx;
                if (k + 1 < kBatchTasks) {
                    nx = issue(U, mt, cm, k + 1);
                } else {
                    cmn = task_max(mn);
                    nx = nxt < U.nbatch ? issue(U, mn, cmn, 0) : no_task();
                }
                process(cur);
                cur = nx;
            }
            batch = nxt;
            mt = mn;
            cm = cmn;
        }
        const int cmf = task_max(mtn);
        const Task first = (nunit < nunits && wave < Un.nbatch) ? issue(Un, mtn, cmf, 0) : no_task();
        __syncthreads();   // every add of the unit has landed
        const int row0 = U.blk * block_rows;
        const int rows_here = min(block_rows, R - row0);
        float* dst = gW + (size_t)row0 * out_cols + U.c * kScCols;
#pragma unroll
        for (int i = 0; i < IT; ++i) {
            const int f = tid + i * NT;
            const int row = f >> 2, q = f & 3;
            d2* src = reinterpret_cast<d2*>(tb + row * kRowBytes + q * 32);
            const d2 lo = src[0], hi = src[1];
            src[0] = d2{0.0, 0.0};
            src[1] = d2{0.0, 0.0};
            if (row < rows_here && q * 4 < U.cols)
                __builtin_nontemporal_store(f4{(float)lo.x, (float)lo.y, (float)hi.x, (float)hi.y},
                                            reinterpret_cast<f4*>(dst + (size_t)row * out_cols + q * 4));
        }
        if (tid == 0) ctr[0] = NW;
        unit = nunit;
        U = Un;
        mt = mtn;
        cm = cmf;
        cur = first;
    }
}

// One wave per pair: a list that names rows of more than one table block was left out by k_scatter_tile and is
// added here, after the tiles have been written.  The test is the sort's (list_facts in fwd_tile.hip): the block
// of the first valid entry, and whether every other valid entry stays inside it.
__global__ __launch_bounds__(256) void k_scatter_foreign(const int32_t* __restrict__ widx,
                                                         const int32_t* __restrict__ bidx,
                                                         const float* __restrict__ G, int g_pitch,
                                                         float* __restrict__ gW, int npairs, int B, int K, int R,
                                                         int out_cols, int block_rows) {
    const int lane = threadIdx.x & 63;
    const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (pair >= npairs) return;
    const int p = pair >= B;
    const int32_t* ix = (p ? bidx : widx) + (size_t)(pair - p * B) * K;
    const int my = lane < K ? ix[lane] : -1;
    const bool ok = my >= 0 && my < R;
    u64 mask = __ballot(ok);
    if (!mask) return;
    const int first = __builtin_amdgcn_readlane(my, __ffsll((long long)mask) - 1);
    const int base = first / block_rows * block_rows;
    if (!__ballot(ok && (my < base || my >= base + block_rows))) return;
    const float* grow = G + (size_t)pair * g_pitch;
    while (mask) {
        float* row = gW + (size_t)bcast_i(my, pop_lane(mask)) * out_cols;
        for (int c0 = lane; c0 < out_cols; c0 += 64) {
            const float v = grow[c0];
            if (v != 0.0f) atomicAdd(row + c0, v);
        }
    }
}

constexpr int kMaxDevices = 64;
std::atomic<int> g_scatter_lds_allowed[kMaxDevices];

int allow_scatter_lds(int device) {
    if (device < 0 || device >= kMaxDevices) return NNUEFT_E_UNSUPPORTED;
    if (g_scatter_lds_allowed[device].load(std::memory_order_acquire)) return 0;
    const hipError_t e = hipFuncSetAttribute((const void*)k_scatter_tile<kScThreads>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, kScLds);
    if (e != hipSuccess) return (int)e;
    g_scatter_lds_allowed[device].store(1, std::memory_order_release);
    return 0;
}

struct ScatterLayout {
    size_t G, partial, sort, end;
    int g_pitch, ntiles;
    Layout L;
};

bool scatter_layout(int B, int K, int R, int out_cols, int n_persp, ScatterLayout* S) {
    if (B <= 0 || B >= (1 << 25) || K <= 0 || K > kSlots || R <= 0 || out_cols <= 0 || out_cols % 4 ||
        (n_persp != 1 && n_persp != 2))
        return false;
    if (!layout(n_persp * B, R, &S->L) || S->L.max_chunks > kMaxChunks) return false;
    S->g_pitch = n_persp == 2 ? nnueft_det_upstream_pitch(out_cols) : out_cols;
    S->ntiles = (B + NNUEFT_BIAS_TILE - 1) / NNUEFT_BIAS_TILE;
    size_t off = 0;
    S->G = off;
    off += up256(n_persp == 2 ? (size_t)2 * B * S->g_pitch * sizeof(float) : 0);
    S->partial = off;
    off += up256((size_t)S->ntiles * out_cols * sizeof(float));
    S->sort = off;
    off += S->L.end;
    S->end = off;
    return true;
}

// gW = scatter of the upstream rows G[npairs, g_pitch] over the lists; every element of gW is written.
int scatter(const int32_t* widx, const int32_t* bidx, const float* G, int g_pitch, float* gW, int B, int K, int R,
            int out_cols, int n_persp, const Layout& L, void* sort_ws, hipStream_t st) {
    int device = 0;
    const nnueft_dev::DeviceInfo* info = nullptr;
    int rc = nnueft_dev::device_info(&device, &info);
    if (rc) return rc;
    if (info->xcds != kXcd || info->cus < kXcd || info->max_lds < kScLds) return NNUEFT_E_UNSUPPORTED;
    rc = allow_scatter_lds(device);
    if (rc) return rc;
    Sorted S;
    rc = launch_sort(widx, bidx, B, K, R, L, sort_ws, st, &S);
    if (rc) return rc;
    const int main_tiles = out_cols / kScCols;
    const int tail_cols = out_cols % kScCols;
    const int tpx = (main_tiles + kXcd - 1) / kXcd;
    const int grid = info->cus / kXcd * kXcd;
    hipLaunchKernelGGL((k_scatter_tile<kScThreads>), dim3(grid), dim3(kScThreads), kScLds, st, S.lists,
                       S.pidcnt, S.loff, S.brec, S.cpool8, S.border, S.sched, G, g_pitch, gW, R, out_cols, main_tiles, tpx,
                       tail_cols, L.nblocks, L.block_rows);
    NNUEFT_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_scatter_foreign, dim3((L.npairs + 3) / 4), dim3(256), 0, st, widx, bidx, G, g_pitch, gW, L.npairs, B,
                       K, R, out_cols, L.block_rows);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}

}  // namespace

}  // namespace nnueft_tile

extern "C" size_t nnueft_atomic_lds_workspace_bytes(int B, int K, int R, int out_cols, int n_persp) {
    nnueft_tile::ScatterLayout S;
    return nnueft_tile::scatter_layout(B, K, R, out_cols, n_persp, &S) ? S.end : 0;
}

extern "C" int nnueft_sparse_bwd_atomic_lds(const int32_t* idx, const float* gout, float* gW, float* gbias, int B, int K,
                                            int R, int out_cols, void* workspace, size_t workspace_bytes, void* stream) {
    if (B <= 0 || K <= 0 || R <= 0 || out_cols <= 0) return NNUEFT_E_ARG;
    if (!idx || !gout || !gW || !gbias) return NNUEFT_E_ARG;
    nnueft_tile::ScatterLayout S;
    if (!nnueft_tile::scatter_layout(B, K, R, out_cols, 1, &S)) return NNUEFT_E_UNSUPPORTED;
    if (!workspace || !aligned256(workspace) || workspace_bytes < S.end) return NNUEFT_E_WORKSPACE;
    if (!aligned16(gW) || !aligned16(gout)) return NNUEFT_E_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    char* ws = (char*)workspace;
    float* partial = (float*)(ws + S.partial);
    int rc = nnueft_det::launch_tile_colsum(gout, partial, B, out_cols, st);
    if (rc) return rc;
    rc = nnueft_tile::scatter(idx, idx, gout, out_cols, gW, B, K, R, out_cols, 1, S.L, ws + S.sort, st);
    if (rc) return rc;
    return nnueft_det::launch_bias_final(partial, gbias, B, out_cols, nullptr, st);
}

extern "C" int nnueft_double_bwd_atomic_lds(const float* us, const float* them, const int32_t* widx,
                                            const int32_t* bidx, const int64_t* psqt_idx, const float* bias,
                                            float max_act, const float* grad_l0, const float* grad_wpsqt,
                                            const float* grad_bpsqt, const float* saved, float* gW, float* gbias,
                                            int B, int K, int R, int L1, int n_psqt, void* workspace,
                                            size_t workspace_bytes, void* stream) {
    if (B < 0 || K <= 0 || R <= 0 || L1 <= 0 || (L1 & 1) || n_psqt < 0) return NNUEFT_E_ARG;
    if (B == 0) return NNUEFT_E_ARG;   // nothing to launch over: an empty batch's gradient is the caller's to zero
    if (!us || !them || !widx || !bidx || !psqt_idx || !bias || !grad_l0 || !grad_wpsqt || !grad_bpsqt || !saved ||
        !gW || !gbias)
        return NNUEFT_E_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int out_cols = L1 + n_psqt;
    nnueft_tile::ScatterLayout S;
    if (!nnueft_tile::scatter_layout(B, K, R, out_cols, 2, &S)) return NNUEFT_E_UNSUPPORTED;
    if (!workspace || !aligned256(workspace) || workspace_bytes < S.end) return NNUEFT_E_WORKSPACE;
    if (!aligned16(gW) || !aligned16(saved) || !aligned16(grad_l0) || !aligned16(bias)) return NNUEFT_E_UNSUPPORTED;
    char* ws = (char*)workspace;
    float* G = (float*)(ws + S.G);
    float* partial = (float*)(ws + S.partial);
    int rc = nnueft_det::launch_bwd_rows(us, them, psqt_idx, bias, max_act, grad_l0, grad_wpsqt, grad_bpsqt, saved, G,
                                         S.g_pitch, partial, B, L1, n_psqt, st);
    if (rc) return rc;
    rc = nnueft_tile::scatter(widx, bidx, G, S.g_pitch, gW, B, K, R, out_cols, 2, S.L, ws + S.sort, st);
    if (rc) return rc;
    return nnueft_det::launch_bias_final(partial, gbias, B, out_cols, nullptr, st);
}
