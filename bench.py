#!/usr/bin/env python3
"""Feature-transformer forward+backward throughput on one MI355X.

A step is one pass of the hot path over one synthetic batch: the fused two-perspective forward
(nnueft_double_fwd) and the backward into a dense weight gradient, through the same autograd
function the trainer calls.  Inputs are resident in HBM before the timed region.

Prints ONE JSON line: positions/s for the workload BASELINE.json's metric is quoted on (L1=3072,
B=16384, HalfKAv2_hm lists, 24576-row table); the roofline of the dominant kernel (k_chain_tile, the
strict order's reduction of the deterministic backward out of LDS tiles; k_seg_reduce, the segmented
reduction through L2, for the windowed order and narrow rows) from HIP event timings of the entry point
that launches it alone, against three bounds (algorithmic bytes against the rate of the path that serves
them, the bytes that must cross HBM, and the counter-measured traffic read from profiles/); the same for the
two entry points and the step; and the reference's CPU path (torch embedding_bag composition) timed on
the host cores on the same workload.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "nnue-pytorch_amd"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# L2: 8 XCDs x 16 channels, one 128-byte line per channel and clock, at the published peak engine clock
L2_CHANNELS = 128
L2_LINE_BYTES = 128
ENGINE_CLOCK_GHZ = 2.4
# LDS: 256 CUs, 256 bytes read per CU and clock
LDS_PEAK_GBS = 256 * 256 * ENGINE_CLOCK_GHZ

WORKLOADS = {
    # name: (L1, B)
    "ft_fwd_bwd_L1_3072_B16384": (3072, 16384),     # BASELINE.json config 3: the metric
    "ft_fwd_bwd_L1_1024_B8192": (1024, 8192),       # config 1
    "ft_fwd_bwd_L1_128_B16384": (128, 16384),       # config 2
    "ft_int16_fwd_L1_3072_B65536": (3072, 65536),   # config 5: quantized forward only
    "full_step_L1_3072_B16384": (3072, 16384),      # config 4: FT + layer stacks + loss + optimizer
    "ref_microbench_L1_264_B8192": (264, 8192),     # the reference's own tests/bench_feature_transformer.py
}
R_ROWS = 24576
N_PSQT = 8
K_SLOTS = 32
MAX_ACT = 255.0 / 256.0


# ------------------------------------------------------------------------------------------------
# byte counts

def algorithmic_bytes(L1, B, sum_a, mode):
    """Logical bytes of one step, no reuse between positions assumed (a = active rows of both lists)."""
    oc = L1 + N_PSQT
    fwd = sum_a * oc * 4 + B * (2 * K_SLOTS * 4 + 16 + L1 * 4 + 2 * L1 * 4 + 8)
    if mode == "atomic":
        bwd = sum_a * oc * 8 + B * (L1 * 4 + 2 * L1 * 4 + 2 * K_SLOTS * 4 + 24) + R_ROWS * oc * 4
    else:
        # read grad_l0 + saved, write the two upstream rows, gather them once per slot, one 8-byte
        # key/value pass for the counting sort, every table row written once
        bwd = B * (3 * L1 * 4 + 2 * oc * 4) + sum_a * oc * 4 + sum_a * 8 + R_ROWS * oc * 4
    return fwd, bwd


def seg_reduce_bytes(L1, B, sum_a):
    """k_seg_reduce's part of the deterministic backward's formula: (algorithmic, of which gathered rows,
    compulsory).  Algorithmic: one upstream row per slot + the slot's list entry + every table row written
    once.  Compulsory: the upstream rows once, the list, the dense gradient."""
    oc = L1 + N_PSQT
    gathered = sum_a * oc * 4
    alg = gathered + sum_a * 4 + R_ROWS * oc * 4
    comp = 2 * B * oc * 4 + sum_a * 4 + (R_ROWS + 1) * 8 + R_ROWS * oc * 4
    return alg, gathered, comp


def compulsory_bytes(L1, B, sum_a):
    """Bytes that have to cross HBM once per kernel that reads or writes them, with this decomposition into
    kernels and nothing kept in a cache between kernels: per entry point."""
    oc = L1 + N_PSQT
    lists = 2 * B * K_SLOTS * 4
    saved = 2 * B * L1 * 4
    small = B * 24
    if forward_path(L1) == "tile_pairs":
        fwd = {
            # + the sides to move and the psqt chains (4 bytes per list entry out of the table's psqt columns)
            "list sort": 2 * lists + sum_a * 2 + 2 * B * 6 + B * 8 + sum_a * 4 + small,
            # table once, packed lists, row sums written, output rows written (the sums of a visit's first tile come
            # back from memory once: they have left the XCD's L2 by the time the second tile's are done)
            "k_acc_tile": R_ROWS * oc * 4 + sum_a * 2 + 2 * B * 6 + saved + saved // 2 + B * L1 * 4,
            "k_mix_rest": B * 8,                                          # a look at the sides to move
        }
    elif forward_path(L1) == "tile":
        fwd = {
            # 16-bit lists at their own length, pair id and list place per list
            "list sort": 2 * lists + sum_a * 2 + 2 * B * 6,               # lists twice, packed lists written
            "k_acc_tile": R_ROWS * oc * 4 + sum_a * 2 + 2 * B * 6 + saved,   # table once, packed lists, row sums written
            "k_mix": saved + B * L1 * 4 + small,                          # row sums read, l0 written
        }
    else:
        fwd = {
            "pair sort": lists + 3 * 2 * B * 4,
            "k_acc_blocked": R_ROWS * oc * 4 + lists + saved,             # table once, row sums written
            "k_mix": saved + B * L1 * 4 + small,                          # row sums read, l0 written
        }
    nchunks = 2 * ((B + 127) // 128)
    tiles16 = (oc + 15) // 16
    bwd_chain = {
        "k_bwd_rows": saved + B * L1 * 4 + 2 * B * oc * 4 + small,    # row sums + grad_l0 read, upstream rows written
        # lists three times (key, place, bit map), pair order written, inverted lists (2 bytes an entry) written
        "sort": 3 * lists + 2 * B * 4 + sum_a * 2,
        # upstream rows once, dense gradient once, the inverted lists once per 16-column tile (out of L2 after the first)
        "k_chain_tile": 2 * B * oc * 4 + R_ROWS * oc * 4 + sum_a * 2,
        "bias": 2 * (B // 32) * oc * 4,
    }
    bwd = {
        "k_bwd_rows": saved + B * L1 * 4 + 2 * B * oc * 4 + small,    # row sums + grad_l0 read, upstream rows written
        "sort": 2 * lists + 3 * nchunks * R_ROWS * 4 + sum_a * 4,     # lists twice, chunk counts w/r/w, sorted list
        "k_seg_reduce": seg_reduce_bytes(L1, B, sum_a)[2],
        "bias": 2 * (B // 32) * oc * 4,
    }
    return fwd, bwd, bwd_chain


# the summaries under profiles/ of one workload by backward mode: no suffix = the headline's (strict) order
PROFILE_SUFFIX = {"deterministic_strict": "", "deterministic": "_windowed", "atomic": "_atomic"}


def read_profile_traffic(workload, positions, mode="deterministic_strict"):
    """Counter-measured bytes per dispatch (FETCH_SIZE, WRITE_SIZE scaled by a copy kernel of known size) from the
    tracked summary profiles/<workload>[_game_like][_windowed|_atomic]_pmc.txt: lines
    `traffic <kernel> fetched_bytes=N written_bytes=N`."""
    name = workload + ("_game_like" if positions == "game" else "") + PROFILE_SUFFIX[mode] + "_pmc.txt"
    path = os.path.join(ROOT, "profiles", name)
    out = {}
    if not os.path.exists(path):
        return out, None
    for line in open(path):
        m = re.match(r"traffic\s+(\S+)\s+fetched_bytes=(\d+)\s+written_bytes=(\d+)", line)
        if m:
            out[m.group(1)] = (int(m.group(2)), int(m.group(3)))
    return out, os.path.relpath(path, ROOT)


def sum_traffic(traffic, kernels):
    """Total of the named kernels (prefix match on the kernel name), or None when one is missing."""
    total = 0
    for k in kernels:
        hit = [v for name, v in traffic.items() if name.startswith(k)]
        if not hit:
            return None
        total += sum(f + w for f, w in hit)
    return total


def forward_path(L1):
    """Which gather nnueft_double_fwd takes with a workspace: out of LDS tiles for wide rows (from L1 = 2048 on it visits
    the column tiles in pairs and writes the output rows itself), else blocked for L2."""
    if L1 >= 2048 and L1 % 64 == 0:
        return "tile_pairs"
    return "tile" if L1 >= 512 and L1 % 32 == 0 else "blocked"


def strict_path(L1):
    """Which reduction the strict order takes: chains summed out of LDS tiles for rows of 256 columns and more (lists of
    up to 32 slots, as all workloads here have), else the segmented reduction through L2."""
    return "chain" if L1 + N_PSQT >= 256 else "segmented"


def bwd_kernels(L1, mode):
    """Kernels of the backward entry point by mode (for summing their counter-measured traffic)."""
    if mode == "deterministic_strict" and strict_path(L1) == "chain":
        # (the sort and the reduction of the other path are launched too and return at once: a batch whose lists
        # the tiles cannot take would run them)
        return ("k_bwd_rows", "k_cs_hist", "k_tl_binscan", "k_cs_place", "k_cs_expand", "k_chain_tile", "k_bias_final")
    return BWD_KERNELS[mode]


def fwd_kernels(L1):
    if forward_path(L1) == "tile_pairs":
        return ("k_tl_hist", "k_tl_binscan", "k_tl_lists", "k_acc_tile", "k_mix_rest")
    if forward_path(L1) == "tile":
        return ("k_tl_hist", "k_tl_binscan", "k_tl_lists", "k_acc_tile", "k_mix<")
    return ("k_pair_hist", "k_pair_scan", "k_pair_scatter", "k_acc_blocked", "k_mix")


# (the windowed order has no k_bias_final launch: the bias gradient's last step rides in k_split_combine)
BWD_KERNELS = {
    "deterministic": ("k_bwd_rows", "k_chunk_hist", "k_col_scan", "k_row_scan", "k_fill", "k_seg_reduce", "k_split_combine"),
    "deterministic_strict": ("k_bwd_rows", "k_chunk_hist", "k_col_scan", "k_row_scan", "k_fill", "k_seg_reduce", "k_bias_final"),
    "atomic": ("k_bwd_rows", "k_tl_hist", "k_tl_binscan", "k_tl_lists", "k_scatter_tile", "k_scatter_foreign", "k_bias_final"),
}


# ------------------------------------------------------------------------------------------------
# inputs

def make_inputs(L1, B, seed, device, positions="uniform"):
    import torch
    from nnueft import halfka_v2_hm as hk

    us, them, white, black, pc = hk.synthetic_batch(B, seed, game_like=(positions == "game"))
    oc = L1 + N_PSQT
    g = torch.Generator(device="cpu").manual_seed(seed)
    W = (torch.randn(R_ROWS, oc, generator=g) * 0.01)
    bias = torch.zeros(oc)
    t = {
        "us": torch.from_numpy(us), "them": torch.from_numpy(them),
        "white": torch.from_numpy(white), "black": torch.from_numpy(black),
        "psqt_idx": torch.from_numpy((pc - 1) // 4),
        "W": W, "bias": bias,
        "g_l0": torch.randn(B, L1, generator=g), "g_wp": torch.randn(B, 1, generator=g),
        "g_bp": torch.randn(B, 1, generator=g),
    }
    sum_a = int((white >= 0).sum() + (black >= 0).sum())
    if device is not None:
        t = {k: v.to(device) for k, v in t.items()}
    return t, sum_a


def host_threads():
    """Threads for the CPU leg: the cores this process may run on, and not more than the share the job was given
    (OMP_NUM_THREADS is that share where a scheduler sets it; on a shared host the affinity mask alone overstates it)."""
    affinity = len(os.sched_getaffinity(0))
    share = os.environ.get("OMP_NUM_THREADS", "")
    threads = min(affinity, int(share)) if share.isdigit() and int(share) > 0 else affinity
    return affinity, threads


def cpu_baseline(workloads, seed, budget_s=12.0):
    """The reference's CPU path (oracle.ref_torch: the torch embedding_bag composition, autograd backward) on the
    whole batch of each workload: 3 warm-up steps, then at least 10 timed steps (fewer only when `budget_s` runs out)."""
    import torch
    from oracle import ref_torch

    affinity, threads = host_threads()
    torch.set_num_threads(threads)
    runs = []
    for name in workloads:
        L1, B = WORKLOADS[name]
        t, _ = make_inputs(L1, B, seed, None)
        W = t["W"].clone().requires_grad_()
        bias = t["bias"].clone().requires_grad_()

        def step():
            W.grad = None
            bias.grad = None
            out = ref_torch.double_feature_transform(t["us"], t["them"], t["white"], t["black"], t["psqt_idx"], W,
                                                     bias, MAX_ACT, L1)
            torch.autograd.backward(list(out), [t["g_l0"], t["g_wp"], t["g_bp"]])

        for _ in range(3):
            step()
        n, t0 = 0, time.perf_counter()
        while True:
            step()
            n += 1
            el = time.perf_counter() - t0
            if (n >= 10 and el > 2.0) or el > budget_s:
                break
        runs.append({"workload": name, "positions_per_s": B * n / el, "ms_per_step": el / n * 1e3, "steps": n,
                     "warmup": 3, "batch": B})
    head = runs[0]
    return {
        "value": head["positions_per_s"], "unit": "positions/s", "cores": threads, "kind": "port",
        "affinity_cores": affinity, "threads_used": threads,
        "sample": f"the whole {head['batch']}-position batch of {head['workload']} (same seeded lists, 24576-row table), "
                  f"{head['steps']} fwd+bwd steps of the torch embedding_bag composition with autograd backward after 3 "
                  f"warm-ups, torch.set_num_threads({threads}) of {affinity} cores in the affinity mask",
        "runs": runs,
    }


def time_steps(fn, steps, warmup):
    """(wall ms per call, HIP-event ms per call); events on torch's current stream, the one every launch here uses."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall / steps * 1e3, e0.elapsed_time(e1) / steps


def l2_peak_gbs():
    return L2_CHANNELS * L2_LINE_BYTES * ENGINE_CLOCK_GHZ


def measured_peaks(lib, dev):
    """What the two memory paths of the gathers deliver on this device, from the library's probe kernels (HIP events,
    one warm-up launch and one timed): random pieces of an L2-resident set (2.5 MB per XCD) and 16-byte reads out of
    a 96 KB LDS tile.  GB/s, whole chip."""
    import ctypes
    import torch

    out = {}
    stream = torch.cuda.current_stream().cuda_stream
    sink = torch.zeros(1, device=dev)
    set_bytes = 2560 * 1024
    src = torch.zeros(8 * set_bytes // 4, device=dev)
    n = ctypes.c_longlong(0)

    def timed(launch):
        assert launch() == 0
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        assert launch() == 0
        e1.record()
        torch.cuda.synchronize()
        return n.value / (e0.elapsed_time(e1) * 1e-3) / 1e9

    for span, depth, key in ((1024, 8, "l2_gather_1KiB_pieces_GBs"), (128, 8, "l2_gather_128B_lines_GBs"),
                             (1024, 16, "l2_gather_1KiB_pieces_depth16_GBs")):
        out[key] = timed(lambda: lib.nnueft_probe_l2_gather(src.data_ptr(), src.numel() * 4, sink.data_ptr(), set_bytes, span,
                                                            depth, 400, ctypes.byref(n), stream))
    for pattern, key in ((0, "lds_read_1KiB_in_a_row_GBs"), (1, "lds_read_random_128B_rows_GBs")):
        out[key] = timed(lambda: lib.nnueft_probe_lds_read(sink.data_ptr(), pattern, 4000, ctypes.byref(n), stream))
    out["l2_gather_measured_GBs"] = max(out["l2_gather_1KiB_pieces_GBs"], out["l2_gather_1KiB_pieces_depth16_GBs"])
    out["how"] = ("nnueft_probe_l2_gather: all CUs, 32 waves each, random pieces of a 2.5 MB set per XCD, 8 (16) loads of 16 "
                  "bytes in flight per lane; nnueft_probe_lds_read: all CUs, 16 waves each, 8 reads of 16 bytes in flight per lane")
    return out


# ------------------------------------------------------------------------------------------------
# other workloads

def run_int16(args, lib, dev):
    """Quantized forward (BASELINE.json config 5): int16 gather-accumulate, clip, product >> 9 -> u8."""
    import numpy as np
    import torch
    from nnueft import halfka_v2_hm as hk
    from nnueft import quantized

    L1, B = WORKLOADS[args.workload]
    R = hk.NUM_INPUTS_EXPORT
    us, them, white, black, pc = hk.synthetic_batch(B, 1239, fold_kings=True)
    g = torch.Generator().manual_seed(5)
    W = torch.randn(R, L1 + N_PSQT, generator=g) * 0.02
    bias = torch.randn(L1 + N_PSQT, generator=g) * 0.1
    w16, b16, p32 = quantized.quantize_feature_transformer(W, bias, L1)
    t = lambda a: torch.from_numpy(a).to(dev)
    stm = t((1 - us[:, 0]).astype(np.uint8))
    wi, bi, pi = t(white), t(black), t((pc - 1) // 4)
    w16, b16, p32 = w16.to(dev), b16.to(dev), p32.to(dev)
    sum_a = int((white >= 0).sum() + (black >= 0).sum())

    from nnueft import model as M

    torch.manual_seed(5)
    stacks = M.LayerStacks(8, M.ModelConfig(L1=L1, L2=32, L3=32), M.QuantizationManager(M.QuantizationConfig()))
    with torch.no_grad():
        stacks.l1.linear.weight.mul_(0.5)
    stack_q = [x.to(dev) for x in quantized.quantize_layer_stacks(stacks)]

    def step():
        return quantized.ft_int16_forward(wi, bi, stm, w16, b16, p32, pi)

    def chain():
        x_u8, psqt = quantized.ft_int16_forward(wi, bi, stm, w16, b16, p32, pi)
        return quantized.stack_int8_forward(x_u8, pi, *stack_q) + psqt

    _, ms = time_steps(step, args.steps, args.warmup)
    _, ms_chain = time_steps(chain, args.steps, args.warmup)
    gathered = sum_a * L1 * 2
    alg = gathered + B * (2 * K_SLOTS * 4 + L1)
    # table once, lists read twice by the sort and once for the psqt sums, packed lists written and read, both
    # lists' sums written and read, u8 out
    comp = (R * L1 * 2 + R * N_PSQT * 4 + 3 * 2 * B * K_SLOTS * 4 + 2 * (sum_a * 2 + 2 * B * 6) + 2 * (2 * B * L1 * 2)
            + B * L1)
    lds_peak = LDS_PEAK_GBS
    gbs = alg / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "quantized FT forward positions/sec (int16 accumulate, L1=3072, B=65536)",
        "value": B / (ms * 1e-3), "unit": "positions/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int16",
        "data": "synthetic",
        "config": {"workload": args.workload, "L1": L1, "batch": B, "table_rows": R,
                   "active_rows_per_position": sum_a / B,
                   "with_int8_layer_stacks_ms": ms_chain, "with_int8_layer_stacks_positions_per_s": B / (ms_chain * 1e-3)},
        "roofline": {"kernel": "nnueft_ft_int16_fwd: k_acc_tile over the int16 table (the gather out of LDS tiles) + "
                               "list sort (with the psqt difference)", "bound": "lds",
                     "achieved": gbs, "peak": lds_peak, "unit": "GB/s", "frac": gbs / lds_peak, "traffic": None,
                     "algorithmic_bytes_per_launch": alg, "avg_launch_ms": ms,
                     "achieved_over_hbm_peak": gbs / HBM_PEAK_GBS,
                     "note": "the gathered rows are LDS reads (a tile of 704 rows x 64 int16 columns per workgroup), so "
                             "the algorithmic rate is held against the LDS read rate; the HBM-side figure is "
                             "roofline_compulsory"},
        "roofline_compulsory": {"bound": "hbm", "bytes_per_launch": comp, "achieved": comp / (ms * 1e-3) / 1e9,
                                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": comp / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "cpu_baseline": None,
    }))


def run_full_step(args, dev):
    """BASELINE.json config 4: the L1=3072 model (FT, pairwise clipped ReLU, 8 bucketed layer stacks),
    WDL-blended sigmoid loss, optimizer step.  The optimizer is the reference's RangerLite in its default
    configuration (positive-negative momentum, lookahead every 5 steps, no decay) running on this build's
    kernels, over the reference's ten parameter groups; --optimizer adam times torch's fused Adam instead."""
    import torch
    import nnueft
    from nnueft import halfka_v2_hm as hk
    from nnueft import model as M

    L1, B = WORKLOADS[args.workload]
    nnueft.set_backward_mode(args.backward)
    nnueft.set_sort_placement(args.sort_placement)
    torch.manual_seed(0)
    model = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(L1=L1, L2=32, L3=32)).to(dev)
    us, them, white, black, pc = [torch.from_numpy(a).to(dev) for a in hk.synthetic_batch(B, 1238)]
    g = torch.Generator().manual_seed(1238)
    score = (torch.randn(B, 1, generator=g) * 400).clamp(-3000, 3000).to(dev)
    outcome = (torch.randint(0, 3, (B, 1), generator=g).float() / 2).to(dev)
    if args.optimizer == "rangerlite":
        from nnueft.optim import RangerLite

        opt = RangerLite(M.optimizer_param_groups(model, lr=8.75e-4), normloss_active=False)
        opt_name = "nnueft.optim.RangerLite(pnm, lookahead 5/0.5, no decay), fused HIP update"
    else:
        opt = torch.optim.Adam(model.parameters(), lr=8.75e-4, fused=True)
        opt_name = "torch.optim.Adam(fused=True)"
    params = M.LossParams()
    fwd = torch.compile(model, backend=args.compile) if args.compile else model

    def step():
        opt.zero_grad(set_to_none=True)
        out = fwd(us, them, white, black, pc)
        loss = M.sf_loss(out * model.quantization.nnue2score, score, outcome, params, 0.75)
        loss.backward()
        opt.step()
        return loss

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    print(json.dumps({
        "metric": "full model training step positions/sec (L1=3072, B=16384)", "value": B / (ms * 1e-3),
        "unit": "positions/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": args.workload, "L1": L1, "L2": 32, "L3": 32, "batch": B, "backward": args.backward,
                   "optimizer": opt_name, "torch_compile": args.compile or None, "lambda": 0.75, "fake_quantization": True,
                   "final_loss": float(loss)},
        "roofline": None, "cpu_baseline": None,
    }))


def run_ref_microbench(args, dev):
    """The reference's own micro-benchmark, tests/bench_feature_transformer.py:22-25,57-133: B=8192, row width 264,
    24 sorted random indices over the whole table + 8 pads per list; the bare sparse-linear function under
    clamp/mean/backward, then the composed feature transformer (fake-quantized weights and activations) with the
    fused backend.  Same loop, same positions/s figure it prints."""
    import torch
    import nnueft
    from nnueft import model as M
    from nnueft.sparse_linear_functions import SparseLinearFunction

    stride, B = WORKLOADS[args.workload]
    nnueft.set_backward_mode(args.backward)
    torch.manual_seed(0)
    quant = M.QuantizationManager(M.QuantizationConfig())
    ft = M.ComposedFeatureTransformer(M.get_feature_cls("HalfKAv2_hm^"), stride, num_psqt_buckets=8,
                                      quantization=quant).to(dev)
    n_in, k = ft.NUM_INPUTS, ft.MAX_ACTIVE_FEATURES

    def fake_indices():
        r = torch.randint(0, n_in, (B, k * 3 // 4), dtype=torch.int32, device=dev)
        r, _ = torch.sort(r, dim=1)
        return torch.cat([r, torch.full((B, k // 4), -1, dtype=torch.int32, device=dev)], dim=1)

    i0, i1 = fake_indices(), fake_indices()
    us = torch.randint(0, 2, (B, 1), device=dev).float()
    them = 1.0 - us
    psqt = (torch.randint(1, 32, (B,), dtype=torch.int64, device=dev) - 1) // 4
    weight = torch.randn(n_in, stride, device=dev, requires_grad=True)
    bias = torch.randn(stride, device=dev, requires_grad=True)

    def direct():
        out = torch.clamp(SparseLinearFunction.apply(i0, weight, bias), 0.0, 1.0)
        out.mean().backward()

    def composed():
        l0, wp, bp = ft(us, them, i0, i1, psqt, fake_quantize_acts=True, fake_quantize_weights=True, backend="fused")
        (l0.sum() + wp.sum() + bp.sum()).backward()

    iters, warm = max(args.steps, 64), max(args.warmup, 10)
    ms_direct, _ = time_steps(direct, iters, warm)
    ms_composed, _ = time_steps(composed, iters, warm)
    print(json.dumps({
        "metric": "reference micro-benchmark (tests/bench_feature_transformer.py): positions/sec, B=8192, row width 264",
        "value": B / (ms_composed * 1e-3), "unit": "positions/s", "n_gpus": 1, "steps": iters, "warmup": warm,
        "ms_per_step": ms_composed, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": args.workload, "batch": B, "row_width": stride, "backward": args.backward,
                   "indices": "24 sorted uniform indices over the whole table + 8 pads per list",
                   "composed_feature_transformer_fused": {"ms": ms_composed, "positions_per_s": B / (ms_composed * 1e-3)},
                   "direct_sparse_linear_function": {"ms": ms_direct, "positions_per_s": B / (ms_direct * 1e-3)}},
        "roofline": None, "cpu_baseline": None,
    }))


def run_handoff(args, dev):
    """The step before the path: batches in host memory laid out as the loader leaves them, staged and
    copied to the GPU by nnueft.batch_handoff, feeding the same forward+backward step.  Reports the cost
    of the hand-off alone and the step rate with every batch crossing PCIe (the headline rate has its
    inputs resident)."""
    import numpy as np
    import torch
    import nnueft
    from nnueft import halfka_v2_hm as hk
    from nnueft.batch_handoff import DevicePrefetcher, SparseBatch
    from nnueft.double_ft_functions import double_feature_transform

    L1, B = WORKLOADS[args.workload]
    nnueft.set_backward_mode(args.backward)
    rng = np.random.default_rng(5)
    batches = []
    for i in range(4):
        us, them, white, black, pc = hk.synthetic_batch(B, 4000 + i)
        batches.append(SparseBatch.from_arrays(hk.NUM_INPUTS, us.reshape(B), rng.random(B, dtype=np.float32),
                                               rng.normal(0, 300, B).astype(np.float32), white, black, pc))
    words = 3 * B + 2 * B * K_SLOTS + B
    g = torch.Generator().manual_seed(0)
    W = (torch.randn(R_ROWS, L1 + N_PSQT, generator=g) * 0.05).to(dev).requires_grad_()
    bias = torch.randn(L1 + N_PSQT, generator=g).to(dev).requires_grad_()
    g_l0 = torch.randn(B, L1, generator=g).to(dev)
    g_p = torch.randn(B, 1, generator=g).to(dev)

    # the hand-off alone, synchronous: host staging + DMA + unpack kernel
    for _ in range(args.warmup):
        batches[0].get_tensors(dev)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        batches[i % 4].get_tensors(dev)
    host_ms = (time.perf_counter() - t0) / args.steps * 1e3
    torch.cuda.synchronize()
    sync_ms = (time.perf_counter() - t0) / args.steps * 1e3

    def step(t):
        us, them, white, black, outcome, score, piece_count = t
        W.grad = None
        bias.grad = None
        out = double_feature_transform(us, them, white, black, (piece_count - 1) // 4, W, bias, MAX_ACT, L1, "fused")
        torch.autograd.backward(list(out), [g_l0, g_p, g_p])

    def rate(source, n):
        it = iter(source)
        for _ in range(args.warmup):
            step(next(it))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            step(next(it))
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e3

    total = args.steps + args.warmup
    resident = batches[0].get_tensors(dev)
    ms_res = rate((resident for _ in range(total)), args.steps)
    pf = DevicePrefetcher((batches[i % 4] for i in range(total)), dev, depth=4)
    ms_pf = rate(pf, args.steps)
    pf.close()
    ms_inline = rate((batches[i % 4].get_tensors(dev) for i in range(total)), args.steps)
    print(json.dumps({
        "metric": "FT fwd+bwd positions/sec with every batch handed over from host memory",
        "config": {"workload": args.workload, "L1": L1, "batch": B, "backward": args.backward,
                   "bytes_per_batch": words * 4},
        "handoff_alone": {"host_ms_per_batch": host_ms, "ms_per_batch_incl_copy": sync_ms,
                          "GBs": words * 4 / (sync_ms * 1e-3) / 1e9},
        "step_ms": {"inputs_resident": ms_res, "prefetcher": ms_pf, "handoff_on_the_training_stream": ms_inline},
        "positions_per_s": {"inputs_resident": B / (ms_res * 1e-3), "prefetcher": B / (ms_pf * 1e-3),
                            "handoff_on_the_training_stream": B / (ms_inline * 1e-3)},
        "steps": args.steps, "warmup": args.warmup, "n_gpus": 1, "data": "synthetic",
    }))


# ------------------------------------------------------------------------------------------------
# the feature-transformer workloads (configs 1-3)

def bound_block(kernel, ms, alg_bytes, gathered_bytes, comp_bytes, traffic_bytes, l2_peak, note=None, measured_peak=None):
    """One launch against its three yardsticks.  measured_peak: what the probe kernel of this run reached on the path
    that serves the algorithmic bytes; `frac` is then against that, `frac_of_nominal_peak` against the nominal rate."""
    s = ms * 1e-3
    alg_gbs = alg_bytes / s / 1e9
    peak = measured_peak if measured_peak else l2_peak
    out = {
        "kernel": kernel, "avg_launch_ms": ms,
        # the algorithmic bytes are served by L2 (the gathers are blocked for it), so that is the bound they are held to
        "bound": "l2", "achieved": alg_gbs, "peak": peak, "unit": "GB/s", "frac": alg_gbs / peak,
        "peak_is": "measured in this run (probe kernel)" if measured_peak else "nominal",
        "nominal_peak": l2_peak, "frac_of_nominal_peak": alg_gbs / l2_peak,
        "algorithmic_bytes_per_launch": alg_bytes, "achieved_over_hbm_peak": alg_gbs / HBM_PEAK_GBS,
        "l2_lines_per_clock_per_channel": gathered_bytes / s / 1e9 / l2_peak if gathered_bytes else None,
        "traffic": traffic_bytes,
        "traffic_GBs": traffic_bytes / s / 1e9 if traffic_bytes else None,
        "traffic_frac_of_hbm_peak": traffic_bytes / s / 1e9 / HBM_PEAK_GBS if traffic_bytes else None,
    }
    if note:
        out["note"] = note
    comp = {"kernel": kernel, "bound": "hbm", "bytes_per_launch": comp_bytes, "achieved": comp_bytes / s / 1e9,
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": comp_bytes / s / 1e9 / HBM_PEAK_GBS,
            "ms_at_peak": comp_bytes / (HBM_PEAK_GBS * 1e9) * 1e3}
    return out, comp


def run_ft(args, lib, dev):
    import torch
    import nnueft
    from nnueft.double_ft_functions import double_feature_transform

    L1, B = WORKLOADS[args.workload]
    oc = L1 + N_PSQT
    seed = 1234 + 3
    t, sum_a = make_inputs(L1, B, seed, dev, args.positions)
    W = t["W"].requires_grad_()
    bias = t["bias"].requires_grad_()
    l2_peak = l2_peak_gbs()
    probes = measured_peaks(lib, dev)

    def step(mode, t=t):
        nnueft.set_backward_mode(mode)
        W.grad = None
        bias.grad = None
        out = double_feature_transform(t["us"], t["them"], t["white"], t["black"], t["psqt_idx"], W, bias,
                                       MAX_ACT, L1, "fused")
        torch.autograd.backward(list(out), [t["g_l0"], t["g_wp"], t["g_bp"]])

    all_modes = ("deterministic", "deterministic_strict", "atomic")
    modes = [args.backward] + [m for m in all_modes if m != args.backward]
    only_mode = {"det": "deterministic", "strict": "deterministic_strict", "atomic": "atomic"}.get(args.only)
    if only_mode:
        modes = [only_mode]
    results = {}
    if args.only not in ("fwd", "reduce"):
        for mode in modes:
            ms_wall, _ = time_steps(lambda: step(mode), args.steps, args.warmup)
            results[mode] = ms_wall

    # the entry points alone, HIP events on the launch stream
    K_ = K_SLOTS
    l0 = torch.empty(B, L1, device=dev)
    wp = torch.empty(B, 1, device=dev)
    bp = torch.empty(B, 1, device=dev)
    saved = torch.empty(2, B, L1, device=dev)
    fwd_ws_bytes = lib.nnueft_fwd_workspace_bytes(B, K_, R_ROWS, L1, N_PSQT)
    fwd_ws = torch.empty(fwd_ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    Wd, bd = W.detach(), bias.detach()
    n_entry = max(args.steps, 10)

    def fwd_only(stream=stream):
        rc = lib.nnueft_double_fwd(t["us"].data_ptr(), t["them"].data_ptr(), t["white"].data_ptr(),
                                   t["black"].data_ptr(), t["psqt_idx"].data_ptr(), Wd.data_ptr(), bd.data_ptr(),
                                   MAX_ACT, l0.data_ptr(), wp.data_ptr(), bp.data_ptr(), saved.data_ptr(),
                                   B, K_, R_ROWS, L1, N_PSQT, fwd_ws.data_ptr(), fwd_ws_bytes, stream)
        assert rc == 0

    _, fwd_ms = time_steps(fwd_only, n_entry, args.warmup)

    bwd_ms = {}
    if args.only != "fwd":
        g_l0, g_wp, g_bp = t["g_l0"], t["g_wp"], t["g_bp"]
        gW = torch.empty(R_ROWS, oc, device=dev)
        gb = torch.empty(oc, device=dev)
        head = (t["us"].data_ptr(), t["them"].data_ptr(), t["white"].data_ptr(), t["black"].data_ptr(),
                t["psqt_idx"].data_ptr(), bd.data_ptr(), MAX_ACT, g_l0.data_ptr(), g_wp.data_ptr(), g_bp.data_ptr(),
                saved.data_ptr())

        from nnueft.sparse_linear_functions import _aux_stream_ptr, row_split_of

        # the entry point as FusedDoubleFtFunction calls it under this sort placement
        aux_stream = _aux_stream_ptr(dev) if args.sort_placement == "backward" else None

        def det_entry(row_split):
            nbytes = lib.nnueft_det_workspace_bytes(B, K_, R_ROWS, oc, 2, row_split)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            sbytes = lib.nnueft_det_sort_bytes(B, K_, R_ROWS, oc, 2)
            lists = torch.empty(sbytes, dtype=torch.uint8, device=dev)
            # upstream rows at the pitch the backward gives its own (whole 128-byte lines)
            g_pitch = lib.nnueft_det_upstream_pitch(oc)
            G = torch.randn(2, B, g_pitch, device=dev)

            def whole(stream=stream, aux_stream=aux_stream):
                rc = lib.nnueft_double_bwd_det(*head, gW.data_ptr(), gb.data_ptr(), B, K_, R_ROWS, L1, N_PSQT,
                                               row_split, ws.data_ptr(), nbytes, None, stream, aux_stream)
                assert rc == 0

            def graph_replay():
                """Forward + this backward captured once into a HIP graph (every buffer allocated beforehand), then
                replayed: what is left of the step when the host launches one graph instead of ~16 kernels."""
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.stream(side):
                    with torch.cuda.graph(graph, stream=side):
                        cap = torch.cuda.current_stream().cuda_stream
                        fwd_only(cap)
                        whole(cap, None)
                torch.cuda.current_stream().wait_stream(side)
                return time_steps(graph.replay, n_entry, args.warmup)[0]

            def sort_only():
                rc = lib.nnueft_det_sort(t["white"].data_ptr(), t["black"].data_ptr(), B, K_, R_ROWS, oc, 2,
                                         row_split, lists.data_ptr(), sbytes, stream)
                assert rc == 0

            def presorted():
                rc = lib.nnueft_double_bwd_det(*head, gW.data_ptr(), gb.data_ptr(), B, K_, R_ROWS, L1, N_PSQT,
                                               row_split, ws.data_ptr(), nbytes, lists.data_ptr(), stream, None)
                assert rc == 0

            def reduce_only():
                # the segmented reduction alone: k_seg_reduce, then the window sums of split rows (k_split_combine)
                # and the rewind of the task counters, a few microseconds together
                rc = lib.nnueft_det_reduce_rows_pitched(G.data_ptr(), g_pitch, gW.data_ptr(), B, K_, R_ROWS, oc, 2,
                                                        row_split, ws.data_ptr(), nbytes, lists.data_ptr(), stream)
                assert rc == 0

            out = {}
            if args.only != "reduce":
                _, out["entry"] = time_steps(whole, n_entry, args.warmup)
                if args.graph:
                    out["graph_replay"] = graph_replay()
            _, out["sort"] = time_steps(sort_only, n_entry, args.warmup)
            if args.only != "reduce":
                _, out["presorted"] = time_steps(presorted, n_entry, args.warmup)
            _, out["reduce"] = time_steps(reduce_only, n_entry, args.warmup)
            return out

        # the atomic mode as the operator runs it: adds in LDS tiles where the shape takes them (the gradient is
        # written, no zero fill), else global atomics on the zeroed gradient
        from nnueft._ops import ATOMIC_LDS_MIN_COLS

        lds_bytes = lib.nnueft_atomic_lds_workspace_bytes(B, K_, R_ROWS, oc, 2) if oc >= ATOMIC_LDS_MIN_COLS else 0
        lds_ws = torch.empty(max(lds_bytes, 1), dtype=torch.uint8, device=dev)

        def bwd_atomic():
            if lds_bytes:
                rc = lib.nnueft_double_bwd_atomic_lds(*head, gW.data_ptr(), gb.data_ptr(), B, K_, R_ROWS, L1, N_PSQT,
                                                      lds_ws.data_ptr(), lds_bytes, stream)
            else:
                gW.zero_()
                gb.zero_()
                rc = lib.nnueft_double_bwd_atomic(*head, gW.data_ptr(), gb.data_ptr(), B, K_, R_ROWS, L1, N_PSQT, stream)
            assert rc == 0

        fwd_only()   # `saved` holds this batch's row sums
        for mode in (["deterministic"] if args.only == "reduce" else modes):
            if mode == "atomic":
                _, ms = time_steps(bwd_atomic, n_entry, args.warmup)
                bwd_ms[mode] = {"entry": ms, "kernel": "k_scatter_tile (atomic adds into LDS tiles of doubles) behind "
                                                       "k_bwd_rows and the list sort" if lds_bytes else
                                "k_double_bwd_atomic (global atomics, + the zero fill of the dense gradient)"}
            else:
                bwd_ms[mode] = det_entry(row_split_of(mode))

    # ---- report
    traffic, traffic_file = read_profile_traffic(args.workload, args.positions, modes[0])
    fwd_bytes, _ = algorithmic_bytes(L1, B, sum_a, "atomic")
    comp_fwd, comp_bwd, comp_bwd_chain = compulsory_bytes(L1, B, sum_a)
    head_mode = modes[0]
    ms_step = results.get(head_mode, float("nan"))
    out = {
        "metric": "FT fwd+bwd positions/sec at L1=3072,B=16384; achieved GB/s vs HBM peak"
        if args.workload == "ft_fwd_bwd_L1_3072_B16384" else f"FT fwd+bwd positions/sec ({args.workload})",
        "value": B / (ms_step * 1e-3) if ms_step == ms_step else None,
        "unit": "positions/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": args.workload, "L1": L1, "batch": B, "table_rows": R_ROWS, "psqt_columns": N_PSQT,
            "slots": K_SLOTS, "active_rows_per_position": sum_a / B, "backward": head_mode,
            "summation_order": {
                "deterministic_strict": "the reference CPU path's: per table row one chain over its slots in (position, slot) "
                                        "order, white + black; bit-equal to torch CPU autograd",
                "deterministic": "this build's default: as strict, except that a row named by more than 512 slots is summed "
                                 "window by window (bit-equal to the oracle and from run to run, to rounding against torch)",
                "atomic": "none (atomic adds into LDS tiles of doubles); 1e-4 relative against the oracle",
            }[head_mode],
            "index_scheme": "HalfKAv2_hm, seeded random positions", "positions": args.positions,
            "sort_placement": args.sort_placement,
        },
        "peaks": {"hbm_GBs": HBM_PEAK_GBS, "l2_nominal_GBs": l2_peak,
                  "l2_nominal": f"{L2_CHANNELS} channels x {L2_LINE_BYTES} B per clock at {ENGINE_CLOCK_GHZ} GHz",
                  "lds_nominal_GBs": LDS_PEAK_GBS, "lds_nominal": f"256 CUs x 256 B per clock at {ENGINE_CLOCK_GHZ} GHz",
                  "measured": probes, "traffic_source": traffic_file},
    }
    if forward_path(L1) in ("tile", "tile_pairs"):
        # the gather reads the table out of LDS tiles: its algorithmic bytes are LDS reads
        fwd_block, fwd_comp = bound_block(
            "nnueft_double_fwd: k_acc_tile (the gather out of LDS tiles; it writes the output rows too) + list sort (with the "
            "psqt chains) + k_mix_rest" if forward_path(L1) == "tile_pairs" else
            "nnueft_double_fwd: k_acc_tile (the gather out of LDS tiles, ~2/3 of the time) + k_mix + list sort", fwd_ms,
            fwd_bytes, None, sum(comp_fwd.values()), sum_traffic(traffic, fwd_kernels(L1)), LDS_PEAK_GBS,
            note="the gathered rows are LDS reads: peak = what 16-byte reads of whole 128-byte rows at random rows of a "
                 "96 KB tile reach on this device (probe kernel, this run); the kernel is bound by its memory side "
                 "(tile fetches and stores of the sums), see roofline_forward_compulsory",
            measured_peak=probes["lds_read_random_128B_rows_GBs"])
        fwd_block["bound"] = "lds"
    else:
        fwd_block, fwd_comp = bound_block(
            "nnueft_double_fwd: k_acc_blocked (the gather, ~3/4 of the time) + k_mix + pair sort", fwd_ms, fwd_bytes,
            sum_a * oc * 4, sum(comp_fwd.values()), sum_traffic(traffic, fwd_kernels(L1)), l2_peak,
            measured_peak=probes["l2_gather_measured_GBs"])
    out["roofline_forward"] = fwd_block
    out["roofline_forward_compulsory"] = fwd_comp
    # the dominant kernel as the headline's order launches it
    det = (bwd_ms.get(head_mode) if head_mode != "atomic" else None) or bwd_ms.get("deterministic") or \
        bwd_ms.get("deterministic_strict")
    if det and head_mode == "deterministic_strict" and strict_path(L1) == "chain":
        # the strict order's reduction out of LDS tiles: the gathered upstream rows are LDS reads
        alg, gathered, _ = seg_reduce_bytes(L1, B, sum_a)
        blk, comp_blk = bound_block(
            "k_chain_tile (timed through nnueft_det_reduce_rows_pitched, which launches it with k_bias_final behind it "
            "and the segmented reduction of the other path, which returns at once)", det["reduce"], alg, None,
            comp_bwd_chain["k_chain_tile"], sum_traffic(traffic, ("k_chain_tile",)), LDS_PEAK_GBS,
            note="dominant kernel of the step; every table row's chain is summed out of a tile of upstream rows in LDS, "
                 "so `achieved` (algorithmic bytes: one 16-column piece of an upstream row per slot) is held against "
                 "what 16-byte LDS reads at random rows reach on this device (probe kernel, this run).  The kernel does "
                 "not run at that bound: a step (one chunk of ~500 pairs x 16 columns) lasts as long as its longest "
                 "chain, the row of the own king, which every pair of the chunk names: ~500 dependent adds fed by LDS "
                 "reads that queue behind those of the other 15 waves.  Against HBM see roofline_compulsory and `traffic`.",
            measured_peak=probes["lds_read_random_128B_rows_GBs"])
        blk["bound"] = "lds"
        out["roofline"], out["roofline_compulsory"] = blk, comp_blk
    elif det:
        alg, gathered, comp = seg_reduce_bytes(L1, B, sum_a)
        seg_traffic = sum_traffic(traffic, ("k_seg_reduce",) + (("k_split_combine",) if head_mode == "deterministic" else ()))
        out["roofline"], out["roofline_compulsory"] = bound_block(
            "k_seg_reduce<4,3> (timed through nnueft_det_reduce_rows_pitched, which launches it with "
            + ("k_split_combine" if head_mode == "deterministic" else "k_bias_final")
            + ", which rewinds the task counters, a few microseconds, behind it)", det["reduce"], alg, gathered, comp,
            seg_traffic, l2_peak,
            note="dominant kernel of the step; it gathers one upstream row per slot through L2 (blocked by king bucket "
                 "and column slice), so `achieved` (algorithmic bytes) is held against what a gather of random 1 KiB "
                 "pieces out of an L2-resident set reaches on this device (probe kernel, this run; the nominal L2 line "
                 "rate is in nominal_peak); against HBM see roofline_compulsory (bytes that must cross HBM once) and "
                 "`traffic` (counter-measured); the L2's channels are busy 95 % of this kernel's time (TCC_BUSY in "
                 "profiles/ft_fwd_bwd_L1_3072_B16384_utilisation_pmc.txt)",
            measured_peak=probes["l2_gather_measured_GBs"])
    elif "atomic" in bwd_ms:
        _, bwd_bytes = algorithmic_bytes(L1, B, sum_a, "atomic")
        gbs = bwd_bytes / (bwd_ms["atomic"]["entry"] * 1e-3) / 1e9
        out["roofline"] = {"kernel": "nnueft_double_bwd_atomic*: " + bwd_ms["atomic"]["kernel"], "bound": "hbm",
                           "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                           "traffic": None, "algorithmic_bytes_per_launch": bwd_bytes,
                           "avg_launch_ms": bwd_ms["atomic"]["entry"]}
    else:
        out["roofline"], out["roofline_compulsory"] = fwd_block, fwd_comp
    step_stats = {}
    for mode in modes:
        if mode not in results:
            continue
        fb, bb = algorithmic_bytes(L1, B, sum_a, mode)
        ms = results[mode]
        st = {"ms_per_step": ms, "positions_per_s": B / (ms * 1e-3), "algorithmic_GBs": (fb + bb) / (ms * 1e-3) / 1e9}
        if mode != "atomic":
            comp_step = sum(comp_fwd.values()) + sum(
                (comp_bwd_chain if mode == "deterministic_strict" and strict_path(L1) == "chain" else comp_bwd).values())
            st["compulsory_bytes"] = comp_step
            st["compulsory_frac_of_hbm_peak"] = comp_step / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS
            tr = sum_traffic(read_profile_traffic(args.workload, args.positions, mode)[0], fwd_kernels(L1) + bwd_kernels(L1, mode))
            st["traffic_bytes"] = tr
            st["traffic_frac_of_hbm_peak"] = tr / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS if tr else None
        else:
            # algorithmic: the formula of the atomic scheme (8 bytes of read-modify-write per gathered float and the
            # zero fill), a ratio since the adds moved into LDS; compulsory: what this decomposition moves through HBM
            # (upstream rows written and read once, lists, the dense gradient written once)
            st["algorithmic_frac_of_hbm_peak"] = st["algorithmic_GBs"] / HBM_PEAK_GBS
            if oc >= 512:
                comp_atomic = (comp_bwd["k_bwd_rows"] + 2 * 2 * B * K_SLOTS * 4 + sum_a * 2 + 2 * B * 6
                               + 2 * B * oc * 4 + sum_a * 2 + R_ROWS * oc * 4 + comp_bwd["bias"])
                comp_step = sum(comp_fwd.values()) + comp_atomic
                st["compulsory_bytes"] = comp_step
                st["compulsory_frac_of_hbm_peak"] = comp_step / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS
                tr = sum_traffic(read_profile_traffic(args.workload, args.positions, mode)[0], fwd_kernels(L1) + bwd_kernels(L1, mode))
                st["traffic_bytes"] = tr
                st["traffic_frac_of_hbm_peak"] = tr / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS if tr else None
        if mode in bwd_ms:
            e = bwd_ms[mode]
            st["backward_entry_ms"] = e.get("entry")
            if "sort" in e:
                st.update(sort_entry_ms=e["sort"], backward_presorted_entry_ms=e.get("presorted"),
                          reduce_stage_ms=e["reduce"])
            if "graph_replay" in e:
                st["fwd_bwd_graph_replay_ms"] = e["graph_replay"]
        step_stats[mode] = st
    out["step"] = step_stats
    if not args.only and args.positions == "uniform":
        # the same step on game-like index lists (not the headline: what real training data looks like)
        tg, sum_g = make_inputs(L1, B, seed, dev, "game")
        game = {"active_rows_per_position": sum_g / B}
        for mode in ("deterministic", "deterministic_strict", "atomic"):
            ms_g, _ = time_steps(lambda: step(mode, tg), args.steps, args.warmup)
            game[mode] = {"ms_per_step": ms_g, "positions_per_s": B / (ms_g * 1e-3)}
        out["game_like_positions"] = game
        del tg
    if not args.no_cpu_baseline and not args.only:
        names = [args.workload] + (["ft_fwd_bwd_L1_1024_B8192"] if args.workload != "ft_fwd_bwd_L1_1024_B8192" else [])
        out["cpu_baseline"] = cpu_baseline(names, seed)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="ft_fwd_bwd_L1_3072_B16384", choices=sorted(WORKLOADS))
    ap.add_argument("--backward", default="deterministic_strict", choices=["deterministic", "deterministic_strict", "atomic"],
                    help="backward mode the headline value is measured with (the others are reported beside it)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--optimizer", default="rangerlite", choices=["rangerlite", "adam"],
                    help="full_step workload only")
    ap.add_argument("--compile", default="", choices=["", "inductor", "aot_eager", "cudagraphs"],
                    help="full_step workload only: torch.compile the model with this backend, as the reference's "
                         "train.py does (the kernels of this build stay opaque to it); off by default")
    ap.add_argument("--sort-placement", default="inline", choices=["inline", "backward", "forward"],
                    help="where the index sort of the deterministic backward runs (nnueft.set_sort_placement); "
                         "the default is the library's")
    ap.add_argument("--positions", default="uniform", choices=["uniform", "game"],
                    help="uniform: kings and pieces uniform over the board (the headline workload); game: piece "
                         "placement statistics of real game positions, where one or two king buckets hold a large "
                         "part of the batch (halfka_v2_hm.game_like_positions); a default run times both")
    ap.add_argument("--graph", action="store_true",
                    help="also capture forward + deterministic backward (through the C ABI, buffers allocated beforehand) "
                         "into one HIP graph and time its replay")
    ap.add_argument("--only", default="", choices=["", "fwd", "det", "strict", "atomic", "reduce", "copy", "handoff"],
                    help="run only this part (for profiling runs); 'reduce' the segmented reduction alone; 'copy' "
                         "launches a plain elementwise kernel reading and writing 1 GiB each, the yardstick the "
                         "FETCH_SIZE/WRITE_SIZE counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    import nnueft
    from nnueft import _native

    nnueft.set_sort_placement(args.sort_placement)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    lib = _native.load()  # raises if libnnueft.so is missing: there is no fallback
    dev = torch.device("cuda:0")
    if args.workload.startswith("ft_int16"):
        run_int16(args, lib, dev)
    elif args.workload.startswith("full_step"):
        run_full_step(args, dev)
    elif args.workload.startswith("ref_microbench"):
        run_ref_microbench(args, dev)
    elif args.only == "copy":
        n = (1 << 30) // 4
        src = torch.ones(n, device=dev)
        dst = torch.empty(n, device=dev)
        for _ in range(args.warmup + args.steps):
            torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "torch.add(src, 1.0, out=dst)", "read_bytes": n * 4, "write_bytes": n * 4,
                          "launches": args.warmup + args.steps}))
    elif args.only == "handoff":
        run_handoff(args, dev)
    else:
        run_ft(args, lib, dev)


if __name__ == "__main__":
    main()
