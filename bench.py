#!/usr/bin/env python3
"""Feature-transformer forward+backward throughput on one MI355X.

A step is one pass of the hot path over one synthetic batch: the fused two-perspective forward
(nnueft_double_fwd) and the backward into a dense weight gradient, through the same autograd
function the trainer calls.  Inputs are resident in HBM before the timed region.

Prints ONE JSON line: positions/s for the workload BASELINE.json's metric is quoted on (L1=3072,
B=16384, HalfKAv2_hm lists, 24576-row table), the roofline of the backward entry point (the dominant
launch of the step; `roofline_forward` is the forward's) from HIP event timings, and the reference's
CPU path (torch embedding_bag composition) timed on the host cores on a bounded sample of the same
workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "nnue-pytorch_amd"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

# Bytes that crossed the L2 boundary per call of an entry point (FETCH_SIZE x2.0 + WRITE_SIZE x1.0 summed over its
# kernels, the scale being what the same counters read for a 1 GiB torch.add), uniform positions:
# profiles/ft_fwd_bwd_L1_3072_B16384_pmc.txt
MEASURED_TRAFFIC = {
    ("ft_fwd_bwd_L1_3072_B16384", "forward"): 1.46e9,
    ("ft_fwd_bwd_L1_3072_B16384", "deterministic"): 2.69e9,
}

WORKLOADS = {
    # name: (L1, B)
    "ft_fwd_bwd_L1_3072_B16384": (3072, 16384),     # BASELINE.json config 3: the metric
    "ft_fwd_bwd_L1_1024_B8192": (1024, 8192),       # config 1
    "ft_fwd_bwd_L1_128_B16384": (128, 16384),       # config 2
    "ft_int16_fwd_L1_3072_B65536": (3072, 65536),   # config 5: quantized forward only
    "full_step_L1_3072_B16384": (3072, 16384),      # config 4: FT + layer stacks + loss + optimizer
}
R_ROWS = 24576
N_PSQT = 8
K_SLOTS = 32


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


def make_inputs(L1, B, seed, device, positions="uniform"):
    import numpy as np
    import torch
    from nnueft import halfka_v2_hm as hk

    us, them, white, black, pc = hk.synthetic_batch(B, seed, game_like=(positions == "game"))
    rng = np.random.default_rng(seed)
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
    del rng
    if device is not None:
        t = {k: v.to(device) for k, v in t.items()}
    return t, sum_a


def cpu_baseline(L1, B_full, seed, budget_s=20.0):
    """The reference's CPU path (oracle.ref_torch) on a sample of the workload's positions."""
    import torch
    from oracle import ref_torch

    cores = len(os.sched_getaffinity(0))
    cores = min(cores, 16) if os.environ.get("GRAFT_REPO_ROOT") else cores
    torch.set_num_threads(cores)
    B = min(B_full, 4096)
    t, _ = make_inputs(L1, B_full, seed, None)
    sl = slice(0, B)
    W = t["W"].clone().requires_grad_()
    bias = t["bias"].clone().requires_grad_()

    def step():
        W.grad = None
        bias.grad = None
        out = ref_torch.double_feature_transform(t["us"][sl], t["them"][sl], t["white"][sl], t["black"][sl],
                                                 t["psqt_idx"][sl], W, bias, 255.0 / 256.0, L1)
        torch.autograd.backward(list(out), [t["g_l0"][sl], t["g_wp"][sl], t["g_bp"][sl]])

    step()  # warm-up
    n, t0 = 0, time.perf_counter()
    while True:
        step()
        n += 1
        el = time.perf_counter() - t0
        if el > budget_s or n >= 8:
            break
    return {
        "value": B * n / el, "unit": "positions/s", "cores": cores, "kind": "port",
        "sample": f"first {B} positions of the {B_full}-position batch, same 24576x{L1 + N_PSQT} table, "
                  f"{n} fwd+bwd steps of the torch embedding_bag composition (autograd backward), 1 warm-up",
    }


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

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    ms = timed(step)
    ms_chain = timed(chain)
    alg = sum_a * L1 * 2 + B * (2 * K_SLOTS * 4 + L1)
    print(json.dumps({
        "metric": "quantized FT forward positions/sec (int16 accumulate, L1=3072, B=65536)",
        "value": B / (ms * 1e-3), "unit": "positions/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int16",
        "data": "synthetic",
        "config": {"workload": args.workload, "L1": L1, "batch": B, "table_rows": R,
                   "active_rows_per_position": sum_a / B,
                   "with_int8_layer_stacks_ms": ms_chain, "with_int8_layer_stacks_positions_per_s": B / (ms_chain * 1e-3)},
        "roofline": {"kernel": "nnueft_ft_int16_fwd", "bound": "hbm", "achieved": alg / (ms * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": None, "algorithmic_bytes_per_launch": alg, "avg_launch_ms": ms},
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
        out = double_feature_transform(us, them, white, black, (piece_count - 1) // 4, W, bias, 255.0 / 256.0, L1,
                                       "fused")
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="ft_fwd_bwd_L1_3072_B16384", choices=sorted(WORKLOADS))
    ap.add_argument("--backward", default="deterministic", choices=["deterministic", "atomic"],
                    help="backward mode the headline value is measured with (the other one is reported beside it)")
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
    ap.add_argument("--only", default="", choices=["", "fwd", "det", "atomic", "copy", "handoff"],
                    help="run only this part (for profiling runs); 'copy' launches a plain elementwise kernel "
                         "reading and writing 1 GiB each, the yardstick the FETCH_SIZE/WRITE_SIZE counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    import nnueft
    from nnueft import _native
    from nnueft.double_ft_functions import double_feature_transform

    nnueft.set_sort_placement(args.sort_placement)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    lib = _native.load()  # raises if libnnueft.so is missing: there is no fallback
    dev = torch.device("cuda:0")
    if args.workload.startswith("ft_int16"):
        run_int16(args, lib, dev)
        return
    if args.workload.startswith("full_step"):
        run_full_step(args, dev)
        return
    if args.only == "copy":
        n = (1 << 30) // 4
        src = torch.ones(n, device=dev)
        dst = torch.empty(n, device=dev)
        for _ in range(args.warmup + args.steps):
            torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "torch.add(src, 1.0, out=dst)", "read_bytes": n * 4, "write_bytes": n * 4,
                          "launches": args.warmup + args.steps}))
        return
    if args.only == "handoff":
        run_handoff(args, dev)
        return
    L1, B = WORKLOADS[args.workload]
    seed = 1234 + 3
    t, sum_a = make_inputs(L1, B, seed, dev, args.positions)
    W = t["W"].requires_grad_()
    bias = t["bias"].requires_grad_()
    max_act = 255.0 / 256.0

    def step(mode, t=t):
        nnueft.set_backward_mode(mode)
        W.grad = None
        bias.grad = None
        out = double_feature_transform(t["us"], t["them"], t["white"], t["black"], t["psqt_idx"], W, bias,
                                       max_act, L1, "fused")
        torch.autograd.backward(list(out), [t["g_l0"], t["g_wp"], t["g_bp"]])

    def time_steps(fn, steps, warmup):
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

    results = {}
    modes = [args.backward] + [m for m in ("deterministic", "atomic") if m != args.backward]
    if args.only in ("det", "atomic"):
        modes = ["deterministic" if args.only == "det" else "atomic"]
    if args.only != "fwd":
        for mode in modes:
            ms_wall, ms_ev = time_steps(lambda: step(mode), args.steps, args.warmup)
            results[mode] = ms_wall

    # the forward kernel alone (one launch per call), HIP events on the launch stream
    B_, K_ = t["white"].shape
    l0 = torch.empty(B, L1, device=dev)
    wp = torch.empty(B, 1, device=dev)
    bp = torch.empty(B, 1, device=dev)
    saved = torch.empty(2, B, L1, device=dev)
    fwd_ws_bytes = lib.nnueft_fwd_workspace_bytes(B, K_SLOTS, R_ROWS, L1, N_PSQT)
    fwd_ws = torch.empty(fwd_ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    Wd, bd = W.detach(), bias.detach()

    def fwd_only():
        rc = lib.nnueft_double_fwd(t["us"].data_ptr(), t["them"].data_ptr(), t["white"].data_ptr(),
                                   t["black"].data_ptr(), t["psqt_idx"].data_ptr(), Wd.data_ptr(), bd.data_ptr(),
                                   max_act, l0.data_ptr(), wp.data_ptr(), bp.data_ptr(), saved.data_ptr(),
                                   B, K_, R_ROWS, L1, N_PSQT, fwd_ws.data_ptr(), fwd_ws_bytes, stream)
        assert rc == 0

    _, fwd_ms = time_steps(fwd_only, max(args.steps, 10), args.warmup)

    # the backward entry points alone
    bwd_ms = {}
    if args.only != "fwd":
        g_l0, g_wp, g_bp = t["g_l0"], t["g_wp"], t["g_bp"]
        oc = L1 + N_PSQT
        row_split = lib.nnueft_row_split()
        nbytes = lib.nnueft_det_workspace_bytes(B, K_, R_ROWS, oc, 2, row_split)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        gW = torch.empty(R_ROWS, oc, device=dev)
        gb = torch.empty(oc, device=dev)
        head = (t["us"].data_ptr(), t["them"].data_ptr(), t["white"].data_ptr(), t["black"].data_ptr(),
                t["psqt_idx"].data_ptr(), bd.data_ptr(), max_act, g_l0.data_ptr(), g_wp.data_ptr(), g_bp.data_ptr(),
                saved.data_ptr())

        from nnueft.sparse_linear_functions import _aux_stream_ptr

        # the entry point as FusedDoubleFtFunction calls it under this sort placement
        aux_stream = _aux_stream_ptr(dev) if args.sort_placement == "backward" else None

        def bwd_det():
            rc = lib.nnueft_double_bwd_det(*head, gW.data_ptr(), gb.data_ptr(), B, K_, R_ROWS, L1, N_PSQT, row_split,
                                           ws.data_ptr(), nbytes, None, stream, aux_stream)
            assert rc == 0

        def bwd_atomic():
            gW.zero_()
            gb.zero_()
            rc = lib.nnueft_double_bwd_atomic(*head, gW.data_ptr(), gb.data_ptr(), B, K_, R_ROWS, L1, N_PSQT, stream)
            assert rc == 0

        for name, fn in (("deterministic", bwd_det), ("atomic", bwd_atomic)):
            if name in modes:
                _, bwd_ms[name] = time_steps(fn, max(args.steps, 10), args.warmup)

        if "deterministic" in modes:
            # with the lists sorted beforehand, as in the step above (the sort runs beside the forward)
            sbytes = lib.nnueft_det_sort_bytes(B, K_, R_ROWS, oc, 2)
            lists = torch.empty(sbytes, dtype=torch.uint8, device=dev)

            def sort_only():
                rc = lib.nnueft_det_sort(t["white"].data_ptr(), t["black"].data_ptr(), B, K_, R_ROWS, oc, 2, row_split,
                                         lists.data_ptr(), sbytes, stream)
                assert rc == 0

            def bwd_presorted():
                rc = lib.nnueft_double_bwd_det(*head, gW.data_ptr(), gb.data_ptr(), B, K_, R_ROWS, L1, N_PSQT,
                                               row_split, ws.data_ptr(), nbytes, lists.data_ptr(), stream, None)
                assert rc == 0

            _, bwd_ms["sort"] = time_steps(sort_only, max(args.steps, 10), args.warmup)
            _, bwd_ms["deterministic_presorted"] = time_steps(bwd_presorted, max(args.steps, 10), args.warmup)

    fwd_bytes, _ = algorithmic_bytes(L1, B, sum_a, "atomic")
    fwd_gbs = fwd_bytes / (fwd_ms * 1e-3) / 1e9
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
            "index_scheme": "HalfKAv2_hm, seeded random positions", "positions": args.positions,
            "sort_placement": args.sort_placement,
        },
        "roofline_forward": {
            "kernel": "nnueft_double_fwd: k_acc_blocked (the gather, ~3/4 of the time) + k_mix + pair sort",
            "bound": "hbm", "achieved": fwd_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": fwd_gbs / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC.get((args.workload, "forward")),
            "algorithmic_bytes_per_launch": fwd_bytes, "avg_launch_ms": fwd_ms,
        },
    }
    # the dominant launch of the step is the backward entry point (about two thirds of it); both gathers are
    # served from L2, so `achieved` (algorithmic bytes) can exceed the HBM peak while `traffic` stays far below
    if head_mode in bwd_ms:
        _, bwd_bytes = algorithmic_bytes(L1, B, sum_a, head_mode)
        bwd_gbs = bwd_bytes / (bwd_ms[head_mode] * 1e-3) / 1e9
        out["roofline"] = {
            "kernel": ("nnueft_double_bwd_det: k_seg_reduce (the gather of the upstream rows, ~60 % of the time) + "
                       "k_bwd_rows + index sort + bias chain") if head_mode == "deterministic"
            else "nnueft_double_bwd_atomic: k_double_bwd_atomic (+ the zero fill of the dense gradient)",
            "bound": "hbm", "achieved": bwd_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": bwd_gbs / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC.get((args.workload, head_mode)),
            "algorithmic_bytes_per_launch": bwd_bytes, "avg_launch_ms": bwd_ms[head_mode],
        }
    else:
        out["roofline"] = out["roofline_forward"]
    step_stats = {}
    for mode in modes:
        if mode not in results:
            continue
        fb, bb = algorithmic_bytes(L1, B, sum_a, mode)
        ms = results[mode]
        step_stats[mode] = {
            "ms_per_step": ms, "positions_per_s": B / (ms * 1e-3),
            "algorithmic_GBs": (fb + bb) / (ms * 1e-3) / 1e9,
            "frac_of_hbm_peak": (fb + bb) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "backward_entry_ms": bwd_ms.get(mode),
            "backward_algorithmic_GBs": bb / (bwd_ms[mode] * 1e-3) / 1e9 if mode in bwd_ms else None,
        }
        if mode == "deterministic" and "sort" in bwd_ms:
            step_stats[mode]["sort_entry_ms"] = bwd_ms["sort"]
            step_stats[mode]["backward_presorted_entry_ms"] = bwd_ms["deterministic_presorted"]
    out["step"] = step_stats
    if not args.only and args.positions == "uniform":
        # the same step on game-like index lists (not the headline: a robustness figure)
        tg, sum_g = make_inputs(L1, B, seed, dev, "game")
        ms_g, _ = time_steps(lambda: step(head_mode, tg), args.steps, args.warmup)
        out["game_like_positions"] = {"ms_per_step": ms_g, "positions_per_s": B / (ms_g * 1e-3),
                                      "active_rows_per_position": sum_g / B, "backward": head_mode}
        del tg
    if not args.no_cpu_baseline and not args.only:
        out["cpu_baseline"] = cpu_baseline(L1, B, seed)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
