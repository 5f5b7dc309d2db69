"""A thin training loop over synthetic batches: everything between the loader's output and the optimizer
step, wired the way the reference's trainer wires it (model/nnue.py:280-364: batch tuple -> model ->
win-rate loss -> optimizer over the parameter groups of :120-177).

  host batches (the loader's SparseBatch layout)  ->  DevicePrefetcher (own thread and stream)
  ->  NNUEModel (feature transformer, layer stacks)  ->  sf_loss  ->  RangerLite

No trainer, logging or checkpointing: `python -m nnueft.train_synthetic --steps 200` prints the loss every
few steps and the positions per second, and `run()` returns the losses for callers and tests.
"""
import argparse
import time

import numpy as np
import torch

from . import halfka_v2_hm as hk
from . import model as M
from .batch_handoff import DevicePrefetcher, SparseBatch
from .optim import RangerLite


def synthetic_host_batches(batch_size: int, distinct: int, seed: int, game_like: bool = False):
    """`distinct` batches in host memory laid out like the loader's.  The score of a position is what a
    fixed random linear teacher over the features says (side to move's list minus the other), plus
    noise, so there is something to learn."""
    rng = np.random.default_rng(seed)
    teacher = np.append(rng.normal(0, 60, hk.NUM_INPUTS), 0.0).astype(np.float32)     # [-1] -> 0 for padding
    batches = []
    for i in range(distinct):
        us, them, white, black, pc = hk.synthetic_batch(batch_size, seed + 1 + i, game_like=game_like)
        side = np.where(us.reshape(-1) > 0.5, 1.0, -1.0)
        value = side * (teacher[white].sum(1) - teacher[black].sum(1))
        score = np.clip(value + rng.normal(0, 50, batch_size), -3000, 3000).astype(np.float32)
        outcome = (np.clip(np.round(np.tanh(score / 400) + rng.normal(0, 0.4, batch_size)), -1, 1) + 1) / 2
        outcome = outcome.astype(np.float32)
        batches.append(SparseBatch.from_arrays(hk.NUM_INPUTS, us.reshape(-1), outcome, score, white, black, pc))
    return batches


def run(steps: int = 50, batch_size: int = 16384, l1: int = 1024, lr: float = 8.75e-4, lam: float = 0.75,
        device: str = "cuda:0", seed: int = 0, distinct: int = 4, game_like: bool = False, log_every: int = 0):
    """Train for `steps` steps; returns (losses, positions per second over the timed steps)."""
    dev = torch.device(device)
    torch.manual_seed(seed)
    model = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(L1=l1, L2=32, L3=32)).to(dev)
    opt = RangerLite(M.optimizer_param_groups(model, lr=lr), normloss_active=False)
    params = M.LossParams()
    host = synthetic_host_batches(batch_size, distinct, seed + 100, game_like)
    feed = DevicePrefetcher((host[i % distinct] for i in range(steps)), dev, depth=3)
    losses = []
    warm = min(5, steps // 2)
    t0 = None
    for step, (us, them, white, black, outcome, score, piece_count) in enumerate(feed):
        if step == warm:
            if dev.type == "cuda":
                torch.cuda.synchronize(dev)
            t0 = time.perf_counter()
        opt.zero_grad(set_to_none=True)
        out = model(us, them, white, black, piece_count)
        loss = M.sf_loss(out * model.quantization.nnue2score, score, outcome, params, lam)
        loss.backward()
        opt.step()
        model.clip_weights(include_input=False)      # the trainer's WeightClipper, after every batch
        losses.append(loss.detach())
        if log_every and step % log_every == 0:
            print(f"step {step:5d}  loss {float(losses[-1]):.6f}", flush=True)
    if dev.type == "cuda":
        torch.cuda.synchronize(dev)
    rate = (steps - warm) * batch_size / (time.perf_counter() - t0) if t0 is not None and steps > warm else 0.0
    feed.close()
    return [float(x) for x in losses], rate


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--batch-size", type=int, default=16384)
    ap.add_argument("--l1", type=int, default=1024)
    ap.add_argument("--lr", type=float, default=8.75e-4)
    ap.add_argument("--lambda", dest="lam", type=float, default=0.75)
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--game-like", action="store_true", help="piece placement drawn from game statistics")
    args = ap.parse_args(argv)
    losses, rate = run(args.steps, args.batch_size, args.l1, args.lr, args.lam, args.device, game_like=args.game_like,
                       log_every=max(1, args.steps // 10))
    print(f"loss {losses[0]:.6f} -> {losses[-1]:.6f} over {args.steps} steps; {rate / 1e6:.2f} M positions/s")


if __name__ == "__main__":
    main()
