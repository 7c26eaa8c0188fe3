"""NotePolicy forward benchmark: eager vs graph-captured, forward and argmax rows.

    python -m beatsaberrl_amd.bench_policy_forward [--ns 2048 16384] [--fp16] [--fused-ffn on]
                                                   [--legacy-arch] [--ckpt runs/perf_ref.pt]

The counterpart of the reference's harness (python/bench_policy_forward.py:72-195) with its
protocol: device-resident seeded obs (randn * 0.7, slot-mask lanes = rand < 0.6, seed 0),
10 warm-ups, best of `reps` x `iters` forwards closed by one device sync, microseconds per
forward, eager next to a captured graph (HIP graph through torch.cuda.CUDAGraph: 3 eager
warm-ups on a side stream, capture, replay)."""
from __future__ import annotations

import argparse
import time

import torch

from . import fp16_linear as _fl
from .policy import N_NOTE_SLOTS, OBS_DIM, OFF_NOTE_MASK, NotePolicy, load_policy


def make_obs(n, device):
    g = torch.Generator().manual_seed(0)
    obs = (torch.randn(n, OBS_DIM, generator=g) * 0.7).to(device)
    obs[:, OFF_NOTE_MASK:OFF_NOTE_MASK + N_NOTE_SLOTS] = (torch.rand(n, N_NOTE_SLOTS, generator=g) < 0.6).float().to(device)
    return obs


class Graphed:
    """Capture fn(static_obs) once, then replay on new obs copied into the static buffer."""

    def __init__(self, fn, example):
        self.s_obs = example.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                fn(self.s_obs)
        torch.cuda.current_stream().wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.out = fn(self.s_obs)

    def __call__(self, obs):
        self.s_obs.copy_(obs)
        self.graph.replay()
        return self.out


def bench(fn, iters, reps, warmup=10):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(reps):
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        best = min(best, (time.perf_counter() - t0) / iters)
    return best * 1e6


def build_policy(args, device):
    try:
        ckpt = torch.load(args.ckpt, map_location="cpu", weights_only=True)
        policy = load_policy(ckpt)
        print(f"weights: {args.ckpt}")
    except FileNotFoundError:              # an incompatible checkpoint is an error, not a reason to time random weights
        torch.manual_seed(0)
        if args.legacy_arch:
            policy = NotePolicy(n_gears=5)
        else:
            policy = NotePolicy(embed=192, trunk_dim=384, n_blocks=6, n_heads=4, n_gears=5, ffn_mult=4, note_geo=True)
        print("weights: random init (checkpoint not found)")
    policy = policy.to(device).eval()
    if args.fp16:
        policy.fp16 = True
        policy.flatten_fp16()
    return policy


@torch.no_grad()
def main(argv=None):
    p = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    p.add_argument("--ckpt", default="runs/perf_ref.pt")
    p.add_argument("--ns", type=int, nargs="+", default=[2048, 16384])
    p.add_argument("--iters", type=int, default=200)
    p.add_argument("--reps", type=int, default=3)
    p.add_argument("--fp16", action="store_true", help="16-bit stream (the production rollout configuration)")
    p.add_argument("--fp16-accum", default=None, choices=_fl.ACCUM_MODES, help="recorded only: accumulate is fp32")
    p.add_argument("--fused-ffn", nargs="+", default=None, choices=_fl.FFN_MODES)
    p.add_argument("--legacy-arch", action="store_true", help="ctor defaults (128 / 256 / 3 blocks) instead of the recipe")
    p.add_argument("--fused-forward", default="auto", choices=("auto", "off"),
                   help="auto: the block stack as one persistent kernel and the pooled critic where the shape has them "
                        "(16-bit stream); off: the per-op launch train with the reference's critic op order, whose "
                        "outputs are the update forward's bits")
    args = p.parse_args(argv)
    device = torch.device("cuda")
    policy = build_policy(args, device)
    policy.fused_blocks = args.fused_forward
    policy.critic_pool = args.fused_forward == "auto"
    if args.fp16_accum is not None:
        policy.fp16_accum = policy.arch["fp16_accum"] = args.fp16_accum
    print(f"gpu: {torch.cuda.get_device_name(0)}  torch {torch.__version__}  fused-forward {args.fused_forward}")
    print(f"best of {args.reps} x {args.iters} iters, us/forward\n")
    hdr = f"{'ffn':<6}{'op':<8}{'N':>6}{'eager':>10}{'graphed':>10}{'vs eager':>10}{'env-samples/s':>16}"
    print(hdr)
    print("-" * len(hdr))
    rows = []
    for mode in (args.fused_ffn or [policy.fused_ffn]):
        policy.fused_ffn = policy.arch["fused_ffn"] = mode
        for n in args.ns:
            obs = make_obs(n, device)
            fwd = lambda o: policy.forward_stacked(o)
            arg = lambda o: policy.forward_stacked(o)[0].argmax(-1)
            for op, fn in (("forward", fwd), ("argmax", arg)):
                te = bench(lambda: fn(obs), args.iters, args.reps)
                g = Graphed(fn, obs)
                tg = bench(lambda: g(obs), args.iters, args.reps)
                print(f"{mode:<6}{op:<8}{n:>6}{te:>10.1f}{tg:>10.1f}{te / tg:>9.2f}x{n / min(te, tg) * 1e6:>16.0f}")
                rows.append((mode, op, n, te, tg))
    return rows


if __name__ == "__main__":
    main()
