"""NotePolicy minibatch UPDATE benchmark: forward + PPO losses + backward + clip + Adam.

    python -m beatsaberrl_amd.bench_policy_update [--mbs 16384] [--fp16] [--iters 20] [--no-step]

The counterpart of the reference's harness (python/bench_policy_update.py:60-160) with its protocol:
a seeded synthetic minibatch (obs randn * 0.7 with 0/1 slot-mask lanes, uniform actions, old
log-probs around the uniform policy's, randn advantages and returns), the eager update body of the
trainer's minibatch loop - get_action_and_value(obs, act) under grad, dual-clip PPO policy loss
(clip 0.3, c 3), entropy bonus 0.03, HL-Gauss critic cross-entropy x 0.5, backward (loss scale
2^12 on the 16-bit stream), grad-norm clip 0.5, Adam lr 7e-4, weights-version bump - warm-up, then best
of `reps` timed loops of `iters` updates closed by one device sync, reported as ms/update and
env-samples/s.  --no-step times forward + backward alone."""
from __future__ import annotations

import argparse
import math
import time

import torch
import torch.nn as nn

from . import fp16_linear as _fl
from .policy import N_ACTION_HEADS, N_NOTE_SLOTS, OBS_DIM, OFF_NOTE_MASK, NotePolicy, hl_loss

ENT_COEF, VF_COEF, CLIP, DUAL_CLIP_C, MAX_GRAD_NORM, LR = 0.03, 0.5, 0.3, 3.0, 0.5, 7e-4


def make_minibatch(n, device, n_gears, seed=0):
    g = torch.Generator().manual_seed(seed)
    obs = (torch.randn(n, OBS_DIM, generator=g) * 0.7).to(device)
    obs[:, OFF_NOTE_MASK:OFF_NOTE_MASK + N_NOTE_SLOTS] = (torch.rand(n, N_NOTE_SLOTS, generator=g) < 0.6).float().to(device)
    act = torch.randint(0, n_gears, (n, N_ACTION_HEADS), generator=g).to(device)
    logp = (torch.randn(n, generator=g) * 0.3 - N_ACTION_HEADS * math.log(n_gears)).to(device)
    return obs, act, logp, torch.randn(n, generator=g).to(device), torch.randn(n, generator=g).to(device)


def pg_loss_fn(ratio, adv):
    """Dual-clip PPO policy loss (reference python/train_batch.py:90-101)."""
    standard = torch.max(-adv * ratio, -adv * torch.clamp(ratio, 1 - CLIP, 1 + CLIP))
    return torch.where(adv < 0, torch.min(standard, -DUAL_CLIP_C * adv), standard).mean()


def eager_update(policy, opt, obs, act, logp, adv, ret, scale=1.0, step=True):
    if opt is not None:
        opt.zero_grad(set_to_none=False)
    a = (adv - adv.mean()) / (adv.std() + 1e-8)
    _, newlogp, entropy, _ = policy.get_action_and_value(obs, act)
    loss = pg_loss_fn((newlogp - logp).exp(), a) - ENT_COEF * entropy.mean() \
        + VF_COEF * hl_loss(policy._value_logits, ret, policy.value_centers, policy.value_sigma)
    (loss * scale).backward()
    if not step:
        return loss.detach()
    if scale != 1.0:                  # unscale in one multi-tensor pass
        torch._foreach_div_([p.grad for p in policy.parameters() if p.grad is not None], scale)
    nn.utils.clip_grad_norm_(policy.parameters(), MAX_GRAD_NORM)
    opt.step()
    _fl.bump_weights_version()
    return loss.detach()


def bench(fn, iters, reps, warmup=3):
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
    return best * 1e3


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--mbs", type=int, nargs="+", default=[16384])
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--reps", type=int, default=3)
    ap.add_argument("--fp16", action="store_true", help="the 16-bit stream (production configuration)")
    ap.add_argument("--bf16", action="store_true", help="bfloat16 as the 16-bit stream dtype")
    ap.add_argument("--legacy-arch", action="store_true", help="ctor defaults (128 / 256 / 3 blocks) instead of the recipe")
    ap.add_argument("--fused-ffn", action="store_true", help="block FFNs forward as the fused kernel, which also writes the hidden for the backward")
    ap.add_argument("--fused-ffn-recompute", action="store_true", help="fused FFN forward that keeps no hidden: the backward recomputes it (less memory)")
    ap.add_argument("--no-step", action="store_true", help="forward + backward only (no clip, no optimizer)")
    ap.add_argument("--update-values", default="rollout", choices=("rollout", "own"),
                    help="rollout (default): the update forward also runs the rollout's fused forward and returns its "
                         "logits / value bits; own: the per-op forward's values (no second forward)")
    args = ap.parse_args(argv)
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    if args.legacy_arch:
        policy = NotePolicy(n_gears=5)
    else:
        policy = NotePolicy(embed=192, trunk_dim=384, n_blocks=6, n_heads=4, n_gears=5, ffn_mult=4, note_geo=True)
    policy = policy.to(dev)
    if args.fp16 or args.bf16:
        policy.fp16 = True
        policy.stream_dtype = torch.bfloat16 if args.bf16 else torch.float16
    if args.fused_ffn or args.fused_ffn_recompute:
        policy.fused_ffn = policy.arch["fused_ffn"] = "recompute" if args.fused_ffn_recompute else "on"
    policy.update_values = args.update_values
    scale = 4096.0 if policy.fp16 else 1.0
    opt = torch.optim.Adam(policy.parameters(), lr=LR)
    print(f"gpu: {torch.cuda.get_device_name(0)}  torch {torch.__version__}  stream "
          f"{policy.stream_dtype if policy.fp16 else torch.float32}")
    rows = []
    for mb in args.mbs:
        data = make_minibatch(mb, dev, policy.n_gears)
        ms = bench(lambda: eager_update(policy, opt, *data, scale=scale, step=not args.no_step), args.iters, args.reps)
        torch.cuda.reset_peak_memory_stats()
        eager_update(policy, opt, *data, scale=scale, step=not args.no_step)
        torch.cuda.synchronize()
        peak = torch.cuda.max_memory_allocated() / 2 ** 30
        print(f"mb {mb:>6}: {ms:8.2f} ms/update  {mb / ms * 1e3:12.0f} env-samples/s  peak {peak:.1f} GiB")
        rows.append((mb, ms))
    return rows


if __name__ == "__main__":
    main()
