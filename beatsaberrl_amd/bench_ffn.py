"""The block FFN `xo = x + act(h2 W0^T + b0) W2^T + b2, ho = LN(xo)` three ways, timed alone on synthetic rows:
the fused kernel on a packed weight image (`bsrl_ffn_packed`, the default of `ops.ffn_fused`), the fused kernel on the
plain weights (`bsrl_ffn_fused`), and two Linears + LayerNorm (hidden through HBM).

    python -m beatsaberrl_amd.bench_ffn [--shapes 128x512x475136 192x768x475136 256x1024x1048576] [--iters 20]

A shape is d x F x rows.  Each variant is timed with HIP events on torch's current stream (the stream the kernels are
launched on) over `iters` calls after 3 warm-ups; FLOPs = 4 d F per row."""
from __future__ import annotations

import argparse
import json
import math

import torch

from . import ops


def avg_us(fn, iters):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters * 1e3


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--shapes", nargs="+", default=["128x512x475136", "192x768x475136", "256x1024x1048576"])
    ap.add_argument("--acts", nargs="+", default=["relu", "gelu"], choices=("relu", "gelu"))
    ap.add_argument("--dtype", default="f16", choices=("f16", "bf16"))
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--only", default=None, choices=("packed", "plain", "linears"), help="time one variant only (for a profiler)")
    args = ap.parse_args(argv)
    dev = torch.device("cuda:0")
    dt = torch.float16 if args.dtype == "f16" else torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rows_out = []
    for shape in args.shapes:
        d, F, rows = (int(v) for v in shape.split("x"))
        x = torch.randn(rows, d, device=dev, generator=g).to(dt)
        h2 = torch.randn(rows, d, device=dev, generator=g).to(dt)
        w0 = (torch.randn(F, d, device=dev, generator=g) / math.sqrt(d)).to(dt)
        w2 = (torch.randn(d, F, device=dev, generator=g) / math.sqrt(F)).to(dt)
        b0 = torch.randn(F, device=dev, generator=g) * 0.1
        b2 = torch.randn(d, device=dev, generator=g) * 0.1
        lw, lb = torch.ones(d, device=dev), torch.zeros(d, device=dev)
        flop = 4.0 * rows * d * F
        for act in args.acts:
            def linears():
                y = ops.linear(ops.linear(h2, w0, b0, act=act), w2, b2, residual=x)
                return ops.ln_fwd(y, lw, lb)
            variants = {
                "packed": lambda: ops.ffn_fused(x, h2, w0, b0, w2, b2, act=act, ln_w=lw, ln_b=lb),
                "plain": lambda: ops.ffn_fused(x, h2, w0, b0, w2, b2, act=act, ln_w=lw, ln_b=lb, packed=False),
                "linears": linears,
            }
            rec = {"d": d, "F": F, "rows": rows, "act": act, "dtype": args.dtype}
            for name, fn in variants.items():
                if args.only and name != args.only:
                    continue
                if name == "packed" and not ops.ffn_pack_supported(d, F, dt):
                    continue
                if name == "plain" and not ops.ffn_fused_supported(d, F, dt):
                    continue
                us = avg_us(fn, args.iters)
                rec[name + "_us"] = round(us, 1)
                rec[name + "_tflops"] = round(flop / us / 1e6, 1)
            rows_out.append(rec)
            print("  ".join(f"{k}={v}" for k, v in rec.items()), flush=True)
    print(json.dumps({"metric": "fused FFN, microseconds per call", "rows": rows_out}))


if __name__ == "__main__":
    main()
