"""Small-batch latency of the benchmark-config policy forward (config[4]): p50 microseconds per
forward at B in {1, 8, 64}, the whole forward as ONE persistent kernel (in its latency form: one env
per wave, weights through a deep direct-to-LDS ring; and in the throughput form) against the two-launch
pruned form and the per-op (multi-kernel) route, eager launches and a captured HIP graph.

    python -m beatsaberrl_amd.bench_latency [--batches 1 8 64] [--iters 300]

Each forward is timed with HIP events on torch's current stream (the stream the kernels are
launched on); p50 over `iters` forwards after 20 warm-ups."""
from __future__ import annotations

import argparse
import json

import torch

from .config_policy import ConfigPolicy


def p50_us(fn, iters, warmup=20):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for s, e in ev:
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    t = sorted(s.elapsed_time(e) for s, e in ev)
    return t[len(t) // 2] * 1e3


def graphed(fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g.replay


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--batches", type=int, nargs="+", default=[1, 8, 64])
    ap.add_argument("--iters", type=int, default=300)
    args = ap.parse_args(argv)
    dev = torch.device("cuda:0")
    torch.manual_seed(5)
    m = ConfigPolicy(dtype="f16").to(dev)
    rows = []
    for B in args.batches:
        obs = torch.randn(B, m.obs_dim, device=dev)
        variants = {
            "persistent kernel, latency form (1 launch)": dict(route="fused", prune=False, latency=True),
            "persistent kernel (1 launch)": dict(route="fused", prune=False),
            "fused, final block pruned (1 launch)": dict(route="fused", prune=True),
            "per-op route (multi-kernel)": dict(route="ops", prune=False),
        }
        for name, v in variants.items():
            m.prune_final = v["prune"]
            m.latency_form = v.get("latency", False)      # False: the throughput forms (small batches default to the latency form)
            fn = lambda: m.forward_stacked(obs, None, route=v["route"])
            eager = p50_us(fn, args.iters)
            replay = graphed(fn)
            gr = p50_us(replay, args.iters)
            rows.append({"B": B, "variant": name, "p50_us_eager": round(eager, 1), "p50_us_graph": round(gr, 1)})
            print(f"B={B:<3d} {name:<44s} eager {eager:8.1f} us   graph {gr:8.1f} us", flush=True)
    print(json.dumps({"metric": "p50 forward latency, config[4] model fp16", "rows": rows}))
    return rows


if __name__ == "__main__":
    main()
