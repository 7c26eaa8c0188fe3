"""Captured policy step: forward + action sampling (+ the env step) as one HIP graph.

The counterpart of the reference's GraphedRollout (python/rollout_graph.py:43-104) for the
kernels of this build, with its contract:

  * the graph is captured once on static storages - the env's observation buffer, the
    16-bit weight replicas / packed images (whose addresses never move, they are recast in
    place per weights version) - and replayed once per env step;
  * `refresh()` MUST run after optimizer steps and before the next replay: it recasts the
    replicas in place, once per weights version, and refuses a drifted `policy.fp16` flag (the
    captured kernels cannot follow a mode switch; python/rollout_graph.py:80-97);
  * sampling noise is fresh on every replay: the in-kernel Philox stream reads its call
    counter from device memory and a one-thread kernel in the graph advances it (torch's
    graph-registered generator offset plays that part for the reference's multinomial);
    `policy.sampler = "torch"` rides torch's generator exactly as the reference does;
  * outputs are static tensors: copy what you keep before the next replay.

`venv` is any object with a device tensor `_obs` (B, 630) it updates in place and, optionally,
a capturable `step(action)` (the reference's CUDA env, python/rollout_graph.py:60-78); without
`step` only the policy half is captured and the caller writes `_obs` between replays.
No memset nodes are recorded by this build's entry points (they allocate nothing and clear
nothing); torch's graph pool owns the intermediate tensors."""
from __future__ import annotations

import torch

from . import fp16_linear as _fl


class GraphedRollout:
    def __init__(self, policy, venv, warmup: int = 3, need_entropy: bool = False):
        if not venv._obs.is_cuda:
            raise RuntimeError("GraphedRollout needs a device-resident observation buffer")
        self.policy, self.venv = policy, venv
        self._version = None
        self.captured_fp16 = bool(getattr(policy, "fp16", False))
        self._step_env = getattr(venv, "step", None)
        self.refresh()                      # replicas must exist (and be stable) before capture
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s), torch.no_grad():
            for _ in range(warmup):         # allocator pools, lazily built caches
                a, _, _, _ = policy.get_action_and_value(venv._obs, need_entropy=need_entropy)
                if self._step_env is not None:
                    self._step_env(a)
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self.graph):
            a, logp, ent, v = policy.get_action_and_value(venv._obs, need_entropy=need_entropy)
            if self._step_env is not None:
                self._step_env(a)
        self.action, self.logp, self.entropy, self.value = a, logp, ent, v

    def refresh(self):
        """In-place refresh of every weight copy the captured kernels read, once per weights version."""
        live = bool(getattr(self.policy, "fp16", False))
        if live != self.captured_fp16:
            raise RuntimeError(f"GraphedRollout was captured with policy.fp16={self.captured_fp16} but the policy is "
                               f"now fp16={live}; the captured kernels cannot follow the mode switch - recapture "
                               "or restore the flag")
        if self._version != _fl._weights_version:
            self.policy.refresh_fp16_caches()
            self._version = _fl._weights_version

    def step(self):
        """One env step: replay, return the static (action, logp, value[, reward, done])."""
        self.graph.replay()
        v = self.venv
        if self._step_env is None:
            return self.action, self.logp, self.value
        return self.action, self.logp, self.value, getattr(v, "_reward", None), getattr(v, "_done", None)
