"""Captured policy step (HIP graph through torch.cuda.CUDAGraph) against the same step run
eagerly: every replay must be bitwise the eager result, with the program's own eager work and
synchronisations between replays; weights refreshed in place per weights version keep their
addresses (the reference's GraphedRollout contract, python/rollout_graph.py:43-104)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from beatsaberrl_amd import fp16_linear as fl  # noqa: E402
from beatsaberrl_amd.config_policy import ConfigPolicy  # noqa: E402
from beatsaberrl_amd.policy import NotePolicy  # noqa: E402
from beatsaberrl_amd.rollout_graph import GraphedRollout  # noqa: E402
from oracle import note_policy_ref as nr  # noqa: E402

DEV = "cuda"


@pytest.fixture(autouse=True)
def _rollout_mode():
    """These tests exercise the forward-only (rollout) routes: grad mode off, as the rollout runs."""
    with torch.no_grad():
        yield


def _obs(n, seed):
    g = torch.Generator().manual_seed(seed)
    obs = torch.randn(n, nr.OBS_DIM, generator=g) * 0.7
    obs[:, nr.OFF_MASK:nr.OFF_MASK + 24] = (torch.rand(n, 24, generator=g) < 0.6).float()
    return obs.to(DEV)


class _Env:
    """A stand-in env whose capturable step writes the next observation in place from the action."""

    def __init__(self, obs):
        self._obs = obs
        self._reward = torch.zeros(obs.shape[0], device=obs.device)
        self._done = torch.zeros(obs.shape[0], dtype=torch.bool, device=obs.device)

    def step(self, a):
        self._obs[:, :29].add_(a.to(self._obs.dtype) * 0.03 - 0.05)
        self._reward.copy_(a.sum(-1).float())


def _eager_work():
    x = torch.randn(257, 129, device=DEV)
    (x @ x.t()).sum().item()            # unrelated kernels + a device sync between replays


@pytest.mark.parametrize("fp16,blocks,ffn", [(True, "auto", "off"), (True, "off", "off"), (False, "off", "off"),
                                             (True, "off", "on")])
def test_replays_match_eager_steps_and_follow_weight_refreshes(fp16, blocks, ffn):
    """ffn = "on" with the block stack per op: the block FFNs run as the packed-image fused kernel, whose images the
    captured graph holds by address - they must be rebuilt in place by refresh(), like the replicas."""
    torch.manual_seed(11)
    m = NotePolicy(embed=128, trunk_dim=256, n_blocks=3, n_heads=4, n_gears=5, ffn_mult=4, note_geo=True,
                   head_gears=tuple(7 if j == 4 else 5 for j in range(29)), fused_ffn=ffn).to(DEV)
    m.fp16, m.fused_blocks = fp16, blocks
    env = _Env(_obs(37, 2))
    gr = GraphedRollout(m, env)
    steps = 4
    o0, c0 = env._obs.clone(), m._sample_ctr.clone()

    def run(step_fn):
        env._obs.copy_(o0)
        m._sample_ctr.copy_(c0)
        out = []
        for _ in range(steps):
            a, lp, v = step_fn()
            out.append((a.clone(), lp.clone(), v.clone(), env._reward.clone(), env._obs.clone()))
            _eager_work()
        return out

    def eager():
        a, lp, _, v = m.get_action_and_value(env._obs, need_entropy=False)
        env.step(a)
        return a, lp, v

    replayed = run(lambda: gr.step()[:3])
    assert int(m._sample_ctr.item()) == int(c0.item()) + steps          # the captured counter kernel ran per replay
    ref = run(eager)
    for i, (r, e) in enumerate(zip(replayed, ref)):
        for got, want in zip(r, e):
            assert torch.equal(got, want), f"replay {i}"
    assert not torch.equal(replayed[0][0], replayed[1][0])               # fresh noise and a new obs per replay
    # an optimizer step: masters change in place, version bumps, refresh() recasts the copies where they are
    with torch.no_grad():
        for p in m.parameters():
            p.mul_(1.03)
    fl.bump_weights_version()
    gr.refresh()
    after = run(lambda: gr.step()[:3])
    ref2 = run(eager)
    for r, e in zip(after, ref2):
        for got, want in zip(r, e):
            assert torch.equal(got, want)
    assert not torch.equal(after[0][1], replayed[0][1])                  # the new weights are what the replay used
    # a drifted stream mode is refused (python/rollout_graph.py:80-97)
    m.fp16 = not fp16
    with pytest.raises(RuntimeError, match="mode switch"):
        gr.refresh()
    m.fp16 = fp16


def test_torch_generator_sampler_under_capture():
    """sampler = "torch": the Exp(1) draws ride torch's default generator, which torch advances per replay."""
    torch.manual_seed(5)
    m = NotePolicy(embed=128, trunk_dim=256, n_blocks=2, n_heads=4, n_gears=5, ffn_mult=4).to(DEV)
    m.fp16, m.sampler = True, "torch"

    class Obs:
        _obs = _obs(64, 3)
    gr = GraphedRollout(m, Obs)
    a1, lp1, _ = (t.clone() for t in gr.step())
    _eager_work()
    a2, lp2, _ = (t.clone() for t in gr.step())
    assert not torch.equal(a1, a2)                                        # same obs, new draws
    for a, lp in ((a1, lp1), (a2, lp2)):                                  # and each replay's log-prob is its action's
        _, lp_e, _, _ = m.get_action_and_value(Obs._obs, action=a, need_entropy=False)
        assert torch.allclose(lp, lp_e, atol=1e-6)


@pytest.mark.parametrize("route", ["fused", "ops"])
def test_config_policy_forward_under_capture(route):
    torch.manual_seed(2)
    m = ConfigPolicy(dtype="f16").to(DEV)
    B = 64
    obs = torch.randn(B, m.obs_dim, device=DEV)
    k = torch.randint(0, 16, (B,), dtype=torch.int32, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            m.forward_stacked(obs, k, route=route)
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        lg, v = m.forward_stacked(obs, k, route=route)
    for seed in range(3):
        obs.copy_(torch.randn(B, m.obs_dim, device=DEV, generator=torch.Generator(DEV).manual_seed(seed)))
        k.copy_(torch.randint(0, 16, (B,), dtype=torch.int32, device=DEV))
        g.replay()
        got = (lg.clone(), v.clone())
        _eager_work()
        want = m.forward_stacked(obs, k, route=route)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), seed
