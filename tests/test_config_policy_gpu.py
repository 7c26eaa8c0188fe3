"""GPU parity of ConfigPolicy.forward_stacked (all kernels through the C ABI)
against the CPU oracle on identical seeded weights and inputs.

Gates (every ceiling is a literal at its call site; nothing is scaled by a quantity
computed at test time):
  * fp32: <= 1e-5 relative (here: |d| <= 1e-5 * (|ref| + max|ref|)).
  * every 16-bit KERNEL holds 2e-3 against the closed form on the same rounded
    operands (tests/test_ops_gpu.py).
  * whole 16-bit forward, three batch maxima per case: logits against the fp32
    oracle, logits against the rounding-emulating oracle of the same precision
    class (pinned by tests/test_oracle_emulate.py), value against that oracle.
    The logits here are O(1..10) (Xavier-uniform heads), and rounding every GEMM
    operand to fp16 / bf16 moves them by ~5e-3 / ~5e-2 at the maximum over a batch
    whatever the implementation: at B = 16384 on the headline config 98.0 % of the
    kernel's logits are within 2e-3 of the fp32 oracle (p99.9 3.0e-3, max 5.4e-3),
    against 98.0 % / 3.0e-3 / 5.1e-3 for the CPU emulation and 92.7 % / 3.9e-3 /
    6.3e-3 for the torch-ROCm eager fp16 forward of the same module.  The
    ceilings are the values measured on these seeded cases (the kernels are
    bitwise reproducible) plus 25 %; the emulated oracle's own distance to fp32 is
    printed beside them for orientation.
  * argmax gear actions identical wherever the oracle's top-2 margin > 1e-2
    (fp16; bf16 cannot decide margins below its own rounding error: a literal
    margin per case, about twice its fp32 ceiling), against both oracles.
"""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

from beatsaberrl_amd.config_policy import ConfigPolicy  # noqa: E402
from oracle import config_model as cm  # noqa: E402

DEV = "cuda"


def _build(spec, seed, dtype, route, randomize_affine=True):
    p = cm.init_params(spec, seed, randomize_affine=randomize_affine)
    m = ConfigPolicy.from_spec(spec, dtype=dtype, route=route)
    m.load_state_dict(p)
    return p, m.to(DEV)


def _check16(lg, v, p, spec, obs, k, dtype, round_residual, ceil, margin=None):
    """ceil = (logits vs fp32 oracle, logits vs same-class oracle, value vs same-class oracle): literal ceilings on
    the batch maximum, written at the call site.  margin: the top-2 margin above which the gear must match."""
    lg, v = lg.float().cpu(), v.float().cpu()
    ref_lg, ref_v = cm.forward(p, spec, obs, k)
    em_lg, em_v = cm.forward(p, spec, obs, k, emulate=dtype, round_residual=round_residual)
    e_class = (lg - em_lg).abs().max().item()
    e_val = (v - em_v).abs().max().item()
    e_mine = (lg - ref_lg).abs().max().item()
    e_emul = (em_lg - ref_lg).abs().max().item()          # printed for orientation only: no gate depends on it
    err = (lg - ref_lg).abs().flatten()
    print(f"\nGATE16 {os.environ.get('PYTEST_CURRENT_TEST', '?').split(' ')[0]} dtype={dtype} B={lg.shape[0]} "
          f"fp32={e_mine:.3e} class={e_class:.3e} value={e_val:.3e} | emulated-oracle-vs-fp32={e_emul:.3e} "
          f"within2e-3={(err <= 2e-3).float().mean().item():.4f} rms={err.pow(2).mean().sqrt().item():.2e}")
    c_fp32, c_class, c_val = ceil
    assert e_mine <= c_fp32, (e_mine, c_fp32)
    assert e_class <= c_class, (e_class, c_class)
    assert e_val <= c_val, (e_val, c_val)
    # argmax gate: identical gear wherever the oracle's top-2 margin > 1e-2 (fp16).  bf16 cannot decide margins below
    # its own operand-rounding error, so its margin is a literal per call site (about twice the fp32 ceiling).
    thr = margin if margin is not None else 1e-2
    assert dtype != "bf16" or margin is not None
    for name, r in (("class", em_lg), ("fp32", ref_lg)):
        decided = cm.top2_margin(r) > thr
        same = lg.argmax(-1) == r.argmax(-1)
        assert bool((same | ~decided).all()), f"argmax differs on a decided head ({name})"
        assert decided.float().mean() > 0.5


def test_config0_fp32_b256():
    c = cm.CONFIGS[0]
    spec = c["spec"]
    p, m = _build(spec, c["w_seed"], "f32", "ops", randomize_affine=False)
    obs, k = cm.make_inputs(spec, c["B"], c["obs_seed"], c["mask"])
    lg, v = m.forward_stacked(obs.to(DEV), None)
    ref_lg, ref_v = cm.forward(p, spec, obs, None)
    assert lg.shape == (256, 29, 7) and lg.dtype is torch.float32 and v.shape == (256,)
    scale = ref_lg.abs().max().item()
    err = (lg.cpu() - ref_lg).abs()
    assert bool((err <= 1e-5 * (ref_lg.abs() + scale)).all()), err.max().item()
    assert bool(((v.cpu() - ref_v).abs() <= 1e-5 * (ref_v.abs() + ref_v.abs().max())).all())
    assert torch.equal(lg.cpu().argmax(-1), ref_lg.argmax(-1)) or bool(
        ((lg.cpu().argmax(-1) == ref_lg.argmax(-1)) | (cm.top2_margin(ref_lg) <= 1e-2)).all())
    # the masked variant of the same model, fp32
    obs2, k2 = cm.make_inputs(spec, 64, 9, "uniform")
    lg2, v2 = m.forward_stacked(obs2.to(DEV), k2.to(DEV))
    r2, rv2 = cm.forward(p, spec, obs2, k2)
    assert bool(((lg2.cpu() - r2).abs() <= 1e-5 * (r2.abs() + r2.abs().max())).all())


@pytest.mark.parametrize("ci,B,ceil,margin", [
    (1, 1024, (7.4e-3, 5.9e-3, 3.0e-3), None), (2, 192, (9.1e-2, 6.6e-2, 4.2e-2), 0.15),
    # config 3, measured: 1.19e-2 / 9.9e-3 / 8.4e-3 with the block FFNs fused (1.22e-2 / 9.2e-3 / 6.6e-3 as two Linears:
    # the same rounding points in another fp32 order; rms 2.78e-3 against 2.80e-3, 53.1 % against 53.0 % within 2e-3)
    (3, 48, (1.6e-2, 1.2e-2, 1.0e-2), None), (4, 64, (4.9e-3, 3.5e-3, 2.3e-3), None),
    (4, 8, (4.9e-3, 3.5e-3, 2.3e-3), None), (4, 1, (4.9e-3, 3.5e-3, 2.3e-3), None)])
def test_configs_16bit_ops_route(ci, B, ceil, margin):
    c = cm.CONFIGS[ci]
    spec = c["spec"]
    p, m = _build(spec, c["w_seed"], c["dtype"], "ops")
    obs, k = cm.make_inputs(spec, B, c["obs_seed"], c["mask"])
    lg, v = m.forward_stacked(obs.to(DEV), k.to(DEV))
    _check16(lg, v, p, spec, obs, k, c["dtype"], round_residual=True, ceil=ceil, margin=margin)


@pytest.mark.parametrize("act,final_ln,dtype", [("relu", True, "f16"), ("gelu", True, "bf16"), ("relu", False, "f32")])
def test_variants_ops_route(act, final_ln, dtype):
    spec = cm.ConfigSpec(3, 128, 4, 256, 16, act=act, final_ln=final_ln)
    p, m = _build(spec, 21, dtype, "ops")
    obs, k = cm.make_inputs(spec, 100, 22, "quarter_empty")
    lg, v = m.forward_stacked(obs.to(DEV), k.to(DEV))
    if dtype == "f32":
        r, rv = cm.forward(p, spec, obs, k)
        assert bool(((lg.cpu() - r).abs() <= 1e-5 * (r.abs() + r.abs().max())).all())
    else:
        ceil, margin = ((4.8e-3, 3.1e-3, 1.7e-3), None) if dtype == "f16" else ((3.5e-2, 2.3e-2, 1.4e-2), 0.07)
        _check16(lg, v, p, spec, obs, k, dtype, round_residual=True, ceil=ceil, margin=margin)


@pytest.mark.parametrize("dtype,tol", [("f32", 2e-6), ("f16", 2.5e-3)])
def test_ops_route_final_block_pruned_to_token0_matches_the_dense_form(dtype, tol):
    """The per-op route computes only token 0 of the final block (keys / values of every token): exact in exact
    arithmetic (the reference's n_queries path, python/policy.py:533-539).  fp32: the same numbers to rounding of a
    different GEMM geometry; fp16: within the stream's own rounding, and against the oracle's pruned form."""
    spec = cm.ConfigSpec(3, 128, 4, 256, 16, act="gelu", final_ln=True)
    p, m = _build(spec, 31, dtype, "ops")
    obs, k = cm.make_inputs(spec, 300, 32, "quarter_empty")
    assert m.prune_final
    lg, v = m.forward_stacked(obs.to(DEV), k.to(DEV))
    m.prune_final = False
    lg_d, v_d = m.forward_stacked(obs.to(DEV), k.to(DEV))
    scale = lg_d.abs().max().item()
    assert (lg - lg_d).abs().max().item() <= tol * max(scale, 1.0), ((lg - lg_d).abs().max().item(), scale)
    assert (v - v_d).abs().max().item() <= tol * max(v_d.abs().max().item(), 1.0)
    r_p, rv_p = cm.forward(p, spec, obs, k, prune_final=True)
    r_d, rv_d = cm.forward(p, spec, obs, k)
    assert (r_p - r_d).abs().max().item() <= 2e-6 * max(r_d.abs().max().item(), 1.0)      # the oracle's own two forms agree
    if dtype == "f32":
        assert bool(((lg.cpu() - r_p).abs() <= 1e-5 * (r_p.abs() + r_p.abs().max())).all())
    # no mask at all: the same
    m.prune_final = True
    lg2, _ = m.forward_stacked(obs.to(DEV), None)
    m.prune_final = False
    lg2_d, _ = m.forward_stacked(obs.to(DEV), None)
    assert (lg2 - lg2_d).abs().max().item() <= tol * max(lg2_d.abs().max().item(), 1.0)


def test_ops_route_block_tail_fusions_keep_the_forward_at_d384():
    """d = 384 per-op route: (a) everything separate, (b) a block's output projection + LN2 + FFN + next LN1 in one kernel,
    (c) also the next block's q|k|v (and block 0's LN1 + q|k|v) from that kernel - the default.  Same rounding points, other
    accumulation orders: the three agree to the stream's rounding, and each holds config 3's ceilings against the oracle."""
    c = cm.CONFIGS[3]
    spec = c["spec"]
    p, m = _build(spec, c["w_seed"], "f16", "ops")
    obs, k = cm.make_inputs(spec, 40, c["obs_seed"], c["mask"])
    od, kd = obs.to(DEV), k.to(DEV)
    assert m.fuse_block_tail and m.fuse_next_proj
    lg_c, v_c = m.forward_stacked(od, kd)
    m.fuse_next_proj = False
    lg_b, v_b = m.forward_stacked(od, kd)
    m.fuse_block_tail = False
    lg_a, v_a = m.forward_stacked(od, kd)
    ref_lg, _ = cm.forward(p, spec, obs, k)
    scale = ref_lg.abs().max().item()
    for lg in (lg_a, lg_b, lg_c):
        assert (lg.cpu() - ref_lg).abs().max().item() <= 1.6e-2            # config 3's literal ceiling (see the 16-bit route test)
    e_a = (lg_a.cpu() - ref_lg).abs().pow(2).mean().sqrt().item()
    for lg in (lg_b, lg_c):
        assert (lg - lg_a).abs().max().item() <= 1.2e-2 and scale > 5.0
        e = (lg.cpu() - ref_lg).abs().pow(2).mean().sqrt().item()
        assert e <= 1.15 * e_a, (e, e_a)                                   # no worse an error class than the separate launches
    assert (v_c - v_a).abs().max().item() <= 1.2e-2 and (v_b - v_a).abs().max().item() <= 1.2e-2
    # unpruned, with the fusions: the last block then also goes through the one-kernel tail (no LayerNorm behind it)
    m.fuse_block_tail = m.fuse_next_proj = True
    m.prune_final = False
    lg_d, _ = m.forward_stacked(od, kd)
    assert (lg_d - lg_c).abs().max().item() <= 1.2e-2


def test_masked_slots_cannot_change_outputs_on_gpu():
    c = cm.CONFIGS[1]
    spec = c["spec"]
    p, m = _build(spec, 1, "f16", "ops")
    obs, k = cm.make_inputs(spec, 64, 3, "uniform")
    lg, v = m.forward_stacked(obs.to(DEV), k.to(DEV))
    obs2 = obs.clone()
    for e in range(64):
        obs2[e, spec.prop_dim + int(k[e]) * spec.obj_dim:] = 77.0
    lg2, v2 = m.forward_stacked(obs2.to(DEV), k.to(DEV))
    assert torch.equal(lg, lg2) and torch.equal(v, v2)


@pytest.mark.parametrize("route", ["ops", "fused"])
def test_weights_version_refreshes_replicas(route):
    """16-bit weight copies are rebuilt only when the weights version is bumped
    (the reference's contract: python/fp16_linear.py:228-246)."""
    c = cm.CONFIGS[1]
    spec = c["spec"]
    p, m = _build(spec, 1, "f16", route)
    obs, k = cm.make_inputs(spec, 16, 3, "uniform")
    a, _ = m.forward_stacked(obs.to(DEV), k.to(DEV))
    with torch.no_grad():
        m.heads.weight.zero_()
    b, _ = m.forward_stacked(obs.to(DEV), k.to(DEV))
    assert torch.equal(a, b)              # stale 16-bit copy until the version is bumped
    m.bump_weights_version()
    c2, _ = m.forward_stacked(obs.to(DEV), k.to(DEV))
    want = m.heads.bias[:-1].view(1, 29, 7).expand(16, 29, 7)
    assert torch.allclose(c2, want, atol=1e-6)


# ------------------------------------------------------------------ fused whole-forward kernel
@pytest.mark.parametrize("prune", [False, True])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("B", [1, 8, 64, 1000, 4096])
def test_fused_route_config1(dtype, B, prune):
    """The throughput forms at every batch size (the latency form that small batches take by default is switched off):
    prune=False: one persistent kernel, every token of the last block; prune=True: the two-launch form with
    final-block query pruning."""
    c = cm.CONFIGS[1]
    spec = c["spec"]
    p, m = _build(spec, c["w_seed"], dtype, "fused")
    m.prune_final = prune
    m.latency_form = False
    assert m.fused_supported()
    obs, k = cm.make_inputs(spec, B, c["obs_seed"], c["mask"])
    lg, v = m.forward_stacked(obs.to(DEV), k.to(DEV))
    assert lg.shape == (B, 29, 7) and lg.dtype is torch.float32 and v.shape == (B,)
    ceil, margin = ((6.4e-3, 4.9e-3, 3.4e-3), None) if dtype == "f16" else ((5.1e-2, 4.2e-2, 2.7e-2), 0.1)
    _check16(lg, v, p, spec, obs, k, dtype, round_residual=False, ceil=ceil, margin=margin)


@pytest.mark.parametrize("w_seed,obs_seed,mask", [(1, 2, "uniform"), (11, 12, "uniform"), (21, 22, "none"), (31, 32, "uniform"),
                                                  (41, 42, "quarter_empty")])
def test_fused_route_error_distribution_over_seeds(w_seed, obs_seed, mask):
    """How close the 16-bit forward is to the fp32 oracle does not hang on one draw of weights and inputs: five
    (weights, observations, mask) draws of the headline model at B = 4096, fp16, each with its share of logits within
    2e-3 of the fp32 oracle, its 99.9th percentile and its maximum under literal bounds (the first draw is the
    benchmark's own; measured over the five: share 0.973-0.993, p99.9 2.5e-3-3.1e-3, max 3.6e-3-5.0e-3)."""
    spec, B = cm.CONFIGS[1]["spec"], 4096
    p, m = _build(spec, w_seed, "f16", "fused", randomize_affine=False)
    obs, k = cm.make_inputs(spec, B, obs_seed, mask)
    lg, v = m.forward_stacked(obs.to(DEV), None if k is None else k.to(DEV))
    ref_lg, ref_v = cm.forward(p, spec, obs, k)
    err = (lg.float().cpu() - ref_lg).abs().flatten()
    share = (err <= 2e-3).float().mean().item()
    p999 = torch.quantile(err[torch.randperm(err.numel(), generator=torch.Generator().manual_seed(0))[:1000000]], 0.999).item()
    print(f"\nDIST w_seed={w_seed} obs_seed={obs_seed} mask={mask}: within2e-3={share:.4f} p99.9={p999:.3e} max={err.max().item():.3e} "
          f"value max={(v.float().cpu() - ref_v).abs().max().item():.3e}")
    assert share >= 0.965 and p999 <= 3.6e-3 and err.max().item() <= 6.3e-3


@pytest.mark.parametrize("act,final_ln,L,ffn,dtype,ceil,margin", [
    ("relu", True, 3, 256, "f16", (3.8e-3, 2.7e-3, 2.1e-3), None), ("gelu", True, 1, 512, "bf16", (2.5e-2, 1.8e-2, 1.1e-2), 0.05),
    ("relu", False, 4, 1024, "f16", (9.1e-3, 7.2e-3, 4.7e-3), None), ("gelu", False, 8, 64, "f16", (1.4e-2, 1.2e-2, 5.9e-3), None)])
def test_fused_route_variants(act, final_ln, L, ffn, dtype, ceil, margin):
    spec = cm.ConfigSpec(L, 128, 4, ffn, 16, act=act, final_ln=final_ln)
    p, m = _build(spec, 31, dtype, "fused")
    m.latency_form = False
    obs, k = cm.make_inputs(spec, 333, 32, "quarter_empty")
    for prune in (False, True):
        m.prune_final = prune
        lg, v = m.forward_stacked(obs.to(DEV), k.to(DEV))
        _check16(lg, v, p, spec, obs, k, dtype, round_residual=False, ceil=ceil, margin=margin)


def test_fused_route_other_obs_layouts_and_no_mask():
    """Smaller proprio/object widths, n_gears 5, obs already in the stream dtype, no mask."""
    spec = cm.ConfigSpec(2, 128, 4, 512, 16, n_gears=5, prop_dim=37, obj_dim=9)
    p, m = _build(spec, 41, "f16", "fused")
    obs, _ = cm.make_inputs(spec, 100, 42, "none")
    lg, v = m.forward_stacked(obs.to(DEV), None)
    assert lg.shape == (100, 29, 5)
    _check16(lg, v, p, spec, obs, None, "f16", round_residual=False, ceil=(4.2e-3, 3.5e-3, 1.9e-3))
    lg2, v2 = m.forward_stacked(obs.half().to(DEV), None)
    assert torch.equal(lg, lg2) and torch.equal(v, v2)       # the kernel rounds fp32 obs to fp16 once on entry


@pytest.mark.parametrize("prune", [False, True])
def test_fused_route_invariants(prune):
    c = cm.CONFIGS[1]
    spec = c["spec"]
    p, m = _build(spec, 1, "f16", "fused")
    m.prune_final = prune
    m.latency_form = False
    obs, k = cm.make_inputs(spec, 700, 3, "uniform")
    od, kd = obs.to(DEV), k.to(DEV)
    lg, v = m.forward_stacked(od, kd)
    # an env's bits do not depend on the batch it sits in or on its tile / wave position
    for lo, hi in ((0, 1), (5, 70), (333, 700)):
        l2, v2 = m.forward_stacked(od[lo:hi].contiguous(), kd[lo:hi].contiguous())
        assert torch.equal(l2, lg[lo:hi]) and torch.equal(v2, v[lo:hi])
    # junk in masked object slots cannot change anything
    obs2 = obs.clone()
    for e in range(700):
        obs2[e, spec.prop_dim + int(k[e]) * spec.obj_dim:] = 99.0
    l3, v3 = m.forward_stacked(obs2.to(DEV), kd)
    assert torch.equal(l3, lg) and torch.equal(v3, v)
    # fused and per-op routes agree to the precision class
    l4, v4 = m.forward_stacked(od, kd, route="ops")
    assert (l4 - lg).abs().max().item() < 1e-2
    # repeated launches are bitwise reproducible
    l5, v5 = m.forward_stacked(od, kd)
    assert torch.equal(l5, lg) and torch.equal(v5, v)
    # pruned and unpruned forms agree to fp32-accumulation-order level on most logits
    m.prune_final = not prune
    l6, _ = m.forward_stacked(od, kd)
    assert (l6 - lg).abs().max().item() < 5e-3


@pytest.mark.parametrize("B", [70001, 270003])
def test_fused_route_packed_tiles_at_a_batch_with_several_envs_per_pairing_thread(B):
    """B > 65536: the tile-table kernel walks several envs per thread (kept in registers up to 4, re-read from memory
    beyond: B > 262144); same bits as one env per tile."""
    c = cm.CONFIGS[1]
    spec = c["spec"]
    _, m = _build(spec, c["w_seed"], "f16", "fused")
    obs, k = cm.make_inputs(spec, B, 77, "uniform")
    od, kd = obs.to(DEV), k.to(DEV)
    lg1, v1 = m.forward_stacked(od, kd)
    m.pack_short = False
    lg0, v0 = m.forward_stacked(od, kd)
    assert torch.equal(lg1, lg0) and torch.equal(v1, v0)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("case", ["uniform", "all_short", "all_long", "one_short", "odd_short", "alternating", "all_tiny",
                                  "all_mid", "five_tiny", "host_tiny", "few_hosts", "many_hosts"])
@pytest.mark.parametrize("B", [1, 9, 700, 4099])
def test_fused_route_packed_tiles_give_the_unpacked_bits(dtype, case, B):
    """`pack_short` (envs of 5..8 tokens two to a 16-row tile, of at most 4 tokens behind an env of 9..12 tokens or four
    to a tile, in the pruned form's first launch) against one env per tile: logits and values are bitwise equal for every mix of short and long envs, and both match the oracle."""
    c = cm.CONFIGS[1]
    spec = c["spec"]
    p, m = _build(spec, c["w_seed"], dtype, "fused")
    m.latency_form = False                       # the packed first launch is a throughput form: keep small batches on it
    obs, k = cm.make_inputs(spec, B, 40 + B, "uniform")
    if case == "all_short":
        k = k % 8
    elif case == "all_long":
        k = 8 + k % 8
    elif case == "one_short":
        k = 8 + k % 8
        k[B // 2] = 3
    elif case == "odd_short":
        k = 8 + k % 8
        k[: min(B, 5)] = torch.tensor([0, 7, 2, 5, 1], dtype=torch.int32)[: min(B, 5)]
    elif case == "all_tiny":
        k = k % 4
    elif case == "all_mid":
        k = 4 + k % 4
    elif case == "five_tiny":
        k = 8 + k % 8
        k[: min(B, 5)] = torch.tensor([0, 3, 2, 1, 3], dtype=torch.int32)[: min(B, 5)]
    elif case == "host_tiny":                     # every tiny env finds a 9..12-token host
        k = torch.where(torch.arange(B) % 2 == 0, 8 + k % 4, k % 4).to(torch.int32)
    elif case == "few_hosts":                     # more tiny envs than hosts: the rest go four to a tile
        k = k % 4
        k[::7] = 9
    elif case == "many_hosts":                    # more hosts than tiny envs
        k = 8 + k % 4
        k[::5] = 2
    elif case == "alternating":
        k = torch.where(torch.arange(B) % 2 == 0, k % 8, 8 + k % 8).to(torch.int32)
    od, kd = obs.to(DEV), k.to(DEV)
    m.pack_short = True
    lg1, v1 = m.forward_stacked(od, kd)
    m.pack_short = False
    lg0, v0 = m.forward_stacked(od, kd)
    assert torch.equal(lg1, lg0) and torch.equal(v1, v0)
    if B == 700:                                  # the class bounds are max statistics: not for a handful of envs
        ceil, margin = ((5.8e-3, 4.8e-3, 3.4e-3), None) if dtype == "f16" else ((5.2e-2, 3.9e-2, 2.9e-2), 0.1)
        _check16(lg1, v1, p, spec, obs, k, dtype, round_residual=False, ceil=ceil, margin=margin)
    # junk in the masked slots of a packed env cannot leak into its tile partner
    obs2 = obs.clone()
    for e in range(B):
        obs2[e, spec.prop_dim + int(k[e]) * spec.obj_dim:] = -77.0
    m.pack_short = True
    lg2, v2 = m.forward_stacked(obs2.to(DEV), kd)
    assert torch.equal(lg2, lg1) and torch.equal(v2, v1)


def test_fused_route_packed_forward_replays_in_a_graph_with_new_key_counts():
    """The packed forward is capturable: the tile table is rebuilt on the device by every replay (its grid does not
    depend on the key counts), so a replay with new obs AND new key counts in the static buffers returns the eager bits."""
    c = cm.CONFIGS[1]
    spec = c["spec"]
    _, m = _build(spec, c["w_seed"], "f16", "fused")
    m.latency_form = False
    B = 3000
    obs0, k0 = cm.make_inputs(spec, B, 1, "uniform")
    s_obs, s_k = obs0.to(DEV), k0.to(DEV)
    m.forward_stacked(s_obs, s_k)                                  # warm-up: image, workspace
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        g_lg, g_v = m.forward_stacked(s_obs, s_k)
    for seed, mask in ((5, "uniform"), (6, "quarter_empty"), (7, "none"), (8, "uniform")):
        obs, k = cm.make_inputs(spec, B, seed, mask)
        s_obs.copy_(obs.to(DEV))
        s_k.copy_(k.to(DEV))
        g.replay()
        got_lg, got_v = g_lg.clone(), g_v.clone()
        x = torch.randn(300, 300, device=DEV)
        (x @ x).sum().item()                                       # unrelated eager work and a sync between replays
        lg, v = m.forward_stacked(obs.to(DEV), k.to(DEV))
        assert torch.equal(got_lg, lg) and torch.equal(got_v, v), seed


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("B", [1, 8, 64, 257, 700, 1024])
def test_fused_route_latency_form(dtype, B):
    """The form small batches take by default (B <= 4 per CU): one persistent launch, one env per wave (1..4 working
    waves per workgroup), weights through the deep direct-to-LDS ring.  Its output BITS are those of both throughput
    forms - so an env's result does not depend on the batch size picking the kernel - and it holds the same literal
    ceilings against the oracle, batch-slice invariance and masked-junk invariance."""
    c = cm.CONFIGS[1]
    spec = c["spec"]
    p, m = _build(spec, c["w_seed"], dtype, "fused")
    assert m.latency_form
    obs, k = cm.make_inputs(spec, B, c["obs_seed"], c["mask"])
    od, kd = obs.to(DEV), k.to(DEV)
    lg, v = m.forward_stacked(od, kd)
    assert lg.shape == (B, 29, 7) and lg.dtype is torch.float32 and v.shape == (B,)
    # (bf16 at B = 1024, a batch the other tests do not run: 4.44e-2 / 2.99e-2 / 2.84e-2)
    ceil, margin = ((6.4e-3, 4.9e-3, 3.4e-3), None) if dtype == "f16" else ((5.6e-2, 4.2e-2, 3.6e-2), 0.11)
    _check16(lg, v, p, spec, obs, k, dtype, round_residual=False, ceil=ceil, margin=margin)
    l2, v2 = m.forward_stacked(od, kd)
    assert torch.equal(l2, lg) and torch.equal(v2, v)                         # reproducible
    if B >= 64:
        for lo, hi in ((0, 1), (5, 9), (33, 64)):
            l3, v3 = m.forward_stacked(od[lo:hi].contiguous(), kd[lo:hi].contiguous())
            assert torch.equal(l3, lg[lo:hi]) and torch.equal(v3, v[lo:hi])   # batch / wave position invariance
    obs2 = obs.clone()
    for e in range(B):
        obs2[e, spec.prop_dim + int(k[e]) * spec.obj_dim:] = 55.0
    l4, v4 = m.forward_stacked(obs2.to(DEV), kd)
    assert torch.equal(l4, lg) and torch.equal(v4, v)                         # masked junk cannot leak
    m.latency_form = False
    for prune in (False, True):                                               # the throughput forms: the same bits
        m.prune_final = prune
        l5, v5 = m.forward_stacked(od, kd)
        assert torch.equal(l5, lg) and torch.equal(v5, v), prune


@pytest.mark.parametrize("act,final_ln,L,ffn,dtype,ceil,margin", [
    ("relu", True, 3, 256, "f16", (3.8e-3, 2.7e-3, 2.1e-3), None), ("gelu", True, 1, 512, "bf16", (2.5e-2, 1.8e-2, 1.1e-2), 0.05),
    ("gelu", False, 6, 64, "f16", (1.4e-2, 1.2e-2, 5.9e-3), None)])
def test_fused_route_latency_form_variants(act, final_ln, L, ffn, dtype, ceil, margin):
    spec = cm.ConfigSpec(L, 128, 4, ffn, 16, act=act, final_ln=final_ln)
    p, m = _build(spec, 31, dtype, "fused")
    obs, k = cm.make_inputs(spec, 333, 32, "quarter_empty")
    lg, v = m.forward_stacked(obs.to(DEV), k.to(DEV))
    _check16(lg, v, p, spec, obs, k, dtype, round_residual=False, ceil=ceil, margin=margin)
    lg0, v0 = m.forward_stacked(obs.to(DEV), None)                             # no mask == full mask
    full = torch.full((333,), spec.T - 1, dtype=torch.int32, device=DEV)
    lg1, v1 = m.forward_stacked(obs.to(DEV), full)
    assert torch.equal(lg0, lg1) and torch.equal(v0, v1)
    m.latency_form = False
    lg2, v2 = m.forward_stacked(obs.to(DEV), k.to(DEV))
    assert torch.equal(lg2, lg) and torch.equal(v2, v)


def test_fused_route_eight_layer_model_has_no_latency_form():
    """Vectors + ring beyond a workgroup's LDS: small batches take the throughput forms, silently."""
    spec = cm.ConfigSpec(8, 128, 4, 2048, 16)
    p, m = _build(spec, 31, "f16", "fused")
    obs, k = cm.make_inputs(spec, 5, 32, "uniform")
    a = m.forward_stacked(obs.to(DEV), k.to(DEV))
    m.latency_form = False
    b = m.forward_stacked(obs.to(DEV), k.to(DEV))
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_fused_route_latency_form_replays_in_a_graph():
    c = cm.CONFIGS[1]
    spec = c["spec"]
    _, m = _build(spec, c["w_seed"], "f16", "fused")
    obs0, k0 = cm.make_inputs(spec, 64, 1, "uniform")
    s_obs, s_k = obs0.to(DEV), k0.to(DEV)
    m.forward_stacked(s_obs, s_k)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        g_lg, g_v = m.forward_stacked(s_obs, s_k)
    for seed in (5, 6, 7):
        obs, k = cm.make_inputs(spec, 64, seed, "uniform")
        s_obs.copy_(obs.to(DEV)); s_k.copy_(k.to(DEV))
        g.replay()
        got_lg, got_v = g_lg.clone(), g_v.clone()
        x = torch.randn(300, 300, device=DEV)
        (x @ x).sum().item()
        lg, v = m.forward_stacked(obs.to(DEV), k.to(DEV))
        assert torch.equal(got_lg, lg) and torch.equal(got_v, v), seed


def test_fused_unsupported_shapes_fall_to_ops_route():
    for ci in (2, 3):
        spec = cm.CONFIGS[ci]["spec"]
        m = ConfigPolicy.from_spec(spec, dtype=cm.CONFIGS[ci]["dtype"])
        assert not m.fused_supported()
    assert not ConfigPolicy.from_spec(cm.CONFIGS[0]["spec"], dtype="f32").fused_supported()
    # config 2 (d = 256, T = 32) has the fused block stack, config 3 (d = 384, T = 48) only the per-op route
    assert ConfigPolicy.from_spec(cm.CONFIGS[2]["spec"], dtype="bf16").blocks_supported()
    assert not ConfigPolicy.from_spec(cm.CONFIGS[3]["spec"], dtype="f16").blocks_supported()
    assert not ConfigPolicy.from_spec(cm.CONFIGS[2]["spec"], dtype="f32").blocks_supported()


@pytest.mark.parametrize("ci,B,ceil,margin", [
    (2, 192, (7.7e-2, 6.3e-2, 4.1e-2), 0.14), (2, 7, (4.4e-2, 4.5e-2, 1.4e-2), 0.14),
    (1, 333, (5.2e-3, 5.0e-3, 3.3e-3), None), (4, 8, (4.2e-3, 3.0e-3, 1.9e-3), None)])
def test_blocks_route(ci, B, ceil, margin):
    """Tokenizer kernel + fused block stack (final block pruned to token 0) + heads: the residual stream stays in
    fp32 registers through the stack, as on the fused route (round_residual=False class)."""
    c = cm.CONFIGS[ci]
    spec = c["spec"]
    p, m = _build(spec, c["w_seed"], c["dtype"], "blocks")
    obs, k = cm.make_inputs(spec, B, c["obs_seed"], c["mask"])
    lg, v = m.forward_stacked(obs.to(DEV), k.to(DEV))
    _check16(lg, v, p, spec, obs, k, c["dtype"], round_residual=False, ceil=ceil, margin=margin)
    # "auto" picks this route for config 2, and no mask == the full mask
    if ci == 2:
        m.route = "auto"
        lg2, v2 = m.forward_stacked(obs.to(DEV), k.to(DEV))
        assert torch.equal(lg, lg2) and torch.equal(v, v2)
    full = torch.full((B,), spec.T - 1, dtype=torch.int32, device=DEV)
    la, va = m.forward_stacked(obs.to(DEV), None, route="blocks")
    lb, vb = m.forward_stacked(obs.to(DEV), full, route="blocks")
    assert torch.equal(la, lb) and torch.equal(va, vb)


@pytest.mark.parametrize("act,final_ln,dtype", [("relu", True, "f16"), ("gelu", True, "bf16")])
def test_blocks_route_variants(act, final_ln, dtype):
    spec = cm.ConfigSpec(3, 256, 8, 512, 32, act=act, final_ln=final_ln, prop_dim=100, obj_dim=16)
    p, m = _build(spec, 23, dtype, "blocks")
    obs, k = cm.make_inputs(spec, 70, 24, "quarter_empty")
    lg, v = m.forward_stacked(obs.to(DEV), k.to(DEV))
    ceil, margin = ((4.2e-3, 4.1e-3, 2.4e-3), None) if dtype == "f16" else ((3.1e-2, 3.0e-2, 1.8e-2), 0.06)
    _check16(lg, v, p, spec, obs, k, dtype, round_residual=False, ceil=ceil, margin=margin)


# ------------------------------------------------------------------ the tolerance asked of the 16-bit forward, on the config's own operands
def _three_way(ci, B, route):
    """Error distributions of one forward against the three references: the fp32 oracle on the fp32 masters, the SAME
    oracle on the config's own 16-bit operands (cm.round_operands: weight matrices and observations rounded once, the
    arithmetic fp32 - the reference's kernel-test idiom, python/tests/test_attn29.py:49-54, 110-111 and
    test_fp16_accum.py:84-89), and the rounding-emulating oracle of the route's precision class.  Weights are the
    config's own draw (Xavier-uniform, LayerNorm 1 / 0)."""
    c = cm.CONFIGS[ci]
    spec, dtype = c["spec"], c["dtype"]
    p, m = _build(spec, c["w_seed"], dtype, route, randomize_affine=False)
    obs, k = cm.make_inputs(spec, B, c["obs_seed"], c["mask"])
    lg, _ = m.forward_stacked(obs.to(DEV), k.to(DEV))
    lg = lg.float().cpu()
    ref, _ = cm.forward(p, spec, obs, k)
    p_sw, obs_sw = cm.round_operands(p, obs, dtype)
    sw, _ = cm.forward(p_sw, spec, obs_sw, k)
    em, _ = cm.forward(p, spec, obs, k, emulate=dtype, round_residual=route == "ops")

    def dist(a, b):
        e = (a - b).abs().flatten().sort().values
        return ((e <= 2e-3).float().mean().item(), e[min(int(0.999 * e.numel()), e.numel() - 1)].item(), e[-1].item())

    def agree(r):
        decided = cm.top2_margin(r) > 1e-2
        return (lg.argmax(-1) == r.argmax(-1))[decided].float().mean().item()

    out = {"fp32": dist(lg, ref), "same": dist(lg, sw), "class": dist(lg, em), "weights_alone": dist(sw, ref),
           "agree_same": agree(sw), "agree_fp32": agree(ref)}
    f = lambda t: f"{t[0]:.5f} / {t[1]:.3e} / {t[2]:.3e}"
    print(f"\nTHREEWAY config {ci} B={B} {route} {dtype} (share within 2e-3 / p99.9 / max): vs fp32 weights {f(out['fp32'])} | "
          f"vs same 16-bit operands {f(out['same'])} | vs class emulation {f(out['class'])} | the operands' rounding alone "
          f"{f(out['weights_alone'])} | argmax where margin > 1e-2: same {out['agree_same']:.5f}, fp32 {out['agree_fp32']:.5f}")
    return out


@pytest.mark.parametrize("ci,B,max_ceiling", [(1, 4096, 4.2e-3), (1, 16384, 4.2e-3), (4, 64, 2.3e-3), (4, 8, 2.1e-3), (4, 1, 1.8e-3)])
def test_fp16_forward_holds_2e_3_on_the_configs_own_operands(ci, B, max_ceiling):
    """The tolerance asked of the fp16 forward - logits within 2e-3 absolute, argmax identical where the top-2 margin
    exceeds 1e-2 - held as literals on the route the fp16 configs of the headline model take ("fused"), against the
    fp32 oracle on the config's own fp16 weights and observations: at least 99.9 % of the logits within 2e-3 and the
    99.9th percentile within 2e-3 (measured at B = 16384: 99.925 %, 1.94e-3); every decided gear identical.  The batch
    MAXIMUM over millions of logits is not inside 2e-3 for any forward that rounds its activations to fp16 (the CPU
    emulation of the same rounding points: 2.98e-3 at B = 4096): it is held under a measured ceiling (3.32e-3 at
    B = 4096, 3.29e-3 at 16384, 1.83e-3 at 64; + 25 %)."""
    r = _three_way(ci, B, "fused")
    share, p999, mx = r["same"]
    assert share >= 0.999, share
    assert p999 <= 2e-3, p999
    assert mx <= max_ceiling, mx
    assert r["agree_same"] == 1.0 and r["agree_fp32"] == 1.0


@pytest.mark.parametrize("ci,B,route,floor_share,ceil_p999,ceil_max,floor_agree", [
    # headline model on the other two routes (measured 0.98856 / 2.68e-3 / 5.44e-3 and 0.99774 / 2.18e-3 / 3.54e-3)
    (1, 4096, "ops", 0.985, 3.4e-3, 6.8e-3, 1.0), (1, 4096, "blocks", 0.996, 2.8e-3, 4.5e-3, 1.0),
    # config 2, bf16 (measured 0.2087 / 2.91e-2 / 4.82e-2, agreement 0.99932) and config 3, fp16, 6 x d = 384
    # (measured 0.638 / 8.2e-3 / 1.26e-2 at B = 512, agreement 1)
    (2, 2048, "blocks", 0.19, 3.7e-2, 6.1e-2, 0.998), (3, 256, "ops", 0.60, 1.05e-2, 1.6e-2, 1.0)])
def test_where_2e_3_is_not_reachable_the_distance_is_bounded(ci, B, route, floor_share, ceil_p999, ceil_max, floor_agree):
    """The same comparison where the 2e-3 clause is NOT met, stated plainly and held under measured literals (+ 25 %):
      * the headline model on the per-op route, whose residual stream is rounded to fp16 between kernels as the
        reference's fp16 stream is (python/policy.py:1200-1209): 98.9 % within 2e-3, p99.9 2.7e-3; on the "blocks"
        route (fp32 residual, 16-bit token tensor in between): 99.8 %, 2.2e-3;
      * config 2 is bf16: an 8-bit significand moves logits of magnitude 1..8 by 1e-2..4e-2 whatever the kernel does
        (the fp32 oracle on the bf16-rounded weights is itself 3.0e-2 at p99.9 from the fp32 oracle), so neither the
        2e-3 clause nor "argmax identical above a 1e-2 margin" is reachable in that dtype: agreement 0.9993;
      * config 3 (6 layers of d = 384, fp16): 64 % within 2e-3, p99.9 8.2e-3, every decided gear identical."""
    r = _three_way(ci, B, route)
    share, p999, mx = r["same"]
    assert share >= floor_share and p999 <= ceil_p999 and mx <= ceil_max, r["same"]
    assert r["agree_same"] >= floor_agree, r["agree_same"]
