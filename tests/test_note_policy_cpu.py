"""Host-side contract of the NotePolicy drop-in, no GPU: parameter names, shapes and
registration order equal the reference's (read from the golden fixtures its own module
wrote), the arch record round-trips, stale layouts are refused."""
import glob
import os

import pytest
import torch

from beatsaberrl_amd import obs_layout as L
from beatsaberrl_amd.policy import NotePolicy, load_policy
from oracle import note_policy_ref as nr

GOLD = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "notepolicy_*.npz")))


@pytest.mark.parametrize("path", GOLD, ids=[os.path.basename(p)[:-4] for p in GOLD])
def test_state_dict_layout_and_arch_match_the_reference(path):
    arch, sd, _, _, _ = nr.load_fixture(path)
    m = load_policy({"arch": arch, "state_dict": sd}, game=arch["game"])
    mine = m.state_dict()
    assert list(mine.keys()) == list(sd.keys())
    for k in sd:
        assert mine[k].shape == sd[k].shape and mine[k].dtype == torch.float32 and torch.equal(mine[k], sd[k])
    assert {k: m.arch[k] for k in arch} == arch and set(m.arch) == set(arch)
    # non-persistent buffers stay out of the state_dict (python/policy.py:933, 1038-1044, 1079-1084)
    assert not any(k.startswith("_") or "value_centers" in k for k in mine)


def test_default_ctor_parameter_count():
    """2,791,734 parameters at 192 / 384 / 3 blocks with note_geo (python/tests/test_trunk_simba.py:37-66)."""
    m = NotePolicy(embed=192, trunk_dim=384, n_blocks=3, n_heads=4, n_gears=5, ffn_mult=4, note_geo=True)
    assert sum(p.numel() for p in m.parameters()) == 2791734


def test_lane_tables_match_the_oracle_restatement():
    assert list(L.SABER_L_IDX) == nr.SABER_L and list(L.SABER_R_IDX) == nr.SABER_R
    assert list(L.TORSO_IDX) == nr.TORSO and list(L.LEG_L_IDX) == nr.LEG_L and list(L.LEG_R_IDX) == nr.LEG_R
    assert L.OFF_NOTE_MASK == 534 and L.OBS_DIM == 630


def test_refusals():
    arch, sd, _, _, _ = nr.load_fixture(GOLD[0])
    with pytest.raises(SystemExit):
        load_policy({"arch": {**arch, "obs_dim": 624}, "state_dict": sd})
    with pytest.raises(SystemExit):
        load_policy({"arch": {**arch, "game": "flux"}, "state_dict": sd})
    with pytest.raises(SystemExit):
        load_policy({"arch": {k: v for k, v in arch.items() if k != "z_asinh"}, "state_dict": sd})
    with pytest.raises(ValueError):
        NotePolicy(trunk_arch="simbav3")
    with pytest.raises(ValueError):
        NotePolicy(n_gears=4)
    with pytest.raises(RuntimeError, match="GPU only"):
        NotePolicy().forward_stacked(torch.zeros(1, 630))


def test_option_modules_exist_only_when_on_and_register_in_the_reference_order():
    """python/tests/test_arch_ab_options.py:131-135, 190-207."""
    kw = dict(embed=64, trunk_dim=96, n_blocks=3, n_heads=2, n_gears=5)
    p = NotePolicy(**kw)
    assert p.emb_ln is None and p.final_ln is None and all(b.vres_a is None for b in p.blocks)
    q = NotePolicy(emb_ln=True, value_residual=True, final_ln=True, trunk_arch="simbav2", **kw)
    assert q.blocks[0].vres_a is None                       # block 0 provides v0
    for blk in q.blocks[1:]:
        assert blk.vres_a.item() == 1.0 and blk.vres_b.item() == 0.0
    order = [n for n, _ in q.named_parameters()]
    assert {"emb_ln.weight", "final_ln.weight", "blocks.1.vres_b", "trunk_alpha", "trunk_in.weight"} <= set(order)
    assert not any(n.startswith(("trunk_proj", "trunk_ln", "trunk_fc")) for n in order)
    assert order.index("emb_ln.bias") < order.index("blocks.0.ln_attn.weight")
    assert order.index("blocks.2.vres_b") < order.index("final_ln.weight") < order.index("trunk_in.weight")
    assert q.arch["value_residual"] is True and q.arch["trunk_arch"] == "simbav2"


def test_simbav2_init_and_projection():
    """python/tests/test_arch_ab_options.py:220-256: unit-norm rows, zero frozen biases, alpha at 0.5."""
    p = NotePolicy(embed=64, trunk_dim=96, n_blocks=2, n_heads=2, n_gears=5, trunk_arch="simbav2", trunk_hidden=128)
    assert [m.weight.shape for m in p.trunk_projected()] == [(96, 320), (128, 96), (96, 128)]
    for m in p.trunk_projected():
        assert torch.allclose(m.weight.norm(dim=1), torch.ones(m.weight.shape[0]), atol=1e-6)
        assert torch.count_nonzero(m.bias) == 0 and not m.bias.requires_grad
    assert torch.allclose(p.trunk_alpha * p._v2_c_alpha, torch.full((96,), 0.5))
    assert torch.allclose(p.trunk_s_in, torch.full((96,), (2.0 / 96) ** 0.5))
    with torch.no_grad():
        p.trunk_w1.weight.mul_(3.0)
        p.trunk_w1.bias.add_(1.0)
    assert p.project_trunk_weights()
    assert torch.allclose(p.trunk_w1.weight.norm(dim=1), torch.ones(128), atol=1e-6)
    assert torch.count_nonzero(p.trunk_w1.bias) == 0
    assert not NotePolicy(embed=64, trunk_dim=96, n_blocks=2, n_heads=2).project_trunk_weights()
