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
    with pytest.raises(NotImplementedError):
        NotePolicy(value_residual=True)
    with pytest.raises(NotImplementedError):
        NotePolicy(trunk_arch="simbav2")
    with pytest.raises(ValueError):
        NotePolicy(n_gears=4)
    with pytest.raises(RuntimeError, match="GPU only"):
        NotePolicy().forward_stacked(torch.zeros(1, 630))
