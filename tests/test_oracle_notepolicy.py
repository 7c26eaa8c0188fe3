"""Pins oracle/note_policy_ref.py (no GPU): golden vectors written by the reference's own
NotePolicy (tests/golden/notepolicy_*.npz), the hand-computed note-geometry cases the
reference's tests hold (python/tests/test_policy.py:141-183, test_i07_blade_geo.py:149-200,
restated from the constants), and the lane-routing / masking invariants."""
import glob
import math
import os

import pytest
import torch

from oracle import note_policy_ref as nr

GOLD = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "notepolicy_*.npz")))


def test_fixtures_exist():
    assert len(GOLD) == 4


@pytest.mark.parametrize("path", GOLD, ids=[os.path.basename(p)[:-4] for p in GOLD])
def test_matches_reference_golden_vectors(path):
    arch, sd, obs, logits, value = nr.load_fixture(path)
    lg, v = nr.forward(sd, arch, obs)
    assert lg.shape == logits.shape and v.shape == value.shape
    live = logits > -1e8
    assert torch.equal(live, lg > -1e8)                        # ragged-head fill in the same lanes
    assert (lg[live] - logits[live]).abs().max().item() < 2e-5
    assert torch.equal(lg[~live], logits[~live])               # exactly -1e9
    assert (v - value).abs().max().item() < 2e-5
    assert logits[live].abs().max() > 0.05                     # the fixture is not degenerate


def test_lane_routing_partitions_the_obs():
    """The reference's module-level asserts (python/policy.py:206, 227-228, 269-275)."""
    assert len(nr.SABER_L) == len(nr.SABER_R) == 47 and len(nr.TORSO) == 29 and len(nr.LEG_L) == len(nr.LEG_R) == 32
    body = set(nr.TORSO) | set(nr.LEG_L) | set(nr.LEG_R)
    assert set(nr.TORSO).isdisjoint(nr.LEG_L) and set(nr.TORSO).isdisjoint(nr.LEG_R)
    assert set(nr.LEG_L) & set(nr.LEG_R) == set(range(618, 624))          # the 6 shared leg torque-scale lanes
    assert set(nr.SABER_L) & set(nr.SABER_R) == set(range(611, 618))      # the 7 shared arm torque-scale lanes
    entity = set(range(nr.OFF_NOTES, nr.OFF_MASK + nr.N_SLOTS))
    assert (body | set(nr.SABER_L) | set(nr.SABER_R) | entity) == set(range(nr.OBS_DIM))
    assert nr.SABER_L[44:47] == [624, 625, 626] and nr.SABER_R[44:47] == [627, 628, 629]
    assert nr.OFF_MASK == 534 and nr.SABER_L[15] == 75 and nr.SABER_R[15] == 86


def _geo_of(obs):
    B = obs.shape[0]
    sab = torch.stack([obs[:, nr.SABER_L], obs[:, nr.SABER_R]], 1)
    notes = obs[:, nr.OFF_NOTES:nr.OFF_MASK].reshape(B, 24, 18)
    return nr.note_geo(notes, sab, 8.0, False, obs[:, nr.OBS_HEAD_Z])


def test_note_geo_known_answers_first_14_lanes():
    obs = torch.zeros(1, nr.OBS_DIM)
    hl = 75                                                    # left-hand derived block
    obs[0, hl:hl + 3] = torch.tensor([0.2, -0.3 / 0.75, -0.5])
    obs[0, hl + 3:hl + 6] = torch.tensor([3.0 / 6.0, 0.0, 0.0])
    obs[0, hl + 6:hl + 9] = torch.tensor([0.0, 1.0, 0.0])
    n0 = nr.OFF_NOTES
    obs[0, n0:n0 + 4] = torch.tensor([0.5, 0.15 / 0.75, math.asinh(4.0 / 8.0), -16.0 / 8.0])
    obs[0, n0 + 6], obs[0, n0 + 7] = 1.0, 0.0
    g = _geo_of(obs)[0, 0]
    dm = torch.tensor([0.3, 0.45, 4.5])
    assert torch.allclose(g[0:3], torch.tensor([0.15, 0.225, math.asinh(4.5 / 8.0)]), atol=1e-5)
    assert abs(g[3] - math.asinh(dm.norm().item() / 8.0)) < 1e-5
    assert abs(g[4] - 4.0 / 16.0 / 3.0) < 1e-5
    assert abs(g[5] - 3.0 / 3.05) < 1e-5 and abs(g[6]) < 1e-6 and abs(g[12]) < 1e-6
    obs[0, n0 + 14] = 1.0                                      # a wall row: direction dots masked
    g2 = _geo_of(obs)[0, 0]
    assert g2[5] == 0 and g2[6] == 0 and torch.allclose(g2[0:3], g[0:3])


def _hand_obs(w, b, tipv=(0.0, 0.0, 0.0)):
    obs = torch.zeros(1, nr.OBS_DIM)
    obs[0, 75:78] = torch.tensor([w[0], w[1] / 0.75, w[2]])
    obs[0, 81:84] = torch.tensor(b)
    obs[0, 624:627] = torch.tensor(tipv) / 6.0
    return obs


def _put_note(obs, slot, p, cut=(1.0, 0.0), wall=False):
    n0 = nr.OFF_NOTES + slot * 18
    obs[0, n0:n0 + 4] = torch.tensor([p[0], p[1] / 0.75, math.asinh(p[2] / 8.0), -2.0])
    obs[0, n0 + 6], obs[0, n0 + 7] = cut
    obs[0, n0 + 14] = 1.0 if wall else 0.0


def _blade(g, hand):
    lanes = g[14 + 4 * hand:18 + 4 * hand].double()
    return [2.0 * math.sinh(lanes[i].item()) for i in range(3)] + [lanes[3].item()]


def test_note_geo_known_answers_blade_frame():
    w = (0.2, -0.3, -0.5)
    b = torch.tensor([0.6, 0.0, 0.8])
    obs = _hand_obs(w, b.tolist())
    for slot, s in enumerate((0.16, 0.66, 1.16, 2.0)):
        _put_note(obs, slot, (torch.tensor(w) + s * b).tolist())
    _put_note(obs, 4, (torch.tensor(w) + 0.7 * b + 0.2 * torch.tensor([0.0, 1.0, 0.0])).tolist())
    g = _geo_of(obs)[0]
    for slot, s in enumerate((0.16, 0.66, 1.16, 2.0)):
        along, perp, _, _ = _blade(g[slot], 0)
        assert abs(perp) < 1e-5 and abs(along - (s - 0.16)) < 1e-5
    along, perp, _, _ = _blade(g[4], 0)
    assert abs(perp - 0.2) < 1e-5 and abs(along - (0.7 - 0.16)) < 1e-5
    # cut-plane sign and the tip-velocity dot (soft normaliser 5 / 5.05)
    obs = _hand_obs((0.0, 0.0, 0.0), (0.0, 1.0, 0.0), tipv=(5.0, 0.0, 0.0))
    _put_note(obs, 0, (0.3, 0.5, -0.2), cut=(1.0, 0.0))
    _put_note(obs, 1, (0.3, 0.5, 0.2), cut=(0.0, -1.0))
    _put_note(obs, 2, (0.3, 0.5, 0.0), cut=(1.0, 0.0), wall=True)
    g = _geo_of(obs)[0]
    assert abs(_blade(g[0], 0)[2] - 0.2 * 5.0 / 5.05) < 1e-5
    assert abs(_blade(g[1], 0)[2] + 0.2 * 5.0 / 5.05) < 1e-5
    assert abs(_blade(g[2], 0)[2]) < 1e-6
    assert abs(_blade(g[0], 0)[3] - 5.0 / 6.0) < 1e-6 and abs(_blade(g[1], 0)[3]) < 1e-6 and _blade(g[2], 0)[3] == 0.0
    assert _blade(g[0], 1)[2] == 0.0 and _blade(g[0], 1)[3] == 0.0


def test_masked_entity_slots_cannot_change_outputs():
    """Junk in masked slots leaves logits / value unchanged (python/tests/test_policy.py:42-63)."""
    arch, sd, obs, _, _ = nr.load_fixture(GOLD[0])
    lg, v = nr.forward(sd, arch, obs)
    obs2 = obs.clone()
    mask = obs[:, nr.OFF_MASK:nr.OFF_MASK + 24] > 0.5
    notes = obs2[:, nr.OFF_NOTES:nr.OFF_MASK].view(-1, 24, 18)
    notes[~mask] = torch.randn_like(notes[~mask]) * 3
    lg2, v2 = nr.forward(sd, arch, obs2)
    assert torch.allclose(lg, lg2, atol=1e-5) and torch.allclose(v, v2, atol=1e-5)


def test_emulated_fp16_stream_is_in_the_reference_tolerance_class():
    """The reference holds its fp16 stream to 2e-2 of max|logit| against the fp32 record
    path (python/tests/test_trunk_simba.py:142-162)."""
    arch, sd, obs, logits, value = nr.load_fixture(GOLD[0])
    lg, v = nr.forward(sd, arch, obs, emulate="f16")
    live = logits > -1e8
    assert (lg[live] - logits[live]).abs().max().item() < 2e-2 * logits[live].abs().max().item()


def test_value_residual_and_simbav2_properties_of_the_oracle():
    """What the reference's own tests hold for the two options (python/tests/test_arch_ab_options.py:
    131-139, 250-256): the mix at (a, b) = (1, 0) is bitwise the plain policy; a SimBaV2 feature row
    is sqrt(D) times a unit vector."""
    path = [p for p in GOLD if p.endswith("notepolicy_vres_v2.npz")][0]
    arch, sd, obs, _, _ = nr.load_fixture(path)
    sd1 = {k: (torch.ones(1) if k.endswith("vres_a") else torch.zeros(1) if k.endswith("vres_b") else v)
           for k, v in sd.items()}
    plain = {k: v for k, v in sd1.items() if "vres" not in k}
    lg1, v1 = nr.forward(sd1, arch, obs)
    lg0, v0 = nr.forward(plain, {**arch, "value_residual": False}, obs)
    assert torch.equal(lg1, lg0) and torch.equal(v1, v0)
    lg, _ = nr.forward(sd, arch, obs)
    assert not torch.equal(lg, lg0)                         # the fixture's (a, b) do move the output
    _, _, parts = nr.forward(sd, arch, obs, return_parts=True)
    rms = parts["h"].square().mean(-1)
    assert torch.allclose(rms, torch.ones_like(rms), atol=1e-5)
