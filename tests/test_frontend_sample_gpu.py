"""GPU parity of the forward's front-end kernel and of the action-epilogue kernel, both through
the C ABI, against the CPU oracle (oracle/note_policy_ref.py::frontend, pinned on the reference's
golden vectors and hand-computed geometry cases; oracle/sampling.py, pinned on Random123's
known-answer vectors and the torch library routines).

Gates: gathered lanes, one-hots and the key bias are data movement -> bit-exact.  The 22 geometry
lanes are fp32 arithmetic (sinh / asinh / sqrt / divide): fp32 outputs within 1e-5 * (|ref| + max|ref|);
16-bit outputs within one unit in the last place of the type (the fp32 value may sit next to a
rounding boundary), and bit-equal on at least 99 % of the lanes.  Epilogue: log-prob / entropy within
1e-5 relative; sampled actions identical wherever the winning score leads by more than 1e-4."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from beatsaberrl_amd import ops  # noqa: E402
from beatsaberrl_amd import obs_layout as L  # noqa: E402
from oracle import note_policy_ref as nr  # noqa: E402
from oracle import sampling as sp  # noqa: E402

DEV = "cuda"
TDT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
ULP = {"f16": 2.0 ** -10, "bf16": 2.0 ** -7}


def _obs(n, seed):
    g = torch.Generator().manual_seed(seed)
    obs = torch.randn(n, nr.OBS_DIM, generator=g) * 0.7
    obs[:, nr.OFF_MASK:nr.OFF_MASK + 24] = (torch.rand(n, 24, generator=g) < 0.6).float()
    notes = obs[:, nr.OFF_NOTES:nr.OFF_MASK].view(n, 24, 18)
    notes[..., 14] = (torch.rand(n, 24, generator=g) < 0.3).float()     # wall flag
    notes[..., 9] = (torch.rand(n, 24, generator=g) < 0.5).float()      # flux bar flag
    return obs


def _tables():
    sab = torch.tensor(L.SABER_L_IDX + L.SABER_R_IDX, dtype=torch.int32, device=DEV)
    body = torch.tensor(L.BODY3_IDX, dtype=torch.int32, device=DEV)
    return sab, body


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("geo,flux", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("B", [1, 7, 8, 1000])
def test_frontend_matches_oracle(dtype, geo, flux, B):
    obs = _obs(B, 100 + B)
    sab, body = _tables()
    got = ops.note_frontend(obs.to(DEV), sab, body, TDT[dtype], note_geo=geo, flux=flux, z_asinh=8.0)
    want = nr.frontend(obs, geo, flux, 8.0, emulate=None if dtype == "f32" else dtype)
    names = ("saber_in", "torso_in", "leg_in", "note_in", "key_bias")
    for name, g_, w_ in zip(names, got, want):
        g_ = g_.float().cpu()
        assert g_.shape == w_.shape, name
        if name != "note_in":
            assert torch.equal(g_, w_), name
            continue
        assert torch.equal(g_[..., :18], w_[..., :18])
        if not geo:
            continue
        gg, wg = g_[..., 18:], w_[..., 18:]
        if dtype == "f32":
            assert bool(((gg - wg).abs() <= 1e-5 * (wg.abs() + wg.abs().max())).all()), (gg - wg).abs().max().item()
        else:
            assert bool(((gg - wg).abs() <= ULP[dtype] * wg.abs() + 1e-7).all()), (gg - wg).abs().max().item()
            assert (gg == wg).float().mean().item() >= 0.99


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("geo", [False, True])
@pytest.mark.parametrize("B", [1, 13, 1000])
def test_frontend_padded_rows_hold_the_same_lanes_and_zeros(dtype, geo, B):
    """The 64-pitch outputs carry the unpadded outputs' bits in their leading lanes and zeros after them (the
    buffers are poisoned first: every pad lane must be written)."""
    obs = _obs(B, 300 + B).to(DEV)
    sab, body = _tables()
    want = ops.note_frontend(obs, sab, body, TDT[dtype], note_geo=geo, flux=geo)
    junk = torch.full((B * 6 * 24 * 64,), float("nan"), device=DEV, dtype=TDT[dtype])
    del junk                                                           # the allocator hands these bytes out next
    got = ops.note_frontend(obs, sab, body, TDT[dtype], note_geo=geo, flux=geo, padded=True)
    for name, g_, w_ in zip(("saber_in", "torso_in", "leg_in", "note_in"), got, want):
        assert g_.shape == (*w_.shape[:-1], ops.FRONT_PITCH), name
        k = w_.shape[-1]
        assert torch.equal(g_[..., :k], w_), name
        assert bool((g_[..., k:] == 0).all()), name
    assert torch.equal(got[4], want[4])


def test_frontend_prerounded_and_strided_obs():
    """fp32 obs and obs already in the stream dtype give the same bits (python/policy.py:1200-1209);
    a row stride larger than 630 is honoured."""
    obs = _obs(33, 5)
    sab, body = _tables()
    a = ops.note_frontend(obs.to(DEV), sab, body, torch.float16, note_geo=True)
    b = ops.note_frontend(obs.half().to(DEV), sab, body, torch.float16, note_geo=True)
    wide = torch.zeros(33, 700, device=DEV)
    wide[:, :630] = obs.to(DEV)
    c = ops.note_frontend(wide[:, :630], sab, body, torch.float16, note_geo=True)
    for x, y, z in zip(a, b, c):
        assert torch.equal(x, y) and torch.equal(x, z)
    with pytest.raises(TypeError):
        ops.note_frontend(obs.half().to(DEV), sab, body, torch.bfloat16)
    with pytest.raises(RuntimeError):
        ops.note_frontend(obs[:, :600].to(DEV), sab, body, torch.float16)


def _logits(B, seed, k=7):
    g = torch.Generator().manual_seed(seed)
    lg = torch.randn(B, 29, k, generator=g) * 2.5
    sizes = np.full(29, k, dtype=np.int32)
    if k == 7:
        sizes[[0, 1, 2, 3]] = 5
        lg[:, :4, 5:] = -1e9
    return lg, sizes


@pytest.mark.parametrize("B,k", [(1, 7), (9, 7), (512, 5), (4099, 3)])
def test_sampling_with_caller_noise_matches_oracle(B, k):
    lg, sizes = _logits(B, 3 + B, k)
    g = torch.Generator().manual_seed(B)
    noise = torch.empty(B, 29, k).exponential_(generator=g)
    hs = torch.from_numpy(sizes).to(DEV)
    act, lp, ent, ent_h, _ = ops.sample_heads(lg.to(DEV), head_sizes=hs, exp_noise=noise.to(DEV), want_ent_h=True)
    act = act.cpu().numpy()
    o_act, _, o_ent_h, o_ent = sp.sample_heads(lg.numpy(), noise.numpy(), sizes)
    assert (act < sizes[None, :]).all() and (act >= 0).all()
    diff = act != o_act
    if diff.any():      # only near-ties may differ: the oracle's top-2 score gap there is tiny
        logsm = sp.log_softmax(lg.numpy().astype(np.float64))
        score = logsm - np.log(noise.numpy().astype(np.float64))
        score = np.where(np.arange(k)[None, None, :] >= sizes[None, :, None], -np.inf, score)
        top2 = np.sort(score, -1)[..., -2:]
        assert ((top2[..., 1] - top2[..., 0])[diff] < 1e-4).all()
    assert diff.mean() < 1e-3
    _, o_lp, _, _ = sp.sample_heads(lg.numpy(), action=act)
    np.testing.assert_allclose(lp.cpu().numpy(), o_lp, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(ent_h.cpu().numpy(), o_ent_h, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(ent.cpu().numpy(), o_ent, rtol=1e-5, atol=1e-5)
    # evaluation mode: int64 and uint8 actions, with and without entropy
    a64 = torch.from_numpy(act).to(DEV)
    for a_in in (a64, a64.to(torch.uint8)):
        a2, lp2, ent2, _, _ = ops.sample_heads(lg.to(DEV), action=a_in, need_entropy=False)
        assert torch.equal(a2, a64) and torch.equal(lp2, lp) and ent2 is None


def test_sampling_kernel_stream_matches_the_documented_philox_mapping():
    B, k = 777, 7
    lg, sizes = _logits(B, 11, k)
    hs = torch.from_numpy(sizes).to(DEV)
    act, lp, _, _, noise = ops.sample_heads(lg.to(DEV), head_sizes=hs, seed=0x1234567890ABCDEF, offset=3,
                                            want_noise=True)
    want = sp.exp1_draws(B * 29, k, 0x1234567890ABCDEF, 3).reshape(B, 29, k)
    got = noise.cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)       # the two logf's may differ in the last place
    # the kernel's actions are the Gumbel-max of its own draws
    o_act, _, _, _ = sp.sample_heads(lg.numpy(), got, sizes)
    assert (act.cpu().numpy() != o_act).mean() < 1e-3
    # same (seed, offset) -> same bits; another offset or seed -> another draw
    act2, lp2, _, _, _ = ops.sample_heads(lg.to(DEV), head_sizes=hs, seed=0x1234567890ABCDEF, offset=3)
    assert torch.equal(act, act2) and torch.equal(lp, lp2)
    act3, _, _, _, _ = ops.sample_heads(lg.to(DEV), head_sizes=hs, seed=0x1234567890ABCDEF, offset=4)
    act4, _, _, _, _ = ops.sample_heads(lg.to(DEV), head_sizes=hs, seed=0x1234567890ABCDEE, offset=3)
    assert not torch.equal(act, act3) and not torch.equal(act, act4)
    # a device-side counter adds to the offset and is advanced by one per sampling launch
    ctr = torch.tensor([2], dtype=torch.int64, device=DEV)
    act5, lp5, _, _, _ = ops.sample_heads(lg.to(DEV), head_sizes=hs, seed=0x1234567890ABCDEF, offset=1, counter=ctr)
    assert torch.equal(act5, act) and torch.equal(lp5, lp) and ctr.item() == 3
    act6, _, _, _, _ = ops.sample_heads(lg.to(DEV), head_sizes=hs, seed=0x1234567890ABCDEF, offset=1, counter=ctr)
    assert torch.equal(act6, act3) and ctr.item() == 4
    ops.sample_heads(lg.to(DEV), head_sizes=hs, action=act, counter=ctr)      # evaluation draws nothing
    assert ctr.item() == 4


def test_sampling_kernel_stream_follows_the_softmax_distribution():
    """Full-size batch, one shared logit row: per-head action frequencies match softmax (chi-square)."""
    B = 16384
    row = torch.tensor([0.3, -1.2, 2.0, 0.0, -0.5, 1.0, -3.0])
    lg = row.expand(B, 29, 7).contiguous()
    act, lp, ent, _, _ = ops.sample_heads(lg.to(DEV), seed=99, offset=0)
    p = torch.softmax(row.double(), -1).numpy()
    cnt = np.bincount(act.cpu().numpy().ravel(), minlength=7)
    n = B * 29
    chi2 = ((cnt - n * p) ** 2 / (n * p)).sum()
    assert chi2 < 35.0            # 6 degrees of freedom: P(chi2 > 35) ~ 4e-6
    want_ent = 29 * float(-(p * np.log(p)).sum())
    assert abs(ent[0].item() - want_ent) < 1e-4 * want_ent
