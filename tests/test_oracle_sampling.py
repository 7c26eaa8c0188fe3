"""Pins of the action-epilogue oracle (CPU)."""
import numpy as np
import torch

from oracle import sampling as sp


def test_philox4x32_10_known_answers():
    """Random123's kat_vectors for philox4x32 with 10 rounds: (counter, key) -> output."""
    kats = [
        ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
        ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
        ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
         (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
    ]
    for ctr, key, want in kats:
        got = sp.philox4x32_10(np.array([ctr], dtype=np.uint64), np.array([key], dtype=np.uint64))[0]
        assert tuple(int(v) for v in got) == want


def test_exp1_draws_are_unit_exponential():
    e = sp.exp1_draws(200000, 7, seed=1234, offset=5).astype(np.float64).ravel()
    assert e.min() >= 0.0
    assert abs(e.mean() - 1.0) < 0.01 and abs(e.var() - 1.0) < 0.03
    # Kolmogorov distance to 1 - exp(-x)
    xs = np.sort(e)
    cdf = 1.0 - np.exp(-xs)
    emp = (np.arange(xs.size) + 0.5) / xs.size
    assert np.abs(cdf - emp).max() < 0.004
    # streams at another offset / seed are different draws
    assert not np.array_equal(sp.exp1_draws(16, 7, 1234, 6), sp.exp1_draws(16, 7, 1234, 5))
    assert not np.array_equal(sp.exp1_draws(16, 7, 1235, 5), sp.exp1_draws(16, 7, 1234, 5))


def test_sample_heads_matches_the_torch_formulas():
    """log_softmax / gather / entropy against the library routines the reference calls
    (python/policy.py:1473, :1497-1513), and Gumbel-max == argmax of the same score in torch."""
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(64, 29, 7, generator=g) * 3
    logits[:, 3, 5:] = -1e9                      # a 5-gear head inside a 7-wide layout
    sizes = np.full(29, 7); sizes[3] = 5
    noise = torch.empty(64, 29, 7).exponential_(generator=g)
    act, lp, ent_h, ent = sp.sample_heads(logits.numpy(), noise.numpy(), sizes)
    logsm = torch.log_softmax(logits.double(), -1)
    score = logsm - noise.double().log()
    score[:, 3, 5:] = -float("inf")
    assert np.array_equal(act, score.argmax(-1).numpy())
    assert (act[:, 3] < 5).all()
    want_lp = logsm.gather(-1, torch.from_numpy(act).unsqueeze(-1)).squeeze(-1).sum(-1)
    np.testing.assert_allclose(lp, want_lp.numpy(), rtol=1e-12, atol=1e-12)
    want_ent_h = -(logsm.exp() * logsm).sum(-1)
    np.testing.assert_allclose(ent_h, want_ent_h.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(ent, want_ent_h.sum(-1).numpy(), rtol=1e-12, atol=1e-12)
    # evaluation of given actions reproduces the sampled log-prob
    _, lp2, _, _ = sp.sample_heads(logits.numpy(), action=act)
    np.testing.assert_array_equal(lp, lp2)


def test_gumbel_max_samples_the_softmax_distribution():
    """Frequencies of argmax(logsm - log E) over many draws match softmax(logits) (chi-square)."""
    logits = np.array([[[0.3, -1.2, 2.0, 0.0, -0.5]]], dtype=np.float32)
    n = 200000
    e = sp.exp1_draws(n, 5, seed=7, offset=0)
    act, _, _, _ = sp.sample_heads(np.broadcast_to(logits, (n, 1, 5)), e[:, None, :])
    p = np.exp(sp.log_softmax(logits.astype(np.float64)))[0, 0]
    cnt = np.bincount(act[:, 0], minlength=5)
    chi2 = ((cnt - n * p) ** 2 / (n * p)).sum()
    assert chi2 < 25.0          # 4 degrees of freedom: P(chi2 > 25) ~ 5e-5
