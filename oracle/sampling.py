"""CPU restatement of the action epilogue (TEST INFRASTRUCTURE: only tests, the smoke check
and the bench's CPU leg may import this package).

`sample_heads` follows the reference's `get_action_and_value` tail
(python/policy.py:1467-1516): log_softmax, Gumbel-max `argmax(logsm - log E)` with the lanes past a
head's gear count pinned to -inf, gathered-and-summed log-probability, per-head entropy
`-(p * logsm).sum(-1)` and its 29-head sum.

`philox4x32_10` is the published counter-based generator (Salmon, Moraes, Dror, Shaw: "Parallel
random numbers: as easy as 1, 2, 3", SC'11; Random123 `philox4x32` with 10 rounds), pinned in
tests/test_oracle_sampling.py by the Random123 known-answer vectors.  `exp1_draws` is the mapping
the HIP kernel documents: key = seed, counter = (row, 2 * offset + block), draw k of a row = word
k & 3 of block k >> 2, E = -log(((word >> 8) + 1) * 2^-24)."""
import numpy as np

M0, M1 = 0xD2511F53, 0xCD9E8D57
W0, W1 = 0x9E3779B9, 0xBB67AE85
MASK32 = 0xFFFFFFFF


def philox4x32_10(ctr, key):
    """ctr (..., 4) uint32-valued, key (..., 2) uint32-valued -> (..., 4) uint32 (numpy uint64 arithmetic)."""
    c = [np.asarray(ctr[..., i], dtype=np.uint64) for i in range(4)]
    k0 = np.asarray(key[..., 0], dtype=np.uint64)
    k1 = np.asarray(key[..., 1], dtype=np.uint64)
    for _ in range(10):
        p0 = np.uint64(M0) * c[0]
        p1 = np.uint64(M1) * c[2]
        n0 = ((p1 >> np.uint64(32)) ^ c[1] ^ k0) & np.uint64(MASK32)
        n1 = p1 & np.uint64(MASK32)
        n2 = ((p0 >> np.uint64(32)) ^ c[3] ^ k1) & np.uint64(MASK32)
        n3 = p0 & np.uint64(MASK32)
        c = [n0, n1, n2, n3]
        k0 = (k0 + np.uint64(W0)) & np.uint64(MASK32)
        k1 = (k1 + np.uint64(W1)) & np.uint64(MASK32)
    return np.stack(c, -1).astype(np.uint32)


def exp1_draws(n_rows, K, seed, offset):
    """(n_rows, K) float32 Exp(1) draws of the kernel's stream."""
    rows = np.arange(n_rows, dtype=np.uint64)
    key = np.broadcast_to(np.array([seed & MASK32, (seed >> 32) & MASK32], dtype=np.uint64), (n_rows, 2))
    words = []
    for blk in range(2):
        hi = (2 * offset + blk) & 0xFFFFFFFFFFFFFFFF
        ctr = np.stack([rows & np.uint64(MASK32), rows >> np.uint64(32),
                        np.full(n_rows, hi & MASK32, dtype=np.uint64), np.full(n_rows, hi >> 32, dtype=np.uint64)], -1)
        words.append(philox4x32_10(ctr, key))
    w = np.concatenate(words, -1)[:, :K]
    u = ((w >> np.uint32(8)).astype(np.float32) + np.float32(1.0)) * np.float32(2.0 ** -24)
    return (-np.log(u.astype(np.float32))).astype(np.float32)


def log_softmax(x):
    m = x.max(-1, keepdims=True)
    z = x - m
    return z - np.log(np.exp(z).sum(-1, keepdims=True))


def sample_heads(logits, exp_noise=None, head_sizes=None, action=None):
    """logits (B, NH, K) float32.  Returns (action int64 (B, NH), logprob (B,), ent_h (B, NH), entropy (B,)),
    computed in float64 from the float32 inputs (the checker's precision)."""
    x = np.asarray(logits, dtype=np.float64)
    B, NH, K = x.shape
    logsm = log_softmax(x)
    if action is None:
        with np.errstate(divide="ignore"):
            score = logsm - np.log(np.asarray(exp_noise, dtype=np.float64))
        if head_sizes is not None:
            invalid = np.arange(K)[None, :] >= np.asarray(head_sizes)[:, None]
            score = np.where(invalid[None], -np.inf, score)
        action = score.argmax(-1)
    action = np.asarray(action).astype(np.int64)
    logprob = np.take_along_axis(logsm, action[..., None], -1)[..., 0].sum(-1)
    ent_h = -(np.exp(logsm) * logsm).sum(-1)
    return action, logprob, ent_h, ent_h.sum(-1)
