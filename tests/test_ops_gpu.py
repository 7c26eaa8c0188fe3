"""GPU parity of the per-op kernels (called through the C ABI via
beatsaberrl_amd.ops) against closed forms / library routines evaluated in
fp64 or fp32 on the same rounded operands - the reference's own test idiom
(python/tests/test_fused_ln.py:29-88, test_attn29.py:49-154,
test_fp16_accum.py:84-89)."""
import math

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

from beatsaberrl_amd import ops  # noqa: E402

DEV = "cuda"
DTS = [torch.float32, torch.float16, torch.bfloat16]
EPS16 = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}


def _rand(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


# ---------------------------------------------------------------- LayerNorm
@pytest.mark.parametrize("dtype", DTS)
@pytest.mark.parametrize("rows,d", [(1, 128), (7, 128), (1000, 128), (257, 192), (64, 256), (33, 384), (5, 512),
                                    (3, 1024), (130, 64), (9, 40)])
def test_ln_fwd(dtype, rows, d):
    x = _rand(rows, d, dtype=dtype, seed=rows + d, scale=2.0) + 0.5
    w = _rand(d, seed=1) * 0.3 + 1.0
    b = _rand(d, seed=2) * 0.3
    y, mean, rstd = ops.ln_fwd(x, w, b, 1e-5, want_stats=True)
    xd = x.double()
    mu = xd.mean(-1)
    var = ((xd - mu[:, None]) ** 2).mean(-1)
    ref = (xd - mu[:, None]) / torch.sqrt(var[:, None] + 1e-5) * w.double() + b.double()
    assert torch.allclose(mean.double(), mu, atol=1e-5, rtol=1e-5)
    assert torch.allclose(rstd.double(), 1 / torch.sqrt(var + 1e-5), atol=1e-5, rtol=1e-5)
    if dtype is torch.float32:
        lib_ref = F.layer_norm(x, (d,), w, b, 1e-5)
        assert torch.allclose(y, lib_ref, atol=1e-5, rtol=1e-5)
        assert torch.allclose(y.double(), ref, atol=1e-5, rtol=1e-5)
    else:
        err = (y.double() - ref).abs().max().item()
        assert err <= EPS16[dtype] * (ref.abs().max().item() + 1.0), err
        # exactly the fp32 formula rounded once
        assert (y.double() - ref.to(dtype).double()).abs().max().item() <= 2 * EPS16[dtype] * ref.abs().max().item()


@pytest.mark.parametrize("dtype", DTS)
@pytest.mark.parametrize("rows,d", [(513, 128), (100, 192), (31, 384)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_ln_fwd_add(dtype, rows, d, with_bias):
    a = _rand(rows, d, dtype=dtype, seed=3)
    b = _rand(rows, d, dtype=dtype, seed=4)
    bb = _rand(d, seed=5) if with_bias else None
    w = _rand(d, seed=1) * 0.3 + 1.0
    bias = _rand(d, seed=2) * 0.3
    x, y = ops.ln_fwd_add(a, b, w, bias, 1e-5, b_bias=bb)
    # x bitwise: a + b in fp32, or round(a + (b + bias)) from fp32 arithmetic
    bf = b.float() if bb is None else b.float() + bb
    x_ref = (a.float() + bf).to(dtype)
    assert torch.equal(x, x_ref)
    y_ref = F.layer_norm(x.float(), (d,), w, bias, 1e-5)
    tol = 1e-5 if dtype is torch.float32 else 2 * EPS16[dtype] * (y_ref.abs().max().item() + 1)
    assert (y.float() - y_ref).abs().max().item() <= tol
    # the plain kernel on the rounded x gives the same bits
    assert torch.equal(ops.ln_fwd(x, w, bias, 1e-5), y)


# ---------------------------------------------------------------- Linear
def _lin_ref(x, w, bias, act, res):
    y = x.double() @ w.double().t()
    if bias is not None:
        y = y + bias.double()
    if act == "relu":
        y = torch.relu(y)
    elif act == "gelu":
        y = 0.5 * y * (1 + torch.erf(y / math.sqrt(2.0)))
    if res is not None:
        y = y + res.double()
    return y


@pytest.mark.parametrize("dtype", DTS)
@pytest.mark.parametrize("rows,K,M", [(1, 128, 128), (127, 128, 384), (129, 128, 512), (1000, 512, 128),
                                      (300, 192, 576), (64, 768, 192), (50, 49, 192), (77, 40, 192),
                                      (33, 128, 204), (65, 384, 145), (19, 640, 101), (256, 100, 128),
                                      (200, 16, 128), (130, 1536, 384)])
def test_linear_shapes(dtype, rows, K, M):
    x = _rand(rows, K, dtype=dtype, seed=rows)
    w = _rand(M, K, dtype=dtype, seed=K, scale=1 / math.sqrt(K))
    b = _rand(M, seed=M)
    y = ops.linear(x, w, b)
    ref = _lin_ref(x, w, b, None, None)
    scale = ref.abs().max().item()
    tol = 1e-5 * scale if dtype is torch.float32 else 1.2 * EPS16[dtype] * scale
    assert y.shape == (rows, M) and y.dtype is dtype
    assert (y.double() - ref).abs().max().item() <= tol


@pytest.mark.parametrize("dtype", DTS)
@pytest.mark.parametrize("act", [None, "relu", "gelu"])
@pytest.mark.parametrize("use_res", [False, True])
def test_linear_epilogues(dtype, act, use_res):
    rows, K, M = 333, 128, 256
    x = _rand(rows, K, dtype=dtype, seed=1)
    w = _rand(M, K, dtype=dtype, seed=2, scale=0.1)
    b = _rand(M, seed=3)
    res = _rand(rows, M, dtype=dtype, seed=4) if use_res else None
    ref = _lin_ref(x, w, b, act, res)
    scale = ref.abs().max().item()
    for out_dtype in (dtype, torch.float32):
        y = ops.linear(x, w, b, act=act, residual=res, out_dtype=out_dtype)
        tol = 2e-5 * scale if out_dtype is torch.float32 and dtype is torch.float32 else (
            1e-4 * scale if out_dtype is torch.float32 else 1.2 * EPS16[dtype] * scale)
        assert y.dtype is out_dtype
        assert (y.double() - ref).abs().max().item() <= tol, (dtype, act, use_res, out_dtype)


@pytest.mark.parametrize("dtype", DTS)
def test_linear_strided_views_split_and_packing(dtype):
    """x as a row-strided view (token 0 of every env), split output, and the
    packed q|k|v GEMM == three separate Linears (column-block identity)."""
    B, T, d = 37, 16, 128
    tok = _rand(B, T, d, dtype=dtype, seed=7)
    w = _rand(204, d, dtype=dtype, seed=8, scale=0.1)
    b = _rand(204, seed=9)
    lg, val = ops.linear(tok[:, 0], w, b, out_dtype=torch.float32, split=203)
    ref = _lin_ref(tok[:, 0], w, b, None, None)
    assert lg.shape == (B, 203) and val.shape == (B, 1)
    assert (torch.cat([lg, val], 1).double() - ref).abs().max().item() <= 1e-4 * ref.abs().max().item()
    ws = [_rand(d, d, dtype=dtype, seed=20 + i, scale=0.1) for i in range(3)]
    bs = [_rand(d, seed=30 + i) for i in range(3)]
    packed = ops.linear(tok, torch.cat(ws).contiguous(), torch.cat(bs).contiguous())
    assert packed.shape == (B, T, 3 * d)
    for i in range(3):
        assert torch.equal(packed[..., i * d:(i + 1) * d], ops.linear(tok, ws[i], bs[i]))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,K,M", [(4096, 128, 128), (5000, 128, 384), (4097, 384, 1152), (8192, 1536, 384),
                                      (6000, 192, 576), (4100, 40, 192), (9000, 256, 1024), (4099, 128, 136),
                                      (4200, 96, 1024), (4500, 512, 1280), (4300, 64, 192), (5000, 64, 256)])
@pytest.mark.parametrize("act,use_res", [(None, False), ("gelu", False), ("relu", True), (None, True)])
def test_linear_large_row_counts_take_the_tiled_kernel(dtype, rows, K, M, act, use_res):
    """rows >= 4096 with aligned shapes run the LDS kernels (K a multiple of 32: the ring-buffered kernel, 256- or
    128-column tiles by M and K; otherwise the register-staged tiled kernel): same closed form, and the same BITS as
    the direct-from-global kernel on a slice (all accumulate k in the same order)."""
    x = _rand(rows, K, dtype=dtype, seed=rows)
    w = _rand(M, K, dtype=dtype, seed=K + M, scale=1 / math.sqrt(K))
    b = _rand(M, seed=M)
    res = _rand(rows, M, dtype=dtype, seed=7) if use_res else None
    y = ops.linear(x, w, b, act=act, residual=res)
    ref = _lin_ref(x, w, b, act, res)
    assert (y.double() - ref).abs().max().item() <= 1.2 * EPS16[dtype] * ref.abs().max().item()
    for lo, hi in ((0, 300), (rows - 257, rows)):
        small = ops.linear(x[lo:hi], w, b, act=act, residual=None if res is None else res[lo:hi])
        assert torch.equal(small, y[lo:hi])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,K,M", [(50, 49, 192), (4096, 29, 192), (32768, 34, 192), (9001, 40, 192), (100000, 40, 192)])
def test_linear_zero_padded_k_gives_the_unpadded_bits(dtype, rows, K, M):
    """Input rows and weight columns zero-padded to K = 64 (the padded encoder inputs): the vector kernels then
    produce the BITS of the odd-K call - the pad lanes add exact zeros to the fp32 accumulators."""
    x = _rand(rows, K, dtype=dtype, seed=rows + K)
    w = _rand(M, K, dtype=dtype, seed=K + M, scale=1 / math.sqrt(K))
    b = _rand(M, seed=M)
    xp = torch.zeros(rows, 64, device=x.device, dtype=dtype)
    xp[:, :K] = x
    wp = torch.zeros(M, 64, device=x.device, dtype=dtype)
    wp[:, :K] = w
    for act in (None, "relu"):
        assert torch.equal(ops.linear(xp, wp, b, act=act), ops.linear(x, w, b, act=act))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,G,K,M,T,t0", [(7, 2, 49, 192, 29, 0), (333, 1, 29, 192, 29, 2), (700, 24, 40, 192, 29, 5),
                                          (64, 31, 16, 256, 32, 1), (3, 5, 128, 136, 8, 3)])
@pytest.mark.parametrize("act", [None, "relu"])
def test_linear_grouped_output_rows_write_a_token_slice(dtype, N, G, K, M, T, t0, act):
    """out = stream[:, t0:t0+G, :] receives the N * G rows in place (direct, vectorised and LDS-tiled kernels):
    the slice holds the same BITS as the plain call, the rest of the stream is untouched."""
    x = _rand(N * G, K, dtype=dtype, seed=N + G)
    w = _rand(M, K, dtype=dtype, seed=K + M, scale=1 / math.sqrt(K))
    b = _rand(M, seed=M)
    plain = ops.linear(x, w, b, act=act)
    stream = torch.full((N, T, M), 7.0, device=DEV, dtype=dtype)
    got = ops.linear(x, w, b, act=act, out=stream[:, t0:t0 + G])
    assert got.data_ptr() == stream[:, t0:t0 + G].data_ptr()
    assert torch.equal(stream[:, t0:t0 + G].reshape(N * G, M), plain)
    rest = torch.ones(T, dtype=torch.bool)
    rest[t0:t0 + G] = False
    assert bool((stream[:, rest] == 7.0).all())
    with pytest.raises(RuntimeError):
        ops.linear(x, w, b, out=stream[:, t0:t0 + G, :M - 1])
    with pytest.raises(RuntimeError):
        ops.linear(x, w, b, out=stream[:, t0:t0 + G], split=8)


def test_linear_rows_are_batch_invariant():
    """A row's bits do not depend on the batch it sits in or on its tile phase
    (the reference holds its kernels to this: tests/test_fused_ffn.py:332-353)."""
    x = _rand(600, 128, dtype=torch.float16, seed=1)
    w = _rand(384, 128, dtype=torch.float16, seed=2, scale=0.1)
    b = _rand(384, seed=3)
    full = ops.linear(x, w, b, act="gelu")
    for lo, hi in ((0, 1), (5, 132), (127, 256), (300, 600)):
        assert torch.equal(ops.linear(x[lo:hi], w, b, act="gelu"), full[lo:hi])


# ---------------------------------------------------------------- Fused FFN
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,d,Fh", [(1, 128, 512), (127, 128, 512), (129, 192, 768), (1000, 192, 768),
                                       (300, 256, 1024), (77, 384, 1536), (513, 128, 64)])
@pytest.mark.parametrize("act,with_ln", [("relu", True), ("gelu", False), ("gelu", True)])
@pytest.mark.parametrize("packed", ["auto", False])
def test_ffn_fused(dtype, rows, d, Fh, act, with_ln, packed):
    """Closed form with the reference's rounding points (python/tests/test_fused_ffn.py:252-266):
    hidden rounded once, fp32 accumulate, out = round(x + (O + b2)), LN on the rounded out.  Both kernels: the one on
    a packed weight image (d = 128 / 192 / 256 / 384 with enough FFN stages; `packed="auto"`) and the one on the plain weights."""
    assert ops.ffn_fused_supported(d, Fh, dtype)
    assert ops.ffn_pack_supported(d, Fh, dtype) == (Fh >= 192)
    x = _rand(rows, d, dtype=dtype, seed=1)
    h2 = _rand(rows, d, dtype=dtype, seed=2)
    w0 = _rand(Fh, d, dtype=dtype, seed=3, scale=1 / math.sqrt(d))
    w2 = _rand(d, Fh, dtype=dtype, seed=4, scale=1 / math.sqrt(Fh))
    b0, b2 = _rand(Fh, seed=5) * 0.3, _rand(d, seed=6) * 0.3
    lw, lb = (_rand(d, seed=7) * 0.2 + 1.0, _rand(d, seed=8) * 0.2) if with_ln else (None, None)
    xo, ho = ops.ffn_fused(x, h2, w0, b0, w2, b2, act=act, ln_w=lw, ln_b=lb, packed=packed)
    pre = h2.double() @ w0.double().t() + b0.double()
    hid = (torch.relu(pre) if act == "relu" else 0.5 * pre * (1 + torch.erf(pre / math.sqrt(2.0)))).to(dtype).double()
    ref = x.double() + hid @ w2.double().t() + b2.double()
    scale = ref.abs().max().item()
    # the hidden's rounding can flip one 16-bit ulp near ties: allow a little over one output ulp
    assert (xo.double() - ref).abs().max().item() <= 1.5 * EPS16[dtype] * scale
    # unfused path through the same library: error class no worse (reference idiom, test_fused_ffn.py:295-306)
    un = ops.linear(ops.linear(h2, w0, b0, act=act), w2, b2, residual=x)
    e_new = (xo.double() - ref).norm() / ref.norm()
    e_old = (un.double() - ref).norm() / ref.norm()
    assert e_new <= max(1.1 * e_old, 2e-3)
    if with_ln:
        ln_ref = F.layer_norm(xo.float(), (d,), lw, lb, 1e-5)
        assert (ho.float() - ln_ref).abs().max().item() <= 2 * EPS16[dtype] * (ln_ref.abs().max().item() + 1)
    else:
        assert ho is None


@pytest.mark.parametrize("packed", ["auto", False])
def test_ffn_fused_rows_are_batch_invariant(packed):
    d, Fh = 192, 768
    x = _rand(400, d, dtype=torch.float16, seed=1)
    h2 = _rand(400, d, dtype=torch.float16, seed=2)
    w0 = _rand(Fh, d, dtype=torch.float16, seed=3, scale=0.07)
    w2 = _rand(d, Fh, dtype=torch.float16, seed=4, scale=0.04)
    b0, b2, lw, lb = _rand(Fh, seed=5), _rand(d, seed=6), _rand(d, seed=7) + 1, _rand(d, seed=8)
    xo, ho = ops.ffn_fused(x, h2, w0, b0, w2, b2, act="relu", ln_w=lw, ln_b=lb, packed=packed)
    for lo, hi in ((0, 1), (3, 130), (127, 256), (271, 400)):
        a, b = ops.ffn_fused(x[lo:hi].contiguous(), h2[lo:hi].contiguous(), w0, b0, w2, b2, act="relu", ln_w=lw, ln_b=lb,
                             packed=packed)
        assert torch.equal(a, xo[lo:hi]) and torch.equal(b, ho[lo:hi])


def test_ffn_fused_packed_image_follows_the_weights_and_large_row_counts():
    """The image cache is keyed by the weight tensors' identity and in-place version: an in-place edit of a weight
    must show in the next call.  Plus a persistent-grid case (more 256-row tiles than CUs, ragged tail)."""
    d, Fh, rows = 128, 512, 70001
    x = _rand(rows, d, dtype=torch.float16, seed=1)
    h2 = _rand(rows, d, dtype=torch.float16, seed=2)
    w0 = _rand(Fh, d, dtype=torch.float16, seed=3, scale=0.09)
    w2 = _rand(d, Fh, dtype=torch.float16, seed=4, scale=0.04)
    b0, b2 = _rand(Fh, seed=5) * 0.3, _rand(d, seed=6) * 0.3
    a1, _ = ops.ffn_fused(x, h2, w0, b0, w2, b2, act="relu")
    ref, _ = ops.ffn_fused(x, h2, w0, b0, w2, b2, act="relu", packed=False)
    scale = ref.float().abs().max().item()
    assert (a1.float() - ref.float()).abs().max().item() <= 2 * EPS16[torch.float16] * scale
    small, _ = ops.ffn_fused(x[69000:].contiguous(), h2[69000:].contiguous(), w0, b0, w2, b2, act="relu")
    assert torch.equal(small, a1[69000:])
    w2.mul_(0.5)
    b0.add_(0.25)
    a2, _ = ops.ffn_fused(x, h2, w0, b0, w2, b2, act="relu")
    ref2, _ = ops.ffn_fused(x, h2, w0, b0, w2, b2, act="relu", packed=False)
    assert not torch.equal(a1, a2)
    assert (a2.float() - ref2.float()).abs().max().item() <= 2 * EPS16[torch.float16] * scale


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,Fh", [(1, 1536), (77, 1536), (1000, 1536), (300, 192), (33000, 768)])
@pytest.mark.parametrize("act,with_ln", [("relu", True), ("gelu", False), ("gelu", True)])
def test_block_tail_in_one_kernel(dtype, rows, Fh, act, with_ln):
    """Output projection + residual, LN2, FFN (+ next LN) as one kernel at d = 384: closed form with the rounding points
    of the separate launches (x1, h2, hidden, xo, ho rounded once each; the reference's Block.forward,
    python/policy.py:650-715, and its fused FFN test's idiom, python/tests/test_fused_ffn.py:252-306), and the error
    class of the separate launches of this library on the same operands."""
    d = 384
    assert ops.proj_ffn_supported(d, Fh, dtype) and not ops.proj_ffn_supported(256, 1024, dtype)
    x = _rand(rows, d, dtype=dtype, seed=1)
    att = _rand(rows, d, dtype=dtype, seed=2)
    wo = _rand(d, d, dtype=dtype, seed=9, scale=1 / math.sqrt(d))
    w0 = _rand(Fh, d, dtype=dtype, seed=3, scale=1 / math.sqrt(d))
    w2 = _rand(d, Fh, dtype=dtype, seed=4, scale=1 / math.sqrt(Fh))
    bo, b0, b2 = _rand(d, seed=10) * 0.3, _rand(Fh, seed=5) * 0.3, _rand(d, seed=6) * 0.3
    l2w, l2b = _rand(d, seed=11) * 0.2 + 1.0, _rand(d, seed=12) * 0.2
    lw, lb = (_rand(d, seed=7) * 0.2 + 1.0, _rand(d, seed=8) * 0.2) if with_ln else (None, None)
    img = ops.proj_ffn_pack(wo, bo, w0, b0, w2, b2)
    xo, ho = ops.proj_ffn_fused(att, x, img, Fh, l2w, l2b, 1e-5, act=act, ln_w=lw, ln_b=lb)
    # the separate launches
    x1_u = ops.linear(att, wo, bo, residual=x)
    h2_u = ops.ln_fwd(x1_u, l2w, l2b, 1e-5)
    xo_u, ho_u = ops.ffn_fused(x1_u, h2_u, w0, b0, w2, b2, act=act, ln_w=lw, ln_b=lb)
    # closed form in double with the same rounding points
    x1 = (x.double() + att.double() @ wo.double().t() + bo.double()).to(dtype)
    h2 = F.layer_norm(x1.double(), (d,), l2w.double(), l2b.double(), 1e-5).to(dtype)
    pre = h2.double() @ w0.double().t() + b0.double()
    hid = (torch.relu(pre) if act == "relu" else 0.5 * pre * (1 + torch.erf(pre / math.sqrt(2.0)))).to(dtype).double()
    ref = x1.double() + hid @ w2.double().t() + b2.double()
    scale = ref.abs().max().item()
    e_new = (xo.double() - ref).norm() / ref.norm()
    e_old = (xo_u.double() - ref).norm() / ref.norm()
    # a one-ulp flip of x1 or h2 near a tie moves a whole row a little: the bound is on the error CLASS, and loosely on the maximum
    assert e_new <= max(1.15 * e_old, 1e-3), (e_new.item(), e_old.item())
    assert (xo.double() - ref).abs().max().item() <= 4 * EPS16[dtype] * scale
    assert (xo.float() - xo_u.float()).abs().max().item() <= 4 * EPS16[dtype] * scale
    if with_ln:
        ln_ref = F.layer_norm(xo.float(), (d,), lw, lb, 1e-5)
        assert (ho.float() - ln_ref).abs().max().item() <= 2 * EPS16[dtype] * (ln_ref.abs().max().item() + 1)
    else:
        assert ho is None
    # a row's bits do not depend on the batch it sits in
    if rows >= 300:
        lo, hi = 130, 290
        a, b = ops.proj_ffn_fused(att[lo:hi].contiguous(), x[lo:hi].contiguous(), img, Fh, l2w, l2b, 1e-5, act=act, ln_w=lw, ln_b=lb)
        assert torch.equal(a, xo[lo:hi]) and (b is None or torch.equal(b, ho[lo:hi]))
    # ... with a projection of the LayerNorm-ed output behind it (the next block's packed q|k|v, or its k|v alone): xo and
    # ho keep their bits, qo is the Linear of the SAME ho to one rounding (another accumulation order: <= 1 ulp, mostly equal)
    if with_ln:
        for n_next, want_ho in ((1152, False), (768, True)):
            assert ops.proj_ffn_supported(d, Fh, dtype, n_next) and not ops.proj_ffn_supported(d, Fh, dtype, 96)
            wn = _rand(n_next, d, dtype=dtype, seed=13, scale=1 / math.sqrt(d))
            bn = _rand(n_next, seed=14) * 0.3
            img_n = ops.proj_ffn_pack(wo, bo, w0, b0, w2, b2, wn, bn)
            xo_n, ho_n, qo = ops.proj_ffn_fused(att, x, img_n, Fh, l2w, l2b, 1e-5, act=act, ln_w=lw, ln_b=lb, n_next=n_next,
                                                want_ho=want_ho)
            assert torch.equal(xo_n, xo) and qo.shape == (rows, n_next)
            assert (ho_n is None) == (not want_ho) and (ho_n is None or torch.equal(ho_n, ho))
            q_ref = ho.double() @ wn.double().t() + bn.double()
            q_lin = ops.linear(ho, wn, bn)
            qs = q_ref.abs().max().item()
            assert (qo.double() - q_ref).abs().max().item() <= 1.01 * EPS16[dtype] * qs
            assert (qo.float() - q_lin.float()).abs().max().item() <= 2 * EPS16[dtype] * qs
            assert (qo == q_lin).float().mean().item() > 0.98


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,n_next,want_ho", [(1, 1152, False), (77, 1152, True), (1000, 768, True), (33000, 1152, False)])
def test_layernorm_and_packed_projection_in_one_kernel(dtype, rows, n_next, want_ho):
    """LN1 + the packed q|k|v Linears of a block (python/policy.py:541-560) as one launch at d = 384: the LayerNorm output
    has ln_fwd's rounding (one flip per thousands of values at most: the statistics are summed in another order), the
    projection is the Linear of that output to one rounding."""
    d = 384
    assert ops.ln_proj_supported(d, n_next, dtype) and not ops.ln_proj_supported(256, 768, dtype) and not ops.ln_proj_supported(d, 96, dtype)
    x = _rand(rows, d, dtype=dtype, seed=1)
    wn = _rand(n_next, d, dtype=dtype, seed=2, scale=1 / math.sqrt(d))
    bn = _rand(n_next, seed=3) * 0.3
    lw, lb = _rand(d, seed=4) * 0.2 + 1.0, _rand(d, seed=5) * 0.2
    img = ops.ln_proj_pack(wn, bn)
    ho, qo = ops.ln_proj_fused(x, img, n_next, lw, lb, 1e-5, want_ho=want_ho)
    h_ref = ops.ln_fwd(x, lw, lb, 1e-5)
    assert (ho is None) == (not want_ho)
    if want_ho:
        assert (ho.float() - h_ref.float()).abs().max().item() <= 1.01 * EPS16[dtype] * h_ref.float().abs().max().item()
        assert (ho == h_ref).float().mean().item() > 0.995
        q_ref = ho.double() @ wn.double().t() + bn.double()
        assert (qo.double() - q_ref).abs().max().item() <= 1.01 * EPS16[dtype] * q_ref.abs().max().item()
    q_lin = ops.linear(h_ref, wn, bn)
    qs = q_lin.float().abs().max().item()
    assert (qo.float() - q_lin.float()).abs().max().item() <= 4 * EPS16[dtype] * qs
    if rows >= 1000:
        lo, hi = 130, 290
        _, b = ops.ln_proj_fused(x[lo:hi].contiguous(), img, n_next, lw, lb, 1e-5)
        assert torch.equal(b, qo[lo:hi])


def test_block_tail_kernel_rejects_what_it_cannot_take():
    d, Fh, rows = 384, 1536, 64
    dt = torch.float16
    x = _rand(rows + 1, d, dtype=dt, seed=1)
    att = _rand(rows + 1, d, dtype=dt, seed=2)
    wo = _rand(d, d, dtype=dt, seed=3, scale=0.05)
    w0 = _rand(Fh, d, dtype=dt, seed=4, scale=0.05)
    w2 = _rand(d, Fh, dtype=dt, seed=5, scale=0.03)
    bo, b0, b2 = _rand(d, seed=6), _rand(Fh, seed=7), _rand(d, seed=8)
    lw, lb = _rand(d, seed=9) + 1, _rand(d, seed=10)
    img = ops.proj_ffn_pack(wo, bo, w0, b0, w2, b2)
    with pytest.raises(RuntimeError):                      # an image packed for another shape
        ops.proj_ffn_fused(att[:rows], x[:rows], img, Fh, lw, lb, n_next=1152, ln_w=lw, ln_b=lb)
    with pytest.raises(RuntimeError):                      # a projection behind needs the LayerNorm it projects
        ops.proj_ffn_fused(att[:rows], x[:rows], img, Fh, lw, lb, n_next=1152)
    with pytest.raises(RuntimeError):                      # att and x of different shapes
        ops.proj_ffn_fused(att[:rows - 1], x[:rows], img, Fh, lw, lb)
    # a hidden width whose vectors do not fit LDS beside the ring is "unsupported", not a launch failure
    assert ops.proj_ffn_supported(d, 4096, dt, 1152) and not ops.proj_ffn_supported(d, 8192, dt, 1152)
    with pytest.raises(ops.Unsupported):                   # d = 256 has no such kernel
        ops.proj_ffn_pack(_rand(256, 256, dtype=dt, seed=1), _rand(256, seed=2), _rand(1024, 256, dtype=dt, seed=3),
                          _rand(1024, seed=4), _rand(256, 1024, dtype=dt, seed=5), _rand(256, seed=6))
    # zero rows: nothing launched, empty outputs
    xo, ho = ops.proj_ffn_fused(att[:0], x[:0], img, Fh, lw, lb, ln_w=lw, ln_b=lb)
    assert xo.shape == (0, d) and ho.shape == (0, d)
    # misaligned rows (a view 8 bytes into the allocation) are an error of the entry point, not a fault
    flat = torch.zeros(rows * d + 8, dtype=dt, device=DEV)
    xm = flat[4:4 + rows * d].view(rows, d)
    with pytest.raises(RuntimeError):
        ops.proj_ffn_fused(att[:rows], xm, img, Fh, lw, lb)


def test_ffn_fused_unsupported_shapes_say_so():
    assert not ops.ffn_fused_supported(160, 640, torch.float16)
    assert not ops.ffn_fused_supported(128, 500, torch.float16)
    assert not ops.ffn_fused_supported(128, 512, torch.float32)


# ---------------------------------------------------------------- Attention
def _attn_ref(q, k, v, H, bias):
    B, TQ, d = q.shape
    T = k.shape[1]
    dh = d // H
    qh = q.double().view(B, TQ, H, dh).transpose(1, 2)
    kh = k.double().view(B, T, H, dh).transpose(1, 2)
    vh = v.double().view(B, T, H, dh).transpose(1, 2)
    s = qh @ kh.transpose(-2, -1) / math.sqrt(dh)
    if bias is not None:
        s = s + bias.double().view(B, 1, 1, T)
    return (torch.softmax(s, -1) @ vh).transpose(1, 2).reshape(B, TQ, d)


@pytest.mark.parametrize("dtype", DTS)
@pytest.mark.parametrize("T,TQ,H,dh", [(16, 16, 4, 32), (29, 29, 4, 48), (29, 5, 4, 48), (29, 1, 4, 48),
                                       (32, 32, 8, 32), (48, 48, 12, 32), (48, 1, 12, 32), (6, 6, 2, 32),
                                       (17, 3, 4, 32)])
@pytest.mark.parametrize("mask", ["none", "n_valid", "bias"])
def test_attention(dtype, T, TQ, H, dh, mask):
    B, d = 11, H * dh
    qkv = _rand(B, T, 3 * d, dtype=dtype, seed=T + TQ)
    q, k, v = qkv[:, :TQ, :d], qkv[..., d:2 * d], qkv[..., 2 * d:]
    g = torch.Generator().manual_seed(5)
    nv = torch.randint(0, T, (B,), generator=g, dtype=torch.int32)
    nv[0] = 0
    nv[1] = T - 1
    valid = (torch.arange(T)[None, :] <= nv[:, None]).float()
    bias = ((valid - 1.0) * 16384.0).to(dtype).to(DEV)
    nvd = nv.to(DEV)
    if mask == "none":
        out = ops.attn_fwd(q, k, v, H)
        ref = _attn_ref(q, k, v, H, None)
    elif mask == "n_valid":
        out = ops.attn_fwd(q, k, v, H, n_valid=nvd)
        ref = _attn_ref(q, k, v, H, bias)
    else:
        out = ops.attn_fwd(q, k, v, H, key_bias=bias)
        ref = _attn_ref(q, k, v, H, bias)
    assert out.shape == (B, TQ, d) and out.is_contiguous()
    tol = 2e-5 if dtype is torch.float32 else 3 * EPS16[dtype] * (ref.abs().max().item() + 1)
    assert (out.double() - ref).abs().max().item() <= tol


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_attention_invariants(dtype):
    B, T, H, dh = 9, 29, 4, 48
    d = H * dh
    q = _rand(B, T, d, dtype=dtype, seed=1)
    k = _rand(B, T, d, dtype=dtype, seed=2)
    v = _rand(B, T, d, dtype=dtype, seed=3)
    nv = torch.tensor([0, 4, 28, 10, 5, 17, 1, 2, 3], dtype=torch.int32, device=DEV)
    out = ops.attn_fwd(q, k, v, H, n_valid=nv)
    # masked keys get exactly zero weight: junk in masked V/K rows changes nothing
    k2, v2 = k.clone(), v.clone()
    for b in range(B):
        v2[b, int(nv[b]) + 1:] = 1000.0
        k2[b, int(nv[b]) + 1:] = 50.0
    assert torch.equal(ops.attn_fwd(q, k2, v2, H, n_valid=nv), out)
    # batch-slice invariance
    assert torch.equal(ops.attn_fwd(q[2:5], k[2:5], v[2:5], H, n_valid=nv[2:5].contiguous()), out[2:5])
    # TQ < T == row slice of the full result (masking is key-side only)
    for tq in (5, 1):
        assert torch.equal(ops.attn_fwd(q[:, :tq], k, v, H, n_valid=nv), out[:, :tq])


# ---------------------------------------------------------------- Tokenizer
@pytest.mark.parametrize("dtype", DTS)
@pytest.mark.parametrize("T,d", [(16, 128), (32, 256), (48, 384), (6, 32)])
def test_cfg_embed(dtype, T, d):
    from oracle import config_model as cm
    spec = cm.ConfigSpec(1, d, d // 32 if d >= 32 else 1, 4 * d, T)
    p = cm.init_params(spec, 3)
    B = 13
    obs, _ = cm.make_inputs(spec, B, 4)
    em = {torch.float32: None, torch.float16: "f16", torch.bfloat16: "bf16"}[dtype]
    ref = cm.tokens_from_obs(p, spec, obs, emulate=em)
    tok = ops.cfg_embed(obs.to(DEV), p["prop_embed.weight"].to(dtype).to(DEV), p["prop_embed.bias"].to(DEV),
                        p["obj_embed.weight"].to(dtype).to(DEV), p["obj_embed.bias"].to(DEV), T, dtype)
    assert tok.shape == (B, T, d)
    tol = 1e-5 if dtype is torch.float32 else 1.2 * EPS16[dtype] * (ref.abs().max().item() + 1)
    assert (tok.float().cpu() - ref).abs().max().item() <= tol


# ---------------------------------------------------------------- value-residual mix
@pytest.mark.parametrize("dtype", DTS)
@pytest.mark.parametrize("B,T,d,packed", [(3, 29, 192, True), (17, 29, 128, True), (5, 7, 20, False), (1, 1, 3, False)])
def test_vres_mix(dtype, B, T, d, packed):
    """torch.addcmul(v * a, v0, b).to(dtype) (python/fp16_linear.py:1002-1006); exact at (a, b) = (1, 0)."""
    if packed:      # v and v0 as column slices of packed q|k|v buffers, mixed in place
        qkv = _rand(B, T, 3 * d, dtype=dtype, seed=11)
        qkv0 = _rand(B, T, 3 * d, dtype=dtype, seed=12)
        v, v0 = qkv[..., 2 * d:], qkv0[..., 2 * d:]
    else:
        v, v0 = _rand(B, T, d, dtype=dtype, seed=11), _rand(B, T, d, dtype=dtype, seed=12)
    a = torch.tensor([0.83], device=DEV)
    b = torch.tensor([-0.41], device=DEV)
    ref = (v.double() * a.double() + v0.double() * b.double())
    keep = v.clone()
    one, zero = torch.ones(1, device=DEV), torch.zeros(1, device=DEV)
    same = ops.vres_mix(v, v0, one, zero, out=torch.empty_like(keep))
    assert torch.equal(same, keep)
    out = ops.vres_mix(v, v0, a, b)                      # in place
    assert out.data_ptr() == v.data_ptr()
    if packed:                                           # the q | k columns of the buffer are untouched
        assert torch.equal(qkv[..., :2 * d], _rand(B, T, 3 * d, dtype=dtype, seed=11)[..., :2 * d])
    if dtype is torch.float32:
        assert torch.allclose(out.double(), ref, rtol=1e-6, atol=1e-6)
    else:
        assert (out.double() - ref).abs().max().item() <= EPS16[dtype] * (ref.abs().max().item() + 1e-3)
        assert (out.double() - ref.to(dtype).double()).abs().max().item() <= 2 * EPS16[dtype] * ref.abs().max().item()


# ---------------------------------------------------------------- SimBaV2 row stages
@pytest.mark.parametrize("dtype", DTS)
@pytest.mark.parametrize("rows,D", [(1, 96), (7, 384), (1001, 256), (5, 50)])
def test_hsphere_stages(dtype, rows, D):
    """The three fp32 row stages against F.normalize (library routine) in fp64
    (python/policy.py:1140-1155); the output rows have RMS 1 (python/tests/test_arch_ab_options.py:250-254)."""
    t = _rand(rows, D, dtype=dtype, seed=21, scale=30.0)
    s = _rand(D, seed=22) * 0.05 + 0.14
    x32, x = ops.hsphere(ops.HS_SCALE_L2N, t, s, 1.5)
    ref_x = F.normalize(t.double() * (s.double() * 1.5), dim=-1, eps=1e-6)
    assert x32.dtype is torch.float32 and x.dtype is dtype
    assert torch.allclose(x32.double(), ref_x, rtol=1e-5, atol=1e-6)
    assert torch.equal(x, x32.to(dtype))
    u = ops.hsphere(ops.HS_SCALE_RELU, t, s, 0.5)
    ref_u = F.relu(t.double() * (s.double() * 0.5))
    tol = 1e-6 if dtype is torch.float32 else EPS16[dtype]
    assert (u.double() - ref_u).abs().max().item() <= tol * (ref_u.abs().max().item() + 1)
    alpha = _rand(D, seed=23) * 0.3 + 0.5
    y_in = _rand(rows, D, dtype=dtype, seed=24, scale=3.0)
    h = ops.hsphere(ops.HS_L2N_LERP, y_in, alpha, 0.9, x32=x32)
    y = F.normalize(y_in.double(), dim=-1, eps=1e-6)
    z = F.normalize(x32.double() + alpha.double() * 0.9 * (y - x32.double()), dim=-1, eps=1e-6)
    ref_h = z * math.sqrt(D)
    assert (h.double() - ref_h).abs().max().item() <= (1e-5 if dtype is torch.float32 else 2 * EPS16[dtype]) * ref_h.abs().max().item()
    rms = h.double().square().mean(-1)
    assert torch.allclose(rms, torch.ones_like(rms), atol=1e-5 if dtype is torch.float32 else 4 * EPS16[dtype])
    # a zero row normalises to zero (eps clamp), not NaN
    z0 = torch.zeros(2, D, dtype=dtype, device=DEV)
    x32z, _ = ops.hsphere(ops.HS_SCALE_L2N, z0, s, 1.0)
    assert torch.equal(x32z, torch.zeros_like(x32z))


# ---------------------------------------------------------------- LayerNorm backward
@pytest.mark.parametrize("dtype", DTS)
@pytest.mark.parametrize("rows,d", [(1, 128), (7, 64), (1000, 128), (257, 192), (4099, 192), (64, 256), (33, 384),
                                    (5, 512), (3, 1024), (9, 40), (70000, 128)])
@pytest.mark.parametrize("with_gx", [False, True])
def test_ln_bwd(dtype, rows, d, with_gx):
    """Against torch autograd through F.layer_norm in fp64 on the same operands (the reference's idiom,
    python/tests/test_fused_ln.py:91-135): dx to the type's rounding, dw / db / dbb to fp32 summation error."""
    x = _rand(rows, d, dtype=dtype, seed=rows + d, scale=2.0) + 0.5
    dy = _rand(rows, d, dtype=dtype, seed=rows + d + 1)
    gx = _rand(rows, d, dtype=dtype, seed=rows + d + 2) if with_gx else None
    w = _rand(d, seed=1) * 0.3 + 1.0
    b = _rand(d, seed=2) * 0.3
    _, mean, rstd = ops.ln_fwd(x, w, b, 1e-5, want_stats=True)
    dx, dw, db, dbb = ops.ln_bwd(x, dy, w, mean, rstd, gx=gx, want_dbb=True)
    assert dx.dtype is dtype and dw.dtype is torch.float32 and dw.shape == (d,)
    xd = x.double().requires_grad_(True)
    wd = w.double().requires_grad_(True)
    bd = b.double().requires_grad_(True)
    F.layer_norm(xd, (d,), wd, bd, 1e-5).backward(dy.double())
    ref_dx = xd.grad + (gx.double() if with_gx else 0.0)
    tol = 2e-5 if dtype is torch.float32 else 1.5 * EPS16[dtype]
    assert (dx.double() - ref_dx).abs().max().item() <= tol * (ref_dx.abs().max().item() + 1.0)
    # column sums: fp32 accumulation over `rows` terms of O(1) magnitude
    tol_c = 3e-6 * max(rows, 64) ** 0.5 * 4
    scale_w = (dy.double().abs() * ((x.double() - mean.double()[:, None]) * rstd.double()[:, None]).abs()).sum(0).max().item()
    assert (dw.double() - wd.grad).abs().max().item() <= tol_c * max(scale_w, 1.0) / max(rows, 64) ** 0.5
    assert (db.double() - bd.grad).abs().max().item() <= tol_c * max(dy.double().abs().sum(0).max().item(), 1.0) / max(rows, 64) ** 0.5
    assert (dbb.double() - dx.double().sum(0)).abs().max().item() <= tol_c * max(dx.double().abs().sum(0).max().item(), 1.0) / max(rows, 64) ** 0.5
    # reproducible: no atomics anywhere in the column sums
    dx2, dw2, db2 = ops.ln_bwd(x, dy, w, mean, rstd, gx=gx)
    assert torch.equal(dx, dx2) and torch.equal(dw, dw2) and torch.equal(db, db2)


def test_ln_bwd_no_rows_and_unsupported_width():
    w = torch.ones(128, device=DEV)
    e = torch.empty(0, 128, device=DEV)
    s = torch.empty(0, device=DEV)
    dx, dw, db = ops.ln_bwd(e, e, w, s, s)
    assert dx.shape == (0, 128) and torch.equal(dw, torch.zeros_like(dw)) and torch.equal(db, torch.zeros_like(db))
    x = torch.zeros(2, 4096, device=DEV, dtype=torch.float16)
    with pytest.raises(ops.Unsupported):
        ops.ln_bwd(x, x, torch.ones(4096, device=DEV), torch.zeros(2, device=DEV), torch.ones(2, device=DEV))


# ---------------------------------------------------------------- Linear weight / bias gradient
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,M,K", [(1, 8, 8), (31, 128, 128), (32, 192, 192), (1000, 576, 192), (5000, 768, 192),
                                      (4097, 192, 768), (70001, 192, 192), (300, 145, 384), (77, 101, 40), (9, 7, 5),
                                      (20000, 384, 256)])
def test_wgrad(dtype, rows, M, K):
    """dy^T x and column sums of dy against fp64 on the same rounded operands (fp32-accumulate class:
    python/tests/test_fp16_accum.py:84-89 uses 2e-3 relative; this is fp32 accumulation of exact products)."""
    dy = _rand(rows, M, dtype=dtype, seed=rows + M)
    x = _rand(rows, K, dtype=dtype, seed=rows + K + 1)
    dw, db = ops.wgrad(dy, x)
    ref_w = dy.double().t() @ x.double()
    ref_b = dy.double().sum(0)
    tol = 2e-6 * max(rows, 16) ** 0.5 + 1e-6
    assert (dw.double() - ref_w).abs().max().item() <= tol * max((dy.double().abs().t() @ x.double().abs()).max().item(), 1.0)
    assert (db.double() - ref_b).abs().max().item() <= tol * max(dy.double().abs().sum(0).max().item(), 1.0)
    dw2, none = ops.wgrad(dy, x, want_db=False)
    assert none is None and torch.equal(dw, dw2)                  # reproducible, and db is optional


def test_wgrad_strided_operands_and_empty_batch():
    """Operands as column slices of packed buffers (the q|k|v gradient, the k|v input), and rows = 0."""
    g = _rand(513, 3 * 192, dtype=torch.float16, seed=5)
    h = _rand(513, 2 * 128, dtype=torch.float16, seed=6)
    dw, db = ops.wgrad(g[:, 192:384], h[:, 128:])
    assert torch.allclose(dw.double(), g[:, 192:384].double().t() @ h[:, 128:].double(), rtol=1e-5, atol=1e-4)
    assert torch.allclose(db.double(), g[:, 192:384].double().sum(0), rtol=1e-5, atol=1e-4)
    e = torch.empty(0, 64, device=DEV, dtype=torch.float16)
    dw, db = ops.wgrad(e, e)
    assert torch.equal(dw, torch.zeros(64, 64, device=DEV)) and torch.equal(db, torch.zeros(64, device=DEV))


# ---------------------------------------------------------------- data gradient through a ReLU
@pytest.mark.parametrize("dtype", DTS)
@pytest.mark.parametrize("rows,K,M", [(1, 8, 8), (77, 192, 768), (5000, 192, 768), (4096, 128, 512), (4300, 768, 192), (333, 40, 101), (129, 256, 96)])
def test_linear_gated(dtype, rows, K, M):
    """(g @ W) * [hidden > 0] == autograd through relu(h @ W1^T) @ W2^T at the hidden (python/fp16_linear.py:719-727)."""
    g = _rand(rows, K, dtype=dtype, seed=rows + K)
    wt = _rand(M, K, dtype=dtype, seed=rows + M + 1, scale=K ** -0.5)          # forward weight (K, M) transposed
    hid = torch.relu(_rand(rows, M, dtype=dtype, seed=rows + 2))
    hid[0, 0] = 0.0                                                             # an exact zero is gated off (relu'(0) = 0)
    out = ops.linear_gated(g, wt, hid)
    ref = (g.double() @ wt.double().t()) * (hid > 0).double()
    assert torch.equal(out == 0, ref == 0) or ((out != 0) != (ref != 0)).sum().item() <= 2       # exact cancellations aside
    tol = 1e-5 if dtype is torch.float32 else 1.5 * EPS16[dtype]
    assert (out.double() - ref).abs().max().item() <= tol * (ref.abs().max().item() + 1.0)
    assert torch.equal(out[hid <= 0], torch.zeros_like(out[hid <= 0]))


# ---------------------------------------------------------------- Attention backward
@pytest.mark.parametrize("dtype", DTS)
@pytest.mark.parametrize("T,TQ,H,dh", [(16, 16, 4, 32), (29, 29, 4, 48), (29, 5, 4, 48), (29, 1, 4, 48),
                                       (32, 32, 8, 32), (48, 48, 12, 32), (48, 1, 12, 32), (6, 6, 2, 32), (17, 3, 4, 32)])
@pytest.mark.parametrize("mask", ["none", "n_valid", "bias"])
def test_attention_backward(dtype, T, TQ, H, dh, mask):
    """dq, dk, dv against torch autograd through the fp64 closed form on the same rounded operands
    (python/tests/test_attn29.py:157-214 compares the same three gradients against the SDPA path)."""
    B, d = 7, H * dh
    qkv = _rand(B, T, 3 * d, dtype=dtype, seed=T + TQ)
    q, k, v = qkv[:, :TQ, :d], qkv[..., d:2 * d], qkv[..., 2 * d:]
    dout = _rand(B, TQ, d, dtype=dtype, seed=T + TQ + 9)
    g = torch.Generator().manual_seed(5)
    nv = torch.randint(0, T, (B,), generator=g, dtype=torch.int32)
    nv[0] = 0
    nv[1] = T - 1
    valid = (torch.arange(T)[None, :] <= nv[:, None]).float()
    bias = ((valid - 1.0) * 16384.0).to(dtype).to(DEV)
    kw = {} if mask == "none" else {"n_valid": nv.to(DEV)} if mask == "n_valid" else {"key_bias": bias}
    # gradients land in the column slices of one packed buffer, as the reference's callers have them
    packed = torch.full((B, T, 3 * d), 7.0, device=DEV, dtype=dtype)
    dq, dk, dv = ops.attn_bwd(q, k, v, dout, H, out=(packed[:, :TQ, :d], packed[..., d:2 * d], packed[..., 2 * d:]), **kw)
    qd, kd, vd = (t.double().detach().clone().requires_grad_(True) for t in (q, k, v))
    _attn_ref(qd, kd, vd, H, None if mask == "none" else bias).backward(dout.double())
    for name, got, want in (("dq", dq, qd.grad), ("dk", dk, kd.grad), ("dv", dv, vd.grad)):
        tol = 3e-5 if dtype is torch.float32 else 4 * EPS16[dtype]
        err = (got.double() - want).abs().max().item()
        assert err <= tol * (want.abs().max().item() + 1.0), (name, err)
    if TQ < T:
        assert torch.equal(packed[:, TQ:, :d], torch.full_like(packed[:, TQ:, :d], 7.0))      # nothing written past the queries
    if mask != "none":                                        # masked keys: exactly zero gradient
        dead = ~(valid.bool().to(DEV))
        assert torch.equal(dk[dead], torch.zeros_like(dk[dead])) and torch.equal(dv[dead], torch.zeros_like(dv[dead]))
    dq2, dk2, dv2 = ops.attn_bwd(q, k, v, dout, H, **kw)      # fresh contiguous outputs, same bits
    assert torch.equal(dq2, dq) and torch.equal(dk2, dk) and torch.equal(dv2, dv)


@pytest.mark.parametrize("TQ", [29, 5, 1])
def test_attention_forward_persistent_workgroups_walk_many_envs(TQ):
    """More envs than resident workgroups of the one-workgroup-per-env forward: an env's output must not depend on
    which other envs share the launch."""
    B, T, H, dh = 3300, 29, 4, 48
    d = H * dh
    qkv = _rand(B, T, 3 * d, dtype=torch.float16, seed=13)
    bias = (((torch.rand(B, T, generator=torch.Generator().manual_seed(16)) < 0.7).float() - 1.0) * 16384.0).half().to(DEV)
    bias[:, :5] = 0
    q, k, v = qkv[:, :TQ, :d], qkv[..., d:2 * d], qkv[..., 2 * d:]
    out = ops.attn_fwd(q, k, v, H, key_bias=bias)
    for lo, hi in ((0, 3), (766, 771), (1534, 1540), (3293, 3300)):
        assert torch.equal(ops.attn_fwd(q[lo:hi], k[lo:hi], v[lo:hi], H, key_bias=bias[lo:hi]), out[lo:hi])


@pytest.mark.parametrize("TQ", [29, 5])
def test_attention_backward_persistent_workgroups_walk_many_envs(TQ):
    """More envs than resident workgroups: every workgroup of the one-workgroup-per-env form processes several envs
    with the next one's rows prefetched.  An env's gradients depend on nothing but that env: the big batch must give the
    bits of the same envs run in small batches."""
    B, T, H, dh = 1500, 29, 4, 48
    d = H * dh
    qkv = _rand(B, T, 3 * d, dtype=torch.float16, seed=3)
    dout = _rand(B, TQ, d, dtype=torch.float16, seed=4)
    bias = (((torch.rand(B, T, generator=torch.Generator().manual_seed(6)) < 0.7).float() - 1.0) * 16384.0).half().to(DEV)
    bias[:, :5] = 0
    q, k, v = qkv[:, :TQ, :d], qkv[..., d:2 * d], qkv[..., 2 * d:]
    dq, dk, dv = ops.attn_bwd(q, k, v, dout, H, key_bias=bias)
    for lo, hi in ((0, 3), (510, 515), (1022, 1030), (1493, 1500)):
        sq, sk, sv = ops.attn_bwd(q[lo:hi], k[lo:hi], v[lo:hi], dout[lo:hi], H, key_bias=bias[lo:hi])
        assert torch.equal(sq, dq[lo:hi]) and torch.equal(sk, dk[lo:hi]) and torch.equal(sv, dv[lo:hi])


# ---------------------------------------------------------------- weight-resident streaming linear
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,K,M", [(8192, 128, 128), (8200, 128, 384), (9001, 192, 192), (8193, 192, 576), (8192, 192, 776),
                                      (8300, 256, 1024), (8192, 384, 384), (8201, 384, 256), (8207, 512, 136), (8192, 768, 192),
                                      (8192, 1024, 256), (8199, 1536, 384)])
@pytest.mark.parametrize("act,use_res,use_bias", [(None, False, True), ("gelu", False, True), ("relu", True, False), (None, True, True)])
def test_linear_many_rows_take_the_streaming_kernel(dtype, rows, K, M, act, use_res, use_bias):
    """rows >= 8192 with K = 128 / 192 / 256 (384 for narrow outputs) run the weight-resident streaming kernel
    (column blocks that overhang M, ragged last row tile; the larger K of the list stay on the tiled kernel): the same closed form, and the
    same BITS as the direct-from-global kernel on row slices (all accumulate k in the same order)."""
    x = _rand(rows, K, dtype=dtype, seed=rows)
    w = _rand(M, K, dtype=dtype, seed=K + M, scale=1 / math.sqrt(K))
    b = _rand(M, seed=M) if use_bias else None
    res = _rand(rows, M, dtype=dtype, seed=7) if use_res else None
    y = ops.linear(x, w, b, act=act, residual=res)
    ref = _lin_ref(x, w, b if use_bias else torch.zeros(M, device=DEV), act, res)
    assert (y.double() - ref).abs().max().item() <= 1.2 * EPS16[dtype] * ref.abs().max().item()
    for lo, hi in ((0, 300), (rows // 2 - 5, rows // 2 + 200), (rows - 257, rows)):
        small = ops.linear(x[lo:hi], w, b, act=act, residual=None if res is None else res[lo:hi])
        assert torch.equal(small, y[lo:hi])


def test_streaming_linear_gate_and_token_slice_output():
    """The ReLU gate and the grouped (token-slice) output through the streaming kernel."""
    rows, K, M = 8192, 192, 768
    g = _rand(rows, K, dtype=torch.float16, seed=1)
    wt = _rand(M, K, dtype=torch.float16, seed=2, scale=K ** -0.5)
    hid = torch.relu(_rand(rows, M, dtype=torch.float16, seed=3))
    out = ops.linear_gated(g, wt, hid)
    assert torch.equal(out[:500], ops.linear_gated(g[:500], wt, hid[:500]))
    assert torch.equal(out[hid <= 0], torch.zeros_like(out[hid <= 0]))
    N, G, T = 512, 24, 29
    x = _rand(N * G, 128, dtype=torch.float16, seed=4)
    w = _rand(192, 128, dtype=torch.float16, seed=5, scale=0.09)
    b = _rand(192, seed=6)
    stream = torch.full((N, T, 192), 7.0, device=DEV, dtype=torch.float16)
    ops.linear(x, w, b, act="relu", out=stream[:, 5:])
    assert torch.equal(stream[:, 5:].reshape(N * G, 192), ops.linear(x, w, b, act="relu"))
    assert torch.equal(stream[:, :5], torch.full_like(stream[:, :5], 7.0))


# ---------------------------------------------------------------- critic attention pool
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,T,d,H", [(1, 29, 192, 4), (37, 29, 192, 4), (9, 29, 128, 4), (5, 32, 128, 2), (4, 16, 256, 8), (3, 17, 192, 3), (6, 7, 256, 16),
                                     (4101, 29, 192, 4)])
@pytest.mark.parametrize("masked", [False, True])
def test_critic_pool(dtype, B, T, d, H, masked):
    """The pooled form against the reference's op order in fp64 (python/policy.py:1346-1403): LN, k = Wk hv + bk,
    v = Wv hv + bv, one query per env, softmax(q.k / sqrt(dh) + bias) v - rebuilt from the pool as Wv pooled + bv."""
    dh = d // H
    x = _rand(B, T, d, dtype=dtype, seed=B + T, scale=1.5)
    lw, lb = _rand(d, seed=1) * 0.3 + 1.0, _rand(d, seed=2) * 0.3
    wk, wv = _rand(d, d, seed=3, scale=d ** -0.5), _rand(d, d, seed=4, scale=d ** -0.5)
    bk, bv = _rand(d, seed=5), _rand(d, seed=6)
    q = _rand(B, d, seed=7)
    bias = None
    if masked:
        valid = torch.rand(B, T, generator=torch.Generator().manual_seed(3)) < 0.6
        valid[:, :5] = True
        bias = ((valid.float() - 1.0) * 16384.0).to(dtype).to(DEV)
    qk = torch.stack([q[:, h * dh:(h + 1) * dh] @ wk[h * dh:(h + 1) * dh] for h in range(H)], 1).to(dtype).contiguous()
    pooled = ops.critic_pool(x, lw, lb, 1e-5, qk, bias, H)
    assert pooled.shape == (B, H, d) and pooled.dtype is dtype
    # reference order on the same rounded operands
    hv = F.layer_norm(x.double(), (d,), lw.double(), lb.double(), 1e-5).to(dtype).double()
    k = hv @ wk.double().t() + bk.double()
    v = hv @ wv.double().t() + bv.double()
    out_ref = torch.empty(B, d, dtype=torch.float64, device=DEV)
    out = torch.empty(B, d, dtype=torch.float64, device=DEV)
    for h in range(H):
        sl = slice(h * dh, (h + 1) * dh)
        s = (k[..., sl] @ q.double()[:, sl, None]).squeeze(-1) / math.sqrt(dh)
        if bias is not None:
            s = s + bias.double()
        p = torch.softmax(s, -1)
        out_ref[:, sl] = (p[:, None, :] @ v[..., sl]).squeeze(1)
        out[:, sl] = pooled[:, h].double() @ wv.double()[sl].t() + bv.double()[sl]
        # the pool itself: rows of probabilities that sum to 1 applied to hv
        s2 = (hv @ qk[:, h].double()[:, :, None]).squeeze(-1) / math.sqrt(dh) + (bias.double() if bias is not None else 0.0)
        ref_pool = (torch.softmax(s2, -1)[:, None, :] @ hv).squeeze(1)
        tol_p = 2e-5 if dtype is torch.float32 else 1.5 * EPS16[dtype]
        assert (pooled[:, h].double() - ref_pool).abs().max().item() <= tol_p * (ref_pool.abs().max().item() + 1.0)
    tol = 1e-4 if dtype is torch.float32 else 6 * EPS16[dtype]
    assert (out - out_ref).abs().max().item() <= tol * (out_ref.abs().max().item() + 1.0)
    if masked:      # junk in masked tokens cannot move the pool
        x2 = x.clone()
        x2[~valid.to(DEV)] = 9.0
        assert torch.equal(ops.critic_pool(x2, lw, lb, 1e-5, qk, bias, H), pooled)


def test_critic_pool_unsupported_shapes_say_so():
    """fp32 streams, T > 32 and widths other than 128 / 192 / 256 are reported, not computed some other way."""
    for dtype, T, d, H in ((torch.float32, 29, 192, 4), (torch.float16, 33, 192, 4), (torch.float16, 29, 96, 3)):
        assert not ops.critic_pool_supported(T, d, H, dtype)
        x = _rand(2, T, d, dtype=dtype, seed=1)
        qk = _rand(2, H, d, dtype=dtype, seed=2)
        with pytest.raises(ops.Unsupported):
            ops.critic_pool(x, _rand(d, seed=3), _rand(d, seed=4), 1e-5, qk, None, H)


@pytest.mark.parametrize("rows,n", [(1, 101), (7, 101), (4099, 101), (33, 64), (5, 1), (3, 257)])
def test_softmax_expect_matches_float64(rows, n):
    """bsrl_softmax_expect = softmax(logits) @ centers (reference python/policy.py:1394-1403): against the same
    expression in float64, 2e-6 of the centers' span (fp32 sums of <= 257 terms); rows of huge and of equal logits."""
    g = torch.Generator().manual_seed(rows * 1000 + n)
    logits = torch.randn(rows, n, generator=g) * 6.0
    logits[0] = 0.0                                     # uniform row: the plain mean of the centers
    if rows > 2:
        logits[1] += 3.0e4                              # max-subtraction keeps this finite
        logits[2, n // 2] = 80.0                        # one bin takes everything
    centers = torch.linspace(-12.5, 37.0, n) if n > 1 else torch.tensor([3.25])
    want = (torch.softmax(logits.double(), -1) @ centers.double())
    got = ops.softmax_expect(logits.to(DEV), centers.to(DEV)).cpu()
    span = float(centers.max() - centers.min()) + float(centers.abs().max())
    assert got.shape == (rows,) and got.dtype is torch.float32
    assert (got.double() - want).abs().max().item() <= 2e-6 * span
    assert abs(got[0].item() - centers.double().mean().item()) <= 2e-6 * span
    with pytest.raises(TypeError):
        ops.softmax_expect(logits.to(DEV).half(), centers.to(DEV))
    with pytest.raises(TypeError):
        ops.softmax_expect(logits.to(DEV), centers[:-1].to(DEV) if n > 1 else torch.zeros(2, device=DEV))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d", [128, 192])
@pytest.mark.parametrize("rows,group", [(1, 0), (77, 0), (4099, 0), (24 * 700, 24), (2 * 9001, 2), (65536, 0)])
def test_mlp2_is_the_two_linears_bit_for_bit(dtype, d, rows, group):
    """bsrl_mlp2 (Linear ReLU Linear on a 64-lane input in one launch, hidden rows never written) against
    linear(act="relu") followed by linear: the same bits, plain and into a token slice of a (B, T, d) stream; and
    against the float64 closed form with the hidden rounded once (python/tests/test_fused_ffn.py:252-266 style)."""
    x = _rand(rows, 64, dtype=dtype, seed=1)
    x[:, 40:] = 0                                                 # the frontend pads the encoder inputs with zeros
    w1 = _rand(d, 64, dtype=dtype, seed=2, scale=1 / math.sqrt(40))
    w2 = _rand(d, d, dtype=dtype, seed=3, scale=1 / math.sqrt(d))
    b1, b2 = _rand(d, seed=4) * 0.3, _rand(d, seed=5) * 0.3
    assert ops.mlp2_supported(64, d, dtype) and not ops.mlp2_supported(40, d, dtype) and not ops.mlp2_supported(64, 256, dtype)
    if group:
        B, T = rows // group, group + 5
        s1 = torch.full((B, T, d), 7.0, device=DEV, dtype=dtype)
        s0 = s1.clone()
        y1 = ops.mlp2(x, w1, b1, w2, b2, out=s1[:, 5:])
        ops.linear(ops.linear(x, w1, b1, act="relu"), w2, b2, out=s0[:, 5:])
        assert y1 is not None and torch.equal(s1, s0)
        assert bool((s1[:, :5] == 7.0).all())                     # rows outside the slice untouched
        got = s1[:, 5:].reshape(rows, d)
    else:
        got = ops.mlp2(x, w1, b1, w2, b2)
        want = ops.linear(ops.linear(x, w1, b1, act="relu"), w2, b2)
        assert got is not None and torch.equal(got, want)
    hid = torch.relu(x.double() @ w1.double().t() + b1.double()).to(dtype).double()
    ref = hid @ w2.double().t() + b2.double()
    scale = ref.abs().max().item()
    assert (got.double() - ref).abs().max().item() <= 1.5 * EPS16[dtype] * scale
