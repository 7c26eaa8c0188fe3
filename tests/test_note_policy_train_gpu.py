"""The update path of the NotePolicy drop-in: forward under autograd + backward on the gradient
kernels (LayerNorm, Linear data / weight / bias gradients, attention), against torch autograd through
the CPU oracle on the same weights and inputs.

  * fp32: every parameter's gradient within 2e-4 of the oracle's (relative to that gradient's largest
    entry), outputs within the forward's 1e-5;
  * 16-bit stream: per-parameter relative Frobenius error against the fp32 oracle under literal ceilings per
    parameter group (`_GRAD_CEIL`), plus the gradient's direction (cosine >= 0.99 fp16 / 0.97 bf16 against the
    oracle's: a flipped sign or a dropped term fails whatever the group's ceiling).  The ceilings are wide for the
    critic because a ReLU unit whose pre-activation sits within a rounding of 0 may flip between two 16-bit
    forwards, and at this batch size ONE flipped unit of the critic MLP (1 of 4608 at B = 48) moves that path's
    gradients by 5 % (measured; the reference's tests note the same effect, python/tests/test_fused_ffn.py:220-224);
  * each Function against torch autograd on the SAME rounded forward (identical masks): 5e-3 (fp16);
  * the update forward is bitwise the per-op rollout forward (the reference's rollout == update contract,
    python/train_batch.py:2364-2372)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from beatsaberrl_amd.policy import NotePolicy  # noqa: E402
from oracle import note_policy_ref as nr  # noqa: E402

DEV = "cuda"


def _obs(n, seed):
    g = torch.Generator().manual_seed(seed)
    obs = torch.randn(n, nr.OBS_DIM, generator=g) * 0.7
    obs[:, nr.OFF_MASK:nr.OFF_MASK + 24] = (torch.rand(n, 24, generator=g) < 0.6).float()
    obs[0, nr.OFF_MASK:nr.OFF_MASK + 24] = 0.0
    notes = obs[:, nr.OFF_NOTES:nr.OFF_MASK].view(n, 24, 18)
    notes[..., 14] = (torch.rand(n, 24, generator=g) < 0.3).float()
    return obs


def _policy(seed, **kw):
    torch.manual_seed(seed)
    m = NotePolicy(**kw)
    with torch.no_grad():
        for p in m.parameters():
            if p.dim() == 1:
                p.add_(0.1 * torch.randn_like(p))
    # these tests hold the update path's OWN forward and backward against the oracle: its own values, not the rollout's
    # (the default "rollout" is covered by test_update_forward_returns_the_rollout_bits_on_the_default_routes)
    m.update_values = "own"
    return m


def _loss(logits, value, action, adv, ret):
    """A PPO-shaped scalar: advantage-weighted log-prob, value regression, entropy bonus."""
    logsm = torch.log_softmax(logits.float(), -1)
    logp = logsm.gather(-1, action.unsqueeze(-1)).squeeze(-1).sum(-1)
    ent = -(logsm.exp() * logsm).sum(-1).sum(-1)
    return -(adv * logp).mean() + 0.5 * ((value - ret) ** 2).mean() - 0.01 * ent.mean()


def _oracle_grads(sd, arch, obs, action, adv, ret, emulate=None):
    leaves = {k: v.clone().requires_grad_(True) for k, v in sd.items()}
    with torch.enable_grad():
        logits, value = nr.forward.__wrapped__(leaves, arch, obs, emulate=emulate)
        _loss(logits, value, action, adv, ret).backward()
    return logits.detach(), value.detach(), {k: v.grad for k, v in leaves.items()}


_KW = [
    dict(embed=64, trunk_dim=96, n_blocks=2, n_heads=2, n_gears=5, ffn_mult=4, note_geo=True),
    dict(embed=128, trunk_dim=256, n_blocks=3, n_heads=4, n_gears=7, ffn_mult=2, emb_ln=True, final_ln=True,
         head_gears=tuple(7 if j in (8, 15) else 5 for j in range(29))),
    dict(embed=192, trunk_dim=384, n_blocks=2, n_heads=4, n_gears=5, ffn_mult=4, note_geo=True,
         value_residual=True, trunk_arch="simbav2", trunk_hidden=256),
]


@pytest.mark.parametrize("kw", _KW, ids=["small_geo", "ragged_ln", "vres_v2"])
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_gradients_match_the_oracle(kw, dtype):
    m = _policy(21, **kw)
    sd = {k: v.detach().clone() for k, v in m.state_dict().items()}
    m = m.to(DEV)
    B = 96
    obs = _obs(B, 6)
    g = torch.Generator().manual_seed(9)
    sizes = torch.tensor(m.head_sizes)
    action = (torch.rand(B, 29, generator=g) * sizes).long()
    adv, ret = torch.randn(B, generator=g), torch.randn(B, generator=g)
    ref_lg, ref_v, ref_g = _oracle_grads(sd, m.arch, obs, action, adv, ret)
    if dtype != "f32":
        m.fp16 = True
        m.stream_dtype = torch.float16 if dtype == "f16" else torch.bfloat16
    _, logp, ent, value = m.get_action_and_value(obs.to(DEV), action.to(DEV))
    assert logp.requires_grad and value.requires_grad and ent.requires_grad
    logits, value2 = m.forward_stacked(obs.to(DEV))
    assert torch.equal(value2, value)
    # the 16-bit gradient stream needs the trainer's loss scaling to stay clear of fp16 subnormals
    lscale = 1.0 if dtype == "f32" else 1024.0
    (_loss(logits, value2, action.to(DEV), adv.to(DEV), ret.to(DEV)) * lscale).backward()
    if lscale != 1.0:
        for p in m.parameters():
            if p.grad is not None:
                p.grad.div_(lscale)
    live = ref_lg > -1e8
    names = [n for n, p in m.named_parameters() if p.requires_grad]
    assert all(m.get_parameter(n).grad is not None for n in names), [n for n in names if m.get_parameter(n).grad is None]
    # a key-projection bias shifts every score of a query alike: its true gradient is 0 and what is
    # computed is rounding noise, so errors are floored relative to the largest gradient of the model
    gmax = max(ref_g[n].abs().max().item() for n in names)
    if dtype == "f32":
        scale = ref_lg[live].abs().max().item()
        assert bool(((logits.cpu()[live] - ref_lg[live]).abs() <= 1e-5 * (ref_lg[live].abs() + scale)).all())
        for n in names:
            got, want = m.get_parameter(n).grad.cpu(), ref_g[n]
            err = (got - want).abs().max().item()
            assert err <= 2e-4 * want.abs().max().item() + 1e-6 * gmax, (n, err, want.abs().max().item())
        return
    _, _, em_g = _oracle_grads(sd, m.arch, obs, action, adv, ret, emulate=dtype)
    worst = []
    for n in names:
        got, want, emu = m.get_parameter(n).grad.cpu().double(), ref_g[n].double(), em_g[n].double()
        if want.abs().max().item() < 1e-5 * gmax:
            assert got.abs().max().item() < 1e-3 * gmax, n
            continue
        den = want.norm().item() + 1e-12
        e_mine, e_emul = (got - want).norm().item() / den, (emu - want).norm().item() / den
        cos = float((got * want).sum() / (got.norm() * want.norm() + 1e-30))
        grp = _group(n)
        worst.append((e_mine / _GRAD_CEIL[dtype][grp], n, e_mine, e_emul, cos))
        assert e_mine <= _GRAD_CEIL[dtype][grp], (n, e_mine, _GRAD_CEIL[dtype][grp], e_emul)
        # direction: a flipped sign gives -1, a dropped term of comparable size ~0.7
        assert cos >= (0.99 if dtype == "f16" else 0.97), (n, cos)
    w = max(worst)
    print(f"\n[{dtype}] gradient closest to its ceiling: {w[1]} error {w[2]:.2e} ({w[0]:.2f} of the ceiling; emulated oracle "
          f"{w[3]:.2e}), cosine {w[4]:.4f}")


# Literal ceilings on the relative Frobenius error of each parameter's gradient against the fp32 oracle's, per stream
# dtype and parameter group: the maxima measured over the three architectures of this test plus 30 %.  The critic's
# gradients are 1e-3 .. 1e-5 of the model's largest (a value loss against a unit-variance target) and carry the
# class's rounding noise at that relative size; vres_a / vres_b are single scalars.
_GRAD_CEIL = {
    "f16": {"heads": 2.2e-3, "trunk": 2.7e-2, "encoder": 5.2e-2, "blocks": 3.1e-2, "vres": 9.0e-2, "critic": 1.3e-1, "ln": 1.0e-2},
    "bf16": {"heads": 1.6e-2, "trunk": 1.05e-1, "encoder": 1.15e-1, "blocks": 1.3e-1, "vres": 2.9e-1, "critic": 1.9e-1, "ln": 4.4e-2},
}


def _group(name):
    if name.startswith("heads"):
        return "heads"
    if name.startswith("trunk"):
        return "trunk"
    if name.startswith("critic"):
        return "critic"
    if name.startswith(("emb_ln", "final_ln")):
        return "ln"
    if name.startswith("blocks"):
        return "vres" if "vres" in name else "blocks"
    assert name.split(".")[0] in ("saber_mlp", "torso_mlp", "leg_mlp", "note_mlp"), name
    return "encoder"


def test_update_forward_returns_the_rollout_bits_on_the_default_routes():
    """The reference holds rollout == update bitwise in every mode (python/tests/test_fp16_accum.py:146-160,
    tests/test_fused_ffn.py:471-495).  Here the DEFAULT rollout (fused block stack + pooled critic) is not the per-op
    route the update differentiates, so the update forward also runs the rollout's forward and returns ITS logits and
    value (`update_values = "rollout"`, the default): identical bits, gradients through the per-op graph.  With
    `update_values = "own"` the update returns its per-op values and the gap is the 16-bit rounding between the two
    routes, bounded here with literal ceilings (measured at B = 4096: log-prob of the 29-head action 8.9e-3, logits
    2.5e-3, value 1.5e-4); `rollout_matches_update = True` closes it from the rollout's side (per-op rollout)."""
    torch.manual_seed(0)
    m = NotePolicy(embed=192, trunk_dim=384, n_blocks=6, n_heads=4, n_gears=5, ffn_mult=4, note_geo=True).to(DEV)
    m.fp16 = True
    assert m.fused_blocks == "auto" and m.critic_pool and not m.rollout_matches_update and m.update_values == "rollout"
    od = _obs(4096, 0).to(DEV)
    with torch.no_grad():
        assert m.fused_blocks_ok(torch.float16)
        act, logp_r, _, v_r = m.get_action_and_value(od)
        lg_r, _ = m.forward_stacked(od)
    # default: the update's outputs ARE the rollout's
    _, logp_u, _, v_u = m.get_action_and_value(od, action=act)
    lg_u, v_u2 = m.forward_stacked(od)
    assert lg_u.requires_grad and v_u.requires_grad
    assert torch.equal(lg_u.detach(), lg_r) and torch.equal(v_u.detach(), v_r) and torch.equal(v_u2.detach(), v_r)
    assert (logp_u.detach() - logp_r).abs().max().item() <= 5e-5     # same logits; kernel vs torch log-softmax summation
    # ... and the gradients are the per-op graph's: the same loss differentiated with update_values = "own" gives
    # gradients that agree to the rounding between the two forwards' values
    def grads(mode):
        m.update_values = mode
        m.zero_grad(set_to_none=True)
        lg, v = m.forward_stacked(od[:512])
        (torch.log_softmax(lg, -1)[..., 0].sum() + v.sum()).backward()
        return {n: p.grad.clone() for n, p in m.named_parameters() if p.grad is not None}
    g_roll, g_own = grads("rollout"), grads("own")
    assert g_roll.keys() == g_own.keys() and len(g_roll) > 50
    gmax = max(g.norm().item() for g in g_own.values())
    for n in g_roll:
        # (k_proj.bias has a zero gradient in exact arithmetic - a softmax does not see a shift of all its keys -: its
        # two rounding-noise vectors are compared on the scale of the model's gradients, like every near-zero one)
        num, den = (g_roll[n] - g_own[n]).norm().item(), g_own[n].norm().item()
        assert num <= 2e-2 * den + 1e-4 * gmax, (n, num, den, gmax)
    # "own": the bounded gap
    m.update_values = "own"
    _, logp_o, _, v_o = m.get_action_and_value(od, action=act)
    lg_o, _ = m.forward_stacked(od)
    logp_o, v_o, lg_o = logp_o.detach(), v_o.detach(), lg_o.detach()
    g_logp, g_lg, g_v = (logp_r - logp_o).abs().max().item(), (lg_r - lg_o).abs().max().item(), (v_r - v_o).abs().max().item()
    print(f"\nrollout(default routes) vs the update's own values: |dlogp| {g_logp:.3e} (ratio off 1 by "
          f"{(torch.exp(logp_o - logp_r) - 1).abs().max().item():.3e}), |dlogit| {g_lg:.3e}, |dvalue| {g_v:.3e}")
    assert 0 < g_logp <= 1.2e-2 and g_lg <= 3.5e-3 and g_v <= 3e-4
    m.rollout_matches_update = True
    with torch.no_grad():
        assert not m.fused_blocks_ok(torch.float16)
        lg_s, v_s = m.forward_stacked(od)
        _, logp_s, _, _ = m.get_action_and_value(od, action=act)
    assert torch.equal(lg_s, lg_o) and torch.equal(v_s, v_o)
    assert (logp_s - logp_o).abs().max().item() <= 5e-5


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_update_forward_is_bitwise_the_per_op_rollout_forward(dtype):
    m = _policy(4, embed=192, trunk_dim=384, n_blocks=3, n_heads=4, n_gears=5, ffn_mult=4, note_geo=True,
                head_gears=tuple(7 if j == 4 else 5 for j in range(29))).to(DEV)
    m.fp16 = dtype == "f16"
    m.fused_blocks = "off"
    m.critic_pool = False          # the update keeps the reference's critic op order; the rollout's pooled form rounds differently
    od = _obs(40, 8).to(DEV)
    with torch.no_grad():
        lg0, v0 = m.forward_stacked(od)
    lg1, v1 = m.forward_stacked(od)
    assert lg1.requires_grad and torch.equal(lg0, lg1.detach()) and torch.equal(v0, v1.detach())
    if dtype == "f16":             # with the pool the logits are untouched and the value moves by rounding only
        m.critic_pool = True
        with torch.no_grad():
            lg2, v2 = m.forward_stacked(od)
        assert torch.equal(lg0, lg2) and (v2 - v0).abs().max().item() <= 5e-3
    # evaluation of given actions: the torch-op log-prob / entropy of the update == the sampling kernel's
    with torch.no_grad():
        act, lp0, ent0, _ = m.get_action_and_value(od)
    _, lp1, ent1, _ = m.get_action_and_value(od, act)
    assert torch.allclose(lp0, lp1.detach(), atol=2e-5, rtol=1e-5) and torch.allclose(ent0, ent1.detach(), atol=2e-5, rtol=1e-5)


def _rel(a, b):
    return ((a.double() - b.double()).norm() / (b.double().norm() + 1e-30)).item()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_functions_match_torch_autograd_on_the_same_forward(dtype):
    """Every autograd Function against plain torch ops that repeat its forward roundings, on identical inputs:
    with the ReLU masks and the softmax probabilities the same on both sides, what is left is the arithmetic of
    the backward kernels."""
    import torch.nn.functional as F
    from beatsaberrl_amd.autograd_ops import AttnPackedFn, AttnQKVFn, ChainFn, LinearFn
    from beatsaberrl_amd.fused_ln import FusedLayerNorm
    torch.manual_seed(0)
    tol = 5e-3 if dtype is torch.float16 else 4e-2 if dtype is torch.bfloat16 else 2e-5    # 16-bit: the gradient stream is rounded too
    r = (lambda t: t) if dtype is torch.float32 else (lambda t: t.to(dtype).float())
    B, T, d, Hd, nh = 40, 29, 64, 101, 2
    leaf = lambda *s, scale=1.0: (torch.randn(*s, device=DEV) * scale).requires_grad_(True)

    def check(mine_out, ref_out, mine_leaves, ref_leaves, gout):
        mine_out.backward(gout.to(mine_out.dtype))
        ref_out.backward(gout)
        assert _rel(mine_out.detach().float(), ref_out.detach()) <= tol
        # a key bias has zero true gradient (it shifts all scores of a query alike): floor the denominators
        floor = 1e-2 * max(b.grad.double().norm().item() for b in ref_leaves)
        for a, b in zip(mine_leaves, ref_leaves):
            err = (a.grad.double() - b.grad.double()).norm().item() / max(b.grad.double().norm().item(), floor)
            assert err <= tol, (tuple(a.shape), err)

    # Linear (ReLU Linear)* chain with a residual on the last layer and an odd output width
    x = (torch.randn(B, T, d, device=DEV)).to(dtype)
    res = torch.randn(B, T, d, device=DEV).to(dtype)
    ws = [leaf(96, d, scale=d ** -0.5), leaf(d, 96, scale=96 ** -0.5)]
    bs = [leaf(96, scale=0.1), leaf(d, scale=0.1)]
    xm, rm = x.detach().clone().requires_grad_(True), res.detach().clone().requires_grad_(True)
    out = ChainFn.apply(xm, rm, False, ws[0], bs[0], ws[1], bs[1])
    w2 = [w.detach().clone().requires_grad_(True) for w in ws]
    b2 = [b.detach().clone().requires_grad_(True) for b in bs]
    xr, rr = x.detach().float().clone().requires_grad_(True), res.detach().float().clone().requires_grad_(True)
    ref = r(rr + F.linear(r(F.relu(F.linear(xr, r(w2[0]), b2[0]))), r(w2[1]), b2[1]))
    check(out, ref, [xm, rm] + ws + bs, [xr, rr] + w2 + b2, torch.randn(B, T, d, device=DEV))
    # three-layer chain, fp32 output of odd width (the critic MLP's shape)
    z = torch.randn(B, 160, device=DEV).to(dtype)
    ws = [leaf(96, 160, scale=160 ** -0.5), leaf(96, 96, scale=0.1), leaf(Hd, 96, scale=0.1)]
    bs = [leaf(96, scale=0.1), leaf(96, scale=0.1), leaf(Hd, scale=0.1)]
    zm = z.detach().clone().requires_grad_(True)
    out = ChainFn.apply(zm, None, True, ws[0], bs[0], ws[1], bs[1], ws[2], bs[2])
    assert out.dtype is torch.float32
    w2 = [w.detach().clone().requires_grad_(True) for w in ws]
    b2 = [b.detach().clone().requires_grad_(True) for b in bs]
    zr = z.detach().float().clone().requires_grad_(True)
    h = r(F.relu(F.linear(zr, r(w2[0]), b2[0])))
    ref = F.linear(r(F.relu(F.linear(h, r(w2[1]), b2[1]))), r(w2[2]), b2[2])
    check(out, ref, [zm] + ws + bs, [zr] + w2 + b2, torch.randn(B, Hd, device=DEV) * 1e-2)
    # packed q|k|v projection (weights concatenated by torch) -> self-attention with a key mask -> output projection
    hx = torch.randn(B, T, d, device=DEV).to(dtype)
    wq, wk, wv, wo = (leaf(d, d, scale=d ** -0.5) for _ in range(4))
    bq, bk, bv, bo = (leaf(d, scale=0.1) for _ in range(4))
    valid = torch.rand(B, T, device=DEV) < 0.7
    valid[:, :5] = True
    bias = ((valid.float() - 1.0) * 16384.0).to(dtype)
    hm = hx.detach().clone().requires_grad_(True)
    qkv = LinearFn.apply(hm, torch.cat([wq, wk, wv]), torch.cat([bq, bk, bv]), None, None, False)
    out = LinearFn.apply(AttnPackedFn.apply(qkv, bias, nh), wo, bo, None, hm, False)
    L2 = [t.detach().clone().requires_grad_(True) for t in (wq, wk, wv, wo, bq, bk, bv, bo)]
    hr = hx.detach().float().clone().requires_grad_(True)

    def attend(q, k, v):
        Bq, Tq = q.shape[0], q.shape[1]
        sp = lambda t: t.view(Bq, -1, nh, d // nh).transpose(1, 2)
        s = sp(q) @ sp(k).transpose(-2, -1) / (d // nh) ** 0.5 + bias.float().view(Bq, 1, 1, T)
        return (r(torch.softmax(s, -1)) @ sp(v)).transpose(1, 2).reshape(Bq, Tq, d)

    q, k, v = (r(F.linear(hr, r(L2[i]), L2[4 + i])) for i in range(3))
    ref = r(hr + F.linear(r(attend(q, k, v)), r(L2[3]), L2[7]))
    check(out, ref, [hm, wq, wk, wv, wo, bq, bk, bv, bo], [hr] + L2, torch.randn(B, T, d, device=DEV))
    # pruned queries over the packed k|v projection
    for t in (wq, wk, wv, bq, bk, bv):
        t.grad = None
    hm = hx.detach().clone().requires_grad_(True)
    kv = LinearFn.apply(hm, torch.cat([wk, wv]), torch.cat([bk, bv]), None, None, False)
    qq = LinearFn.apply(hm[:, :5], wq, bq, None, None, False)
    out = AttnQKVFn.apply(qq, kv, bias, nh)
    L2 = [t.detach().clone().requires_grad_(True) for t in (wq, wk, wv, bq, bk, bv)]
    hr = hx.detach().float().clone().requires_grad_(True)
    ref = r(attend(r(F.linear(hr[:, :5], r(L2[0]), L2[3])), r(F.linear(hr, r(L2[1]), L2[4])), r(F.linear(hr, r(L2[2]), L2[5]))))
    check(out, ref, [hm, wq, wk, wv, bq, bk, bv], [hr] + L2, torch.randn(B, 5, d, device=DEV))
    # LayerNorm and residual-add + LayerNorm with a folded bias
    ln = FusedLayerNorm(d).to(DEV)
    with torch.no_grad():
        ln.weight.add_(0.2 * torch.randn(d, device=DEV))
        ln.bias.add_(0.2 * torch.randn(d, device=DEV))
    a0, b0 = torch.randn(B, T, d, device=DEV).to(dtype), torch.randn(B, T, d, device=DEV).to(dtype)
    bb = leaf(d, scale=0.3)
    am, bm = a0.detach().clone().requires_grad_(True), b0.detach().clone().requires_grad_(True)
    xs, ys = ln.forward_add(am, bm, bb)
    wl, bl, bb2 = (t.detach().clone().requires_grad_(True) for t in (ln.weight, ln.bias, bb))
    ar, br = a0.detach().float().clone().requires_grad_(True), b0.detach().float().clone().requires_grad_(True)
    xr2 = r(ar + (br + bb2))
    yr = r(F.layer_norm(xr2, (d,), wl, bl, 1e-5))
    g1, g2 = torch.randn(B, T, d, device=DEV), torch.randn(B, T, d, device=DEV)
    (xs.float() * g1 + ys.float() * g2).sum().backward()
    (xr2 * g1 + yr * g2).sum().backward()
    for got, want in ((am.grad, ar.grad), (bm.grad, br.grad), (ln.weight.grad, wl.grad), (ln.bias.grad, bl.grad), (bb.grad, bb2.grad)):
        assert _rel(got.float(), want) <= tol


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,d,F", [(70, 128, 512), (4133, 192, 768)])
@pytest.mark.parametrize("save", [False, True])
def test_fused_ffn_function_matches_the_unfused_chain(dtype, rows, d, F, save):
    """FusedFfnFn (fused forward kernel; chain backward over the hidden the kernel wrote - `save` - or over a
    recomputed one; reference
    python/fp16_linear.py:1197-1251) against ChainFn on the same operands: outputs to 16-bit rounding of the
    stream, every gradient to 2 % of its largest entry (the two forwards accumulate in different k orders, so a
    hidden unit within a rounding of 0 may sit on the other side of the ReLU)."""
    from beatsaberrl_amd.autograd_ops import ChainFn, FusedFfnFn
    g = torch.Generator().manual_seed(rows)
    mk = lambda *s, sc=1.0: (torch.randn(*s, generator=g) * sc).to(DEV)
    w0, b0, w2, b2 = mk(F, d, sc=d ** -0.5), mk(F, sc=0.1), mk(d, F, sc=F ** -0.5), mk(d, sc=0.1)
    x0, h0, go = mk(rows, d).to(dtype), mk(rows, d).to(dtype), mk(rows, d).to(dtype)
    outs = []
    for fn in ("fused", "chain"):
        leaves = [t.clone().requires_grad_(True) for t in (x0, h0, w0, b0, w2, b2)]
        x, h, a0, c0, a2, c2 = leaves
        y = FusedFfnFn.apply(x, h, a0, c0, a2, c2, save) if fn == "fused" else ChainFn.apply(h, x, False, a0, c0, a2, c2)
        y.backward(go)
        outs.append((y.detach(), [t.grad for t in leaves]))
    (yf, gf), (yc, gc) = outs
    eps = 2.0 ** -10 if dtype is torch.float16 else 2.0 ** -7
    assert (yf.float() - yc.float()).abs().max().item() <= 2 * eps * yc.float().abs().max().item()
    for name, a, b in zip(("dx", "dh2", "dw0", "db0", "dw2", "db2"), gf, gc):
        assert a.dtype == b.dtype and a.shape == b.shape, name
        err = (a.float() - b.float()).abs().max().item()
        assert err <= 2e-2 * b.float().abs().max().item(), (name, err)
    assert torch.equal(gf[0], go)                               # the residual branch passes the gradient through


def test_fused_ffn_saved_hidden_is_the_hidden_the_kernel_used():
    """want_hidden: the (rows, F) tensor the packed kernel writes is relu(h2 W0^T + b0) rounded once - within one
    16-bit ulp of the Linear kernel's (another k order) - and the backward over it equals the backward over the
    recomputed hidden wherever the two hiddens agree bitwise (here: gradients to 1e-3 of their largest entry)."""
    from beatsaberrl_amd import ops
    from beatsaberrl_amd.autograd_ops import FusedFfnFn
    rows, d, F, dtype = 1000, 192, 768, torch.float16
    g = torch.Generator().manual_seed(9)
    mk = lambda *s, sc=1.0: (torch.randn(*s, generator=g) * sc).to(DEV)
    w0, b0, w2, b2 = mk(F, d, sc=d ** -0.5), mk(F, sc=0.1), mk(d, F, sc=F ** -0.5), mk(d, sc=0.1)
    x0, h0, go = mk(rows, d).to(dtype), mk(rows, d).to(dtype), mk(rows, d).to(dtype)
    xo, ho, hid = ops.ffn_fused(x0, h0, w0.to(dtype), b0, w2.to(dtype), b2, act="relu", want_hidden=True)
    ref = ops.linear(h0, w0.to(dtype), b0, act="relu")
    assert hid.shape == (rows, F) and hid.dtype is dtype and ho is None
    assert (hid.float() - ref.float()).abs().max().item() <= 2.0 ** -10 * ref.float().abs().max().item()
    assert (hid == ref).float().mean().item() > 0.99
    plain, _ = ops.ffn_fused(x0, h0, w0.to(dtype), b0, w2.to(dtype), b2, act="relu")
    assert torch.equal(plain, xo)                               # writing the hidden changes nothing else
    grads = []
    for save in (True, False):
        leaves = [t.clone().requires_grad_(True) for t in (x0, h0, w0, b0, w2, b2)]
        FusedFfnFn.apply(*leaves, save).backward(go)
        grads.append([t.grad for t in leaves])
    for name, a, b in zip(("dx", "dh2", "dw0", "db0", "dw2", "db2"), *grads):
        assert (a.float() - b.float()).abs().max().item() <= 1e-3 * b.float().abs().max().item(), name


def test_update_path_with_the_fused_ffn_follows_the_unfused_update():
    """fused_ffn = "on": the update forward's block FFNs run as the fused kernel; logits, value and every
    parameter gradient stay within the 16-bit class of the unfused update on the same weights and batch."""
    kw = dict(embed=192, trunk_dim=384, n_blocks=3, n_heads=4, n_gears=5, ffn_mult=4, note_geo=True)
    m = _policy(5, **kw).to(DEV)
    m.fp16 = True
    B = 64
    obs = _obs(B, 3).to(DEV)
    g = torch.Generator().manual_seed(2)
    action = (torch.rand(B, 29, generator=g) * 5).long().to(DEV)
    adv, ret = torch.randn(B, generator=g).to(DEV), torch.randn(B, generator=g).to(DEV)
    res = []
    for mode in ("off", "on", "recompute"):
        m.fused_ffn = mode
        m.zero_grad(set_to_none=True)
        logits, value = m.forward_stacked(obs)
        (_loss(logits, value, action, adv, ret) * 1024.0).backward()
        res.append((logits.detach(), value.detach(), {n: p.grad.detach().clone() / 1024.0 for n, p in m.named_parameters()}))
    (l0, v0, g0), (l1, v1, g1), (l2, v2, g2) = res
    assert torch.equal(l1, l2) and torch.equal(v1, v2)         # one forward kernel, with or without the hidden written
    for n in g1:                                                # and the same chain backward up to the hidden's k order
        assert (g1[n] - g2[n]).norm().item() <= 2e-2 * g2[n].norm().item() + 1e-12, n
    assert not torch.equal(l0, l1)                              # the fused kernel did run
    assert (l0 - l1).abs().max().item() < 2e-2 and (v0 - v1).abs().max().item() < 2e-2
    gmax = max(t.abs().max().item() for t in g0.values())
    for n in g0:
        den = g0[n].norm().item()
        if g0[n].abs().max().item() < 1e-5 * gmax:
            continue
        assert (g1[n] - g0[n]).norm().item() <= 6e-2 * den, (n, (g1[n] - g0[n]).norm().item() / den)     # measured maximum 4.4e-2 (critic_q.weight)
