"""Pins the config-model oracle (oracle/config_model.py) without any GPU:
a library routine (torch.nn.TransformerEncoderLayer), a float64 loop
implementation written from the formulas, and the domain's invariants."""
import math

import numpy as np
import pytest
import torch

from oracle import config_model as cm


def _tiny(act="gelu", final_ln=False, T=6, L=2):
    return cm.ConfigSpec(n_layers=L, d=32, n_heads=2, ffn=64, T=T, n_gears=7,
                         act=act, final_ln=final_ln, prop_dim=10, obj_dim=4)


def test_shapes_and_layout():
    spec = cm.CONFIGS[1]["spec"]
    assert spec.obs_dim == 340 and spec.n_out == 204 and spec.dh == 32
    assert cm.CONFIGS[2]["spec"].obs_dim == 596 and cm.CONFIGS[3]["spec"].obs_dim == 852
    p = cm.init_params(spec, 1)
    assert [k for k, _ in cm.param_shapes(spec)] == list(p.keys())
    obs, k = cm.make_inputs(spec, 8, 2)
    lg, v = cm.forward(p, spec, obs, k)
    assert lg.shape == (8, 29, 7) and v.shape == (8,) and lg.dtype == torch.float32
    # 12.98 MFLOP / env on the headline config
    assert abs(cm.flops_per_env(spec) / 1e6 - 12.98) < 0.01
    assert abs(cm.flops_per_env(cm.CONFIGS[2]["spec"]) / 1e6 - 205.9) < 0.1
    assert abs(cm.flops_per_env(cm.CONFIGS[3]["spec"]) / 1e9 - 1.0413) < 0.001


def test_xavier_bounds():
    spec = _tiny()
    p = cm.init_params(spec, 3)
    for name, w in p.items():
        if name.endswith("weight") and w.dim() == 2:
            a = math.sqrt(6.0 / sum(w.shape))
            assert w.abs().max() <= a and w.abs().max() > 0.8 * a


@pytest.mark.parametrize("masked", [False, True])
def test_block_matches_torch_encoder_layer(masked):
    """One block == nn.TransformerEncoderLayer(norm_first=True, gelu) with the
    same weights; key-padding mask == our additive -2^14 key bias."""
    spec = _tiny(L=1)
    p = cm.init_params(spec, 5, randomize_affine=True)
    torch.manual_seed(0)
    B = 5
    x = torch.randn(B, spec.T, spec.d)
    n_valid = torch.tensor([0, 1, 3, 5, 2], dtype=torch.int32) if masked else None
    bias = cm.key_bias(spec, n_valid, B)
    mine = cm.block(p, "blocks.0.", spec, x, bias)

    layer = torch.nn.TransformerEncoderLayer(spec.d, spec.n_heads, spec.ffn, dropout=0.0,
                                             activation="gelu", batch_first=True,
                                             norm_first=True)
    pre = "blocks.0."
    with torch.no_grad():
        layer.self_attn.in_proj_weight.copy_(torch.cat(
            [p[pre + n + ".weight"] for n in ("q_proj", "k_proj", "v_proj")]))
        layer.self_attn.in_proj_bias.copy_(torch.cat(
            [p[pre + n + ".bias"] for n in ("q_proj", "k_proj", "v_proj")]))
        layer.self_attn.out_proj.weight.copy_(p[pre + "out_proj.weight"])
        layer.self_attn.out_proj.bias.copy_(p[pre + "out_proj.bias"])
        layer.linear1.weight.copy_(p[pre + "ffn.0.weight"]); layer.linear1.bias.copy_(p[pre + "ffn.0.bias"])
        layer.linear2.weight.copy_(p[pre + "ffn.2.weight"]); layer.linear2.bias.copy_(p[pre + "ffn.2.bias"])
        layer.norm1.weight.copy_(p[pre + "ln_attn.weight"]); layer.norm1.bias.copy_(p[pre + "ln_attn.bias"])
        layer.norm2.weight.copy_(p[pre + "ln_ffn.weight"]); layer.norm2.bias.copy_(p[pre + "ln_ffn.bias"])
    layer.train()        # the training path is the plain (non-fused, non-nested) arithmetic
    pad = (bias < 0) if masked else None
    with torch.no_grad():
        ref = layer(x, src_key_padding_mask=pad)
    assert torch.allclose(mine, ref, atol=2e-6, rtol=1e-5), (mine - ref).abs().max()


def _forward_f64(p, spec, obs, n_valid):
    """Per-env, per-head, per-query loops in float64, written from the formulas."""
    P = {k: v.double().numpy() for k, v in p.items()}
    obs = obs.double().numpy()
    B = obs.shape[0]
    d, T, H, dh = spec.d, spec.T, spec.n_heads, spec.dh
    logits = np.zeros((B, 29, spec.n_gears)); value = np.zeros(B)

    def ln(v, w, b):
        mu = v.mean(); var = ((v - mu) ** 2).mean()
        return (v - mu) / math.sqrt(var + 1e-5) * w + b

    def act(v):
        if spec.act == "relu":
            return np.maximum(v, 0.0)
        return np.array([0.5 * t * (1.0 + math.erf(t / math.sqrt(2.0))) for t in v])

    for e in range(B):
        x = np.zeros((T, d))
        x[0] = P["prop_embed.weight"] @ obs[e, :spec.prop_dim] + P["prop_embed.bias"]
        for j in range(1, T):
            o = obs[e, spec.prop_dim + (j - 1) * spec.obj_dim: spec.prop_dim + j * spec.obj_dim]
            x[j] = P["obj_embed.weight"] @ o + P["obj_embed.bias"]
        nv = T - 1 if n_valid is None else int(n_valid[e])
        valid = [j <= nv for j in range(T)]
        for i in range(spec.n_layers):
            pre = f"blocks.{i}."
            h = np.stack([ln(x[t], P[pre + "ln_attn.weight"], P[pre + "ln_attn.bias"]) for t in range(T)])
            q = h @ P[pre + "q_proj.weight"].T + P[pre + "q_proj.bias"]
            k = h @ P[pre + "k_proj.weight"].T + P[pre + "k_proj.bias"]
            v = h @ P[pre + "v_proj.weight"].T + P[pre + "v_proj.bias"]
            att = np.zeros((T, d))
            for hh in range(H):
                sl = slice(hh * dh, (hh + 1) * dh)
                for t in range(T):
                    s = np.array([q[t, sl] @ k[u, sl] / math.sqrt(dh) if valid[u] else -np.inf
                                  for u in range(T)])
                    w = np.exp(s - s.max()); w /= w.sum()
                    att[t, sl] = sum(w[u] * v[u, sl] for u in range(T))
            x = x + att @ P[pre + "out_proj.weight"].T + P[pre + "out_proj.bias"]
            h2 = np.stack([ln(x[t], P[pre + "ln_ffn.weight"], P[pre + "ln_ffn.bias"]) for t in range(T)])
            hid = np.stack([act(P[pre + "ffn.0.weight"] @ h2[t] + P[pre + "ffn.0.bias"]) for t in range(T)])
            x = x + hid @ P[pre + "ffn.2.weight"].T + P[pre + "ffn.2.bias"]
        r = x[0]
        if spec.final_ln:
            r = ln(r, P["final_ln.weight"], P["final_ln.bias"])
        out = P["heads.weight"] @ r + P["heads.bias"]
        logits[e] = out[:-1].reshape(29, spec.n_gears); value[e] = out[-1]
    return logits, value


@pytest.mark.parametrize("act,final_ln", [("gelu", False), ("relu", True)])
def test_forward_matches_float64_loops(act, final_ln):
    spec = _tiny(act=act, final_ln=final_ln)
    p = cm.init_params(spec, 7, randomize_affine=True)
    obs, k = cm.make_inputs(spec, 4, 11)
    k = torch.tensor([0, 2, 5, 3], dtype=torch.int32)
    lg, v = cm.forward(p, spec, obs, k)
    lg64, v64 = _forward_f64(p, spec, obs, k)
    assert np.abs(lg.numpy() - lg64).max() < 2e-5
    assert np.abs(v.numpy() - v64).max() < 2e-5


def test_masked_slots_cannot_change_outputs():
    """Junk in masked object slots leaves logits/value unchanged (the reference
    holds its policy to this in python/tests/test_policy.py:42-63, atol 1e-5)."""
    spec = _tiny()
    p = cm.init_params(spec, 9)
    obs, _ = cm.make_inputs(spec, 6, 4)
    k = torch.tensor([0, 1, 2, 3, 4, 5], dtype=torch.int32)
    lg, v = cm.forward(p, spec, obs, k)
    obs2 = obs.clone()
    for e in range(6):
        lo = spec.prop_dim + int(k[e]) * spec.obj_dim
        obs2[e, lo:] = 1000.0
    lg2, v2 = cm.forward(p, spec, obs2, k)
    assert torch.allclose(lg, lg2, atol=1e-5) and torch.allclose(v, v2, atol=1e-5)


def test_full_mask_equals_no_mask_and_pruning_is_exact():
    spec = _tiny()
    p = cm.init_params(spec, 13)
    obs, _ = cm.make_inputs(spec, 5, 6, mask="none")
    full = torch.full((5,), spec.T - 1, dtype=torch.int32)
    a = cm.forward(p, spec, obs, None)
    b = cm.forward(p, spec, obs, full)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    k = torch.tensor([0, 1, 2, 3, 4], dtype=torch.int32)
    c = cm.forward(p, spec, obs, k)
    dd = cm.forward(p, spec, obs, k, prune_final=True)
    assert torch.allclose(c[0], dd[0], atol=1e-5) and torch.allclose(c[1], dd[1], atol=1e-5)


def test_masked_weights_are_exactly_zero():
    """exp(-2^14 + s - max) underflows to exactly 0.0 in fp32 (reference
    python/policy.py:422-428)."""
    s = torch.tensor([[0.3, -16384.0 + 5.0, 1.2]])
    w = torch.softmax(s, -1)
    assert w[0, 1].item() == 0.0


def test_emulated_16bit_is_close_to_fp32():
    spec = cm.CONFIGS[1]["spec"]
    p = cm.init_params(spec, 1)
    obs, k = cm.make_inputs(spec, 64, 2)
    lg, v = cm.forward(p, spec, obs, k)
    lg16, v16 = cm.forward(p, spec, obs, k, emulate="f16")
    assert (lg - lg16).abs().max() < 2e-3 * 2
    assert lg.abs().max() > 0.1
