"""Pins the 16-bit `emulate=` branches of both oracles (oracle/config_model.py,
oracle/note_policy_ref.py) without a GPU.  Every 16-bit GPU gate compares a kernel
path against these branches, so a doubled or a missed rounding in them would move
the gates silently.

How they are pinned:
  * the casts themselves: float16 through numpy's own type, bfloat16 through a
    round-to-nearest-even written on the bit pattern here, both checked on
    hand-picked values (ties, carries into the exponent) and against torch's;
  * a float64 restatement of each forward, written from the formulas, with an
    explicit cast at every documented rounding point of the 16-bit stream
    (python/fp16_linear.py:1-18: 16-bit storage of every GEMM operand and
    result, fp32 accumulate; python/fused_ln.py:134-164: fp32 statistics, one
    rounding of the LayerNorm output; python/policy.py:1200-1209: the obs is
    rounded once; csrc/small_attn.cu:15-21: fp32 scores and softmax, 16-bit
    probabilities into P.V);
  * mutation checks: the same restatement with ONE rounding point left out (or
    one added) must land measurably further from the oracle than the faithful
    one - so the tolerance is shown to separate "same rounding points" from
    "one differs";
  * one library cross-check per op: torch's CPU float16 / bfloat16 kernels
    (matmul, layer_norm, softmax, gelu, relu) on the same rounded operands.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import config_model as cm
from oracle import note_policy_ref as nr


# ---- the casts -------------------------------------------------------------------
def _bf16_rne(x):
    """float32 -> nearest bfloat16 (ties to even) -> float32, on the bit pattern."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    u = (u + 0x7FFF + lsb) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def _cast(x, dtype):
    """float64 array -> fp32 (the accumulator's own rounding) -> 16-bit type -> float64."""
    x32 = np.asarray(x, dtype=np.float64).astype(np.float32)
    if dtype == "f16":
        return x32.astype(np.float16).astype(np.float64)
    return _bf16_rne(x32).astype(np.float64)


def test_casts_on_known_values():
    # bf16 keeps 8 significand bits: 1 + 2^-8 is a tie between 1 and 1 + 2^-7 -> even (1); 1 + 3 * 2^-8 ties up
    assert _bf16_rne(np.float32(1 + 2 ** -8)) == np.float32(1.0)
    assert _bf16_rne(np.float32(1 + 3 * 2 ** -8)) == np.float32(1 + 2 ** -6)
    assert _bf16_rne(np.float32(1 + 2 ** -8 + 2 ** -20)) == np.float32(1 + 2 ** -7)
    assert _bf16_rne(np.float32(2 - 2 ** -9)) == np.float32(2.0)              # carry into the exponent
    assert _bf16_rne(np.float32(-3.140625)) == np.float32(-3.140625)          # representable: unchanged
    # fp16 keeps 11: 1 + 2^-11 ties to 1, 2049 ties to 2048, 2051 to 2052, 65519 stays finite (65504)
    assert _cast(1 + 2 ** -11, "f16") == 1.0 and _cast(2049.0, "f16") == 2048.0 and _cast(2051.0, "f16") == 2052.0
    assert _cast(65519.0, "f16") == 65504.0
    g = torch.Generator().manual_seed(0)
    x = torch.randn(20000, generator=g) * torch.logspace(-6, 4, 20000)
    for dtype, tdt in (("f16", torch.float16), ("bf16", torch.bfloat16)):
        mine = _cast(x.double().numpy(), dtype)
        assert np.array_equal(mine, x.to(tdt).double().numpy())
        assert np.array_equal(mine, cm._round(x, dtype).double().numpy())
        assert np.array_equal(mine, nr._round(x, dtype).double().numpy())
    assert cm._round(x, None) is x and nr._round(x, None) is x


# ---- config model ----------------------------------------------------------------
def _tiny(act="gelu", final_ln=False, T=6, L=2):
    return cm.ConfigSpec(n_layers=L, d=32, n_heads=2, ffn=64, T=T, n_gears=7,
                         act=act, final_ln=final_ln, prop_dim=10, obj_dim=4)


def _ln64(x, w, b):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + 1e-5) * w + b


def _act64(x, kind):
    if kind == "relu":
        return np.maximum(x, 0.0)
    return 0.5 * x * (1.0 + np.vectorize(math.erf)(x / math.sqrt(2.0)))


# the rounding points of the 16-bit config forward, by name
CFG_POINTS = ("obs", "weights", "ln_attn", "q", "k", "v", "probs", "att", "ln_ffn", "hidden", "readout")
CFG_RESIDUAL_POINTS = ("tokens", "res_attn", "res_ffn")        # only with a 16-bit residual stream


def _cfg_forward_f64(p, spec, obs, n_valid, dtype, round_residual, skip=(), extra=()):
    """Per-env float64 restatement with explicit casts.  skip: rounding points left out;
    extra: 'scores' rounds the attention scores too (a point the 16-bit stream does NOT have)."""
    def r(x, point):
        return x if point in skip else _cast(x, dtype)

    def rr(x, point):
        return r(x, point) if round_residual else x

    P = {k: v.double().numpy() for k, v in p.items()}
    W = {k: r(v, "weights") for k, v in P.items() if k.endswith("weight") and v.ndim == 2}
    obs = r(obs.double().numpy(), "obs")
    B, d, T, H, dh = obs.shape[0], spec.d, spec.T, spec.n_heads, spec.dh
    out = np.zeros((B, spec.n_out))
    for e in range(B):
        x = np.zeros((T, d))
        x[0] = W["prop_embed.weight"] @ obs[e, :spec.prop_dim] + P["prop_embed.bias"]
        for j in range(1, T):
            o = obs[e, spec.prop_dim + (j - 1) * spec.obj_dim: spec.prop_dim + j * spec.obj_dim]
            x[j] = W["obj_embed.weight"] @ o + P["obj_embed.bias"]
        x = rr(x, "tokens")
        nv = T - 1 if n_valid is None else int(n_valid[e])
        for i in range(spec.n_layers):
            pre = f"blocks.{i}."
            h = r(_ln64(x, P[pre + "ln_attn.weight"], P[pre + "ln_attn.bias"]), "ln_attn")
            q = r(h @ W[pre + "q_proj.weight"].T + P[pre + "q_proj.bias"], "q")
            k = r(h @ W[pre + "k_proj.weight"].T + P[pre + "k_proj.bias"], "k")
            v = r(h @ W[pre + "v_proj.weight"].T + P[pre + "v_proj.bias"], "v")
            att = np.zeros((T, d))
            for hh in range(H):
                sl = slice(hh * dh, (hh + 1) * dh)
                s = q[:, sl] @ k[:, sl].T / math.sqrt(dh)
                if "scores" in extra:
                    s = _cast(s, dtype)
                s[:, nv + 1:] = -np.inf
                w = np.exp(s - s.max(-1, keepdims=True))
                w = r(w / w.sum(-1, keepdims=True), "probs")
                att[:, sl] = w @ v[:, sl]
            att = r(att, "att")
            x = rr(x + att @ W[pre + "out_proj.weight"].T + P[pre + "out_proj.bias"], "res_attn")
            h2 = r(_ln64(x, P[pre + "ln_ffn.weight"], P[pre + "ln_ffn.bias"]), "ln_ffn")
            hid = r(_act64(h2 @ W[pre + "ffn.0.weight"].T + P[pre + "ffn.0.bias"], spec.act), "hidden")
            x = rr(x + hid @ W[pre + "ffn.2.weight"].T + P[pre + "ffn.2.bias"], "res_ffn")
        t0 = x[0]
        if spec.final_ln:
            t0 = _ln64(t0, P["final_ln.weight"], P["final_ln.bias"])
        out[e] = W["heads.weight"] @ r(t0, "readout") + P["heads.bias"]
    return out


def _cfg_case(dtype, act, final_ln, seed):
    spec = _tiny(act=act, final_ln=final_ln)
    p = cm.init_params(spec, seed, randomize_affine=True)
    obs, _ = cm.make_inputs(spec, 6, seed + 100)
    k = torch.tensor([0, 2, 5, 3, 1, 4], dtype=torch.int32)
    return spec, p, obs, k


def _oracle_flat(p, spec, obs, k, dtype, round_residual):
    lg, v = cm.forward(p, spec, obs, k, emulate=dtype, round_residual=round_residual)
    return torch.cat([lg.reshape(lg.shape[0], -1), v[:, None]], 1).double().numpy()


# Faithful restatement and oracle differ in two ways only: fp32 against float64 accumulation (~1e-4 of a 16-bit unit
# roundoff on the outputs), and - rarely, about one env in five at these sizes - an intermediate whose fp32 and
# float64 values land on opposite sides of a 16-bit rounding boundary (a single-ulp flip, which then moves that env's
# outputs by a good fraction of a unit roundoff).  One missing or added rounding point moves EVERY env.  So the gate
# is on the MEDIAN env: faithful <= 1e-3 u, every mutant >= 0.05 u (measured: faithful 0 .. 2e-4 u, mutants >= 0.2 u),
# plus a cap on how many envs may carry a flip.
_U = {"f16": 2.0 ** -11, "bf16": 2.0 ** -8}


def _rms(a, b):
    return float(np.sqrt(np.mean((a - b) ** 2)))


def _env_rms(a, b):
    return np.sqrt(np.mean((a - b) ** 2, axis=1))


@pytest.mark.parametrize("round_residual", [False, True])
@pytest.mark.parametrize("act,final_ln", [("gelu", False), ("relu", True)])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_config_emulate_matches_float64_restatement(dtype, act, final_ln, round_residual):
    u = _U[dtype]
    points = CFG_POINTS + (CFG_RESIDUAL_POINTS if round_residual else ())
    if round_residual and not final_ln:
        points = tuple(pt for pt in points if pt != "readout")     # the stream is already 16-bit there
    faithful, mutants = [], {pt: [] for pt in points + ("+scores",)}
    for seed in (7, 8, 9):
        spec, p, obs, k = _cfg_case(dtype, act, final_ln, seed)
        orc = _oracle_flat(p, spec, obs, k, dtype, round_residual)
        faithful.append(_env_rms(orc, _cfg_forward_f64(p, spec, obs, k, dtype, round_residual)))
        for pt in points:
            mutants[pt].append(_env_rms(orc, _cfg_forward_f64(p, spec, obs, k, dtype, round_residual, skip=(pt,))))
        mutants["+scores"].append(_env_rms(orc, _cfg_forward_f64(p, spec, obs, k, dtype, round_residual, extra=("scores",))))
    faithful = np.concatenate(faithful) / u
    med = {pt: float(np.median(np.concatenate(v))) / u for pt, v in mutants.items()}
    nearest = min(med, key=med.get)
    print(f"\n[{dtype} {act} final_ln={final_ln} rr={round_residual}] faithful: median env {np.median(faithful):.1e} u, "
          f"{int((faithful > 0.01).sum())}/{faithful.size} envs with a flip (worst {faithful.max():.2f} u); "
          f"nearest mutant '{nearest}': median env {med[nearest]:.3f} u")
    assert np.median(faithful) <= 1e-3
    assert (faithful > 0.01).mean() <= 0.34 and faithful.max() <= 1.5
    assert med[nearest] >= 0.05, med


def test_config_emulate_residual_switch_and_fp32_limit():
    """round_residual=False must differ from True only by the three stream roundings, and with the casts
    replaced by the identity the emulate branch IS the fp32 forward (same code path, bit for bit)."""
    spec, p, obs, k = _cfg_case("f16", "gelu", False, 7)
    a = _oracle_flat(p, spec, obs, k, "f16", False)
    b = _oracle_flat(p, spec, obs, k, "f16", True)
    assert _rms(a, b) > 0.25 * _U["f16"]
    orig = cm._round
    try:
        cm._round = lambda x, emulate: x
        ident = _oracle_flat(p, spec, obs, k, "f16", True)
    finally:
        cm._round = orig
    lg, v = cm.forward(p, spec, obs, k)
    assert np.array_equal(ident, torch.cat([lg.reshape(6, -1), v[:, None]], 1).double().numpy())


# ---- library cross-checks, one per op --------------------------------------------
@pytest.mark.parametrize("dtype,tdt", [("f16", torch.float16), ("bf16", torch.bfloat16)])
def test_emulated_ops_match_torch_16bit_cpu_kernels(dtype, tdt):
    """The emulation's rule for one op - round the operands, compute in fp32, round the result - against torch's own
    CPU kernels on 16-bit tensors (which accumulate in fp32 and round on store)."""
    g = torch.Generator().manual_seed(3)
    r = lambda t: cm._round(t, dtype)
    x, w = torch.randn(96, 128, generator=g), torch.randn(64, 128, generator=g) * 0.1

    def agree(mine, lib, what, min_equal=0.995):
        lib = lib.float()
        same = (mine == lib).float().mean().item()
        ulp = (mine - lib).abs().max().item() / (mine.abs().max().item() * _U[dtype] * 2)
        print(f"[{dtype}] {what}: {same:.4f} bit-equal, max diff {ulp:.2f} ulp of the largest value")
        assert same >= min_equal and ulp <= 1.0, what

    agree(r(F.linear(r(x), r(w))), F.linear(x.to(tdt), w.to(tdt)), "matmul")
    gm, bt = torch.rand(128, generator=g) + 0.5, torch.randn(128, generator=g) * 0.1
    # 16-bit LayerNorm: statistics and affine in fp32 on the 16-bit operands, one rounding of the output
    agree(r(F.layer_norm(r(x), (128,), r(gm), r(bt), 1e-5)), F.layer_norm(x.to(tdt), (128,), gm.to(tdt), bt.to(tdt), 1e-5),
          "layer_norm", min_equal=0.99)
    s = torch.randn(96, 16, generator=g) * 3
    agree(r(torch.softmax(r(s), -1)), torch.softmax(s.to(tdt), -1), "softmax", min_equal=0.99)
    agree(r(F.gelu(r(x))), F.gelu(x.to(tdt)), "gelu", min_equal=0.99)
    agree(r(F.relu(r(x))), F.relu(x.to(tdt)), "relu", min_equal=1.0)


# ---- NotePolicy oracle -----------------------------------------------------------
# At this model's size (29 tokens, 2-3 blocks, trunk, critic) every env carries several single-ulp flips, so
# outputs cannot separate "faithful" from "one rounding point off".  Instead every rounding the oracle performs is
# recorded (input and output of its cast, in call order) and a float64 restatement is walked along that tape: at each
# of its own rounding points it must meet the oracle's NEXT recorded cast, with the same shape and - before the cast,
# where no flip can occur - the same values to fp32-accumulate precision; it then continues from the oracle's rounded
# tensor.  A rounding point the oracle lacks, has twice, or has elsewhere breaks the walk; wrong arithmetic between
# two points shows as a pre-cast mismatch (a missed upstream rounding is ~5e-4 relative, the gate 2e-5).
class _Tape:
    def __init__(self, dtype):
        self.dtype, self.calls, self.i, self.skip_call = dtype, [], 0, None

    def record(self, x, emulate):
        if emulate is None:
            return x
        n = len(self.calls)
        if n == self.skip_call:                # mutation: the oracle "forgets" this rounding
            self.skip_call = None
            return x
        out = x.to({"f16": torch.float16, "bf16": torch.bfloat16}[emulate]).float()
        self.calls.append((x.detach().clone(), out))
        return out

    def meet(self, x64, what):
        """The restatement's value before one of its rounding points -> the oracle's rounded tensor."""
        assert self.i < len(self.calls), f"{what}: the oracle performs no further rounding"
        inp, out = self.calls[self.i]
        self.i += 1
        x64 = np.asarray(x64, dtype=np.float64)
        assert tuple(inp.shape) == x64.shape, f"{what}: oracle rounds a {tuple(inp.shape)} tensor here, expected {x64.shape}"
        ref = inp.double().numpy()
        tol = 2e-5 * max(float(np.abs(ref).max()), 1e-3)
        err = float(np.abs(ref - x64).max())
        assert err <= tol, f"{what}: pre-rounding values differ by {err:.3e} (gate {tol:.3e})"
        assert np.array_equal(out.double().numpy(), _cast(ref, self.dtype)), f"{what}: not one round-to-nearest-even"
        return out.double().numpy()


def _blocks_walk(P, arch, x, bias, r, round_residual=True):
    """The block stack of the walk: blocks 0..L-2 on all rows, the last on the lead rows; returns (lead, x_res, attend)."""
    B, d, H, L = x.shape[0], arch["embed"], arch["n_heads"], arch["n_blocks"]
    dh = d // H
    rr = r if round_residual else (lambda v, what: v)

    def lin(n, v):
        return v @ r(P[n + ".weight"], n + ".weight").T + P[n + ".bias"]

    ln = lambda n, v: _ln64(v, P[n + ".weight"], P[n + ".bias"])
    mlp2 = lambda n, v: lin(n + ".2", r(np.maximum(lin(n + ".0", v), 0.0), n + " hidden"))

    def attend(q, k, v, what):
        Tq, T = q.shape[1], k.shape[1]
        s = np.einsum("bqhd,bkhd->bhqk", q.reshape(B, Tq, H, dh), k.reshape(B, T, H, dh)) / math.sqrt(dh) + bias[:, None, None, :]
        w = np.exp(s - s.max(-1, keepdims=True))
        w = r(w / w.sum(-1, keepdims=True), what + " probabilities")
        return np.einsum("bhqk,bkhd->bqhd", w, v.reshape(B, T, H, dh)).reshape(B, Tq, d)

    x_res, v0, vres = None, None, bool(arch.get("value_residual", False))
    for i in range(L):
        p = f"blocks.{i}."
        h = r(ln(p + "ln_attn", x), p + "ln_attn")
        k = r(lin(p + "k_proj", h), p + "k")
        v = r(lin(p + "v_proj", h), p + "v")
        if vres and i == 0:
            v0 = v                              # block 0 hands its values to every later block
        elif vres:
            v = r(v * P[p + "vres_a"] + v0 * P[p + "vres_b"], p + "value-residual mix")
        if i == L - 1:
            x_res = x
            x, h = x[:, :nr.N_LEAD], h[:, :nr.N_LEAD]
        q = r(lin(p + "q_proj", h), p + "q")
        att = r(attend(q, k, v, p + "attention"), p + "attention output")
        x = rr(x + lin(p + "out_proj", att), p + "stream after attention")
        h2 = r(ln(p + "ln_ffn", x), p + "ln_ffn")
        x = rr(x + mlp2(p + "ffn", h2), p + "stream after ffn")
    return r(x, "lead rows"), r(x_res, "x_res"), attend


def _np_walk(sd, arch, obs, tape):
    """float64 restatement of NotePolicy's 16-bit forward walked along the oracle's tape.  Rounding points, in the
    order the forward meets them: obs; encoder inputs with geometry lanes; per Linear its weight, then its result
    where the result is stored (every Linear but the second of a residual pair and the last of the critic MLP);
    encoder / FFN / trunk hidden after ReLU; token stream; every LayerNorm output; q, k, v, probabilities, attention
    output; residual stream after each add; the two outputs of the block stack; trunk sum; critic activations."""
    P = {k: v.double().numpy() for k, v in sd.items()}
    r = tape.meet

    def lin(n, x):
        return x @ r(P[n + ".weight"], n + ".weight").T + P[n + ".bias"]

    ln = lambda n, x: _ln64(x, P[n + ".weight"], P[n + ".bias"])
    mlp2 = lambda n, x: lin(n + ".2", r(np.maximum(lin(n + ".0", x), 0.0), n + " hidden"))
    B, d, H, L = obs.shape[0], arch["embed"], arch["n_heads"], arch["n_blocks"]
    dh = d // H
    o = r(obs.double().numpy(), "obs")
    sab = np.stack([o[:, nr.SABER_L], o[:, nr.SABER_R]], 1)
    notes = o[:, nr.OFF_NOTES:nr.OFF_MASK].reshape(B, nr.N_SLOTS, nr.NOTE_FEAT)
    mask = o[:, nr.OFF_MASK:nr.OFF_MASK + nr.N_SLOTS]
    if arch.get("note_geo", False):
        # the geometry lanes are fp32 arithmetic (pinned on its own); what is checked here is where it is rounded
        geo = nr.note_geo(torch.from_numpy(notes).float(), torch.from_numpy(sab).float(), float(arch["z_asinh"]),
                          arch.get("game", "standard") == "flux", torch.from_numpy(o[:, nr.OBS_HEAD_Z]).float())
        notes = r(np.concatenate([notes, geo.double().numpy()], -1), "note lanes + geometry")
    eye = np.broadcast_to(np.eye(2), (B, 2, 2))
    legs = np.stack([o[:, nr.LEG_L], o[:, nr.LEG_R]], 1)
    x = np.concatenate([mlp2("saber_mlp", np.concatenate([sab, eye], -1)), mlp2("torso_mlp", o[:, nr.TORSO])[:, None],
                        mlp2("leg_mlp", np.concatenate([legs, eye], -1)), mlp2("note_mlp", notes)], 1)
    x = r(x, "tokens")
    bias = np.concatenate([np.zeros((B, nr.N_LEAD)), (mask - 1.0) * nr.MASK_BIAS], 1)
    if arch.get("emb_ln", False):
        x = r(ln("emb_ln", x), "emb_ln")

    lead, x_res, attend = _blocks_walk(P, arch, x, bias, r)
    if arch.get("final_ln", False):
        lead = r(ln("final_ln", lead), "final_ln")
    if arch.get("trunk_arch", "simba") == "simbav2":
        # SimBaV2 (python/policy.py:1140-1155): GEMM results and GEMM inputs are stored 16-bit; scalers, ReLU, the
        # row normalisations and the LERP are fp32 in between; one rounding of the feature row at the end
        l2n = lambda v: v / np.maximum(np.sqrt((v * v).sum(-1, keepdims=True)), 1e-6)
        D = arch["trunk_dim"]
        xx = l2n(r(lin("trunk_in", lead.reshape(B, -1)), "trunk_in") * P["trunk_s_in"])
        xr = r(xx, "trunk_w1 input")
        uu = np.maximum(r(lin("trunk_w1", xr), "trunk_w1") * P["trunk_s_1"], 0.0)
        ur = r(uu, "trunk_w2 input")
        yy = l2n(r(lin("trunk_w2", ur), "trunk_w2"))
        xx = l2n(xx + P["trunk_alpha"] * (0.5 * math.sqrt(D)) * (yy - xx))
        hfeat = r(xx * math.sqrt(D), "trunk feature")
    else:
        t = r(lin("trunk_proj", lead.reshape(B, -1)), "trunk_proj")
        u = r(ln("trunk_ln1", t), "trunk_ln1")
        dlt = lin("trunk_fc2", r(np.maximum(lin("trunk_fc1", u), 0.0), "trunk hidden"))
        hfeat = r(ln("trunk_ln2", r(t + dlt, "trunk sum")), "trunk_ln2")
    wh = r(np.concatenate([P[f"heads.{j}.weight"] for j in range(nr.N_HEADS_OUT)]), "packed head weights")
    flat = hfeat @ wh.T + np.concatenate([P[f"heads.{j}.bias"] for j in range(nr.N_HEADS_OUT)])
    hv = r(ln("critic_ln", x_res), "critic_ln")
    q = r(lin("critic_q", hv[:, 2:3]), "critic q")
    k = r(lin("critic_k", hv), "critic k")
    v = r(lin("critic_v", hv), "critic v")
    a = r(attend(q, k, v, "critic attention"), "critic attention output").reshape(B, d)
    a = r(lin("critic_out", a), "critic_out")
    z = r(np.maximum(lin("critic_mlp.0", np.concatenate([a, hfeat], -1)), 0.0), "critic_mlp.0")
    z = r(np.maximum(lin("critic_mlp.2", z), 0.0), "critic_mlp.2")
    vlog = lin("critic_mlp.4", z)
    centers = np.linspace(-float(arch["value_vmax"]), float(arch["value_vmax"]), int(arch["value_bins"]))
    pv = np.exp(vlog - vlog.max(-1, keepdims=True))
    value = (pv / pv.sum(-1, keepdims=True)) @ centers
    assert tape.i == len(tape.calls), f"the oracle rounds {len(tape.calls) - tape.i} more tensors than the 16-bit stream has"
    return flat, value


def _np_taped_oracle(sd, arch, obs, dtype, skip_call=None):
    tape = _Tape(dtype)
    tape.skip_call = skip_call
    orig = nr._round
    try:
        nr._round = tape.record
        lg, v = nr.forward(sd, arch, obs, emulate=dtype)
    finally:
        nr._round = orig
    sizes = arch.get("head_gears") or [arch["n_gears"]] * nr.N_HEADS_OUT
    flat = torch.cat([lg[:, j, :n] for j, n in enumerate(sizes)], 1)
    return tape, flat.double().numpy(), v.double().numpy()


def _fixture(name):
    import os
    arch, sd, obs, _, _ = nr.load_fixture(os.path.join(os.path.dirname(__file__), "golden", name + ".npz"))
    return arch, sd, obs[:3]


@pytest.mark.parametrize("fixture", ["notepolicy_geo", "notepolicy_ragged_ln", "notepolicy_flux", "notepolicy_vres_v2"])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_notepolicy_emulate_walks_the_float64_restatement(dtype, fixture):
    arch, sd, obs = _fixture(fixture)
    tape, flat, value = _np_taped_oracle(sd, arch, obs, dtype)
    my_flat, my_value = _np_walk(sd, arch, obs, tape)
    print(f"\n[{dtype} {fixture}] {len(tape.calls)} rounding points walked")
    # downstream of the last rounding point nothing can flip: fp32 against float64 arithmetic only
    assert np.abs(flat - my_flat).max() <= 2e-5 * np.abs(flat).max()
    assert np.abs(value - my_value).max() <= 2e-5 * float(arch["value_vmax"])
    # and the untaped oracle gives the same bits as the taped one (the recorder changes nothing)
    lg, v = nr.forward(sd, arch, obs, emulate=dtype)
    assert np.array_equal(v.double().numpy(), value)


@pytest.mark.parametrize("round_residual", [True, False])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_blocks_forward_emulate_walks_the_float64_restatement(dtype, round_residual):
    """nr.blocks_forward is the class oracle of the fused block-stack kernel; round_residual=False is the form for a
    kernel that carries the residual stream in fp32 registers: the same walk minus the two stream roundings per block."""
    arch, sd, _ = _fixture("notepolicy_geo")
    g = torch.Generator().manual_seed(21)
    B, T, d = 3, nr.N_LEAD + nr.N_SLOTS, arch["embed"]
    x = torch.randn(B, T, d, generator=g)
    bias = torch.cat([torch.zeros(B, nr.N_LEAD), ((torch.rand(B, nr.N_SLOTS, generator=g) < 0.6).float() - 1) * nr.MASK_BIAS], 1)
    tape = _Tape(dtype)
    orig = nr._round
    try:
        nr._round = tape.record
        lead, x_res = nr.blocks_forward(sd, arch, x, bias, emulate=dtype, round_residual=round_residual)
    finally:
        nr._round = orig
    P = {k: v.double().numpy() for k, v in sd.items()}
    x64 = tape.meet(x.double().numpy(), "tokens")
    my_lead, my_res, _ = _blocks_walk(P, arch, x64, bias.double().numpy(), tape.meet, round_residual)
    assert tape.i == len(tape.calls)
    assert np.array_equal(my_lead, lead.double().numpy()) and np.array_equal(my_res, x_res.double().numpy())


def test_notepolicy_walk_detects_a_missing_rounding_point():
    """Mutation check of the walk itself: an oracle that forgets any ONE of its roundings must fail it (except where
    the forgotten cast was a no-op: a value that is already on the 16-bit grid)."""
    arch, sd, obs = _fixture("notepolicy_geo")
    tape, _, _ = _np_taped_oracle(sd, arch, obs, "f16")
    n = len(tape.calls)
    noop = [bool(torch.equal(i, o)) for i, o in tape.calls]
    caught = 0
    tried = [c for c in range(n) if not noop[c]]
    for c in tried:
        t2, _, _ = _np_taped_oracle(sd, arch, obs, "f16", skip_call=c)
        try:
            _np_walk(sd, arch, obs, t2)
        except AssertionError:
            caught += 1
    print(f"\n{caught}/{len(tried)} single forgotten roundings caught ({n - len(tried)} casts were no-ops)")
    assert caught == len(tried) and len(tried) >= 0.8 * n


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_notepolicy_frontend_emulate_rounding_points(dtype):
    """The front end's 16-bit rule, bit for bit: the obs is rounded ONCE (python/policy.py:1200-1209), gathered lanes
    are copies of rounded lanes, the geometry is fp32 arithmetic on the rounded lanes with one rounding on store, the
    key bias is exact.  note_geo itself is pinned on the reference tests' hand cases (tests/test_oracle_notepolicy.py)."""
    g = torch.Generator().manual_seed(5)
    obs = torch.randn(4, nr.OBS_DIM, generator=g) * 0.7
    obs[:, nr.OFF_MASK:nr.OFF_MASK + nr.N_SLOTS] = (torch.rand(4, nr.N_SLOTS, generator=g) < 0.6).float()
    sab, torso, leg, note, bias = nr.frontend(obs, True, False, 8.0, emulate=dtype)
    o = torch.from_numpy(_cast(obs.double().numpy(), dtype)).float()
    assert torch.equal(sab[..., :47], torch.stack([o[:, nr.SABER_L], o[:, nr.SABER_R]], 1))
    assert torch.equal(torso, o[:, nr.TORSO]) and torch.equal(leg[..., :32], torch.stack([o[:, nr.LEG_L], o[:, nr.LEG_R]], 1))
    assert torch.equal(sab[..., 47:], torch.eye(2).expand(4, 2, 2)) and torch.equal(leg[..., 32:], torch.eye(2).expand(4, 2, 2))
    notes = o[:, nr.OFF_NOTES:nr.OFF_MASK].reshape(4, nr.N_SLOTS, nr.NOTE_FEAT)
    assert torch.equal(note[..., :18], notes)
    geo = nr.note_geo(notes, sab[..., :47], 8.0, False, o[:, nr.OBS_HEAD_Z])
    assert np.array_equal(note[..., 18:].double().numpy(), _cast(geo.double().numpy(), dtype))
    mask = o[:, nr.OFF_MASK:nr.OFF_MASK + nr.N_SLOTS]
    assert torch.equal(bias[:, :5], torch.zeros(4, 5)) and torch.equal(bias[:, 5:], (mask - 1) * 16384.0)
