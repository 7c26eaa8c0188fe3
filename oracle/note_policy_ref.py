"""TEST INFRASTRUCTURE - CPU oracle for the reference's NotePolicy forward.

The checker, never the product: only tests/, the smoke entry point and the
CPU-baseline leg of bench.py may import it.  A functional, plain-torch fp32
restatement of NotePolicy.forward_stacked from a state_dict and an arch record,
following the reference's fp32 record path:

  * obs lane routing           reference python/policy.py:174-275, 1099-1105
  * note-geometry lanes        reference python/policy.py:329-404
  * token encoders + order     reference python/policy.py:1224-1249
  * key bias                   reference python/policy.py:428, 1257-1260
  * blocks, final-block pruning reference python/policy.py:524-715 (`else` arms), 1267-1305
  * SimBa readout trunk        reference python/policy.py:1107-1138
  * SimBaV2 readout trunk      reference python/policy.py:1140-1155 (scalers :1003-1014)
  * value residual (a v + b v0) reference python/policy.py:568-611, 1264-1275; fp16_linear.py:1002-1006
  * packed heads + ragged fill reference python/policy.py:1311-1344, 430-434
  * adapool critic             reference python/policy.py:1346-1403

Pinned (tests/test_oracle_notepolicy.py) against tests/golden/notepolicy_*.npz, vectors
written by the reference module itself (tests/golden/make_notepolicy_golden.py), and
against the hand-computed note-geometry cases the reference's own tests hold
(python/tests/test_policy.py:141-183, test_i07_blade_geo.py:149-200 - restated there).
The value-residual mix and the SimBaV2 trunk are pinned by the notepolicy_vres_v2 vector and
by the reference's own properties (python/tests/test_arch_ab_options.py:131-139, 250-256:
(a, b) = (1, 0) is bitwise the plain policy; the SimBaV2 feature has RMS 1 per row).

`forward(..., emulate="f16")` restates the rounding points of the 16-bit stream (obs,
weights and every GEMM operand rounded, fp32 accumulate, fp32 LayerNorm / softmax /
geometry) for comparing a 16-bit kernel path against its own precision class.  Pinned by
tests/test_oracle_emulate.py: every cast the branch performs is recorded and a float64
restatement with explicit casts is walked along that record (same rounding points in the same
places, same arithmetic between them to fp32-accumulate precision); an oracle that forgets
any single rounding fails the walk; the value-residual and SimBaV2 options are walked too.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

OBS_DIM = 630
N_SLOTS, NOTE_FEAT = 24, 18
OFF_NOTES = 102
OFF_MASK = OFF_NOTES + N_SLOTS * NOTE_FEAT          # 534
N_HEADS_OUT = 29
MASK_BIAS = 16384.0
MASKED_LOGIT = -1e9
N_LEAD = 5
SABER_FEAT, TORSO_FEAT, LEG_FEAT = 47, 29, 32


def _r(*spans):
    out = []
    for lo, hi in spans:
        out += list(range(lo, hi))
    return out


# obs blocks after the slot mask: ground contact (4), body points (18), their velocities (18),
# previous-note L / R (5 + 5), torque-limit scales (16), blade-tip velocity L / R (3 + 3)
_GI = OFF_MASK + N_SLOTS            # 558
_BP = _GI + 4                       # 562
_BPV = _BP + 18                     # 580
_PREV_L = _BPV + 18                 # 598
_PREV_R = _PREV_L + 5               # 603
_TAU = _PREV_R + 5                  # 608
_TIP = _TAU + 16                    # 624
assert _TIP + 6 == OBS_DIM
_TAU_ARM = (_TAU + 3, _TAU + 10)
SABER_L = _r((18, 26), (49, 56), (75, 86), (_BP, _BP + 3), (_BPV, _BPV + 3), (_PREV_L, _PREV_L + 5), _TAU_ARM,
             (_TIP, _TIP + 3))
SABER_R = _r((26, 34), (56, 63), (86, 97), (_BP + 3, _BP + 6), (_BPV + 3, _BPV + 6), (_PREV_R, _PREV_R + 5),
             _TAU_ARM, (_TIP + 3, _TIP + 6))
TORSO = _r((0, 18), (46, 49), (97, 102), (_TAU, _TAU + 3))
_TAU_LEG = (_TAU + 10, _TAU + 16)
LEG_L = _r((34, 40), (63, 69), (_GI, _GI + 2), (_BP + 6, _BP + 9), (_BP + 12, _BP + 15), (_BPV + 6, _BPV + 9),
           (_BPV + 12, _BPV + 15), _TAU_LEG)
LEG_R = _r((40, 46), (69, 75), (_GI + 2, _GI + 4), (_BP + 9, _BP + 12), (_BP + 15, _BP + 18), (_BPV + 9, _BPV + 12),
           (_BPV + 15, _BPV + 18), _TAU_LEG)
assert len(SABER_L) == len(SABER_R) == SABER_FEAT and len(TORSO) == TORSO_FEAT and len(LEG_L) == len(LEG_R) == LEG_FEAT

X_NORM, Y_NORM, Z_SCALE, V_NORM, HANDLE_LEN = 1.0, 0.75, 8.0, 6.0, 0.16
OBS_HEAD_Z = 99
S_WPOS, S_WVEL, S_BLADE, S_TIPV = 15, 18, 21, 44


def note_geo(notes, sabers, z_asinh, flux, z_off):
    """(B,24,18) notes, (B,2,47) saber lanes, (B,) head z offset -> (B,24,22):
    [hand L (7), hand R (7), blade-frame L (4), blade-frame R (4)].
    Reference python/policy.py:329-404."""
    z_m = torch.sinh(notes[..., 2]) * z_asinh
    tx, ty = notes[..., 0], notes[..., 1]
    if flux:
        bar = notes[..., 9] > 0.5
        tx = torch.where(bar, notes[..., 12], tx)
        ty = torch.where(bar, notes[..., 13], ty)
    npos = torch.stack([tx * X_NORM, ty * Y_NORM, z_m], -1)
    cutd = torch.stack([notes[..., 6], notes[..., 7], torch.zeros_like(tx)], -1)
    not_wall = 1.0 - notes[..., 14:15]
    speed = (-notes[..., 3:4] * Z_SCALE).clamp_min(1e-3)
    zrel = z_m - (z_off * X_NORM)[:, None]
    tpl = (zrel[..., None] / speed).clamp(-0.5, 3.0) / 3.0
    first, second = [], []
    for h in range(2):
        w = sabers[:, h]
        wpos = torch.stack([w[:, S_WPOS] * X_NORM, w[:, S_WPOS + 1] * Y_NORM, w[:, S_WPOS + 2]], -1)
        dpm = npos - wpos[:, None]
        dp = dpm * 0.5
        dist = torch.asinh(dp.norm(dim=-1, keepdim=True) * 0.25)
        dp = torch.cat([dp[..., :2], torch.asinh(dp[..., 2:3] * 0.25)], -1)
        v = w[:, S_WVEL:S_WVEL + 3] * V_NORM
        vhat = v / (v.norm(dim=-1, keepdim=True) + 0.05)
        vdot = (vhat[:, None] * cutd).sum(-1, keepdim=True) * not_wall
        b = w[:, S_BLADE:S_BLADE + 3]
        bdot = (b[:, None] * cutd).sum(-1, keepdim=True) * not_wall
        first += [dp, dist, tpl, vdot, bdot]
        ab = (dpm * b[:, None]).sum(-1, keepdim=True)
        along = torch.asinh((ab - HANDLE_LEN) * 0.5)
        perp = torch.asinh((dpm - ab * b[:, None]).norm(dim=-1, keepdim=True) * 0.5)
        vt = w[:, S_TIPV:S_TIPV + 3]
        pn = torch.linalg.cross(b, vt * V_NORM)
        nhat = pn / (pn.norm(dim=-1, keepdim=True) + 0.05)
        cut = torch.asinh((dpm * nhat[:, None]).sum(-1, keepdim=True) * 0.5)
        vtdot = (vt[:, None] * cutd).sum(-1, keepdim=True) * not_wall
        second += [along, perp, cut, vtdot]
    return torch.cat(first + second, -1)


def _round(x, emulate):
    if emulate is None:
        return x
    return x.to({"f16": torch.float16, "bf16": torch.bfloat16}[emulate]).float()


class _Net:
    """state_dict accessors with the 16-bit rounding rule (weights rounded, biases / LN fp32)."""

    def __init__(self, sd, emulate):
        self.sd, self.em = sd, emulate

    def r(self, x):
        return _round(x, self.em)

    def lin(self, name, x):
        return F.linear(x, self.r(self.sd[name + ".weight"]), self.sd[name + ".bias"])

    def ln(self, name, x):
        w = self.sd[name + ".weight"]
        return F.layer_norm(x, (w.shape[0],), w, self.sd[name + ".bias"], 1e-5)

    def mlp2(self, name, x):
        """Linear - ReLU - Linear (an encoder or FFN Sequential [0, 2])."""
        return self.lin(name + ".2", self.r(F.relu(self.lin(name + ".0", x))))


def _attend(q, k, v, bias, n_heads, r):
    B, Tq, d = q.shape
    T = k.shape[1]
    dh = d // n_heads
    qh = q.view(B, Tq, n_heads, dh).transpose(1, 2)
    kh = k.view(B, T, n_heads, dh).transpose(1, 2)
    vh = v.view(B, T, n_heads, dh).transpose(1, 2)
    s = qh @ kh.transpose(-2, -1) / (dh ** 0.5) + bias.view(B, 1, 1, T)
    return (r(torch.softmax(s, -1)) @ vh).transpose(1, 2).reshape(B, Tq, d)


def _blocks(net, arch, x, bias, round_residual=True):
    """The block stack (reference python/policy.py:1262-1306, Block.forward :524-715): blocks
    0..L-2 over all T rows, the final block on the N_LEAD lead rows only.  Returns (lead (B,5,d),
    x_res (B,T,d) = the stream entering the final block).  round_residual=False keeps the
    residual stream unrounded between blocks (a kernel that carries it in fp32 registers)."""
    r = net.r
    rr = r if round_residual else (lambda t: t)
    H, L = arch["n_heads"], arch["n_blocks"]

    vres = bool(arch.get("value_residual", False))
    v0 = [None]

    def block(i, x, n_q):
        p = f"blocks.{i}."
        h = r(net.ln(p + "ln_attn", x))
        k, v = r(net.lin(p + "k_proj", h)), r(net.lin(p + "v_proj", h))
        if vres and i == 0:
            v0[0] = v                       # block 0 hands its values to every later block
        elif vres:
            v = r(v * net.sd[p + "vres_a"] + v0[0] * net.sd[p + "vres_b"])
        x_full = x
        if n_q:
            x, h = x[:, :n_q], h[:, :n_q]
        q = r(net.lin(p + "q_proj", h))
        att = r(_attend(q, k, v, bias, H, r))
        x = rr(x + net.lin(p + "out_proj", att))
        h2 = r(net.ln(p + "ln_ffn", x))
        x = rr(x + net.mlp2(p + "ffn", h2))
        return x, x_full

    for i in range(L - 1):
        x, _ = block(i, x, 0)
    lead, x_res = block(L - 1, x, N_LEAD)
    return r(lead), r(x_res)


@torch.no_grad()
def blocks_forward(sd, arch, x, bias, emulate=None, round_residual=True):
    """Public form of the block stack for kernel tests: x (B,T,d) tokens, bias (B,T) additive key bias."""
    return _blocks(_Net(sd, emulate), arch, _round(x.float(), emulate), bias.float(), round_residual)


@torch.no_grad()
def frontend(obs, note_geo_on=False, flux=False, z_asinh=8.0, emulate=None):
    """The forward's preamble on its own (reference python/policy.py:1199-1260): obs rounded once
    to the stream dtype, then (saber_in (B,2,49), torso_in (B,29), leg_in (B,2,34),
    note_in (B,24,18|40), key_bias (B,29)), every output rounded to the stream dtype."""
    r = lambda x: _round(x, emulate)
    B = obs.shape[0]
    obs = r(obs.float())
    sab = torch.stack([obs[:, SABER_L], obs[:, SABER_R]], 1)
    notes = obs[:, OFF_NOTES:OFF_MASK].reshape(B, N_SLOTS, NOTE_FEAT)
    mask = obs[:, OFF_MASK:OFF_MASK + N_SLOTS]
    if note_geo_on:
        notes = r(torch.cat([notes, note_geo(notes, sab, float(z_asinh), flux, obs[:, OBS_HEAD_Z])], -1))
    eye = torch.eye(2).expand(B, 2, 2)
    legs = torch.stack([obs[:, LEG_L], obs[:, LEG_R]], 1)
    bias = F.pad((mask - 1.0) * MASK_BIAS, (N_LEAD, 0))
    return torch.cat([sab, eye], -1), obs[:, TORSO], torch.cat([legs, eye], -1), notes, r(bias)


def _l2n(x):
    return x / x.norm(dim=-1, keepdim=True).clamp_min(1e-6)


def _trunk_v2(net, arch, z):
    """SimBaV2 readout (reference python/policy.py:1140-1155): x = l2n(s_in * W_in z);
    y = l2n(W2 relu(s_1 * W1 x)); x = l2n(x + alpha (y - x)); h = sqrt(D) x.  GEMM outputs are
    rounded to the stream dtype; scalers, ReLU, normalisations and the LERP stay fp32 and are
    rounded once before each GEMM and at the output.  Scaler factors (:1003-1014): s_in and s_1
    enter as they are, alpha times 0.5 * sqrt(D)."""
    r, sd = net.r, net.sd
    D = arch["trunk_dim"]
    x = _l2n(r(net.lin("trunk_in", z)) * sd["trunk_s_in"])
    u = F.relu(r(net.lin("trunk_w1", r(x))) * sd["trunk_s_1"])
    y = _l2n(r(net.lin("trunk_w2", r(u))))
    alpha = sd["trunk_alpha"] * (0.5 * math.sqrt(D))
    x = _l2n(x + alpha * (y - x))
    return r(x * math.sqrt(D))


@torch.no_grad()
def forward(sd, arch, obs, emulate=None, return_parts=False):
    """obs (B, 630) -> logits (B, 29, k_max) fp32, value (B,) fp32."""
    net = _Net(sd, emulate)
    r = net.r
    d, H = arch["embed"], arch["n_heads"]
    L = arch["n_blocks"]
    B = obs.shape[0]
    obs = r(obs.float())
    sab = torch.stack([obs[:, SABER_L], obs[:, SABER_R]], 1)                  # (B,2,47)
    notes = obs[:, OFF_NOTES:OFF_MASK].reshape(B, N_SLOTS, NOTE_FEAT)
    mask = obs[:, OFF_MASK:OFF_MASK + N_SLOTS]
    if arch.get("note_geo", False):
        geo = note_geo(notes, sab, float(arch["z_asinh"]), arch.get("game", "standard") == "flux", obs[:, OBS_HEAD_Z])
        notes = r(torch.cat([notes, geo], -1))
    eye = torch.eye(2).expand(B, 2, 2)
    tok_saber = net.mlp2("saber_mlp", torch.cat([sab, eye], -1))
    tok_torso = net.mlp2("torso_mlp", obs[:, TORSO]).unsqueeze(1)
    legs = torch.stack([obs[:, LEG_L], obs[:, LEG_R]], 1)
    tok_leg = net.mlp2("leg_mlp", torch.cat([legs, eye], -1))
    tok_note = net.mlp2("note_mlp", notes)
    x = r(torch.cat([tok_saber, tok_torso, tok_leg, tok_note], 1))            # (B,29,d)
    bias = F.pad((mask - 1.0) * MASK_BIAS, (N_LEAD, 0))                        # (B,29)
    if arch.get("emb_ln", False):
        x = r(net.ln("emb_ln", x))

    lead, x_res = _blocks(net, arch, x, bias)
    if arch.get("final_ln", False):
        lead = r(net.ln("final_ln", lead))
    if arch.get("trunk_arch", "simba") == "simbav2":
        h = _trunk_v2(net, arch, lead.reshape(B, N_LEAD * d))
    else:
        # SimBa readout trunk
        t = r(net.lin("trunk_proj", lead.reshape(B, N_LEAD * d)))
        u = r(net.ln("trunk_ln1", t))
        dlt = net.lin("trunk_fc2", r(F.relu(net.lin("trunk_fc1", u))))
        h = r(net.ln("trunk_ln2", r(t + dlt)))
    # packed heads
    sizes = arch.get("head_gears") or [arch["n_gears"]] * N_HEADS_OUT
    w = torch.cat([sd[f"heads.{j}.weight"] for j in range(N_HEADS_OUT)])
    b = torch.cat([sd[f"heads.{j}.bias"] for j in range(N_HEADS_OUT)])
    flat = F.linear(h, r(w), b)
    kmax = max(sizes)
    logits = torch.full((B, N_HEADS_OUT, kmax), MASKED_LOGIT)
    o = 0
    for j, n in enumerate(sizes):
        logits[:, j, :n] = flat[:, o:o + n]
        o += n
    # adapool critic
    hv = r(net.ln("critic_ln", x_res))
    q = r(net.lin("critic_q", hv[:, 2:3]))
    k, v = r(net.lin("critic_k", hv)), r(net.lin("critic_v", hv))
    a = r(_attend(q, k, v, bias, H, r)).reshape(B, d)
    a = r(net.lin("critic_out", a))
    z = torch.cat([a, h], -1)
    z = r(F.relu(net.lin("critic_mlp.0", z)))
    z = r(F.relu(net.lin("critic_mlp.2", z)))
    vlog = net.lin("critic_mlp.4", z)
    centers = torch.linspace(-float(arch["value_vmax"]), float(arch["value_vmax"]), int(arch["value_bins"]))
    value = torch.softmax(vlog, -1) @ centers
    if return_parts:
        return logits, value, {"tokens": x, "x_res": x_res, "lead": lead, "h": h, "value_logits": vlog, "critic_a": a}
    return logits, value


def load_fixture(path):
    """(arch, state_dict, obs, logits, value) from a tests/golden/notepolicy_*.npz file."""
    import json
    import numpy as np
    z = np.load(path)
    arch = json.loads(bytes(z["arch_json"]).decode())
    keys = json.loads(bytes(z["sd_keys_json"]).decode())
    sd = {k: torch.from_numpy(z["sd." + k]) for k in keys}
    return arch, sd, torch.from_numpy(z["obs"]), torch.from_numpy(z["logits"]), torch.from_numpy(z["value"])


def flops_per_env(arch) -> int:
    """Executed FLOPs per env of the reference forward (final block pruned to the 5 lead tokens)."""
    d, D, L, T = arch["embed"], arch["trunk_dim"], arch["n_blocks"], N_LEAD + N_SLOTS
    Fh = arch["ffn_mult"] * d
    Hd = arch.get("trunk_hidden") or D
    note_in = NOTE_FEAT + (22 if arch.get("note_geo") else 0)
    enc = N_SLOTS * (note_in * d + d * d) + 2 * ((SABER_FEAT + 2) * d + d * d) + (TORSO_FEAT * d + d * d) \
        + 2 * ((LEG_FEAT + 2) * d + d * d)
    full = 3 * T * d * d + 2 * T * T * d + T * d * d + 2 * T * d * Fh
    last = 2 * T * d * d + N_LEAD * d * d + 2 * N_LEAD * T * d + N_LEAD * d * d + 2 * N_LEAD * d * Fh
    sizes = arch.get("head_gears") or [arch["n_gears"]] * N_HEADS_OUT
    trunk = N_LEAD * d * D + 2 * D * Hd + D * sum(sizes)
    critic = d * d + 2 * T * d * d + 2 * T * d + d * d + (d + D) * D + D * D + D * int(arch["value_bins"])
    return 2 * (enc + (L - 1) * full + last + trunk + critic)
