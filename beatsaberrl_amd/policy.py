"""NotePolicy on the HIP kernels: a drop-in for the reference's policy module (forward).

Same constructor arguments, parameter names / shapes / registration order (hence the
same state_dict and checkpoints) and the same `forward_stacked(obs) -> (logits
(B, 29, k_max) fp32, value (B,) fp32)` contract as the reference (python/policy.py:
784-1097 ctor, :1179-1344 forward, :1346-1403 critic).  What runs where:

  * on the C-ABI kernels: every Linear (token encoders, packed q|k|v, output
    projections with the residual add in the epilogue, FFNs - fused with the next
    block's LayerNorm when `fused_ffn` is on -, SimBa trunk, packed heads, critic
    projections and MLP), every LayerNorm, every attention (blocks, the final block's
    5 lead queries, the critic's single query), the forward's preamble (obs rounding,
    lane gathers, the 22 note-geometry lanes, one-hots, key bias: one front-end kernel)
    and the action epilogue (log-softmax, Gumbel-max sampling, log-prob, entropy: one
    kernel);
  * in torch on the GPU (pure data movement): token concatenation, the ragged-head
    scatter and the 101-bin value expectation.

Grad mode selects the path, as in the reference: under torch.no_grad() (rollout, evaluation) the
forward-only routes above run; with grad mode on (the update), `forward_stacked` /
`get_action_and_value(obs, action)` run op for op the per-op route as autograd Functions over the
backward kernels (autograd_ops.py: LayerNorm, Linear data / weight / bias gradients, attention),
so parameters receive fp32 gradients and the update forward is bitwise the per-op rollout forward
(`fused_ffn` off; with it on, the block FFNs of the update run forward as the fused kernel and
recompute their hidden in the backward - less activation memory, one more GEMM per block).

Stream dtype: `policy.fp16 = True` runs the 16-bit stream (fp16; set `stream_dtype =
torch.bfloat16` for bf16) exactly as the reference's switch does (python/policy.py:
1085-1090); otherwise fp32 kernels.  There is no CPU path and no torch fallback for
the kernel ops.  Architecture options: emb_ln, final_ln, ragged per-joint heads, the
value-residual mix (per-op route; its row kernel mixes inside the packed q|k|v buffer)
and the SimBaV2 trunk (three GEMMs + three fp32 row kernels)."""
from __future__ import annotations

import contextlib
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import fp16_linear as _fl
from . import obs_layout as L
from . import ops
from .autograd_ops import AttnPackedFn, AttnQKVFn, ChainFn, FusedFfnFn, LinearFn, LnResFn
from .fused_ln import FusedLayerNorm

OBS_DIM = L.OBS_DIM
N_NOTE_SLOTS = L.N_NOTE_SLOTS
NOTE_FEAT = L.NOTE_FEAT
OFF_NOTES = L.OFF_NOTES
OFF_NOTE_MASK = L.OFF_NOTE_MASK
SABER_FEAT, TORSO_FEAT, LEG_FEAT = L.SABER_FEAT, L.TORSO_FEAT, L.LEG_FEAT
NOTE_GEO_FEAT = L.NOTE_GEO_FEAT
N_ACTION_HEADS = L.N_ACTION_HEADS
MASK_BIAS = L.MASK_BIAS
MASKED_LOGIT = L.MASKED_LOGIT
TRUNK_ARCHS = ("simba", "simbav2")


_SIDE_STREAMS = {}      # device index -> the forward's second stream


def _mlp(sizes, act=nn.ReLU):
    layers = []
    for i in range(len(sizes) - 1):
        layers.append(nn.Linear(sizes[i], sizes[i + 1]))
        if i < len(sizes) - 2:
            layers.append(act())
    return nn.Sequential(*layers)


def _lin(m: nn.Linear, x, act=None, residual=None, out=None):
    """A Linear on the kernels in x's dtype (fp32 master weights, 16-bit replica when needed)."""
    return ops.linear(x, _fl._replica(m.weight, x.dtype), _fl._bias32(m.bias), act=act, residual=residual, out=out)


def _seq(seq: nn.Sequential, x, out=None):
    """Linear (ReLU Linear)* with each ReLU in its producer's epilogue (reference
    python/policy.py:76-145, `_seq` / `_run`).  out: a (N, G, M) slice of the token stream that
    receives the last Linear's rows directly.  x may be wider than the first Linear's input (rows
    zero-padded by the producer): the first weight's columns are then padded to match."""
    ms = list(seq)
    if (len(ms) == 3 and isinstance(ms[0], nn.Linear) and isinstance(ms[1], nn.ReLU) and isinstance(ms[2], nn.Linear)
            and x.shape[-1] >= ms[0].in_features and ms[0].bias is not None and ms[2].bias is not None
            and ops.mlp2_supported(x.shape[-1], ms[2].out_features, x.dtype) and ms[0].out_features == ms[2].in_features == ms[2].out_features):
        # Linear ReLU Linear on a 64-lane input: one launch, the hidden rows never written (same bits as the two below)
        w1 = _fl._replica_padded(ms[0].weight, x.dtype, x.shape[-1]) if x.shape[-1] != ms[0].in_features else _fl._replica(ms[0].weight, x.dtype)
        y = ops.mlp2(x.contiguous(), w1, _fl._bias32(ms[0].bias), _fl._replica(ms[2].weight, x.dtype), _fl._bias32(ms[2].bias), out=out)
        if y is not None:
            return y
    i = 0
    while i < len(ms):
        m = ms[i]
        if not isinstance(m, nn.Linear):
            raise RuntimeError(f"unsupported module in Sequential: {type(m).__name__}")
        relu = i + 1 < len(ms) and isinstance(ms[i + 1], nn.ReLU)
        last = i + (2 if relu else 1) >= len(ms)
        if x.shape[-1] != m.in_features:
            if i or x.shape[-1] < m.in_features or x.dtype is torch.float32:
                raise RuntimeError(f"_seq: input has {x.shape[-1]} lanes, the Linear takes {m.in_features}")
            x = ops.linear(x, _fl._replica_padded(m.weight, x.dtype, x.shape[-1]), _fl._bias32(m.bias),
                           act="relu" if relu else None, out=out if last else None)
        else:
            x = _lin(m, x, act="relu" if relu else None, out=out if last else None)
        i += 2 if relu else 1
    return x


def _lin_t(m: nn.Linear, x, act=None, residual=None, out_f32=False):
    """_lin under autograd: forward on the same kernel, backward on the gradient kernels."""
    return LinearFn.apply(x, m.weight, m.bias, act, residual, out_f32)


def _seq_t(seq: nn.Sequential, x, residual=None, out_f32=False):
    """_seq under autograd: the whole Linear (ReLU Linear)* chain as one Function."""
    lins = [m for m in seq if isinstance(m, nn.Linear)]
    if len(lins) != (len(seq) + 1) // 2 or not all(isinstance(m, nn.ReLU) for m in list(seq)[1::2]):
        raise RuntimeError("training path: Sequential must be Linear (ReLU Linear)*")
    return ChainFn.apply(x, residual, out_f32, *[t for m in lins for t in (m.weight, m.bias)])


def _packed_t(ms, x):
    """Several same-input Linears as one GEMM under autograd: the concatenation is a torch op, so each
    master receives its row block of the packed gradient (reference python/fp16_linear.py:459-470)."""
    return LinearFn.apply(x, torch.cat([m.weight for m in ms]), torch.cat([m.bias for m in ms]), None, None, False)


def note_geo(notes, sabers, z_asinh, flux, z_off):
    """The 22 hand-relative geometry lanes per entity slot, fp32 (reference
    python/policy.py:329-404): per hand [dp x, dp y (half-metres), asinh(dp z / 8),
    asinh(|dp| / 8), seconds-to-plane / 3, v.d, b.d], then per hand the blade-frame
    block [along, perp, cut (asinh(m / 2)), vt.d]."""
    z_m = torch.sinh(notes[..., 2]) * float(z_asinh)
    tx, ty = notes[..., 0], notes[..., 1]
    if flux:
        bar = notes[..., 9] > 0.5
        tx, ty = torch.where(bar, notes[..., 12], tx), torch.where(bar, notes[..., 13], ty)
    npos = torch.stack([tx * L.X_NORM, ty * L.Y_NORM, z_m], -1)
    cutd = torch.stack([notes[..., 6], notes[..., 7], torch.zeros_like(tx)], -1)
    not_wall = 1.0 - notes[..., 14:15]
    speed = (-notes[..., 3:4] * L.Z_SCALE).clamp_min(1e-3)
    tpl = ((z_m - (z_off * L.X_NORM)[:, None])[..., None] / speed).clamp(-0.5, 3.0) / 3.0
    base, blade = [], []
    for hand in range(2):
        w = sabers[:, hand]
        wpos = torch.stack([w[:, L.S_WPOS] * L.X_NORM, w[:, L.S_WPOS + 1] * L.Y_NORM, w[:, L.S_WPOS + 2]], -1)
        dpm = npos - wpos[:, None]
        dp = dpm * 0.5
        dist = torch.asinh(dp.norm(dim=-1, keepdim=True) * 0.25)
        dp = torch.cat([dp[..., :2], torch.asinh(dp[..., 2:3] * 0.25)], -1)
        v = w[:, L.S_WVEL:L.S_WVEL + 3] * L.V_NORM
        vhat = v / (v.norm(dim=-1, keepdim=True) + 0.05)
        b = w[:, L.S_BLADE:L.S_BLADE + 3]
        base += [dp, dist, tpl, (vhat[:, None] * cutd).sum(-1, keepdim=True) * not_wall,
                 (b[:, None] * cutd).sum(-1, keepdim=True) * not_wall]
        ab = (dpm * b[:, None]).sum(-1, keepdim=True)
        vt = w[:, L.S_TIPV:L.S_TIPV + 3]
        pn = torch.linalg.cross(b, vt * L.V_NORM)
        nhat = pn / (pn.norm(dim=-1, keepdim=True) + 0.05)
        blade += [torch.asinh((ab - L.HANDLE_LEN) * 0.5),
                  torch.asinh((dpm - ab * b[:, None]).norm(dim=-1, keepdim=True) * 0.5),
                  torch.asinh((dpm * nhat[:, None]).sum(-1, keepdim=True) * 0.5),
                  (vt[:, None] * cutd).sum(-1, keepdim=True) * not_wall]
    return torch.cat(base + blade, -1)


def hl_target(v, centers, sigma: float):
    """HL-Gauss target (reference python/policy.py:759-773): the mass of N(v, sigma^2) inside each of the K
    equally spaced histogram bins, v clamped into the support, rows renormalised to 1.  v (B,) -> (B, K)."""
    v = v.float()
    width = centers[1] - centers[0]
    edges = torch.cat([centers[:1] - 0.5 * width, centers + 0.5 * width])
    v = v.clamp(edges[0], edges[-1])
    cdf = 0.5 * (1.0 + torch.erf((edges.unsqueeze(0) - v.unsqueeze(1)) / (sigma * math.sqrt(2.0))))
    p = cdf[:, 1:] - cdf[:, :-1]
    return p / p.sum(-1, keepdim=True)


def hl_loss(logits, v_tgt, centers, sigma: float):
    """Cross-entropy between the critic's bin distribution and the HL-Gauss target, batch mean
    (reference python/policy.py:776-781); logits (B, K) fp32 = `policy._value_logits` of the update forward."""
    return -(hl_target(v_tgt, centers, sigma) * F.log_softmax(logits.float(), dim=-1)).sum(-1).mean()


class Block(nn.Module):
    """Pre-LN transformer block; parameters as the reference's Block
    (python/policy.py:492-522): ln_attn, q/k/v/out_proj, ln_ffn, ffn.{0,2}."""

    def __init__(self, d: int, n_heads: int = 4, ffn_mult: int = 4, value_residual: bool = False):
        super().__init__()
        if n_heads < 2 or d % n_heads:
            raise ValueError(f"embed {d} must split into >= 2 heads, got n_heads={n_heads}")
        # value residual (python/policy.py:511-522): v <- a v + b v0 with block 0's values v0;
        # (a, b) = (1, 0) at init is bitwise the plain block
        if value_residual:
            self.vres_a = nn.Parameter(torch.ones(1))
            self.vres_b = nn.Parameter(torch.zeros(1))
        else:
            self.vres_a = self.vres_b = None
        self.ln_attn = FusedLayerNorm(d)
        self.q_proj = nn.Linear(d, d)
        self.k_proj = nn.Linear(d, d)
        self.v_proj = nn.Linear(d, d)
        self.out_proj = nn.Linear(d, d)
        self.ln_ffn = FusedLayerNorm(d)
        self.ffn = _mlp([d, ffn_mult * d, d])
        self.d, self.n_heads, self.dh = d, n_heads, d // n_heads

    def forward(self, x, attn_bias, h=None, n_queries=0, next_ln=None, v0=None, want_v=False):
        """x (B, T, d); attn_bias (B, T) additive key bias; h = ln_attn(x) if the
        previous block's fused FFN already produced it.  n_queries > 0 computes only
        the first n_queries rows (keys / values still span all T): exact, masking is
        key-side only (reference python/policy.py:533-539).  v0: block 0's attention
        values, mixed into this block's (a v + b v0, python/policy.py:568-611) before the
        attention.  Returns (x_out, h_next) with h_next = next_ln(x_out) when the fused FFN
        produced it, else None; with want_v (block 0 of a value-residual stack) a third element,
        this block's values as a view of its packed projection."""
        d = self.d
        if h is None:
            h = self.ln_attn(x)
        if n_queries:
            wkv, bkv = _fl.packed_halves([self.k_proj, self.v_proj], x.dtype)
            kv = ops.linear(h, wkv, bkv)                                   # (B, T, 2d)
            v = kv[..., d:]
            if v0 is not None:
                ops.vres_mix(v, v0, self.vres_a, self.vres_b)              # in place in the packed buffer
            hq = h[:, :n_queries]
            q = _lin(self.q_proj, hq)                                      # (B, nq, d)
            att = ops.attn_fwd(q, kv[..., :d], kv[..., d:], self.n_heads, key_bias=attn_bias)
            x = x[:, :n_queries].contiguous()
        else:
            wqkv, bqkv = _fl.packed_halves([self.q_proj, self.k_proj, self.v_proj], x.dtype)
            qkv = ops.linear(h, wqkv, bqkv)                                # (B, T, 3d)
            v = qkv[..., 2 * d:]
            if v0 is not None:
                ops.vres_mix(v, v0, self.vres_a, self.vres_b)
            att = ops.attn_fwd(qkv[..., :d], qkv[..., d:2 * d], qkv[..., 2 * d:], self.n_heads, key_bias=attn_bias)
        x = _lin(self.out_proj, att, residual=x)                           # x + out(att), one rounding
        h2 = self.ln_ffn(x)
        if _fl.fused_ffn_ok(x, self.ffn, next_ln):
            r = _fl.fused_ffn(x, h2, self.ffn, next_ln)
            r = (r, None) if next_ln is None else tuple(r)
        else:
            hid = _lin(self.ffn[0], h2, act="relu")
            r = (_lin(self.ffn[2], hid, residual=x), None)
        return r + (v,) if want_v else r


class _ValuesOf(torch.autograd.Function):
    """forward: `values`, bit for bit; backward: the incoming gradient goes to `graph` (same shape), the tensor whose
    autograd graph stands in for the way `values` were computed."""

    @staticmethod
    def forward(ctx, graph, values):
        return values.detach().clone()

    @staticmethod
    def backward(ctx, g):
        return g, None


def _block_train(self, x, attn_bias, n_queries=0, v0=None, want_v=False, fused_ffn=False):
    """Block.forward under autograd (update path): the same kernels in the same order as the per-op
    rollout route without the fused FFN, each paired with its backward; returns x_out (, v).
    fused_ffn: the FFN's forward as the fused kernel (reference python/fp16_linear.py:1197-1275; its
    bits are the fused rollout route's, not the unfused chain's)."""
    d = self.d
    # each LayerNorm hands the stream back with it: the residual branch's gradient joins LN's inside ln_bwd
    x, h = LnResFn.apply(x.contiguous(), self.ln_attn.weight, self.ln_attn.bias, self.ln_attn.eps)
    if n_queries:
        kv = _packed_t([self.k_proj, self.v_proj], h)
        v = kv[..., d:]
        if v0 is not None:
            kv = torch.cat([kv[..., :d], torch.addcmul(v * self.vres_a, v0, self.vres_b).to(v.dtype)], -1)
        q = _lin_t(self.q_proj, h[:, :n_queries])
        att = AttnQKVFn.apply(q, kv, attn_bias, self.n_heads)
        x = x[:, :n_queries].contiguous()
    else:
        qkv = _packed_t([self.q_proj, self.k_proj, self.v_proj], h)
        v = qkv[..., 2 * d:]
        if v0 is not None:
            qkv = torch.cat([qkv[..., :2 * d], torch.addcmul(v * self.vres_a, v0, self.vres_b).to(v.dtype)], -1)
        att = AttnPackedFn.apply(qkv, attn_bias, self.n_heads)
    x = _lin_t(self.out_proj, att, residual=x)
    x, h2 = LnResFn.apply(x, self.ln_ffn.weight, self.ln_ffn.bias, self.ln_ffn.eps)
    if fused_ffn:
        x = FusedFfnFn.apply(x, h2, self.ffn[0].weight, self.ffn[0].bias, self.ffn[2].weight, self.ffn[2].bias,
                             fused_ffn != "recompute")
    else:
        x = _seq_t(self.ffn, h2, residual=x)
    return (x, v) if want_v else x


Block.forward_train = _block_train


def build_head_gears(n_gears: int) -> tuple:
    """Per-joint gear counts of this build: uniform (the reference falls back to the
    same when its env constants are not importable, python/policy.py:1555-1564)."""
    return (n_gears,) * N_ACTION_HEADS


class NotePolicy(nn.Module):
    def __init__(self, embed: int = 128, trunk_dim: int = 256, encoder: str = "transformer", n_blocks: int = 3,
                 n_heads: int = 4, n_gears: int = 3, ffn_mult: int = 4, note_geo: bool = False,
                 value_bins: int = 101, value_vmax: float = 6.0, value_sigma: float = 0.75,
                 trunk_hidden: int | None = None, z_asinh: float = 8.0, game: str = "standard",
                 fp16_accum: str = "off", fused_ffn: str = "off", emb_ln: bool = False,
                 value_residual: bool = False, final_ln: bool = False, trunk_arch: str = "simba",
                 head_gears: tuple | list | None = None):
        super().__init__()
        if trunk_arch not in TRUNK_ARCHS:
            raise ValueError(f"trunk_arch must be one of {TRUNK_ARCHS}, got {trunk_arch!r}")
        if game not in ("standard", "flux"):
            raise ValueError(f"game must be 'standard' or 'flux', got {game!r}")
        if not float(z_asinh) > 0:
            raise ValueError(f"z_asinh must be > 0 (metres), got {z_asinh}")
        if fp16_accum not in _fl.ACCUM_MODES:
            raise ValueError(f"fp16_accum must be one of {_fl.ACCUM_MODES}, got {fp16_accum!r}")
        if fused_ffn not in _fl.FFN_MODES:
            raise ValueError(f"fused_ffn must be one of {_fl.FFN_MODES}, got {fused_ffn!r}")
        if encoder != "transformer":
            raise ValueError(f"unknown encoder: {encoder}")
        if n_gears not in (3, 5, 7):
            raise ValueError(f"n_gears must be 3/5/7, got {n_gears}")
        if value_bins <= 1:
            raise ValueError(f"value_bins must be > 1, got {value_bins}")
        self.encoder, self.embed, self.n_heads, self.n_gears = encoder, embed, n_heads, n_gears
        head_gears = tuple(int(k) for k in (head_gears if head_gears is not None else build_head_gears(n_gears)))
        if len(head_gears) != N_ACTION_HEADS or not all(3 <= k <= 7 for k in head_gears):
            raise ValueError(f"head_gears must be {N_ACTION_HEADS} counts in [3, 7], got {head_gears}")
        self.head_sizes = head_gears
        self.k_max = max(head_gears)
        H = int(trunk_hidden) if trunk_hidden else trunk_dim
        # arch record, key for key the reference's (python/policy.py:857-928)
        self.arch = {"embed": embed, "trunk_dim": trunk_dim, "n_blocks": n_blocks, "n_heads": n_heads,
                     "n_gears": n_gears, "obs_dim": OBS_DIM, "ffn_mult": ffn_mult, "critic": "adapool_v1",
                     "n_action_heads": N_ACTION_HEADS, "body_token": True, "body_tokens": 3,
                     "note_geo": bool(note_geo), "note_geo_norm": True, "blade_geo": 1, "z_asinh": float(z_asinh),
                     "trunk_arch": trunk_arch, "trunk_hidden": H, "value_bins": int(value_bins),
                     "value_vmax": float(value_vmax), "value_sigma": float(value_sigma), "game": game,
                     "fp16_accum": fp16_accum, "fused_ffn": fused_ffn, "emb_ln": bool(emb_ln),
                     "value_residual": bool(value_residual), "final_ln": bool(final_ln)}
        if head_gears != (n_gears,) * N_ACTION_HEADS:
            self.arch["head_gears"] = list(head_gears)
        self.value_bins = int(value_bins)
        self.value_sigma_bins = float(value_sigma)
        centers = torch.linspace(-float(value_vmax), float(value_vmax), self.value_bins)
        self.register_buffer("value_centers", centers, persistent=False)
        self.value_sigma = float(value_sigma) * float(centers[1] - centers[0])
        self.note_geo, self.z_asinh, self.game = bool(note_geo), float(z_asinh), game
        # parameter registration order == the reference's (state_dict layout contract)
        self.note_mlp = _mlp([NOTE_FEAT + (NOTE_GEO_FEAT if note_geo else 0), embed, embed])
        self.saber_mlp = _mlp([SABER_FEAT + 2, embed, embed])
        self.body_tokens, self.n_lead = 3, L.N_LEAD
        self.torso_mlp = _mlp([TORSO_FEAT, embed, embed])
        self.leg_mlp = _mlp([LEG_FEAT + 2, embed, embed])
        self.value_residual = bool(value_residual)
        self.emb_ln = FusedLayerNorm(embed) if emb_ln else None
        self.blocks = nn.ModuleList(Block(embed, n_heads, ffn_mult, value_residual=self.value_residual and i > 0)
                                    for i in range(n_blocks))
        self.final_ln = FusedLayerNorm(embed) if final_ln else None
        self.trunk_arch = trunk_arch
        if trunk_arch == "simba":
            self.trunk_proj = nn.Linear(self.n_lead * embed, trunk_dim)
            self.trunk_ln1 = FusedLayerNorm(trunk_dim)
            self.trunk_fc1 = nn.Linear(trunk_dim, H)
            self.trunk_fc2 = nn.Linear(H, trunk_dim)
            self.trunk_ln2 = FusedLayerNorm(trunk_dim)
        else:
            # SimBaV2 readout (python/policy.py:990-1014): three bias-free (zero, frozen bias)
            # Linears with unit-norm rows and orthogonal init, per-lane scalers s_in / s_1 at
            # sqrt(2 / width) and the LERP rate alpha at 0.5 (stored as alpha / (0.5 sqrt(D)))
            D = trunk_dim
            self.trunk_in = nn.Linear(self.n_lead * embed, D)
            self.trunk_w1 = nn.Linear(D, H)
            self.trunk_w2 = nn.Linear(H, D)
            for lin in (self.trunk_in, self.trunk_w1, self.trunk_w2):
                nn.init.orthogonal_(lin.weight)
                nn.init.zeros_(lin.bias)
                lin.bias.requires_grad_(False)
            self._v2_c_in = self._v2_c_1 = 1.0
            self.trunk_s_in = nn.Parameter(torch.full((D,), math.sqrt(2.0 / D)))
            self.trunk_s_1 = nn.Parameter(torch.full((H,), math.sqrt(2.0 / H)))
            a_init, a_scale = 0.5, 1.0 / math.sqrt(D)
            self._v2_c_alpha = a_init / a_scale
            self.trunk_alpha = nn.Parameter(torch.full((D,), a_scale))
            self.project_trunk_weights()
        self.heads = nn.ModuleList(nn.Linear(trunk_dim, n) for n in self.head_sizes)
        if min(self.head_sizes) < self.k_max:
            self.register_buffer("_gear_valid", torch.tensor([[a < k for a in range(self.k_max)]
                                                              for k in self.head_sizes]), persistent=False)
            self.register_buffer("_gear_idx", torch.tensor([j * self.k_max + a for j, k in enumerate(self.head_sizes)
                                                            for a in range(k)], dtype=torch.long), persistent=False)
        else:
            self._gear_valid = self._gear_idx = None
        self.critic_ln = FusedLayerNorm(embed)
        self.critic_q = nn.Linear(embed, embed)
        self.critic_k = nn.Linear(embed, embed)
        self.critic_v = nn.Linear(embed, embed)
        self.critic_out = nn.Linear(embed, embed)
        self.critic_mlp = _mlp([embed + trunk_dim, trunk_dim, trunk_dim, self.value_bins])
        self.register_buffer("_saber_idx", torch.tensor(L.SABER_L_IDX + L.SABER_R_IDX, dtype=torch.long),
                             persistent=False)
        self.register_buffer("_body_idx", torch.tensor(L.BODY3_IDX, dtype=torch.long), persistent=False)
        self.register_buffer("_hand_id", torch.eye(2), persistent=False)
        # int32 copies of the lane tables and the per-head gear counts for the kernels
        self.register_buffer("_saber_idx32", self._saber_idx.to(torch.int32), persistent=False)
        self.register_buffer("_body_idx32", self._body_idx.to(torch.int32), persistent=False)
        self.register_buffer("_head_sizes32", torch.tensor(self.head_sizes, dtype=torch.int32), persistent=False)
        self.sampler = "kernel"                 # "kernel": in-kernel Philox stream; "torch": torch's generator
        # "auto": the 16-bit stream runs the whole block stack as one persistent kernel when the
        # shape has one (ops.blocks_pack_size > 0); "off": always the per-op launch train
        self.fused_blocks = "auto"
        self._blocks_image = None               # [weights version, dtype, uint8 image]
        # True: the critic's one-query attention runs as a pool over LN(x_res) with the k | v projections folded
        # around it (no (B T, 2d) keys / values); False: the reference's op order
        self.critic_pool = True
        # batches from this size on run the critic's attention pool on a second stream beside the trunk and heads (smaller
        # ones are launch-bound on the host, where the fork and join only add calls)
        self.critic_overlap_min_batch = 2048
        self._critic_pool_cache = None
        # The reference keeps the grad-free rollout forward and the grad-mode update forward bit-identical
        # (python/tests/test_fp16_accum.py:146-160): PPO's first-epoch ratio is then exactly 1.  The two fast rollout
        # routes above (fused block stack: fp32 residual in registers; pooled critic: k / v never rounded) differ from
        # the update forward, which is the per-op route, by 16-bit rounding (log-prob of a 29-head action to ~1e-2,
        # value to ~2e-4 at the recipe shape).  True: the rollout takes the per-op route and the reference's critic op
        # order whatever the two switches say - same bits as the update forward, at the per-op route's speed.
        self.rollout_matches_update = False
        # The same contract from the other side, at the fast routes' rollout speed: "rollout" = the update forward
        # RETURNS the rollout forward's logits and value - it runs that forward too, grad-free, on the routes the
        # rollout takes - and sends their gradients through its own per-op graph (a function that differs from the
        # rollout's by 16-bit rounding, as any two 16-bit evaluations do).  Rollout and update outputs are then the
        # same bits in every mode and PPO's first-epoch ratio is exactly 1, for one more (fused, ~3 ms at the recipe
        # shape and 16384 envs) forward per update pass.  "own": the update returns its own per-op values (the gap
        # bounded in the tests).  No effect on the fp32 stream, whose two forwards are the same ops.
        self.update_values = "rollout"
        # sampling-call counter of the in-kernel Philox stream; on the device so that a captured
        # get_action_and_value draws fresh noise on every replay
        self.register_buffer("_sample_ctr", torch.zeros(1, dtype=torch.int64), persistent=False)
        self.fp16 = False                       # True: 16-bit stream (python/policy.py:1085-1090)
        self.stream_dtype = torch.float16       # the 16-bit type used when fp16 is on
        self.fp16_accum = fp16_accum
        self.fused_ffn = fused_ffn
        self.upgraded_from = None
        self._value_logits = None
        self._ent_h = None

    # ---- weights ---------------------------------------------------------------------
    def flatten_fp16(self):
        """The reference repacks every master into one flat buffer here
        (python/policy.py:1405-1423); this build keeps per-tensor replicas that are
        recast in place per weights version, so only the replicas are (re)built."""
        self.refresh_fp16_caches()

    def _blocks_desc(self, dt):
        b0 = self.blocks[0]
        act = "gelu" if isinstance(b0.ffn[1], nn.GELU) else "relu"
        return dict(d=self.embed, n_heads=self.n_heads, ffn=b0.ffn[0].out_features, T=self.n_lead + N_NOTE_SLOTS,
                    act=act, n_queries=self.n_lead, dtype=dt)

    def fused_blocks_ok(self, dt) -> bool:
        """True when the block stack of this architecture has a fused kernel in dtype dt."""
        if self.fused_blocks == "off" or self.rollout_matches_update or dt is torch.float32 or self.value_residual:
            return False                    # the value-residual mix has no place in the fused stack
        if self.fused_blocks != "auto":
            raise ValueError(f"fused_blocks must be 'auto' or 'off', got {self.fused_blocks!r}")
        return ops.blocks_pack_size(len(self.blocks), **self._blocks_desc(dt)) > 0

    def blocks_image(self, dt):
        """The fused block stack's weight image for the current weights version: rebuilt IN PLACE
        (one cast + permute launch pair) when `bump_weights_version` has been called, so its
        address is stable under a captured graph - the contract of the reference's flat replica
        buffer (python/fp16_linear.py:249-346, :367-375)."""
        desc = self._blocks_desc(dt)
        c = self._blocks_image
        dev = self.blocks[0].q_proj.weight.device
        if c is None or c[1] is not dt or c[2].device != dev:
            nbytes = ops.blocks_pack_size(len(self.blocks), **desc)
            c = self._blocks_image = [-1, dt, torch.empty(nbytes, dtype=torch.uint8, device=dev)]
        if c[0] != _fl._weights_version:
            params = [[blk.ln_attn.weight, blk.ln_attn.bias, blk.q_proj.weight, blk.q_proj.bias, blk.k_proj.weight,
                       blk.k_proj.bias, blk.v_proj.weight, blk.v_proj.bias, blk.out_proj.weight, blk.out_proj.bias,
                       blk.ln_ffn.weight, blk.ln_ffn.bias, blk.ffn[0].weight, blk.ffn[0].bias, blk.ffn[2].weight,
                       blk.ffn[2].bias] for blk in self.blocks]
            ops.blocks_pack(params, c[2], **desc)
            c[0] = _fl._weights_version
        return c[2]

    def _heads_packed(self, dt):
        """The 29 action heads as ONE packed (29 k_max, trunk_dim) matrix + fp32 bias (python/policy.py:1311-1335).  With
        per-joint gear counts every head's block is padded to k_max rows - zero weights, the masked-logit constant as
        bias - so the GEMM's output IS the (29, k_max) layout with its masked lanes (python/policy.py:1337-1344 scatters
        over a constant fill instead)."""
        ragged = self._gear_idx is not None
        return _fl.packed_halves(list(self.heads), dt, pad_rows=self.k_max if ragged else None, pad_bias=MASKED_LOGIT)

    def refresh_fp16_caches(self):
        """Force every weight copy the kernels read up to date for the current weights version
        (python/policy.py:1448-1461): call after optimizer steps under a captured graph.  On the
        16-bit stream these are the replicas (the encoders' column-padded first-layer copies among
        them), the fused block image and, with `fused_ffn` on, each block FFN's packed image; on the fp32 stream only
        the concatenated q|k|v / k|v / head matrices (single Linears read the masters)."""
        dt = self.stream_dtype if self.fp16 else torch.float32
        if self.fused_blocks_ok(dt):
            self.blocks_image(dt)
        if dt is not torch.float32:
            for m in self.modules():
                if isinstance(m, nn.Linear):
                    _fl._replica(m.weight, dt)
            for enc in (self.saber_mlp, self.torso_mlp, self.leg_mlp, self.note_mlp):   # padded first-layer copies
                _fl._replica_padded(enc[0].weight, dt, ops.FRONT_PITCH)
            if self.fused_ffn != "off":                     # the per-op route's fused block FFNs read packed images
                for blk in self.blocks:
                    _fl.ffn_image(blk.ffn, dt)
        for blk in self.blocks:
            _fl.packed_halves([blk.q_proj, blk.k_proj, blk.v_proj], dt)
            _fl.packed_halves([blk.k_proj, blk.v_proj], dt)
        _fl.packed_halves([self.critic_k, self.critic_v], dt)
        self._heads_packed(dt)
        if self.critic_pool:
            self._critic_pool_weights(dt)

    def load_state_dict(self, *a, **k):
        r = super().load_state_dict(*a, **k)
        _fl.bump_weights_version()
        return r

    # ---- forward -----------------------------------------------------------------------
    def _split(self, obs):
        sabers = obs.index_select(1, self._saber_idx)
        body = obs.index_select(1, self._body_idx)
        notes = obs[:, OFF_NOTES:OFF_NOTE_MASK].reshape(-1, N_NOTE_SLOTS, NOTE_FEAT)
        note_mask = obs[:, OFF_NOTE_MASK:OFF_NOTE_MASK + N_NOTE_SLOTS]
        return sabers, body, notes, note_mask

    def forward_stacked(self, obs):
        """obs (B, 630) on the GPU -> logits (B, 29, k_max) fp32, value (B,) fp32.  Under
        torch.no_grad() (rollout, evaluation) the forward-only routes run, fused kernels included; with
        grad mode on (the update) every op runs as an autograd Function over the backward kernels."""
        if not obs.is_cuda:
            raise RuntimeError("NotePolicy.forward_stacked runs on the GPU only (no CPU path)")
        if obs.dim() != 2 or obs.shape[1] != OBS_DIM:
            raise RuntimeError(f"obs must be (B, {OBS_DIM}), got {tuple(obs.shape)}")
        if torch.is_grad_enabled():
            if self.update_values not in ("rollout", "own"):
                raise ValueError(f"update_values must be 'rollout' or 'own', got {self.update_values!r}")
            if self.update_values == "rollout" and self.fp16 and not self.rollout_matches_update:
                with torch.no_grad():
                    r_out, r_value = self.forward_stacked(obs)       # the rollout's own routes, grad-free
                out, value = self._forward_train(obs)
                return _ValuesOf.apply(out, r_out), _ValuesOf.apply(value, r_value)
            return self._forward_train(obs)
        with contextlib.ExitStack() as modes:
            if self.fp16 and self.fp16_accum != "off":
                modes.enter_context(_fl.fp16_accum(self.fp16_accum))
            if self.fp16 and self.fused_ffn != "off":
                modes.enter_context(_fl.ffn_fusion(self.fused_ffn))
            return self._forward_stacked(obs)

    def _forward_stacked(self, obs):
        dt = self.stream_dtype if self.fp16 else torch.float32
        B, d = obs.shape[0], self.embed
        # preamble in one kernel: the obs is rounded once to the stream dtype (policy.py:1200-1209),
        # gathered into the four encoder inputs (+ note-geometry lanes, one-hots) and the key bias
        if obs.dtype is not torch.float32 and obs.dtype is not dt:
            obs = obs.float()
        if obs.stride(1) != 1:
            obs = obs.contiguous()
        sab_in, torso_in, leg_in, note_in, attn_bias = ops.note_frontend(
            obs, self._saber_idx32, self._body_idx32, dt, note_geo=self.note_geo, flux=self.game == "flux",
            z_asinh=self.z_asinh, padded=dt is not torch.float32)
        # 16-bit streams: the encoder inputs arrive 64 lanes wide (zero past 49 / 29 / 34 / 40), so each first
        # Linear is a K = 64 GEMM on the vector kernels instead of an odd-K one on the element-wise path.
        # every encoder writes its tokens straight into their rows of the (B, 29, d) stream
        # [saber_L, saber_R, torso, leg_L, leg_R, notes...] (the reference concatenates, policy.py:1247-1249)
        x = torch.empty(B, self.n_lead + N_NOTE_SLOTS, d, device=obs.device, dtype=dt)
        _seq(self.saber_mlp, sab_in, out=x[:, 0:2])
        _seq(self.torso_mlp, torso_in, out=x[:, 2:3])
        _seq(self.leg_mlp, leg_in, out=x[:, 3:5])
        _seq(self.note_mlp, note_in, out=x[:, 5:])
        if self.emb_ln is not None:
            x = self.emb_ln(x)
        if self.fused_blocks_ok(dt):
            # the whole stack in one persistent kernel; x_res = the stream entering the final block
            b0 = self.blocks[0]
            lead, x_res = ops.blocks_forward(self.blocks_image(dt), x.contiguous(), attn_bias, len(self.blocks),
                                             self.n_heads, b0.ffn[0].out_features,
                                             "gelu" if isinstance(b0.ffn[1], nn.GELU) else "relu", self.n_lead)
        else:
            h = None
            nb = len(self.blocks)
            v0 = None
            for i in range(nb - 1):
                if self.value_residual and i == 0:                         # block 0's values feed every later block
                    x, h, v0 = self.blocks[0](x, attn_bias, h=h, next_ln=self.blocks[1].ln_attn, want_v=True)
                else:
                    x, h = self.blocks[i](x, attn_bias, h=h, next_ln=self.blocks[i + 1].ln_attn, v0=v0)
            x_res = x                                                      # the stream entering the final block
            lead, _ = self.blocks[-1](x, attn_bias, h=h, n_queries=self.n_lead, v0=v0)
        if self.final_ln is not None:
            lead = self.final_ln(lead)
        # the critic's attention pool needs only the stream entering the final block: for a large batch it runs on a
        # second stream beside the trunk and the action heads (every kernel of either chain is a small GEMM or a row op
        # that leaves most of the chip idle), and joins before the value MLP, which needs the trunk's features
        side = self._side_stream(obs.device) if B >= self.critic_overlap_min_batch else None
        if side is not None:
            main = torch.cuda.current_stream(obs.device)
            side.wait_stream(main)
            with torch.cuda.stream(side):
                attended = self._critic_attend(x_res, attn_bias)
        hfeat = self._trunk(lead.reshape(B, self.n_lead * d))
        wh, bh = self._heads_packed(dt)
        out = ops.linear(hfeat, wh, bh, out_dtype=torch.float32)           # (B, 29 k_max) fp32, masked lanes included
        if side is not None:
            main.wait_stream(side)
            # the pool's outputs were allocated on the side stream and are read on this one: tell the allocator, so that
            # their blocks are not handed out again on the side stream while this stream's reads are still pending
            for t in (attended if isinstance(attended, (tuple, list)) else (attended,)):
                if torch.is_tensor(t):
                    t.record_stream(main)
        else:
            attended = self._critic_attend(x_res, attn_bias)
        value = self._critic_value(attended, hfeat)
        return out.view(B, N_ACTION_HEADS, self.k_max), value

    def _forward_train(self, obs):
        """The update-path forward: op for op the per-op rollout route (no fused block stack), so its
        outputs are that route's bits, with autograd Functions instead of bare kernels.  With
        `fused_ffn` on (16-bit stream, a width the fused kernel takes - here the switch buys activation
        memory, so it applies wherever the kernel exists, not only where it is the faster forward) the
        block FFNs run forward as the fused kernel, as in the reference (python/fp16_linear.py:1254-1275); the outputs then follow the
        fused per-op rollout route to 16-bit rounding (that route also folds the next LayerNorm in)."""
        dt = self.stream_dtype if self.fp16 else torch.float32
        B, d = obs.shape[0], self.embed
        obs = obs.detach()
        if obs.dtype is not torch.float32 and obs.dtype is not dt:
            obs = obs.float()
        if obs.stride(1) != 1:
            obs = obs.contiguous()
        sab_in, torso_in, leg_in, note_in, attn_bias = ops.note_frontend(
            obs, self._saber_idx32, self._body_idx32, dt, note_geo=self.note_geo, flux=self.game == "flux",
            z_asinh=self.z_asinh)
        x = torch.cat([_seq_t(self.saber_mlp, sab_in), _seq_t(self.torso_mlp, torso_in).unsqueeze(1),
                       _seq_t(self.leg_mlp, leg_in), _seq_t(self.note_mlp, note_in)], 1)
        if self.emb_ln is not None:
            x = self.emb_ln(x)
        v0 = None
        ffn = self.blocks[0].ffn
        # "on" / "up16": the forward kernel writes the hidden for the backward (the reference's form); "recompute":
        # it keeps the block input only and the backward recomputes the hidden (less memory, one more GEMM)
        fuse = (self.fp16 and self.fused_ffn != "off" and isinstance(ffn[1], nn.ReLU)
                and ops.ffn_fused_supported(ffn[0].in_features, ffn[0].out_features, dt)) and self.fused_ffn
        for i, blk in enumerate(self.blocks[:-1]):
            if self.value_residual and i == 0:
                x, v0 = blk.forward_train(x, attn_bias, want_v=True, fused_ffn=fuse)
            else:
                x = blk.forward_train(x, attn_bias, v0=v0, fused_ffn=fuse)
        x_res = x
        lead = self.blocks[-1].forward_train(x, attn_bias, n_queries=self.n_lead, v0=v0, fused_ffn=fuse)
        if self.final_ln is not None:
            lead = self.final_ln(lead)
        z = lead.reshape(B, self.n_lead * d)
        if self.trunk_arch == "simbav2":
            hfeat = self._trunk_v2_train(z)
        else:
            t = _lin_t(self.trunk_proj, z)
            hfeat = self.trunk_ln2(ChainFn.apply(self.trunk_ln1(t), t, False, self.trunk_fc1.weight, self.trunk_fc1.bias,
                                                 self.trunk_fc2.weight, self.trunk_fc2.bias))
        if self._gear_idx is None:
            w_heads, b_heads = torch.cat([m.weight for m in self.heads]), torch.cat([m.bias for m in self.heads])
        else:       # per-joint gear counts: every head padded to k_max rows (zero weights, the masked-logit constant as bias)
            w_heads = torch.cat([torch.cat([m.weight, m.weight.new_zeros(self.k_max - m.out_features, m.in_features)])
                                 for m in self.heads])
            b_heads = torch.cat([torch.cat([m.bias, m.bias.new_full((self.k_max - m.out_features,), MASKED_LOGIT)])
                                 for m in self.heads])
        out = LinearFn.apply(hfeat, w_heads, b_heads, None, None, True)
        # critic (adapool_v1)
        hv = self.critic_ln(x_res)
        q = _lin_t(self.critic_q, hv[:, 2:3])
        kv = _packed_t([self.critic_k, self.critic_v], hv)
        a = _lin_t(self.critic_out, AttnQKVFn.apply(q, kv, attn_bias, self.n_heads).view(B, d))
        vlogits = _seq_t(self.critic_mlp, torch.cat([a, hfeat], dim=-1), out_f32=True)
        self._value_logits = vlogits
        value = torch.softmax(vlogits, dim=-1) @ self.value_centers
        return out.view(B, N_ACTION_HEADS, self.k_max), value

    def _trunk_v2_train(self, z):
        """SimBaV2 readout under autograd: the three GEMMs on the gradient-aware Linear, the fp32 row work
        (scalers, ReLU, normalisations, LERP) in torch ops on B rows, as the reference writes it
        (python/policy.py:1146-1155)."""
        dt = z.dtype
        l2n = lambda t: F.normalize(t, dim=-1, eps=1e-6)
        x = l2n(_lin_t(self.trunk_in, z).float() * (self.trunk_s_in * self._v2_c_in))
        u = F.relu(_lin_t(self.trunk_w1, x.to(dt)).float() * (self.trunk_s_1 * self._v2_c_1))
        y = l2n(_lin_t(self.trunk_w2, u.to(dt)).float())
        x = l2n(x + (self.trunk_alpha * self._v2_c_alpha) * (y - x))
        return (x * math.sqrt(x.shape[-1])).to(dt)

    def trunk_projected(self):
        """The Linears whose rows `project_trunk_weights` keeps unit-norm (python/policy.py:1157-1162)."""
        return [self.trunk_in, self.trunk_w1, self.trunk_w2] if self.trunk_arch == "simbav2" else []

    @torch.no_grad()
    def project_trunk_weights(self) -> bool:
        """SimBaV2 weight projection, in place on the fp32 masters (python/policy.py:1164-1178): every
        output row back onto the unit sphere, frozen biases at 0.  The caller bumps the weights
        version afterwards, as after an optimizer step.  No-op (False) for the SimBa trunk."""
        lins = self.trunk_projected()
        for lin in lins:
            w = lin.weight
            w.div_(w.norm(dim=1, keepdim=True).clamp_min(1e-12))
            lin.bias.zero_()
        return bool(lins)

    def _trunk_v2(self, z):
        """SimBaV2 readout (python/policy.py:1140-1155): GEMMs on the stream dtype, the fp32 row
        work between them (scalers, ReLU, l2 normalisation, LERP) in one kernel per stage."""
        x32, x = ops.hsphere(ops.HS_SCALE_L2N, _lin(self.trunk_in, z), self.trunk_s_in, self._v2_c_in)
        u = ops.hsphere(ops.HS_SCALE_RELU, _lin(self.trunk_w1, x), self.trunk_s_1, self._v2_c_1)
        return ops.hsphere(ops.HS_L2N_LERP, _lin(self.trunk_w2, u), self.trunk_alpha, self._v2_c_alpha, x32=x32)

    def _trunk(self, x):
        """SimBa readout: proj -> LN1 -> fc1 -> ReLU -> fc2 -> (+proj) -> LN2 (policy.py:1107-1138)."""
        if self.trunk_arch == "simbav2":
            return self._trunk_v2(x)
        t = _lin(self.trunk_proj, x)
        u = self.trunk_ln1(t)
        r = _lin(self.trunk_fc1, u, act="relu")
        return self.trunk_ln2(_lin(self.trunk_fc2, r, residual=t))

    def _critic_pool_weights(self, dt):
        """Block-structured weights of the pooled critic attention, rebuilt in place per weights version (their
        addresses stay put under a captured graph): wqk (H d, d) with wqk[h d + e, h dh + c] = Wk[h dh + c, e] maps the
        query to the H per-head key-space vectors, wvo (d, H d) with wvo[h dh + c, h d + e] = Wv[h dh + c, e] maps the H
        pooled vectors to the attention output; zeros elsewhere."""
        d, H = self.embed, self.n_heads
        dh = d // H
        c = self._critic_pool_cache
        dev = self.critic_k.weight.device
        if c is None or c[1] is not dt or c[2].device != dev:
            c = self._critic_pool_cache = [-1, dt, torch.zeros(H, d, H, dh, device=dev, dtype=dt),
                                           torch.zeros(H, dh, H, d, device=dev, dtype=dt),
                                           torch.empty(d, device=dev, dtype=torch.float32)]
        if c[0] != _fl._weights_version:
            wk, wv = self.critic_k.weight.detach(), self.critic_v.weight.detach()
            for h in range(H):
                c[2][h, :, h, :].copy_(wk[h * dh:(h + 1) * dh].t())
                c[3][h, :, h, :].copy_(wv[h * dh:(h + 1) * dh])
            c[4].copy_(self.critic_v.bias.detach())
            c[0] = _fl._weights_version
        return c[2].view(H * d, d), c[3].view(d, H * d), c[4]

    @staticmethod
    def _side_stream(device):
        """The second stream of the forward (default priority), one per device and process, made on first use."""
        key = torch.device(device).index
        key = torch.cuda.current_device() if key is None else key
        s = _SIDE_STREAMS.get(key)
        if s is None:
            s = _SIDE_STREAMS[key] = torch.cuda.Stream(device=device)
        return s

    def _critic(self, x_res, hfeat, attn_bias):
        """adapool_v1 value path (policy.py:1346-1403): LN -> query from the torso token ->
        packed k|v -> 1-query attention pool -> out -> MLP -> HL-Gauss expectation."""
        return self._critic_value(self._critic_attend(x_res, attn_bias), hfeat)

    def _critic_attend(self, x_res, attn_bias):
        """The attention half of the value path: ((B, d) pooled and out-projected, whether the pooled kernel ran);
        independent of the trunk."""
        B, T, d = x_res.shape
        H = self.n_heads
        pooled_route = self.critic_pool and not self.rollout_matches_update and ops.critic_pool_supported(T, d, H, x_res.dtype)
        if pooled_route:
            # one query per env: the k | v projections commute with the pool, so keys and values are never formed
            wqk, wvo, bvo = self._critic_pool_weights(x_res.dtype)
            q = _lin(self.critic_q, self.critic_ln(x_res[:, 2].contiguous()))          # (B, d), the torso token's query
            qk = ops.linear(q, wqk).view(B, H, d)                                      # Wk_h^T q_h per head
            pooled = ops.critic_pool(x_res.contiguous(), self.critic_ln.weight.detach(), self.critic_ln.bias.detach(),
                                     self.critic_ln.eps, qk, attn_bias, H)
            a = ops.linear(pooled.view(B, H * d), wvo, bvo)                            # Wv_h pooled_h + bv_h
        else:
            hv = self.critic_ln(x_res)
            q = _lin(self.critic_q, hv[:, 2:3])                                # (B, 1, d)
            wkv, bkv = _fl.packed_halves([self.critic_k, self.critic_v], x_res.dtype)
            kv = ops.linear(hv, wkv, bkv)
            a = ops.attn_fwd(q, kv[..., :d], kv[..., d:], H, key_bias=attn_bias).view(B, d)
        return _lin(self.critic_out, a), pooled_route

    def _critic_value(self, attended, hfeat):
        """The value MLP over [attended | trunk features] and the HL-Gauss expectation."""
        a, pooled_route = attended
        z = torch.cat([a, hfeat], dim=-1)
        z = _lin(self.critic_mlp[0], z, act="relu")
        z = _lin(self.critic_mlp[2], z, act="relu")
        m = self.critic_mlp[4]
        logits = ops.linear(z, _fl._replica(m.weight, z.dtype), _fl._bias32(m.bias), out_dtype=torch.float32)
        self._value_logits = None
        if not pooled_route:
            # the reference's op order: the update path evaluates this very expression, and the two stay bit-equal
            return torch.softmax(logits, dim=-1) @ self.value_centers
        return ops.softmax_expect(logits, self.value_centers)

    def forward(self, obs):
        logits, value = self.forward_stacked(obs)
        return list(logits.unbind(1)), value

    def get_action_and_value(self, obs, action=None, need_entropy=True):
        """With grad mode on and an action given (the update): log-prob and entropy of that action from
        the training forward, in torch ops on the fp32 logits so that they carry gradients.  Otherwise:
        log_softmax + Gumbel-max sampling + log-prob (+ per-head entropy) in one kernel on
        the forward's fp32 logits (reference python/policy.py:1467-1516).  `self.sampler`:
        "kernel" draws inside the kernel (Philox keyed by torch's seed and a per-module call
        counter that lives on the device and is advanced on the stream, so a captured call draws
        fresh noise on every replay); "torch" feeds the kernel Exp(1) draws from torch's default
        generator, the stream the reference rides."""
        if torch.is_grad_enabled() and action is not None:
            logits, value = self.forward_stacked(obs)
            logsm = torch.log_softmax(logits, dim=-1)
            logprob = logsm.gather(-1, action.long().unsqueeze(-1)).squeeze(-1).sum(-1)
            entropy = None
            if need_entropy:
                ent_h = -(logsm.exp() * logsm).sum(-1)
                # detached (a view, no copy): the stash outlives the backward and must not pin the micro-batch's
                # autograd graph (reference python/policy.py:1509-1515)
                self._ent_h = ent_h.detach()
                entropy = ent_h.sum(-1)
            return action, logprob, entropy, value
        with torch.no_grad():
            return self._act_rollout(obs, action, need_entropy)

    def _act_rollout(self, obs, action, need_entropy):
        logits, value = self.forward_stacked(obs)
        logits = logits.contiguous()
        if action is not None and action.dtype not in (torch.int64, torch.uint8):
            action = action.long()
        noise = None
        if action is None and self.sampler == "torch":
            noise = torch.empty_like(logits).exponential_()
        elif action is None and self.sampler != "kernel":
            raise ValueError(f"sampler must be 'kernel' or 'torch', got {self.sampler!r}")
        sizes = self._head_sizes32 if self._gear_valid is not None else None
        act, logprob, entropy, ent_h, _ = ops.sample_heads(
            logits, head_sizes=sizes, exp_noise=noise, seed=torch.initial_seed(), counter=self._sample_ctr,
            action=None if action is None else action.contiguous(), need_entropy=need_entropy,
            want_ent_h=need_entropy)
        if need_entropy:
            self._ent_h = ent_h
        return act, logprob, entropy, value


def load_policy(ckpt, game: str = "standard") -> NotePolicy:
    """Rebuild a NotePolicy from a checkpoint dict {"arch", "state_dict"} written by the
    reference trainer (python/policy.py:1589-1696); refuses the same stale layouts."""
    arch = ckpt.get("arch", {})
    if arch.get("blade_geo", 0) != 1:
        raise SystemExit("only obs-630 (blade_geo 1) checkpoints are supported by this build")
    if arch.get("game", "standard") != game:
        raise SystemExit(f"checkpoint plays game {arch.get('game', 'standard')!r} but this tool plays {game!r}")
    if (arch.get("body_tokens", 1) != 3 or arch.get("obs_dim") != OBS_DIM
            or arch.get("n_action_heads") != N_ACTION_HEADS or "ffn_mult" not in arch
            or not arch.get("body_token", False)):
        raise SystemExit(f"checkpoint is not the obs-{OBS_DIM} / 29-head / 3-body-token layout: {dict(arch)}")
    z_asinh = arch.get("z_asinh")
    if z_asinh is None or not float(z_asinh) > 0:
        raise SystemExit(f"checkpoint arch has z_asinh {z_asinh!r}")
    if arch.get("note_geo", False) and not arch.get("note_geo_norm", False):
        raise SystemExit("checkpoint has the raw-metre note-geo lanes (no note_geo_norm marker)")
    if arch.get("dwa"):
        raise ValueError("checkpoint uses --dwa, which no code path can rebuild")
    policy = NotePolicy(
        embed=arch["embed"], trunk_dim=arch["trunk_dim"], n_blocks=arch["n_blocks"], n_heads=arch["n_heads"],
        n_gears=arch["n_gears"], ffn_mult=arch["ffn_mult"], note_geo=arch.get("note_geo", False),
        trunk_hidden=arch.get("trunk_hidden"), value_bins=arch["value_bins"],
        value_vmax=arch.get("value_vmax", 6.0), value_sigma=arch.get("value_sigma", 0.75),
        z_asinh=float(z_asinh), game=game, fp16_accum=arch.get("fp16_accum", "off"),
        fused_ffn=arch.get("fused_ffn", "off"), emb_ln=arch.get("emb_ln", False),
        value_residual=arch.get("value_residual", False), final_ln=arch.get("final_ln", False),
        trunk_arch=arch.get("trunk_arch", "simba"),
        head_gears=(arch.get("head_gears") or (arch["n_gears"],) * N_ACTION_HEADS))
    policy.load_state_dict(ckpt["state_dict"])
    return policy
