"""TEST INFRASTRUCTURE - CPU oracle for the benchmark-config policy forward.

This module is the checker, never the product: only tests/, the smoke entry
point and the CPU-baseline leg of bench.py may import it.  It restates, in
plain torch fp32 on the CPU, the textbook pre-LN transformer policy that the
benchmark configs describe, following the arithmetic of the reference's fp32
"record path":

  * Linear          = x @ W.T + b          (reference python/policy.py:67-73, `_lin`)
  * LayerNorm       = eps 1e-5, affine     (reference python/fused_ln.py:126-138)
  * attention       = softmax(q k^T / sqrt(dh) + bias) v, bias = (valid-1)*2^14
                      (reference python/policy.py:686-690 and :422-428, :1257-1260)
  * block           = x += out(MHA(LN(x))); x += W2 act(W1 LN(x) + b1) + b2
                      (reference python/policy.py:524-715, the `else` arms)
  * heads           = one packed projection whose rows are the 29 gear heads
                      (reference python/policy.py:1311-1335); here the last row is
                      the scalar value.

Builder decisions the configs leave open (recorded here because every fixture
and every parity test depends on them):
  * obs = [proprio (100 lanes) | (T-1) object tokens x 16 lanes]; token 0 is
    the proprio token, token j>=1 object j-1; both embedded by one Linear.
  * the first `n_valid[b]` object tokens of env b are attendable, token 0 always.
  * activation: exact-erf GELU (configs) or ReLU (the reference's own FFN).
  * readout = final-block output of token 0 (optionally LayerNormed), projected
    by one (29*7+1, d) matrix: rows 0..202 = logits (29,7), row 203 = value.
  * init: Xavier-uniform weights, biases U(-1/sqrt(fan_in), 1/sqrt(fan_in)),
    LayerNorm weight 1 / bias 0, from one torch.Generator seeded per config.

Pins (tests/test_oracle_config.py): torch.nn.TransformerEncoderLayer
(norm_first, gelu) with the same weights and key-padding mask; a float64
per-env, per-head loop implementation written from the formulas; the
invariants "masked slots cannot change outputs", "full mask == no mask" and
"final-block pruning == full block".

`forward(..., emulate=...)` additionally restates the rounding points of the
16-bit stream (weights and every GEMM operand rounded to fp16/bf16, fp32
accumulate, fp32 LayerNorm/softmax statistics) so a 16-bit kernel can be
compared against its own precision class as well as against fp32.  That branch is
pinned too (tests/test_oracle_emulate.py): the casts on hand-picked ties and against
an independent bit-pattern rounding; a float64 restatement with an explicit cast at
each rounding point, matched on the median env (single-ulp flips aside) while every
one-rounding-point mutant of it is rejected; torch's own CPU 16-bit kernels per op.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, asdict

import torch
import torch.nn.functional as F

MASK_BIAS = 16384.0          # reference python/policy.py:428
N_HEADS_OUT = 29             # reference python/policy.py:409
PROP_DIM = 100
OBJ_DIM = 16


@dataclass(frozen=True)
class ConfigSpec:
    n_layers: int = 2
    d: int = 128
    n_heads: int = 4
    ffn: int = 512
    T: int = 16
    n_gears: int = 7
    act: str = "gelu"
    final_ln: bool = False
    prop_dim: int = PROP_DIM
    obj_dim: int = OBJ_DIM

    @property
    def obs_dim(self) -> int:
        return self.prop_dim + (self.T - 1) * self.obj_dim

    @property
    def dh(self) -> int:
        return self.d // self.n_heads

    @property
    def n_out(self) -> int:
        return N_HEADS_OUT * self.n_gears + 1

    def asdict(self):
        return asdict(self)


# the five benchmark configs (index = position in the benchmark's config list)
CONFIGS = {
    0: dict(spec=ConfigSpec(2, 128, 4, 512, 16), B=256, dtype="f32", obs_seed=0, w_seed=1, mask="none"),
    1: dict(spec=ConfigSpec(2, 128, 4, 512, 16), B=16384, dtype="f16", obs_seed=2, w_seed=1, mask="uniform"),
    2: dict(spec=ConfigSpec(4, 256, 8, 1024, 32), B=32768, dtype="bf16", obs_seed=3, w_seed=3, mask="uniform"),
    3: dict(spec=ConfigSpec(6, 384, 12, 1536, 48), B=65536, dtype="f16", obs_seed=4, w_seed=4, mask="quarter_empty"),
    4: dict(spec=ConfigSpec(2, 128, 4, 512, 16), B=64, dtype="f16", obs_seed=5, w_seed=1, mask="none"),
}


def param_shapes(spec: ConfigSpec):
    """Ordered (name, shape) list = the config model's state_dict layout."""
    d, Fh = spec.d, spec.ffn
    out = [("prop_embed.weight", (d, spec.prop_dim)), ("prop_embed.bias", (d,)),
           ("obj_embed.weight", (d, spec.obj_dim)), ("obj_embed.bias", (d,))]
    for i in range(spec.n_layers):
        p = f"blocks.{i}."
        out += [(p + "ln_attn.weight", (d,)), (p + "ln_attn.bias", (d,))]
        for n in ("q_proj", "k_proj", "v_proj", "out_proj"):
            out += [(p + n + ".weight", (d, d)), (p + n + ".bias", (d,))]
        out += [(p + "ln_ffn.weight", (d,)), (p + "ln_ffn.bias", (d,)),
                (p + "ffn.0.weight", (Fh, d)), (p + "ffn.0.bias", (Fh,)),
                (p + "ffn.2.weight", (d, Fh)), (p + "ffn.2.bias", (d,))]
    if spec.final_ln:
        out += [("final_ln.weight", (d,)), ("final_ln.bias", (d,))]
    out += [("heads.weight", (spec.n_out, d)), ("heads.bias", (spec.n_out,))]
    return out


def init_params(spec: ConfigSpec, seed: int, randomize_affine: bool = False):
    """Xavier-uniform weights / fan-in-uniform biases from one seeded CPU
    generator, drawn in state_dict order.  randomize_affine=True also perturbs
    the LayerNorm weight/bias (tests use it so an ignored affine term fails)."""
    g = torch.Generator().manual_seed(seed)
    p = {}
    for name, shape in param_shapes(spec):
        is_ln = ".ln_" in name or name.startswith("final_ln")
        if is_ln:
            if randomize_affine:
                base = 1.0 if name.endswith("weight") else 0.0
                p[name] = base + 0.2 * (torch.rand(shape, generator=g) * 2 - 1)
            else:
                p[name] = torch.ones(shape) if name.endswith("weight") else torch.zeros(shape)
        elif name.endswith("weight"):
            fan_out, fan_in = shape
            a = math.sqrt(6.0 / (fan_in + fan_out))
            p[name] = (torch.rand(shape, generator=g) * 2 - 1) * a
        else:
            wname = name[:-4] + "weight"
            fan_in = p[wname].shape[1]
            a = 1.0 / math.sqrt(fan_in)
            p[name] = (torch.rand(shape, generator=g) * 2 - 1) * a
    return p


def make_inputs(spec: ConfigSpec, B: int, seed: int, mask: str = "uniform"):
    """Seeded synthetic obs (B, obs_dim) ~ N(0,1) and valid object counts (B,)
    int32.  mask: "none" (all T-1 valid), "uniform" (k ~ U{0..T-1}),
    "quarter_empty" (25% of envs k = 0, the rest k ~ U{1..T-1})."""
    g = torch.Generator().manual_seed(seed)
    obs = torch.randn(B, spec.obs_dim, generator=g)
    nobj = spec.T - 1
    if mask == "none":
        k = torch.full((B,), nobj, dtype=torch.int32)
    elif mask == "uniform":
        k = torch.randint(0, nobj + 1, (B,), generator=g, dtype=torch.int32)
    elif mask == "quarter_empty":
        k = torch.randint(1, nobj + 1, (B,), generator=g, dtype=torch.int32)
        empty = torch.rand(B, generator=g) < 0.25
        k = torch.where(empty, torch.zeros_like(k), k)
    else:
        raise ValueError(mask)
    return obs, k


def key_bias(spec: ConfigSpec, n_valid: torch.Tensor | None, B: int):
    """(B, T) additive key bias: 0 for token 0 and the first n_valid object
    tokens, -2^14 elsewhere (reference python/policy.py:1257-1260)."""
    if n_valid is None:
        return torch.zeros(B, spec.T)
    idx = torch.arange(spec.T).unsqueeze(0)
    valid = (idx <= n_valid.to(torch.int64).unsqueeze(1)).float()
    return (valid - 1.0) * MASK_BIAS


def _round(x: torch.Tensor, emulate):
    if emulate is None:
        return x
    dt = {"f16": torch.float16, "bf16": torch.bfloat16}[emulate]
    return x.to(dt).float()


def _act(x, kind):
    if kind == "gelu":
        return F.gelu(x)                      # exact erf form
    if kind == "relu":
        return F.relu(x)
    raise ValueError(kind)


def tokens_from_obs(p, spec: ConfigSpec, obs: torch.Tensor, emulate=None):
    B = obs.shape[0]
    r = lambda t: _round(t, emulate)
    o = r(obs.float())
    prop = o[:, :spec.prop_dim]
    objs = o[:, spec.prop_dim:].reshape(B, spec.T - 1, spec.obj_dim)
    t0 = F.linear(prop, r(p["prop_embed.weight"]), p["prop_embed.bias"]).unsqueeze(1)
    tj = F.linear(objs, r(p["obj_embed.weight"]), p["obj_embed.bias"])
    return torch.cat([t0, tj], dim=1)          # (B, T, d) fp32


def attention(q, k, v, bias, n_heads, emulate=None):
    """q (B,Tq,d), k/v (B,T,d), bias (B,T) -> (B,Tq,d).  The reference's fp32
    arithmetic, python/policy.py:677-691.  Under `emulate` the normalised
    probabilities are rounded to the 16-bit type before the P.V product (they
    are an MFMA operand in the 16-bit kernels)."""
    B, Tq, d = q.shape
    T = k.shape[1]
    dh = d // n_heads
    qh = q.view(B, Tq, n_heads, dh).transpose(1, 2)
    kh = k.view(B, T, n_heads, dh).transpose(1, 2)
    vh = v.view(B, T, n_heads, dh).transpose(1, 2)
    scores = qh @ kh.transpose(-2, -1) / (dh ** 0.5)
    scores = scores + bias.view(B, 1, 1, T)
    att = _round(torch.softmax(scores, dim=-1), emulate) @ vh
    return att.transpose(1, 2).reshape(B, Tq, d)


def block(p, prefix, spec: ConfigSpec, x, bias, n_queries=0, emulate=None,
          round_residual=False):
    """One pre-LN block.  n_queries>0 restricts the output to the first
    n_queries rows (keys/values still span all T) - exact because masking is
    key-side only (reference python/policy.py:533-539)."""
    r = lambda t: _round(t, emulate)
    rr = (lambda t: _round(t, emulate)) if round_residual else (lambda t: t)
    d = spec.d
    W = lambda n: r(p[prefix + n + ".weight"])
    b = lambda n: p[prefix + n + ".bias"]
    h = r(F.layer_norm(x, (d,), p[prefix + "ln_attn.weight"], p[prefix + "ln_attn.bias"], 1e-5))
    k = r(F.linear(h, W("k_proj"), b("k_proj")))
    v = r(F.linear(h, W("v_proj"), b("v_proj")))
    if n_queries:
        x = x[:, :n_queries]
        h = h[:, :n_queries]
    q = r(F.linear(h, W("q_proj"), b("q_proj")))
    att = r(attention(q, k, v, bias, spec.n_heads, emulate))
    x = rr(x + F.linear(att, W("out_proj"), b("out_proj")))
    h2 = r(F.layer_norm(x, (d,), p[prefix + "ln_ffn.weight"], p[prefix + "ln_ffn.bias"], 1e-5))
    hid = r(_act(F.linear(h2, W("ffn.0"), b("ffn.0")), spec.act))
    x = rr(x + F.linear(hid, W("ffn.2"), b("ffn.2")))
    return x


@torch.no_grad()
def forward(p, spec: ConfigSpec, obs, n_valid=None, emulate=None,
            round_residual=False, prune_final=False, return_tokens=False):
    """obs (B, obs_dim) -> logits (B, 29, n_gears) fp32, value (B,) fp32."""
    B = obs.shape[0]
    bias = key_bias(spec, n_valid, B)
    x = tokens_from_obs(p, spec, obs, emulate)
    if round_residual:
        x = _round(x, emulate)
    for i in range(spec.n_layers):
        last = i == spec.n_layers - 1
        x = block(p, f"blocks.{i}.", spec, x, bias,
                  n_queries=1 if (last and prune_final) else 0,
                  emulate=emulate, round_residual=round_residual)
    if return_tokens:
        return x
    h = x[:, 0]
    if spec.final_ln:
        h = F.layer_norm(h, (spec.d,), p["final_ln.weight"], p["final_ln.bias"], 1e-5)
    h = _round(h, emulate)
    out = F.linear(h, _round(p["heads.weight"], emulate), p["heads.bias"])
    n_log = N_HEADS_OUT * spec.n_gears
    return out[:, :n_log].reshape(B, N_HEADS_OUT, spec.n_gears).contiguous(), out[:, n_log].contiguous()


def round_operands(p, obs, dtype: str):
    """The config's own 16-bit storage, with the arithmetic left in fp32: every weight MATRIX and the observations
    rounded once to fp16 / bf16 and widened again (biases and LayerNorm affine stay fp32, as in every 16-bit stream
    here and in the reference, python/fp16_linear.py:1-18).  `forward(*round_operands(...))` is then the reference's
    own kernel-test idiom - a closed form "on the same fp16-rounded inputs" (python/tests/test_attn29.py:49-54,
    python/tests/test_fp16_accum.py:84-89) - applied to the whole forward: what is left between it and a 16-bit
    forward is the forward's own activation rounding, not the rounding of weights the config declares to BE 16-bit.
    No arithmetic of the oracle changes: the same `forward` runs on other inputs."""
    dt = {"f16": torch.float16, "bf16": torch.bfloat16}[dtype]
    pr = {k: (v.to(dt).float() if v.dim() == 2 else v) for k, v in p.items()}
    return pr, obs.to(dt).float()


def top2_margin(logits: torch.Tensor) -> torch.Tensor:
    """(B, 29) gap between the best and second-best logit of every head."""
    t = logits.topk(2, dim=-1).values
    return t[..., 0] - t[..., 1]


def flops_per_env(spec: ConfigSpec) -> int:
    """Dense algorithmic FLOPs per env (all T slots, 2 FLOPs per MAC)."""
    d, T, Fh, L = spec.d, spec.T, spec.ffn, spec.n_layers
    E = spec.prop_dim * d + (T - 1) * spec.obj_dim * d
    per_layer = 3 * T * d * d + 2 * T * T * d + T * d * d + 2 * T * d * Fh
    return 2 * (E + L * per_layer + d * spec.n_out)
