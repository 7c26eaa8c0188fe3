"""16-bit-stream op layer on the HIP kernels (forward paths).

Mirrors the forward surface of the reference's op layer (python/fp16_linear.py):
Linears whose fp32 master weights are used through 16-bit replicas that are rebuilt
only when the weights version changes (`bump_weights_version`, reference :228-246,
:349-376), several same-input Linears packed into one GEMM (`packed_halves`,
`fp16_packed_linear`, :411-427, :506-517), Linear + ReLU with the activation in the
GEMM epilogue (`fp16_linear_relu`, `fp16_relu_chain`, :633-641, :732-767), the fused
short-sequence attention straight off the packed projection (`attn29_packed`,
`attn29_qkv`, :967-989) and the fused block FFN (`fused_ffn_ok`, `fused_ffn`,
:1143-1275).

Differences, all deliberate:
  * every GEMM runs the library's MFMA kernel with fp32 accumulate - there is no
    fp16-accumulate mode here; `fp16_accum(...)` is accepted and recorded so callers
    written against the reference keep working, and is a no-op;
  * biases are never rounded: the kernels read the fp32 master bias;
  * the attention kernel covers any T <= 48 with 32- or 48-wide heads, not only the
    (29, 192, 4) shape, so `attn29_ok` is true for all of them;
  * the stream dtype may be bfloat16 as well as float16 (the replica follows x.dtype);
  * forward only (rollout / evaluation); there is no torch fallback - a missing kernel
    library raises."""
from __future__ import annotations

import torch
import torch.nn as nn

from . import ops

ACCUM_MODES = ("off", "fwd", "all")
FFN_MODES = ("off", "on", "up16", "recompute")

_weights_version = 0
_accum_mode = "off"
_ffn_mode = "off"


def bump_weights_version():
    """Call after every in-place update of the fp32 masters (optimizer step, load):
    16-bit replicas are recast, in place, on their next use."""
    global _weights_version
    _weights_version += 1


def ext_ok() -> bool:
    """True when the kernel library loads (the reference's `ext_ok`, :644)."""
    from . import _lib
    try:
        _lib.load()
        return True
    except (RuntimeError, OSError, AttributeError):
        return False


class fp16_accum:
    """Context manager kept for API compatibility (reference :98-119): the mode is
    validated and recorded, the arithmetic is always fp32-accumulate."""

    def __init__(self, mode):
        if mode not in ACCUM_MODES:
            raise ValueError(f"fp16_accum mode must be one of {ACCUM_MODES}, got {mode!r}")
        self.mode = mode

    def __enter__(self):
        global _accum_mode
        self._prev, _accum_mode = _accum_mode, self.mode
        return self

    def __exit__(self, *exc):
        global _accum_mode
        _accum_mode = self._prev


class ffn_fusion:
    """Selects the fused block-FFN kernel inside the context (reference :1120-1140).
    "up16" (fp16-accumulated up-projection in the reference) maps to "on"; "recompute" differs from "on" in the
    update path only (the fused forward keeps no hidden and the backward recomputes it)."""

    def __init__(self, mode):
        if mode not in FFN_MODES:
            raise ValueError(f"ffn_fusion mode must be one of {FFN_MODES}, got {mode!r}")
        self.mode = mode

    def __enter__(self):
        global _ffn_mode
        self._prev, _ffn_mode = _ffn_mode, self.mode
        return self

    def __exit__(self, *exc):
        global _ffn_mode
        _ffn_mode = self._prev


# ---- replicas ----------------------------------------------------------------------
def _replica(w: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Version-checked 16-bit copy of a master weight, refreshed IN PLACE so its
    address never moves (graph-capture contract, reference :367-375)."""
    if dtype is torch.float32:
        return w.detach()
    cache = getattr(w, "_bsrl_replica", None)
    if cache is None or cache[1].dtype is not dtype or cache[1].device != w.device:
        cache = [_weights_version, w.detach().to(dtype).contiguous()]
        w._bsrl_replica = cache
    elif cache[0] != _weights_version:
        cache[1].copy_(w.detach())
        cache[0] = _weights_version
    return cache[1]


def _replica_padded(w: torch.Tensor, dtype: torch.dtype, k_pad: int) -> torch.Tensor:
    """_replica with the (M, K) weight's columns zero-padded to k_pad: the operand of a Linear whose input
    rows arrive padded the same way.  Refreshed in place like _replica."""
    M, K = w.shape
    cache = getattr(w, "_bsrl_replica_padded", None)
    if cache is None or cache[1].dtype is not dtype or cache[1].device != w.device or cache[1].shape[1] != k_pad:
        wp = torch.zeros(M, k_pad, device=w.device, dtype=dtype)
        wp[:, :K].copy_(w.detach())
        cache = [_weights_version, wp]
        w._bsrl_replica_padded = cache
    elif cache[0] != _weights_version:
        cache[1][:, :K].copy_(w.detach())
        cache[0] = _weights_version
    return cache[1]


def packed_halves(ms, dtype=torch.float16, pad_rows=None, pad_bias=0.0):
    """(w_cat in `dtype`, b_cat fp32) for an ordered group of same-input Linears.  16-bit copies are refreshed per
    weights version (bump_weights_version), like every replica.  The fp32 "copy" is a plain concatenation of the
    masters: the reference's fp32 forward reads the masters themselves (python/policy.py:1371-1376), so it is also
    rebuilt whenever torch's own in-place counters of the members move (any in-place edit, with or without a bump).
    pad_rows: every member's block is padded to that many output rows with zero weights and bias `pad_bias` - the
    packed action heads with per-joint gear counts come out of ONE GEMM already in the (29, k_max) layout, the lanes past
    a head's count holding the masked-logit constant exactly (0 + pad_bias in fp32), where the reference scatters the
    ragged GEMM output over a constant fill (python/policy.py:1337-1344)."""
    key = ms[0].weight
    ident = tuple(id(m) for m in ms)                      # the members, not just the first one and the count
    table = getattr(key, "_bsrl_packed", None)
    if table is None:
        table = key._bsrl_packed = {}
    cache = table.get((ident, dtype, pad_rows))
    tv = tuple((m.weight._version, m.bias._version) for m in ms) if dtype is torch.float32 else None

    def cat_w():
        if pad_rows is None:
            return torch.cat([m.weight.detach() for m in ms])
        return torch.cat([torch.cat([m.weight.detach(), m.weight.new_zeros(pad_rows - m.out_features, m.in_features)])
                          for m in ms])

    def cat_b():
        if pad_rows is None:
            return torch.cat([m.bias.detach() for m in ms])
        return torch.cat([torch.cat([m.bias.detach(), m.bias.new_full((pad_rows - m.out_features,), pad_bias)]) for m in ms])

    if cache is None or cache[1].device != key.device:
        cache = [_weights_version, cat_w().to(dtype).contiguous(), cat_b().float().contiguous(), tv]
        table[(ident, dtype, pad_rows)] = cache
    elif cache[0] != _weights_version or cache[3] != tv:
        cache[1].copy_(cat_w())
        cache[2].copy_(cat_b())
        cache[0], cache[3] = _weights_version, tv
    return cache[1], cache[2]


def _bias32(b):
    if b is None:
        return None
    b = b.detach()
    return b if b.dtype is torch.float32 and b.is_contiguous() else b.float().contiguous()


# ---- Linears ---------------------------------------------------------------------------
def fp16_linear(x, w, b):
    """x @ w.T + b with w a fp32 master (reference :794-805)."""
    return ops.linear(x, _replica(w, x.dtype), _bias32(b))


def fp16_linear_nobias(x, w, b):
    """x @ w.T, the bias left to the consumer's fused pass (reference :581-587)."""
    return ops.linear(x, _replica(w, x.dtype), None)


def fp16_linear_relu(x, w, b):
    """relu(x @ w.T + b) in one kernel (reference :633-641)."""
    return ops.linear(x, _replica(w, x.dtype), _bias32(b), act="relu")


def fp16_relu_chain(x, ms, tail_bias=True):
    """Linear (ReLU Linear)+ with every ReLU in a GEMM epilogue (reference :732-767);
    tail_bias=False runs the last Linear bias-free."""
    for m in ms[:-1]:
        x = fp16_linear_relu(x, m.weight, m.bias)
    tail = ms[-1]
    return fp16_linear(x, tail.weight, tail.bias) if tail_bias else fp16_linear_nobias(x, tail.weight, tail.bias)


def fp16_packed_linear(x, wh, bh, ms=None):
    """One GEMM against concatenated replicas (reference :506-517); wh, bh from packed_halves."""
    return ops.linear(x, wh, bh)


def linear_residual(x, w, b, residual):
    """residual + (x @ w.T + b) with the add in the GEMM epilogue (one rounding)."""
    return ops.linear(x, _replica(w, x.dtype), _bias32(b), residual=residual)


# ---- attention -------------------------------------------------------------------------
def attn29_ok(T, d, n_heads) -> bool:
    """Shapes the fused attention kernel covers (the reference's gate is the single
    production shape, :925-928)."""
    return T <= 48 and d % n_heads == 0 and d // n_heads in (32, 48)


def attn29_packed(qkv, attn_bias, n_heads=4):
    """Self-attention straight off the packed (B, T, 3d) projection -> (B, T, d);
    attn_bias (B, 1, T) or (B, T) additive key bias (reference :967-977; its kernel is
    hard-wired to 4 heads, here the head count is a parameter)."""
    d = qkv.shape[-1] // 3
    B, T = qkv.shape[0], qkv.shape[1]
    return ops.attn_fwd(qkv[..., :d], qkv[..., d:2 * d], qkv[..., 2 * d:], n_heads,
                        key_bias=attn_bias.reshape(B, T).contiguous())


def attn29_qkv(q, kv, attn_bias, n_heads=4):
    """q (B, TQ, d) over the packed (B, T, 2d) k|v projection (reference :979-989)."""
    d = q.shape[-1]
    B, T = kv.shape[0], kv.shape[1]
    return ops.attn_fwd(q, kv[..., :d], kv[..., d:], n_heads, key_bias=attn_bias.reshape(B, T).contiguous())


# ---- fused FFN --------------------------------------------------------------------------
def fused_ffn_ok(x, ffn, ln=None) -> bool:
    """Can `fused_ffn` run on this input? (reference :1143-1174): the fusion is on,
    16-bit contiguous rows, a Linear-ReLU/GELU-Linear Sequential of a width at which the
    fused kernel is the faster route (ops.ffn_fused_profitable)."""
    if _ffn_mode == "off" or x.dtype not in (torch.float16, torch.bfloat16) or not x.is_cuda:
        return False
    if len(ffn) != 3 or not isinstance(ffn[0], nn.Linear) or not isinstance(ffn[2], nn.Linear):
        return False
    if not isinstance(ffn[1], (nn.ReLU, nn.GELU)):
        return False
    return ops.ffn_fused_profitable(ffn[0].in_features, ffn[0].out_features, x.dtype)


def ffn_image(ffn, dtype):
    """The packed fused FFN's weight image of a Linear-act-Linear Sequential, or None where the shape has no packed
    kernel.  ONE buffer per module, rebuilt IN PLACE from the (in-place) replicas once per weights version: like the
    replicas themselves (reference :367-375) its address never moves, so a captured graph that holds it follows every
    refresh_fp16_caches / bump_weights_version."""
    w0, w2 = ffn[0].weight, ffn[2].weight
    if dtype is torch.float32 or not ops.ffn_pack_supported(ffn[0].in_features, ffn[0].out_features, dtype):
        return None
    cache = getattr(w0, "_bsrl_ffn_image", None)
    if cache is None or cache[1] is not dtype or cache[2].device != w0.device:
        cache = [-1, dtype, None]
        w0._bsrl_ffn_image = cache
    if cache[0] != _weights_version or cache[2] is None:
        cache[2] = ops.ffn_pack_into(cache[2], _replica(w0, dtype), _bias32(ffn[0].bias), _replica(w2, dtype),
                                     _bias32(ffn[2].bias))
        cache[0] = _weights_version
    return cache[2]


def fused_ffn(x, h2, ffn, ln=None):
    """out = x + ffn(h2) [, LayerNorm_ln(out)] in one kernel (reference :1254-1275).
    Returns out, or (out, ln(out)) when ln is given."""
    act = "gelu" if isinstance(ffn[1], nn.GELU) else "relu"
    r = ops.ffn_fused(x.contiguous(), h2.contiguous(), _replica(ffn[0].weight, x.dtype), _bias32(ffn[0].bias),
                      _replica(ffn[2].weight, x.dtype), _bias32(ffn[2].bias), act=act,
                      ln_w=None if ln is None else ln.weight, ln_b=None if ln is None else ln.bias,
                      eps=1e-5 if ln is None else ln.eps, image=ffn_image(ffn, x.dtype))
    if r is None:
        raise ops.Unsupported("fused_ffn: call fused_ffn_ok first")
    return r[0] if ln is None else r
