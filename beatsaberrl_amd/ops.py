"""Tensor-level wrappers of the C-ABI entry points.

Each function checks what the kernel assumes (device, dtype, contiguity),
allocates the outputs with torch (device memory + stream are torch's; the
arithmetic is not), and enqueues on torch's current stream.  Outputs are fresh
tensors and inputs are only borrowed - the ownership convention of the
reference's extension ops (python/beat_arena_env/csrc/layer_norm.cu:545-547).
A False / None return means "the kernel set does not cover this shape"
(the reference signals the same with an empty list, fp16_gemm.cu:346-357)."""
from __future__ import annotations

import torch

from . import _lib
from ._lib import ACT_GELU, ACT_NONE, ACT_RELU, BF16, F16, F32

_DT = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}
_ACT = {None: ACT_NONE, "none": ACT_NONE, "relu": ACT_RELU, "gelu": ACT_GELU}


class Unsupported(RuntimeError):
    """The kernel set has no kernel for the requested shape/dtype."""


def dt_code(dtype: torch.dtype) -> int:
    try:
        return _DT[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}") from None


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("bsrl ops need device tensors (there is no CPU path)")


def _ptr(t):
    return None if t is None else t.data_ptr()


def _f32c(t, name):
    if t is None:
        return None
    if t.dtype is not torch.float32 or not t.is_contiguous():
        raise TypeError(f"{name} must be a contiguous fp32 tensor")
    return t


def ln_fwd(x, weight, bias, eps=1e-5, want_stats=False):
    """y = LayerNorm(x) over the last dim; fp32 weight/bias/stats."""
    _need_cuda(x, weight, bias)
    d = x.shape[-1]
    if not x.is_contiguous():
        raise RuntimeError("ln_fwd: x must be contiguous")
    if weight.numel() != d or bias.numel() != d:
        raise RuntimeError(f"ln_fwd: weight / bias must have {d} elements")
    rows = x.numel() // d
    y = torch.empty_like(x)
    mean = rstd = None
    if want_stats:
        mean = torch.empty(rows, device=x.device, dtype=torch.float32)
        rstd = torch.empty(rows, device=x.device, dtype=torch.float32)
    with torch.cuda.device(x.device):
        rc = _lib.load().bsrl_ln_fwd(x.data_ptr(), _f32c(weight, "weight").data_ptr(), _f32c(bias, "bias").data_ptr(),
                                     y.data_ptr(), _ptr(mean), _ptr(rstd), rows, d, float(eps), dt_code(x.dtype),
                                     _stream(x))
    if not _lib.check(rc, "bsrl_ln_fwd"):
        raise Unsupported(f"ln_fwd d={d} dtype={x.dtype}")
    return (y, mean, rstd) if want_stats else y


def ln_fwd_add(a, b, weight, bias, eps=1e-5, b_bias=None, want_stats=False):
    """x = round(a + (b + b_bias)); y = LayerNorm(x).  Returns (x, y[, mean, rstd])."""
    _need_cuda(a, b, weight, bias, b_bias)
    if a.shape != b.shape or a.dtype is not b.dtype or not (a.is_contiguous() and b.is_contiguous()):
        raise RuntimeError("ln_fwd_add: a and b must be contiguous with equal shape and dtype")
    d = a.shape[-1]
    if weight.numel() != d or bias.numel() != d or (b_bias is not None and b_bias.numel() != d):
        raise RuntimeError(f"ln_fwd_add: weight / bias / b_bias must have {d} elements")
    rows = a.numel() // d
    x = torch.empty_like(a)
    y = torch.empty_like(a)
    mean = rstd = None
    if want_stats:
        mean = torch.empty(rows, device=a.device, dtype=torch.float32)
        rstd = torch.empty(rows, device=a.device, dtype=torch.float32)
    with torch.cuda.device(a.device):
        rc = _lib.load().bsrl_ln_fwd_add(a.data_ptr(), b.data_ptr(), _ptr(_f32c(b_bias, "b_bias")),
                                         _f32c(weight, "weight").data_ptr(), _f32c(bias, "bias").data_ptr(),
                                         x.data_ptr(), y.data_ptr(), _ptr(mean), _ptr(rstd), rows, d, float(eps),
                                         dt_code(a.dtype), _stream(a))
    if not _lib.check(rc, "bsrl_ln_fwd_add"):
        raise Unsupported(f"ln_fwd_add d={d} dtype={a.dtype}")
    return (x, y, mean, rstd) if want_stats else (x, y)


def ln_bwd(x, dy, weight, mean, rstd, gx=None, want_dbb=False):
    """LayerNorm backward (reference layer_norm_cuda.ln_bwd, layer_norm.cu:645-729):
    returns [dx, dw, db] (+ [dbb] with want_dbb: column sums of the stored dx).  gx, if given,
    is added into dx before its one rounding (the residual-path gradient of ln_fwd_add)."""
    _need_cuda(x, dy, weight, mean, rstd, gx)
    if not (x.is_contiguous() and dy.is_contiguous()) or dy.shape != x.shape or dy.dtype is not x.dtype:
        raise TypeError("ln_bwd: x and dy must be contiguous with one shape and dtype")
    if gx is not None and (not gx.is_contiguous() or gx.shape != x.shape or gx.dtype is not x.dtype):
        raise TypeError("ln_bwd: gx must be contiguous with x's shape and dtype")
    d = x.shape[-1]
    rows = x.numel() // d if d else 0
    weight, mean, rstd = _f32c(weight, "ln weight"), _f32c(mean, "ln mean"), _f32c(rstd, "ln rstd")
    if weight.numel() != d or mean.numel() != rows or rstd.numel() != rows:
        raise TypeError("ln_bwd: weight must be (d), mean / rstd (rows)")
    dev = x.device
    dx = torch.empty_like(x)
    dw = torch.empty(d, device=dev, dtype=torch.float32)
    db = torch.empty(d, device=dev, dtype=torch.float32)
    dbb = torch.empty(d, device=dev, dtype=torch.float32) if want_dbb else None
    lib = _lib.load()
    ws = _workspace(dev, _stream(x), lib.bsrl_ln_bwd_workspace_size(d))
    with torch.cuda.device(dev):
        rc = lib.bsrl_ln_bwd(x.data_ptr(), dy.data_ptr(), weight.data_ptr(), mean.data_ptr(), rstd.data_ptr(),
                             _ptr(gx), dx.data_ptr(), dw.data_ptr(), db.data_ptr(), _ptr(dbb), ws.data_ptr(),
                             rows, d, dt_code(x.dtype), _stream(x))
    if not _lib.check(rc, "bsrl_ln_bwd"):
        raise Unsupported(f"ln_bwd: no kernel for d={d} {x.dtype}")
    return [dx, dw, db] + ([dbb] if want_dbb else [])


_WS = {}


def _workspace(dev, stream, nbytes):
    """One scratch buffer per (device, stream), grown on demand: calls on one stream are ordered,
    so they may share it (the C entry points never allocate)."""
    key = (dev, stream)
    ws = _WS.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = _WS[key] = torch.empty(nbytes, device=dev, dtype=torch.uint8)
    return ws


def wgrad(dy, x, want_db=True):
    """(dW (M, K) fp32, db (M) fp32 | None) of a Linear from dy (rows, M) and its input x (rows, K),
    16-bit operands with fp32 accumulation (reference fp16_gemm.wgrad / wgrad_bgrad,
    fp16_gemm.cu:189-277, 404-476)."""
    _need_cuda(dy, x)
    if dy.dim() != 2 or x.dim() != 2 or dy.shape[0] != x.shape[0] or dy.dtype is not x.dtype:
        raise TypeError("wgrad: dy (rows, M) and x (rows, K) must share rows and dtype")
    if dy.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError("wgrad: 16-bit operands only (the fp32 stream uses the vendor GEMM)")
    if dy.stride(1) != 1 or x.stride(1) != 1:
        raise TypeError("wgrad: unit-stride rows needed")
    rows, M = dy.shape
    K = x.shape[1]
    dev = dy.device
    dw = torch.empty(M, K, device=dev, dtype=torch.float32)
    db = torch.empty(M, device=dev, dtype=torch.float32) if want_db else None
    lib = _lib.load()
    ws = _workspace(dev, _stream(dy), lib.bsrl_wgrad_workspace_size(M, K))
    with torch.cuda.device(dev):
        rc = lib.bsrl_wgrad(dy.data_ptr(), dy.stride(0) if rows > 1 else M, x.data_ptr(), x.stride(0) if rows > 1 else K,
                            dw.data_ptr(), _ptr(db), ws.data_ptr(), rows, M, K, dt_code(dy.dtype), _stream(dy))
    _lib.check(rc, "bsrl_wgrad")
    return dw, db


def _rows2d(t):
    """View t (..., K) as rows with one row stride; returns (tensor, rows, ld)."""
    K = t.shape[-1]
    if t.stride(-1) != 1:
        t = t.contiguous()
    if t.dim() == 1:
        return t, 1, K
    if t.dim() == 2:
        return t, t.shape[0], t.stride(0)
    # collapse leading dims if they form one stride
    lead = t.shape[:-1]
    st = t.stride()[:-1]
    ld = st[-1]
    ok = all(st[i] == st[i + 1] * lead[i + 1] for i in range(len(lead) - 1))
    if not ok:
        t = t.contiguous()
        ld = K
    rows = 1
    for n in lead:
        rows *= n
    return t, rows, ld


def linear(x, w, bias=None, act=None, residual=None, out_dtype=None, split=None, out=None):
    """act(x @ w.T + bias) (+ residual).  x (..., K) in w's dtype, w (M, K)
    contiguous, bias fp32.  split=s returns (y[..., :s], y[..., s:]) as two
    separately stored tensors.  out: a (N, G, M) view with unit last stride (e.g. a
    token slice `stream[:, a:b, :]` of a (B, T, d) tensor) that receives the N * G
    output rows in place of a fresh tensor - the kernel writes the slice directly, there
    is no concatenation pass."""
    _need_cuda(x, w, bias, residual, out)
    if x.dtype is not w.dtype:
        raise TypeError(f"linear: x is {x.dtype} but w is {w.dtype}")
    if not w.is_contiguous() or w.dim() != 2:
        raise RuntimeError("linear: w must be a contiguous (M, K) matrix")
    M, K = w.shape
    if x.shape[-1] != K:
        raise RuntimeError(f"linear: x has K={x.shape[-1]}, w has K={K}")
    out_dtype = out_dtype or x.dtype
    lead = x.shape[:-1]
    x2, rows, ldx = _rows2d(x)
    r2, ldr = None, 0
    if residual is not None:
        if residual.dtype is not x.dtype or residual.shape != (*lead, M):
            raise RuntimeError("linear: residual must be (..., M) in x's dtype")
        r2, _, ldr = _rows2d(residual)
    group, gstride = 0, 0
    if out is not None:
        if split is not None or out.dim() != 3 or out.shape[2] != M or out.stride(2) != 1 or out.dtype is not out_dtype \
                or out.shape[0] * out.shape[1] != rows:
            raise RuntimeError("linear: out must be a (N, G, M) view with unit last stride holding all output rows")
        y, y2, ld2, sp = out, None, 0, 0
        group, gstride = out.shape[1], out.stride(0)
        ldy = out.stride(1) if group > 1 else M
    elif split is None:
        y = torch.empty(*lead, M, device=x.device, dtype=out_dtype)
        y2, ld2, sp = None, 0, 0
        ldy = M
    else:
        y = torch.empty(*lead, split, device=x.device, dtype=out_dtype)
        y2 = torch.empty(*lead, M - split, device=x.device, dtype=out_dtype)
        ldy, ld2, sp = split, M - split, split
    with torch.cuda.device(x.device):
        rc = _lib.load().bsrl_linear_grouped(x2.data_ptr(), ldx, w.data_ptr(), _ptr(_f32c(bias, "bias")), _ptr(r2), ldr,
                                             y.data_ptr(), ldy, _ptr(y2), ld2, sp, rows, K, M, _ACT[act],
                                             dt_code(x.dtype), dt_code(out_dtype), group, gstride, _stream(x))
    if not _lib.check(rc, "bsrl_linear"):
        raise Unsupported(f"linear rows={rows} K={K} M={M} dtype={x.dtype}")
    return y if split is None else (y, y2)


def mlp2_supported(K1, d, dtype) -> bool:
    """Shapes bsrl_mlp2 covers: a 64-lane input, d = 128 / 192, 16-bit stream."""
    return dtype in (torch.float16, torch.bfloat16) and K1 == 64 and d in (128, 192)


def mlp2(x, w1, b1, w2, b2, out=None):
    """relu(x w1^T + b1) w2^T + b2 in one launch (bsrl_mlp2; the hidden rows stay on the chip): bit for bit
    linear(linear(x, w1, b1, act="relu"), w2, b2, out=out).  x (.., K1) contiguous, w1 (d, K1), w2 (d, d) in x's dtype,
    b1 / b2 fp32; out: a (N, G, d) slice of a token stream that receives the rows (as in `linear`).  Returns None where
    the shape has no kernel (the caller runs the two Linears)."""
    _need_cuda(x, w1, w2, b1, b2)
    K1, d = x.shape[-1], w2.shape[0]
    if not mlp2_supported(K1, d, x.dtype):
        return None
    if not (x.is_contiguous() and w1.is_contiguous() and w2.is_contiguous()) or w1.dtype is not x.dtype or w2.dtype is not x.dtype:
        raise TypeError("mlp2: x, w1, w2 must be contiguous in one dtype")
    if tuple(w1.shape) != (d, K1) or tuple(w2.shape) != (d, d) or b1.numel() != d or b2.numel() != d:
        raise TypeError(f"mlp2: expected w1 ({d}, {K1}), w2 ({d}, {d}), b1 / b2 ({d},)")
    rows = x.numel() // K1
    group, gstride = 0, 0
    if out is None:
        y = torch.empty(*x.shape[:-1], d, device=x.device, dtype=x.dtype)
        ldy = d
    else:
        if out.dim() != 3 or out.shape[2] != d or out.stride(2) != 1 or out.dtype is not x.dtype or out.shape[0] * out.shape[1] != rows:
            raise TypeError("mlp2: out must be a (N, G, d) view with unit last stride and N * G rows in x's dtype")
        y = out
        group, gstride = out.shape[1], out.stride(0)
        ldy = out.stride(1) if group > 1 else d
    with torch.cuda.device(x.device):
        rc = _lib.load().bsrl_mlp2(x.data_ptr(), K1, w1.data_ptr(), _ptr(_f32c(b1, "b1")), K1, w2.data_ptr(),
                                   _ptr(_f32c(b2, "b2")), y.data_ptr(), ldy, rows, d, dt_code(x.dtype), group, gstride, _stream(x))
    return y if _lib.check(rc, "bsrl_mlp2") else None


def linear_gated(x, w, gate):
    """(x @ w.T) * [gate > 0]: the data gradient of a Linear masked by the ReLU before it, in one
    GEMM (reference fp16_gemm.dgrad_drelu, fp16_gemm.cu:479-518).  x (..., K), w (M, K) contiguous
    (the forward weight transposed), gate (..., M) = the ReLU's forward output; one dtype."""
    _need_cuda(x, w, gate)
    if x.dtype is not w.dtype or gate.dtype is not x.dtype:
        raise TypeError("linear_gated: x, w and gate must share one dtype")
    if not w.is_contiguous() or w.dim() != 2 or x.shape[-1] != w.shape[1]:
        raise RuntimeError("linear_gated: w must be a contiguous (M, K) matrix matching x's K")
    M, K = w.shape
    if gate.shape != (*x.shape[:-1], M):
        raise RuntimeError("linear_gated: gate must be (..., M)")
    x2, rows, ldx = _rows2d(x)
    g2, _, ldg = _rows2d(gate)
    y = torch.empty(*x.shape[:-1], M, device=x.device, dtype=x.dtype)
    with torch.cuda.device(x.device):
        rc = _lib.load().bsrl_linear_gated(x2.data_ptr(), ldx, w.data_ptr(), g2.data_ptr(), ldg, y.data_ptr(), M,
                                           rows, K, M, dt_code(x.dtype), _stream(x))
    if not _lib.check(rc, "bsrl_linear_gated"):
        raise Unsupported(f"linear_gated rows={rows} K={K} M={M} dtype={x.dtype}")
    return y


def attn_fwd(q, k, v, n_heads, key_bias=None, n_valid=None):
    """softmax(q k^T / sqrt(dh) + key_bias) v per head.  q (B, TQ, d), k/v
    (B, T, d): any batch/row strides (views of a packed projection are fine),
    unit last stride.  key_bias (B, T) additive in q's dtype, or n_valid (B,)
    int32 (keys 0..n_valid[b] attendable).  Returns (B, TQ, d) contiguous."""
    _need_cuda(q, k, v, key_bias, n_valid)
    B, TQ, d = q.shape
    T = k.shape[1]
    if k.shape != (B, T, d) or v.shape != (B, T, d) or d % n_heads:
        raise RuntimeError("attn_fwd: shape mismatch")
    for t in (q, k, v):
        if t.stride(2) != 1 or t.dtype is not q.dtype:
            raise RuntimeError("attn_fwd: q/k/v need unit last stride and one dtype")
    if key_bias is not None:
        if key_bias.shape != (B, T) or key_bias.dtype is not q.dtype or not key_bias.is_contiguous():
            raise RuntimeError("attn_fwd: key_bias must be contiguous (B, T) in q's dtype")
    if n_valid is not None:
        if n_valid.shape != (B,) or n_valid.dtype is not torch.int32 or not n_valid.is_contiguous():
            raise RuntimeError("attn_fwd: n_valid must be contiguous int32 (B,)")
    out = torch.empty(B, TQ, d, device=q.device, dtype=q.dtype)
    with torch.cuda.device(q.device):
        rc = _lib.load().bsrl_attn_fwd(q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), k.stride(0), k.stride(1),
                                       v.data_ptr(), v.stride(0), v.stride(1), _ptr(key_bias), _ptr(n_valid),
                                       out.data_ptr(), B, T, TQ, n_heads, d // n_heads, dt_code(q.dtype), _stream(q))
    if not _lib.check(rc, "bsrl_attn_fwd"):
        raise Unsupported(f"attn_fwd T={T} TQ={TQ} H={n_heads} dh={d // n_heads} dtype={q.dtype}")
    return out


def attn_bwd(q, k, v, dout, n_heads, key_bias=None, n_valid=None, out=None):
    """(dq, dk, dv) of attn_fwd for the output gradient dout (B, TQ, d) (reference fp16_gemm.attn29_bwd,
    small_attn.cu:539-571).  q / k / v / dout: any batch / row strides, unit last stride.  out: optional
    (dq, dk, dv) views to write into (e.g. the column slices of one packed q|k|v gradient buffer)."""
    _need_cuda(q, k, v, dout, key_bias, n_valid)
    B, TQ, d = q.shape
    T = k.shape[1]
    if k.shape != (B, T, d) or v.shape != (B, T, d) or dout.shape != (B, TQ, d) or d % n_heads:
        raise RuntimeError("attn_bwd: shape mismatch")
    if out is None:
        out = (torch.empty(B, TQ, d, device=q.device, dtype=q.dtype), torch.empty(B, T, d, device=q.device, dtype=q.dtype),
               torch.empty(B, T, d, device=q.device, dtype=q.dtype))
    dq, dk, dv = out
    if dq.shape != q.shape or dk.shape != k.shape or dv.shape != v.shape:
        raise RuntimeError("attn_bwd: gradient views must have the shapes of q, k, v")
    for t in (q, k, v, dout, dq, dk, dv):
        if t.stride(2) != 1 or t.dtype is not q.dtype:
            raise RuntimeError("attn_bwd: every tensor needs unit last stride and one dtype")
    if key_bias is not None and (key_bias.shape != (B, T) or key_bias.dtype is not q.dtype or not key_bias.is_contiguous()):
        raise RuntimeError("attn_bwd: key_bias must be contiguous (B, T) in q's dtype")
    if n_valid is not None and (n_valid.shape != (B,) or n_valid.dtype is not torch.int32 or not n_valid.is_contiguous()):
        raise RuntimeError("attn_bwd: n_valid must be contiguous int32 (B,)")
    st = lambda t: (t.data_ptr(), t.stride(0), t.stride(1))
    with torch.cuda.device(q.device):
        rc = _lib.load().bsrl_attn_bwd(*st(q), *st(k), *st(v), _ptr(key_bias), _ptr(n_valid), *st(dout), *st(dq), *st(dk),
                                       *st(dv), B, T, TQ, n_heads, d // n_heads, dt_code(q.dtype), _stream(q))
    if not _lib.check(rc, "bsrl_attn_bwd"):
        raise Unsupported(f"attn_bwd T={T} TQ={TQ} H={n_heads} dh={d // n_heads} dtype={q.dtype}")
    return dq, dk, dv


def critic_pool_supported(T, d, n_heads, dtype) -> bool:
    """Shapes bsrl_critic_pool covers (16-bit streams; the fp32 parity path keeps the reference's op order)."""
    return dtype in (torch.float16, torch.bfloat16) and T <= 32 and n_heads <= 16 and d in (128, 192, 256) and d % n_heads == 0


def critic_pool(x_res, ln_weight, ln_bias, eps, qk, key_bias, n_heads):
    """pooled (B, H, d) = per-head attention pool of LN(x_res) under the single query folded into qk (B, H, d)
    (see bsrl_critic_pool: the adapool critic's attention without materialised keys / values)."""
    _need_cuda(x_res, ln_weight, ln_bias, qk, key_bias)
    B, T, d = x_res.shape
    if qk.shape != (B, n_heads, d) or qk.dtype is not x_res.dtype or not (x_res.is_contiguous() and qk.is_contiguous()):
        raise TypeError("critic_pool: x_res (B, T, d) and qk (B, H, d) must be contiguous in one dtype")
    if key_bias is not None and (key_bias.shape != (B, T) or key_bias.dtype is not x_res.dtype or not key_bias.is_contiguous()):
        raise TypeError("critic_pool: key_bias must be contiguous (B, T) in x_res's dtype")
    pooled = torch.empty(B, n_heads, d, device=x_res.device, dtype=x_res.dtype)
    with torch.cuda.device(x_res.device):
        rc = _lib.load().bsrl_critic_pool(x_res.data_ptr(), _f32c(ln_weight, "ln weight").data_ptr(),
                                          _f32c(ln_bias, "ln bias").data_ptr(), float(eps), qk.data_ptr(), _ptr(key_bias),
                                          pooled.data_ptr(), B, T, d, n_heads, dt_code(x_res.dtype), _stream(x_res))
    if not _lib.check(rc, "bsrl_critic_pool"):
        raise Unsupported(f"critic_pool T={T} d={d} H={n_heads} dtype={x_res.dtype}")
    return pooled


def ffn_fused_supported(d, F, dtype) -> bool:
    return bool(_lib.load().bsrl_ffn_fused_supported(d, F, dt_code(dtype)))


def ffn_fused_profitable(d, F, dtype) -> bool:
    """Is the fused FFN kernel the faster route?  Measured on MI355X (fp16, FFN + next LayerNorm): the packed-image
    kernel wins wherever it exists - 0.25 ms against 0.38 for two Linears + LayerNorm at d = 128 (F = 512, 475k rows),
    0.39 against 0.62 at d = 192, 1.27 against 1.80 at d = 256 (1M rows), 10.3 against 11.7 at d = 384 (3.1M rows, GELU);
    the kernel on the plain weights only at d = 128 (0.33 against 0.38 ms; 0.82 against 0.62 at d = 192, 44 against 11.7 at
    d = 384: its per-workgroup row tile is too small for the weight stream)."""
    if ffn_pack_supported(d, F, dtype):
        return True
    return d <= 128 and ffn_fused_supported(d, F, dtype)


def ffn_pack_supported(d, F, dtype) -> bool:
    return dtype in (torch.float16, torch.bfloat16) and _lib.load().bsrl_ffn_pack_size(d, F, dt_code(dtype)) > 0


def ffn_pack_into(img, w0, b0, w2, b2):
    """(Re)build the packed fused FFN's weight image (bsrl_ffn_pack) from w0 (F, d), w2 (d, F) in a 16-bit dtype and
    the fp32 biases INTO `img` (a uint8 buffer of bsrl_ffn_pack_size bytes; None: a new one is allocated) and return
    it.  The owner of a stable image - a module whose forward a captured graph may replay - calls this once per weights
    version with the same buffer, so the address the graph holds never moves and never goes stale."""
    Fh, d = w0.shape
    n = _lib.load().bsrl_ffn_pack_size(d, Fh, dt_code(w0.dtype))
    if n <= 0:
        raise Unsupported(f"ffn_pack d={d} F={Fh} dtype={w0.dtype}")
    if img is None or img.numel() != n or img.device != w0.device:
        img = torch.empty(n, dtype=torch.uint8, device=w0.device)
    with torch.cuda.device(w0.device):
        rc = _lib.load().bsrl_ffn_pack(w0.data_ptr(), _f32c(b0, "b0").data_ptr(), w2.data_ptr(), _f32c(b2, "b2").data_ptr(),
                                       d, Fh, dt_code(w0.dtype), img.data_ptr(), _stream(w0))
    if not _lib.check(rc, "bsrl_ffn_pack"):
        raise Unsupported(f"ffn_pack d={d} F={Fh} dtype={w0.dtype}")
    return img


# Weight images for EAGER callers that hand ffn_fused bare tensors (tests, ConfigPolicy's per-op route), keyed by the
# identity and in-place version of the four tensors.  A refresh of the tensors changes the key and a NEW image is
# built, and old entries are dropped one by one: nothing here is safe to hold in a captured graph - callers that
# capture pass `image=` (fp16_linear.ffn_image keeps one per module at a stable address).
_FFN_IMAGES: dict = {}
_FFN_IMAGES_MAX = 64


def ffn_pack(w0, b0, w2, b2):
    """Weight image of the packed fused FFN for bare tensors; cached while the four tensors are unchanged."""
    key = tuple((t.data_ptr(), t._version, tuple(t.shape), t.dtype) for t in (w0, b0, w2, b2))
    img = _FFN_IMAGES.get(key)
    if img is not None:
        return img
    img = ffn_pack_into(None, w0, b0, w2, b2)
    while len(_FFN_IMAGES) >= _FFN_IMAGES_MAX:
        _FFN_IMAGES.pop(next(iter(_FFN_IMAGES)))          # oldest entry first
    # the key's data pointers stay valid only while the tensors live: hold them with the image
    _FFN_IMAGES[key] = img
    img._bsrl_sources = (w0, b0, w2, b2)
    return img


def ffn_fused(x, h2, w0, b0, w2, b2, act="relu", ln_w=None, ln_b=None, eps=1e-5, packed="auto", want_hidden=False,
              image=None):
    """xo = x + act(h2 w0^T + b0) w2^T + b2; ho = LN(xo) when ln_w is given.
    Returns (xo, ho) (ho None without LN), or None when unsupported.
    want_hidden (packed route only; None is returned where that route has no kernel): (xo, ho, hid) with hid (.., F) the
    activated hidden as the down-projection consumed it, for a backward (the reference's save mode).
    packed: "auto" takes the packed-image kernel (bsrl_ffn_packed: d in {128, 192, 256, 384}, weights streamed straight
    into LDS, 32 rows per wave) where the shape has one, else the kernel on the plain weights; False forces the latter.
    image: the caller's own weight image of (w0, b0, w2, b2) (ffn_pack_into) for the packed kernel - the form for
    callers whose launches a graph replays; without it the image comes from the identity-keyed cache of ffn_pack."""
    _need_cuda(x, h2, w0, w2)
    d = x.shape[-1]
    Fh = w0.shape[0]
    if not (x.is_contiguous() and h2.is_contiguous() and w0.is_contiguous() and w2.is_contiguous()):
        raise RuntimeError("ffn_fused: contiguous tensors required")
    if h2.shape != x.shape or not (h2.dtype is x.dtype and w0.dtype is x.dtype and w2.dtype is x.dtype):
        raise RuntimeError("ffn_fused: h2 must have x's shape, and h2 / w0 / w2 x's dtype")
    if tuple(w0.shape) != (Fh, d) or tuple(w2.shape) != (d, Fh) or b0.numel() != Fh or b2.numel() != d:
        raise RuntimeError(f"ffn_fused: expected w0 ({Fh}, {d}), w2 ({d}, {Fh}), b0 ({Fh},), b2 ({d},)")
    if (ln_w is None) != (ln_b is None) or (ln_w is not None and (ln_w.numel() != d or ln_b.numel() != d)):
        raise RuntimeError(f"ffn_fused: ln_w and ln_b come together, {d} elements each")
    rows = x.numel() // d
    xo = torch.empty_like(x)
    ho = torch.empty_like(x) if ln_w is not None else None
    if packed and ffn_pack_supported(d, Fh, x.dtype):
        img = image if image is not None else ffn_pack(w0, _f32c(b0, "b0"), w2, _f32c(b2, "b2"))
        if img.numel() != _lib.load().bsrl_ffn_pack_size(d, Fh, dt_code(x.dtype)) or img.device != x.device:
            raise RuntimeError("ffn_fused: image does not belong to this shape / dtype / device")
        hid = torch.empty(*x.shape[:-1], Fh, device=x.device, dtype=x.dtype) if want_hidden else None
        with torch.cuda.device(x.device):
            rc = _lib.load().bsrl_ffn_packed(img.data_ptr(), x.data_ptr(), h2.data_ptr(), _ptr(_f32c(ln_w, "ln_w")),
                                             _ptr(_f32c(ln_b, "ln_b")), float(eps), xo.data_ptr(), _ptr(ho), _ptr(hid),
                                             rows, d, Fh, _ACT[act], dt_code(x.dtype), _stream(x))
        if not _lib.check(rc, "bsrl_ffn_packed"):
            return None
        return (xo, ho, hid) if want_hidden else (xo, ho)
    if want_hidden:
        return None
    with torch.cuda.device(x.device):
        rc = _lib.load().bsrl_ffn_fused(x.data_ptr(), h2.data_ptr(), w0.data_ptr(), _f32c(b0, "b0").data_ptr(),
                                        w2.data_ptr(), _f32c(b2, "b2").data_ptr(), _ptr(_f32c(ln_w, "ln_w")),
                                        _ptr(_f32c(ln_b, "ln_b")), float(eps), xo.data_ptr(), _ptr(ho), rows, d, Fh,
                                        _ACT[act], dt_code(x.dtype), _stream(x))
    if not _lib.check(rc, "bsrl_ffn_fused"):
        return None
    return xo, ho


def proj_ffn_supported(d, F, dtype, n_next=0) -> bool:
    """True where the block tail (output projection + LN2 + FFN, optionally the next block's packed projection of
    n_next columns behind it) has a one-kernel form (bsrl_proj_ffn_packed)."""
    return dtype is not torch.float32 and _lib.load().bsrl_proj_ffn_pack_size(d, F, n_next, dt_code(dtype)) > 0


def proj_ffn_pack(wo, bo, w0, b0, w2, b2, wn=None, bn=None):
    """Weight image of proj_ffn_fused (bsrl_proj_ffn_pack) from wo (d, d), w0 (F, d), w2 (d, F), optionally wn
    (n_next, d) - the projection applied to the LayerNorm-ed output, e.g. the next block's packed q|k|v - in a 16-bit
    dtype and the fp32 biases; rebuild once per weights version."""
    _need_cuda(wo, w0, w2, wn)
    Fh, d = w0.shape
    n_next = 0 if wn is None else wn.shape[0]
    n = _lib.load().bsrl_proj_ffn_pack_size(d, Fh, n_next, dt_code(w0.dtype))
    if n <= 0 or tuple(wo.shape) != (d, d) or tuple(w2.shape) != (d, Fh) or not (wo.is_contiguous() and w0.is_contiguous() and w2.is_contiguous()) \
            or (wn is not None and (wn.shape[1] != d or not wn.is_contiguous() or wn.dtype is not w0.dtype or bn is None or bn.numel() != n_next)):
        raise Unsupported(f"proj_ffn_pack d={d} F={Fh} n_next={n_next} dtype={w0.dtype}")
    img = torch.empty(n, dtype=torch.uint8, device=w0.device)
    with torch.cuda.device(w0.device):
        rc = _lib.load().bsrl_proj_ffn_pack(wo.data_ptr(), _f32c(bo, "bo").data_ptr(), w0.data_ptr(), _f32c(b0, "b0").data_ptr(),
                                            w2.data_ptr(), _f32c(b2, "b2").data_ptr(), _ptr(wn), _ptr(_f32c(bn, "bn")), n_next,
                                            d, Fh, dt_code(w0.dtype), img.data_ptr(), _stream(w0))
    if not _lib.check(rc, "bsrl_proj_ffn_pack"):
        raise Unsupported(f"proj_ffn_pack d={d} F={Fh} n_next={n_next} dtype={w0.dtype}")
    return img


def proj_ffn_fused(att, x, image, F, ln2_w, ln2_b, eps2=1e-5, act="relu", ln_w=None, ln_b=None, eps=1e-5, n_next=0,
                   want_ho=True):
    """The tail of a block from the attention output on: x1 = x + att Wo^T + bo, h2 = LN(x1; ln2), xo = x1 +
    act(h2 W0^T + b0) W2^T + b2, ho = LN(xo; ln) when ln_w is given - one kernel, x1 and h2 in registers.  att, x
    (.., d) contiguous; image from proj_ffn_pack; F the hidden width.  n_next > 0 (the image was packed with wn): also
    qo (.., n_next) = ho Wn^T + bn from the same launch; want_ho=False then leaves ho unwritten.
    Returns (xo, ho) or (xo, ho, qo) (ho None where not written)."""
    _need_cuda(att, x, image)
    d = x.shape[-1]
    if not (x.is_contiguous() and att.is_contiguous()) or att.shape != x.shape or att.dtype is not x.dtype:
        raise RuntimeError("proj_ffn_fused: att and x contiguous, one shape, one dtype")
    if image.numel() != _lib.load().bsrl_proj_ffn_pack_size(d, F, n_next, dt_code(x.dtype)) or image.device != x.device:
        raise RuntimeError("proj_ffn_fused: image does not belong to this shape / dtype / device")
    if ln2_w.numel() != d or ln2_b.numel() != d or (ln_w is None) != (ln_b is None) or (n_next > 0 and ln_w is None):
        raise RuntimeError(f"proj_ffn_fused: ln2_w / ln2_b of {d} elements; ln_w and ln_b come together, and with n_next")
    rows = x.numel() // d
    xo = torch.empty_like(x)
    ho = torch.empty_like(x) if ln_w is not None and (want_ho or n_next == 0) else None
    qo = torch.empty(*x.shape[:-1], n_next, device=x.device, dtype=x.dtype) if n_next > 0 else None
    if rows == 0:                      # nothing to launch (an empty tensor has no address to hand over)
        return (xo, ho, qo) if n_next > 0 else (xo, ho)
    with torch.cuda.device(x.device):
        rc = _lib.load().bsrl_proj_ffn_packed(image.data_ptr(), att.data_ptr(), x.data_ptr(), _f32c(ln2_w, "ln2_w").data_ptr(),
                                              _f32c(ln2_b, "ln2_b").data_ptr(), float(eps2), _ptr(_f32c(ln_w, "ln_w")),
                                              _ptr(_f32c(ln_b, "ln_b")), float(eps), xo.data_ptr(), _ptr(ho), _ptr(qo), n_next,
                                              rows, d, F, _ACT[act], dt_code(x.dtype), _stream(x))
    if not _lib.check(rc, "bsrl_proj_ffn_packed"):
        raise Unsupported(f"proj_ffn_fused d={d} F={F} n_next={n_next} dtype={x.dtype}")
    return (xo, ho, qo) if n_next > 0 else (xo, ho)


def ln_proj_supported(d, n_next, dtype) -> bool:
    """True where LayerNorm + a packed projection of n_next columns has a one-kernel form (bsrl_ln_proj_packed)."""
    return dtype is not torch.float32 and _lib.load().bsrl_ln_proj_pack_size(d, n_next, dt_code(dtype)) > 0


def ln_proj_pack(wn, bn):
    """Weight image of ln_proj_fused (bsrl_ln_proj_pack) from wn (n_next, d) in a 16-bit dtype and bn fp32."""
    _need_cuda(wn, bn)
    n_next, d = wn.shape
    n = _lib.load().bsrl_ln_proj_pack_size(d, n_next, dt_code(wn.dtype))
    if n <= 0 or not wn.is_contiguous() or bn.numel() != n_next:
        raise Unsupported(f"ln_proj_pack d={d} n_next={n_next} dtype={wn.dtype}")
    img = torch.empty(n, dtype=torch.uint8, device=wn.device)
    with torch.cuda.device(wn.device):
        rc = _lib.load().bsrl_ln_proj_pack(wn.data_ptr(), _f32c(bn, "bn").data_ptr(), n_next, d, dt_code(wn.dtype), img.data_ptr(),
                                           _stream(wn))
    if not _lib.check(rc, "bsrl_ln_proj_pack"):
        raise Unsupported(f"ln_proj_pack d={d} n_next={n_next} dtype={wn.dtype}")
    return img


def ln_proj_fused(x, image, n_next, ln_w, ln_b, eps=1e-5, want_ho=False):
    """qo (.., n_next) = LayerNorm(x; ln_w, ln_b) Wn^T + bn in one kernel (image from ln_proj_pack); x (.., d)
    contiguous.  Returns (ho, qo): ho = the LayerNorm output when want_ho, else None."""
    _need_cuda(x, image)
    d = x.shape[-1]
    if not x.is_contiguous() or ln_w.numel() != d or ln_b.numel() != d:
        raise RuntimeError(f"ln_proj_fused: x contiguous, ln_w / ln_b of {d} elements")
    if image.numel() != _lib.load().bsrl_ln_proj_pack_size(d, n_next, dt_code(x.dtype)) or image.device != x.device:
        raise RuntimeError("ln_proj_fused: image does not belong to this shape / dtype / device")
    rows = x.numel() // d
    ho = torch.empty_like(x) if want_ho else None
    qo = torch.empty(*x.shape[:-1], n_next, device=x.device, dtype=x.dtype)
    if rows == 0:
        return ho, qo
    with torch.cuda.device(x.device):
        rc = _lib.load().bsrl_ln_proj_packed(image.data_ptr(), x.data_ptr(), _f32c(ln_w, "ln_w").data_ptr(),
                                             _f32c(ln_b, "ln_b").data_ptr(), float(eps), _ptr(ho), qo.data_ptr(), n_next, rows, d,
                                             dt_code(x.dtype), _stream(x))
    if not _lib.check(rc, "bsrl_ln_proj_packed"):
        raise Unsupported(f"ln_proj_fused d={d} n_next={n_next} dtype={x.dtype}")
    return ho, qo


def cfg_embed(obs, wp, bp, wo, bo, T, dtype):
    """Config-model tokenizer: obs (B, obs_dim) fp32 or `dtype` -> tokens (B, T, d)."""
    _need_cuda(obs, wp, wo)
    B = obs.shape[0]
    d, prop_dim = wp.shape
    obj_dim = wo.shape[1]
    if obs.stride(1) != 1 or not (wp.is_contiguous() and wo.is_contiguous()):
        raise RuntimeError("cfg_embed: contiguous rows required")
    if wp.dtype is not dtype or wo.dtype is not dtype:
        raise TypeError("cfg_embed: weights must be in the stream dtype")
    tokens = torch.empty(B, T, d, device=obs.device, dtype=dtype)
    with torch.cuda.device(obs.device):
        rc = _lib.load().bsrl_cfg_embed(obs.data_ptr(), obs.stride(0), dt_code(obs.dtype), wp.data_ptr(),
                                        _ptr(_f32c(bp, "bp")), wo.data_ptr(), _ptr(_f32c(bo, "bo")),
                                        tokens.data_ptr(), B, T, d, prop_dim, obj_dim, dt_code(dtype), _stream(obs))
    if not _lib.check(rc, "bsrl_cfg_embed"):
        raise Unsupported(f"cfg_embed T={T} d={d}")
    return tokens


FRONT_PITCH = 64        # row pitch of note_frontend's padded encoder inputs


def note_frontend(obs, saber_idx, body_idx, dtype, note_geo=False, flux=False, z_asinh=8.0, padded=False):
    """obs (B, 630) fp32 or `dtype` -> (saber_in (B, 2, 49), torso_in (B, 29), leg_in (B, 2, 34),
    note_in (B, 24, 18 | 40), key_bias (B, 29)), all in `dtype`: the forward's preamble in one
    kernel (obs rounding, lane gathers, note-geometry lanes, one-hots, key bias).  padded=True: every
    encoder-input row is 64 wide, zero past its natural width (for a first Linear whose weight columns
    are padded the same way)."""
    _need_cuda(obs, saber_idx, body_idx)
    if obs.dim() != 2 or obs.shape[1] != 630 or obs.stride(1) != 1:
        raise RuntimeError(f"note_frontend: obs must be (B, 630) with unit last stride, got {tuple(obs.shape)}")
    if obs.dtype is not torch.float32 and obs.dtype is not dtype:
        raise TypeError("note_frontend: obs must be fp32 or already in the stream dtype")
    if saber_idx.dtype is not torch.int32 or body_idx.dtype is not torch.int32 or saber_idx.numel() != 94 \
            or body_idx.numel() != 93 or not (saber_idx.is_contiguous() and body_idx.is_contiguous()):
        raise TypeError("note_frontend: saber_idx (94) / body_idx (93) must be contiguous int32 tables")
    B = obs.shape[0]
    mk = lambda *s: torch.empty(*s, device=obs.device, dtype=dtype)
    if padded:
        saber_in, torso_in, leg_in, note_in = mk(B, 2, FRONT_PITCH), mk(B, FRONT_PITCH), mk(B, 2, FRONT_PITCH), mk(B, 24, FRONT_PITCH)
    else:
        saber_in, torso_in, leg_in = mk(B, 2, 49), mk(B, 29), mk(B, 2, 34)
        note_in = mk(B, 24, 40 if note_geo else 18)
    key_bias = mk(B, 29)
    lib = _lib.load()
    entry = lib.bsrl_note_frontend_padded if padded else lib.bsrl_note_frontend
    with torch.cuda.device(obs.device):
        rc = entry(obs.data_ptr(), obs.stride(0), dt_code(obs.dtype), saber_idx.data_ptr(),
                                            body_idx.data_ptr(), int(bool(note_geo)), int(bool(flux)), float(z_asinh),
                                            saber_in.data_ptr(), torso_in.data_ptr(), leg_in.data_ptr(),
                                            note_in.data_ptr(), key_bias.data_ptr(), B, dt_code(dtype), _stream(obs))
    _lib.check(rc, "bsrl_note_frontend_padded" if padded else "bsrl_note_frontend")
    return saber_in, torso_in, leg_in, note_in, key_bias


def sample_heads(logits, head_sizes=None, exp_noise=None, seed=0, offset=0, action=None,
                 need_entropy=True, want_ent_h=False, want_noise=False, counter=None, validate_action=False):
    """Action epilogue on fp32 logits (B, n_heads, K).  action=None samples (Gumbel-max with the
    caller's Exp(1) draws `exp_noise`, or the kernel's Philox stream keyed by (seed, offset));
    otherwise evaluates the given (B, n_heads) int64 / uint8 actions.  counter: a one-element
    int64 device tensor whose value is added to `offset` on the device and advanced by one after
    a sampling launch (a captured launch then draws fresh noise on every replay).
    Returns (action int64, logprob, entropy | None, ent_h | None, noise | None)."""
    _need_cuda(logits, head_sizes, exp_noise, action)
    if logits.dtype is not torch.float32 or logits.dim() != 3 or not logits.is_contiguous():
        raise TypeError("sample_heads: logits must be a contiguous fp32 (B, n_heads, K) tensor")
    B, NH, K = logits.shape
    if head_sizes is not None and (head_sizes.dtype is not torch.int32 or head_sizes.numel() != NH
                                   or not head_sizes.is_contiguous()):
        raise TypeError("sample_heads: head_sizes must be a contiguous int32 (n_heads,) tensor")
    if exp_noise is not None and (exp_noise.dtype is not torch.float32 or exp_noise.shape != logits.shape
                                  or not exp_noise.is_contiguous()):
        raise TypeError("sample_heads: exp_noise must be contiguous fp32 of the logits' shape")
    u8 = 0
    if action is not None:
        if action.shape != (B, NH) or action.dtype not in (torch.int64, torch.uint8) or not action.is_contiguous():
            raise TypeError("sample_heads: action must be a contiguous (B, n_heads) int64 or uint8 tensor")
        u8 = int(action.dtype is torch.uint8)
        if validate_action:             # a host round trip (synchronises): off on the rollout / captured paths
            lo, hi = int(action.min()), int(action.max())
            if lo < 0 or hi >= K:
                raise IndexError(f"sample_heads: action values in [{lo}, {hi}] outside [0, {K}) (the kernel would clamp them)")
    if counter is not None and (counter.dtype is not torch.int64 or counter.numel() != 1 or not counter.is_cuda):
        raise TypeError("sample_heads: counter must be a one-element int64 device tensor")
    dev = logits.device
    act_out = torch.empty(B, NH, device=dev, dtype=torch.int64)
    logprob = torch.empty(B, device=dev, dtype=torch.float32)
    entropy = torch.empty(B, device=dev, dtype=torch.float32) if need_entropy else None
    ent_h = torch.empty(B, NH, device=dev, dtype=torch.float32) if want_ent_h else None
    noise = torch.empty_like(logits) if (want_noise and action is None) else None
    with torch.cuda.device(dev):
        rc = _lib.load().bsrl_sample_heads(logits.data_ptr(), B, NH, K, _ptr(head_sizes), _ptr(exp_noise),
                                           int(seed) & (2 ** 64 - 1), int(offset) & (2 ** 64 - 1), _ptr(counter),
                                           _ptr(action), u8, act_out.data_ptr(), logprob.data_ptr(), _ptr(entropy),
                                           _ptr(ent_h), _ptr(noise), _stream(logits))
        _lib.check(rc, "bsrl_sample_heads")
        if counter is not None and action is None and exp_noise is None:
            rc = _lib.load().bsrl_counter_add(counter.data_ptr(), 1, _stream(logits))
    _lib.check(rc, "bsrl_sample_heads")
    return act_out, logprob, entropy, ent_h, noise


# ---- architecture options: value-residual mix, SimBaV2 row stages -------------------------
def _view2d(t, name):
    """(rows, d, pitch) of a tensor whose last dim is dense and whose leading dims form one
    uniform row pitch (a column slice of a packed q|k|v buffer qualifies)."""
    if t.dim() < 2 or t.stride(-1) != 1:
        raise TypeError(f"{name}: need a tensor with a unit-stride last dim")
    lead = [(n, st) for n, st in zip(t.shape[:-1], t.stride()[:-1]) if n != 1]
    pitch = lead[-1][1] if lead else t.shape[-1]
    for (_, st_outer), (n_inner, st_inner) in zip(lead[:-1], lead[1:]):
        if st_outer != st_inner * n_inner:
            raise TypeError(f"{name}: rows must have one uniform pitch")
    rows = 1
    for n in t.shape[:-1]:
        rows *= n
    return rows, t.shape[-1], pitch


def vres_mix(v, v0, a, b, out=None):
    """out = a * v + b * v0 in fp32, rounded once to v's dtype (reference fp16_linear.vres_mix,
    python/fp16_linear.py:1002-1006).  a, b: fp32 (1,) device tensors.  v / v0 / out may be
    column slices of packed projection buffers; out=None mixes in place into v."""
    _need_cuda(v, v0, a, b, out)
    out = v if out is None else out
    if v0.shape != v.shape or out.shape != v.shape or v0.dtype is not v.dtype or out.dtype is not v.dtype:
        raise TypeError("vres_mix: v, v0 and out must share shape and dtype")
    for s in (a, b):
        if s.dtype is not torch.float32 or s.numel() != 1:
            raise TypeError("vres_mix: a and b must be fp32 tensors with one element")
    rows, d, ldv = _view2d(v, "vres_mix v")
    _, _, ldv0 = _view2d(v0, "vres_mix v0")
    _, _, ldo = _view2d(out, "vres_mix out")
    with torch.cuda.device(v.device):
        rc = _lib.load().bsrl_vres_mix(v.data_ptr(), ldv, v0.data_ptr(), ldv0, a.data_ptr(), b.data_ptr(),
                                       out.data_ptr(), ldo, rows, d, dt_code(v.dtype), _stream(v))
    _lib.check(rc, "bsrl_vres_mix")
    return out


def relu_bwd(g, y):
    """g * [y > 0] (reference fp16_gemm.relu_bwd): the gradient through a ReLU from its saved output."""
    _need_cuda(g, y)
    if g.shape != y.shape or g.dtype is not y.dtype:
        raise TypeError("relu_bwd: g and y must share shape and dtype")
    rows, d, ldg = _view2d(g, "relu_bwd g")
    _, _, ldy = _view2d(y, "relu_bwd y")
    out = torch.empty(g.shape, device=g.device, dtype=g.dtype)
    with torch.cuda.device(g.device):
        rc = _lib.load().bsrl_relu_bwd(g.data_ptr(), ldg, y.data_ptr(), ldy, out.data_ptr(), d, rows, d,
                                       dt_code(g.dtype), _stream(g))
    _lib.check(rc, "bsrl_relu_bwd")
    return out


HS_SCALE_L2N, HS_SCALE_RELU, HS_L2N_LERP = 0, 1, 2


def softmax_expect(logits, centers):
    """sum_i softmax(logits)_i * centers_i per row: the HL-Gauss value readout (reference
    NotePolicy._critic, python/policy.py:1394-1403, `softmax(logits) @ value_centers`).
    logits (rows, n) fp32, centers (n) fp32 -> (rows,) fp32."""
    _need_cuda(logits, centers)
    if logits.dim() != 2 or logits.dtype is not torch.float32 or not logits.is_contiguous():
        raise TypeError("softmax_expect: logits must be a contiguous fp32 (rows, n) tensor")
    rows, n = logits.shape
    if centers.dtype is not torch.float32 or centers.numel() != n or not centers.is_contiguous():
        raise TypeError(f"softmax_expect: centers must be {n} contiguous fp32 values")
    out = torch.empty(rows, device=logits.device, dtype=torch.float32)
    with torch.cuda.device(logits.device):
        rc = _lib.load().bsrl_softmax_expect(logits.data_ptr(), centers.data_ptr(), out.data_ptr(), rows, n, _stream(logits))
    if not _lib.check(rc, "bsrl_softmax_expect"):
        raise Unsupported(f"softmax_expect rows={rows} n={n}")
    return out


def hsphere(op, t, s, c=1.0, x32=None):
    """One fp32 row stage of the SimBaV2 trunk on a GEMM output t (rows, D)
    (reference NotePolicy._trunk_v2, python/policy.py:1140-1155):
      HS_SCALE_L2N  -> (x32 fp32, x in t's dtype) = l2n(t * (s * c))
      HS_SCALE_RELU -> relu(t * (s * c)) in t's dtype
      HS_L2N_LERP   -> sqrt(D) * l2n(x32 + (s * c) * (l2n(t) - x32)) in t's dtype"""
    _need_cuda(t, s, x32)
    if t.dim() != 2 or not t.is_contiguous():
        raise TypeError("hsphere: t must be a contiguous (rows, D) tensor")
    rows, D = t.shape
    s = _f32c(s, "hsphere scaler")
    if s.numel() != D:
        raise TypeError(f"hsphere: scaler has {s.numel()} lanes, rows have {D}")
    x32_in = x32_out = None
    out = torch.empty_like(t)
    if op == HS_SCALE_L2N:
        x32_out = torch.empty(rows, D, device=t.device, dtype=torch.float32)
    elif op == HS_L2N_LERP:
        if x32 is None or x32.dtype is not torch.float32 or x32.shape != t.shape or not x32.is_contiguous():
            raise TypeError("hsphere: HS_L2N_LERP needs the contiguous fp32 x32 of the first stage")
        x32_in = x32
    elif op != HS_SCALE_RELU:
        raise ValueError(f"hsphere: unknown op {op}")
    with torch.cuda.device(t.device):
        rc = _lib.load().bsrl_hsphere(op, t.data_ptr(), s.data_ptr(), float(c), _ptr(x32_in), _ptr(x32_out),
                                      out.data_ptr(), rows, D, dt_code(t.dtype), _stream(t))
    _lib.check(rc, "bsrl_hsphere")
    return (x32_out, out) if op == HS_SCALE_L2N else out


# ---- fused transformer block stack ----------------------------------------------------
def _blocks_desc(n_layers, d, n_heads, ffn, T, act, n_queries, dtype):
    return _lib.BlocksDesc(n_layers=n_layers, d=d, n_heads=n_heads, ffn=ffn, T=T, act=_ACT[act],
                           n_queries=n_queries, dtype=dt_code(dtype))


def blocks_pack_size(n_layers, d, n_heads, ffn, T, act, n_queries, dtype) -> int:
    """Bytes of the fused block stack's weight image; 0 = this shape has no fused kernel."""
    desc = _blocks_desc(n_layers, d, n_heads, ffn, T, act, n_queries, dtype)
    return int(_lib.load().bsrl_blocks_pack_size(desc))


_BLK_FIELDS = ("ln_attn_w", "ln_attn_b", "q_w", "q_b", "k_w", "k_b", "v_w", "v_b", "out_w", "out_b",
               "ln_ffn_w", "ln_ffn_b", "ffn0_w", "ffn0_b", "ffn2_w", "ffn2_b")


def blocks_pack(block_params, image, d, n_heads, ffn, T, act, n_queries, dtype):
    """block_params: per block, the 16 fp32 master tensors in `_BLK_FIELDS` order (contiguous,
    on the device).  Writes the MFMA-fragment-major image into `image` (uint8 tensor of
    blocks_pack_size bytes, 16-byte aligned)."""
    desc = _blocks_desc(len(block_params), d, n_heads, ffn, T, act, n_queries, dtype)
    params = _lib.BlocksParams()
    for l, tensors in enumerate(block_params):
        if len(tensors) != 16:
            raise ValueError("blocks_pack: 16 tensors per block expected")
        for name, t in zip(_BLK_FIELDS, tensors):
            _need_cuda(t)
            setattr(params.blk[l], name, _f32c(t.detach(), name).data_ptr())
    with torch.cuda.device(image.device):
        rc = _lib.load().bsrl_blocks_pack(desc, params, image.data_ptr(), _stream(image))
    if not _lib.check(rc, "bsrl_blocks_pack"):
        raise Unsupported("blocks_pack: shape not covered by the fused block stack")


def blocks_forward(image, x, key_bias, n_layers, n_heads, ffn, act, n_queries, want_res=True):
    """x (B, T, d) 16-bit tokens, key_bias (B, T) same dtype -> (x_out, x_res | None): the whole
    block stack in one launch; x_out is (B, n_queries, d) when n_queries > 0 else (B, T, d)."""
    _need_cuda(image, x, key_bias)
    if x.dim() != 3 or not x.is_contiguous() or not key_bias.is_contiguous() or key_bias.dtype is not x.dtype \
            or key_bias.shape != x.shape[:2]:
        raise RuntimeError("blocks_forward: x (B, T, d) and key_bias (B, T) must be contiguous and of one dtype")
    B, T, d = x.shape
    desc = _blocks_desc(n_layers, d, n_heads, ffn, T, act, n_queries, x.dtype)
    out = torch.empty(B, n_queries if n_queries else T, d, device=x.device, dtype=x.dtype)
    res = torch.empty_like(x) if (want_res and n_queries) else None
    with torch.cuda.device(x.device):
        rc = _lib.load().bsrl_blocks_forward(desc, image.data_ptr(), x.data_ptr(), key_bias.data_ptr(), _ptr(res),
                                             out.data_ptr(), B, _stream(x))
    if not _lib.check(rc, "bsrl_blocks_forward"):
        raise Unsupported("blocks_forward: shape not covered by the fused block stack")
    return out, res
