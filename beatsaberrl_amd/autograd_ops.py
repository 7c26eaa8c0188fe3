"""torch.autograd Functions over the kernel ops: the update (training) side of the op layer.

Each Function pairs a forward kernel with its backward kernels, the way the reference's op layer
does (python/fused_ln.py:56-112 `_LnFn` / `_LnAddFn`; python/fp16_linear.py:442-640 the Linear
Functions with `wgrad` / `wgrad_bgrad` / `dgrad_drelu`; :930-1000 the attention Functions over
`attn29_bwd`).  Gradients of weights and biases are fp32 (they feed fp32 masters), activations'
gradients are in the stream dtype.

What runs where in a backward pass:
  * LayerNorm: `ops.ln_bwd` (dx with the residual-path gradient folded in, dw, db, folded-bias dbb);
  * Linear data gradient: `ops.linear` against the transposed replica, or `ops.linear_gated` when the
    Linear follows a ReLU (the mask rides the GEMM epilogue);
  * Linear weight / bias gradient: `ops.wgrad` on the 16-bit stream (MFMA, LDS transpose loads); on the
    fp32 stream the vendor GEMM through torch (`g.t() @ x`), as the reference does;
  * attention: `ops.attn_bwd`, writing dq | dk | dv into one packed gradient buffer;
  * block FFN with the fused forward kernel (`FusedFfnFn`): the chain's backward over the hidden the kernel wrote, or over
    a recomputed one.
"""
from __future__ import annotations

import torch

from . import fp16_linear as _fl
from . import ops


def _w_for(w: torch.Tensor, dtype):
    """The weight in the stream dtype: fp32 masters are cast per call here (the update path casts once per
    forward; the rollout path's in-place replicas live in fp16_linear)."""
    w = w.detach()
    return w.contiguous() if w.dtype is dtype else w.to(dtype).contiguous()


def _wgrad(g2, x2, need_w, need_b):
    """(dW, db) fp32 for dy = g2 (rows, M), x = x2 (rows, K)."""
    if not (need_w or need_b):
        return None, None
    if g2.dtype is torch.float32:
        dw = g2.t() @ x2 if need_w else None
        db = g2.sum(0) if need_b else None
        return dw, db
    if need_w:
        dw, db = ops.wgrad(g2, x2, want_db=need_b)
        return dw, db
    return None, g2.sum(0, dtype=torch.float32)


def _rows(t):
    return t.reshape(-1, t.shape[-1])


class LnFn(torch.autograd.Function):
    """y = LayerNorm(x) (reference python/fused_ln.py:56-68)."""

    @staticmethod
    def forward(ctx, x, weight, bias, eps):
        y, mean, rstd = ops.ln_fwd(x, weight.detach(), bias.detach(), eps, want_stats=True)
        ctx.save_for_backward(x, weight, mean, rstd)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, mean, rstd = ctx.saved_tensors
        dx, dw, db = ops.ln_bwd(x, dy.contiguous(), weight.detach(), mean, rstd)
        return dx, dw, db, None


class LnResFn(torch.autograd.Function):
    """(x, LayerNorm(x)) for a pre-LN residual stream: x is handed back as it came so that the residual branch
    hangs off this node, and the backward forms grad(x) + LN's dx in ln_bwd's store loop (one rounding, no
    separate add pass over the stream) - the saving the reference takes through `_LnAddFn`
    (python/fused_ln.py:71-108) on its deferred-residual block layout."""

    @staticmethod
    def forward(ctx, x, weight, bias, eps):
        y, mean, rstd = ops.ln_fwd(x, weight.detach(), bias.detach(), eps, want_stats=True)
        ctx.save_for_backward(x, weight, mean, rstd)
        return x.view_as(x), y

    @staticmethod
    def backward(ctx, gx, gy):
        x, weight, mean, rstd = ctx.saved_tensors
        dx, dw, db = ops.ln_bwd(x, gy.contiguous(), weight.detach(), mean, rstd, gx=gx.contiguous())
        return dx, dw, db, None


class LnAddFn(torch.autograd.Function):
    """(x, y) = (a + b (+ b_bias), LayerNorm(x)) (reference python/fused_ln.py:71-108): d/da == d/db ==
    grad(x) + LN's dx, formed in one rounding inside ln_bwd; d/d(b_bias) = its column sums."""

    @staticmethod
    def forward(ctx, a, b, weight, bias, eps, b_bias):
        x, y, mean, rstd = ops.ln_fwd_add(a, b, weight.detach(), bias.detach(), eps,
                                          None if b_bias is None else b_bias.detach(), want_stats=True)
        ctx.save_for_backward(x, weight, mean, rstd)
        return x, y

    @staticmethod
    def backward(ctx, gx, gy):
        x, weight, mean, rstd = ctx.saved_tensors
        want = ctx.needs_input_grad[5]
        r = ops.ln_bwd(x, gy.contiguous(), weight.detach(), mean, rstd, gx=gx.contiguous(), want_dbb=want)
        dx, dw, db = r[:3]
        return dx, dx, dw, db, None, (r[3] if want else None)


class LinearFn(torch.autograd.Function):
    """act(x @ w.T + b) (+ residual), act in {None, "relu"}; w (M, K) and b fp32 masters or any tensors
    autograd tracks (a torch.cat of several masters for a packed projection)."""

    @staticmethod
    def forward(ctx, x, w, b, act, residual, out_f32=False):
        if act not in (None, "relu"):
            raise NotImplementedError("training path: only ReLU epilogues have a backward")
        if act == "relu" and residual is not None:
            raise NotImplementedError("relu + residual epilogue has no backward here")
        w16 = _w_for(w, x.dtype)
        bias = None if b is None else b.detach().float().contiguous()
        y = ops.linear(x, w16, bias, act=act, residual=residual, out_dtype=torch.float32 if out_f32 else None)
        ctx.act = act
        ctx.has_b = b is not None
        ctx.save_for_backward(x, w16, y if act == "relu" else None)
        return y

    @staticmethod
    def backward(ctx, g):
        x, w16, y = ctx.saved_tensors
        g = g.to(x.dtype).contiguous()                         # an fp32 output's gradient re-enters the stream dtype
        if ctx.act == "relu":
            g = ops.relu_bwd(g, y)
        need_x, need_w, need_b, _, need_r = ctx.needs_input_grad[:5]
        dx = ops.linear(g, w16.t().contiguous()) if need_x else None
        dw, db = _wgrad(_rows(g), _rows(x), need_w, need_b and ctx.has_b)
        return dx, dw, db, None, (g if need_r else None), None


class ChainFn(torch.autograd.Function):
    """Linear (ReLU Linear)+ with every ReLU in a GEMM epilogue (reference python/fp16_linear.py:668-767
    `_chain_forward` / backward): forward keeps the post-ReLU hiddens; backward runs, last layer first,
    (dW, db) = wgrad(g, input) and g = (g @ W) * [hidden > 0] as ONE gated GEMM per layer."""

    @staticmethod
    def forward(ctx, x, residual, out_f32, *wb):
        n = len(wb) // 2
        ws = [_w_for(w, x.dtype) for w in wb[0::2]]
        hs = [x]
        h = x
        for i in range(n):
            last = i == n - 1
            bias = wb[2 * i + 1]
            bias = None if bias is None else bias.detach().float().contiguous()
            h = ops.linear(h, ws[i], bias, act=None if last else "relu", residual=residual if last else None,
                           out_dtype=torch.float32 if (last and out_f32) else None)
            if not last:
                hs.append(h)
        ctx.n = n
        ctx.has_b = [wb[2 * i + 1] is not None for i in range(n)]
        ctx.save_for_backward(*hs, *ws)
        return h

    @staticmethod
    def backward(ctx, g):
        n = ctx.n
        hs, ws = ctx.saved_tensors[:n], ctx.saved_tensors[n:]
        g = g.to(hs[0].dtype).contiguous()
        need = ctx.needs_input_grad
        grads = [None] * (2 * n)
        g_res = g if need[1] else None
        for i in range(n - 1, -1, -1):
            dw, db = _wgrad(_rows(g), _rows(hs[i]), need[3 + 2 * i], need[4 + 2 * i] and ctx.has_b[i])
            grads[2 * i], grads[2 * i + 1] = dw, db
            wt = ws[i].t().contiguous()                       # (K_in, M_out): the data gradient is g @ W
            if i > 0:
                g = ops.linear_gated(g, wt, hs[i])             # through the ReLU that produced hs[i]
            elif need[0]:
                g = ops.linear(g, wt)
            else:
                g = None
        return (g, g_res, None, *grads)


class FusedFfnFn(torch.autograd.Function):
    """x + W2 relu(W0 h2 + b0) + b2 with the forward as ONE kernel, the block FFN of the update path when the
    fused FFN is on (reference python/fp16_linear.py:1197-1251 `_FusedFfn`).  The backward is the unfused chain's:
    (dW2, db2) = wgrad(g, hidden), gm = (g @ W2) * [hidden > 0] as one gated GEMM, (dW0, db0) = wgrad(gm, h2),
    dh2 = gm @ W0, dx = g.  save_hidden: the forward kernel also writes the activated hidden for the backward, as the
    reference's does (its mask is hidden > 0); otherwise the forward keeps h2 only and the backward recomputes the
    hidden with the Linear kernel (one more rows x d x F GEMM per step, rows x F activations less held between
    forward and backward).  Shapes without the packed-image kernel always recompute."""

    @staticmethod
    def _image(w0, b0, w2, b2, w0h, b0f, w2h, b2f):
        """The packed kernel's weight image for the update path: one buffer per FFN (held on its first master
        weight), repacked only when a master has changed - torch's in-place counters of the four masters (every
        optimizer step and load moves them) and the global weights version make the key - instead of once per
        forward call from the freshly cast copies."""
        if not ops.ffn_pack_supported(w0h.shape[1], w0h.shape[0], w0h.dtype):
            return None
        key = (_fl._weights_version, w0._version, b0._version, w2._version, b2._version, w0h.dtype, str(w0h.device))
        cache = getattr(w0, "_bsrl_ffn_image_train", None)
        if cache is None:
            cache = w0._bsrl_ffn_image_train = [None, None]
        if cache[0] != key:
            cache[1] = ops.ffn_pack_into(cache[1], w0h, b0f, w2h, b2f)
            cache[0] = key
        return cache[1]

    @staticmethod
    def forward(ctx, x, h2, w0, b0, w2, b2, save_hidden=False):
        w0h, w2h = _w_for(w0, x.dtype), _w_for(w2, x.dtype)
        b0f, b2f = b0.detach().float().contiguous(), b2.detach().float().contiguous()
        xc, hc = x.contiguous(), h2.contiguous()
        img = FusedFfnFn._image(w0, b0, w2, b2, w0h, b0f, w2h, b2f)
        r = ops.ffn_fused(xc, hc, w0h, b0f, w2h, b2f, act="relu", want_hidden=True, image=img) if save_hidden else None
        hid = None
        if r is not None:
            hid = r[2]
        else:
            r = ops.ffn_fused(xc, hc, w0h, b0f, w2h, b2f, act="relu", image=img)
        if r is None:
            raise ops.Unsupported(f"fused FFN d={x.shape[-1]} F={w0.shape[0]} dtype={x.dtype}")
        ctx.has_hid = hid is not None
        if hid is not None:
            ctx.save_for_backward(h2, w0h, w2h, b0f, hid)
        else:
            ctx.save_for_backward(h2, w0h, w2h, b0f)
        return r[0]

    @staticmethod
    def backward(ctx, g):
        if ctx.has_hid:
            h2, w0h, w2h, b0f, hid = ctx.saved_tensors
        else:
            h2, w0h, w2h, b0f = ctx.saved_tensors
            hid = ops.linear(h2, w0h, b0f, act="relu")
        need = ctx.needs_input_grad                              # x, h2, w0, b0, w2, b2
        g = g.contiguous()
        dw2, db2 = _wgrad(_rows(g), _rows(hid), need[4], need[5])
        gm = ops.linear_gated(g, w2h.t().contiguous(), hid)
        del hid
        dw0, db0 = _wgrad(_rows(gm), _rows(h2), need[2], need[3])
        dh2 = ops.linear(gm, w0h.t().contiguous()) if need[1] else None
        return (g if need[0] else None), dh2, dw0, db0, dw2, db2, None


class AttnPackedFn(torch.autograd.Function):
    """Self-attention off the packed (B, T, 3d) projection (reference python/fp16_linear.py:930-965
    `_Attn29Packed`): ONE packed gradient comes back."""

    @staticmethod
    def forward(ctx, qkv, key_bias, n_heads):
        d = qkv.shape[-1] // 3
        out = ops.attn_fwd(qkv[..., :d], qkv[..., d:2 * d], qkv[..., 2 * d:], n_heads, key_bias=key_bias)
        ctx.n_heads = n_heads
        ctx.save_for_backward(qkv, key_bias)
        return out

    @staticmethod
    def backward(ctx, dout):
        qkv, key_bias = ctx.saved_tensors
        d = qkv.shape[-1] // 3
        dqkv = torch.empty_like(qkv)
        ops.attn_bwd(qkv[..., :d], qkv[..., d:2 * d], qkv[..., 2 * d:], dout.contiguous(), ctx.n_heads, key_bias=key_bias,
                     out=(dqkv[..., :d], dqkv[..., d:2 * d], dqkv[..., 2 * d:]))
        return dqkv, None, None


class AttnQKVFn(torch.autograd.Function):
    """q (B, TQ, d) over the packed (B, T, 2d) k|v projection (reference python/fp16_linear.py:967-1000
    `_Attn29QKV`): the final block's lead queries and the critic's single query."""

    @staticmethod
    def forward(ctx, q, kv, key_bias, n_heads):
        d = q.shape[-1]
        out = ops.attn_fwd(q, kv[..., :d], kv[..., d:], n_heads, key_bias=key_bias)
        ctx.n_heads = n_heads
        ctx.save_for_backward(q, kv, key_bias)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, kv, key_bias = ctx.saved_tensors
        d = q.shape[-1]
        dq = torch.empty_like(q)
        dkv = torch.empty_like(kv)
        ops.attn_bwd(q, kv[..., :d], kv[..., d:], dout.contiguous(), ctx.n_heads, key_bias=key_bias,
                     out=(dq, dkv[..., :d], dkv[..., d:]))
        return dq, dkv, None, None
