"""FusedLayerNorm: nn.LayerNorm parameters, HIP kernels for the arithmetic.

Mirrors the reference's module of the same name (python/fused_ln.py:110-164):
a subclass of nn.LayerNorm, so state_dict keys, parameter names and
checkpoints are unchanged; weight/bias stay fp32 whatever the activation
dtype; `forward_add(a, b, b_bias)` returns (a + b, LayerNorm(a + b)) from one
pass.  With grad mode on, both run as autograd Functions over the backward
kernel (the reference's `_LnFn` / `_LnAddFn`, python/fused_ln.py:56-108).  Unlike
the reference there is no stock-torch fallback: a tensor that is not on the GPU,
or a missing kernel library, raises."""
from __future__ import annotations

import torch
import torch.nn as nn

from . import ops
from .autograd_ops import LnAddFn, LnFn


class FusedLayerNorm(nn.LayerNorm):
    def _check(self, x):
        if len(self.normalized_shape) != 1 or not self.elementwise_affine:
            raise RuntimeError("FusedLayerNorm: 1-D affine LayerNorm only")
        if not x.is_cuda:
            raise RuntimeError("FusedLayerNorm runs on the GPU only (no CPU path)")
        if x.shape[-1] != self.normalized_shape[0]:
            raise RuntimeError(f"FusedLayerNorm: last dim {x.shape[-1]} != {self.normalized_shape[0]}")

    def forward(self, x):
        self._check(x)
        if torch.is_grad_enabled() and (x.requires_grad or self.weight.requires_grad):
            return LnFn.apply(x.contiguous(), self.weight, self.bias, self.eps)
        return ops.ln_fwd(x.contiguous(), self.weight.detach(), self.bias.detach(), self.eps)

    def forward_add(self, a, b, b_bias=None):
        """(x, LayerNorm(x)) with x = round(a + (b + b_bias)); b_bias is an
        optional fp32 (d,) vector (the producer Linear's un-added bias)."""
        self._check(a)
        if torch.is_grad_enabled() and (a.requires_grad or b.requires_grad or self.weight.requires_grad):
            return LnAddFn.apply(a.contiguous(), b.contiguous(), self.weight, self.bias, self.eps, b_bias)
        return ops.ln_fwd_add(a.contiguous(), b.contiguous(), self.weight.detach(), self.bias.detach(), self.eps,
                              None if b_bias is None else b_bias.detach())
