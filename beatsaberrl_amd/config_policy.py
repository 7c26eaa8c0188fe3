"""ConfigPolicy: the benchmark-config transformer policy on the HIP kernels.

Same module contract as the reference's NotePolicy (python/policy.py:784,
:1179): fp32 master parameters in a state_dict, `forward_stacked(obs) ->
(logits (B, 29, K) fp32, value (B,) fp32)`, a stream dtype switched by an
attribute (`.dtype`; the reference's `.fp16`), 16-bit weight replicas refreshed
per weights version (python/fp16_linear.py:228-246, 349-376).  The
architecture is the textbook pre-LN transformer of the benchmark configs:
one Linear per token type, L blocks, one packed (29*K + 1, d) output matrix
whose last row is the value.

Three routes, all entirely on the C-ABI kernels:
  * "ops":    one kernel per op (tokenizer, LayerNorm, packed QKV linear,
              attention, out-proj + residual, LayerNorm, FFN - one fused
              kernel where the shape has one, else up + act and down +
              residual -, heads; final block pruned to token 0) - any
              supported shape and dtype;
  * "fused":  the whole forward in one persistent kernel reading a packed
              weight image (16-bit dtypes, T = 16 / d = 128);
  * "blocks": tokenizer kernel, then the whole block stack in one persistent
              kernel (final block pruned to token 0), then final LayerNorm and
              heads on the B token-0 rows (16-bit dtypes, T <= 32, d = 128 / 256).
`route="auto"` takes "fused", else "blocks", else "ops", by what the library
supports for the shape."""
from __future__ import annotations

import ctypes

import torch
import torch.nn as nn

from . import _lib, ops
from .fused_ln import FusedLayerNorm

N_ACTION_HEADS = 29      # reference python/policy.py:409
_DTYPES = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


class CfgBlock(nn.Module):
    """Pre-LN block; parameter names follow the reference's Block
    (python/policy.py:492-522): ln_attn, q/k/v/out_proj, ln_ffn, ffn.0, ffn.2."""

    def __init__(self, d, ffn, act):
        super().__init__()
        self.ln_attn = FusedLayerNorm(d)
        self.q_proj = nn.Linear(d, d)
        self.k_proj = nn.Linear(d, d)
        self.v_proj = nn.Linear(d, d)
        self.out_proj = nn.Linear(d, d)
        self.ln_ffn = FusedLayerNorm(d)
        self.ffn = nn.Sequential(nn.Linear(d, ffn), nn.GELU() if act == "gelu" else nn.ReLU(), nn.Linear(ffn, d))


class ConfigPolicy(nn.Module):
    def __init__(self, n_layers=2, d=128, n_heads=4, ffn=512, T=16, n_gears=7, act="gelu", final_ln=False,
                 prop_dim=100, obj_dim=16, dtype="f16", route="auto"):
        super().__init__()
        if act not in ("gelu", "relu"):
            raise ValueError(f"act must be gelu or relu, got {act!r}")
        if d % n_heads:
            raise ValueError(f"d={d} not divisible by n_heads={n_heads}")
        if n_layers > _lib.MAX_LAYERS:
            raise ValueError(f"n_layers <= {_lib.MAX_LAYERS}")
        self.n_layers, self.d, self.n_heads, self.ffn_dim, self.T = n_layers, d, n_heads, ffn, T
        self.n_gears, self.act, self.prop_dim, self.obj_dim = n_gears, act, prop_dim, obj_dim
        self.obs_dim = prop_dim + (T - 1) * obj_dim
        self.n_out = N_ACTION_HEADS * n_gears + 1
        self.prop_embed = nn.Linear(prop_dim, d)
        self.obj_embed = nn.Linear(obj_dim, d)
        self.blocks = nn.ModuleList(CfgBlock(d, ffn, act) for _ in range(n_layers))
        self.final_ln = FusedLayerNorm(d) if final_ln else None
        self.heads = nn.Linear(d, self.n_out)
        self.dtype = dtype            # stream dtype: "f32" | "f16" | "bf16"
        self.route = route            # "auto" | "ops" | "fused" | "blocks"
        self._blocks_image = None     # (key, uint8 image) of the fused block stack
        self._version = 0             # bumped by bump_weights_version()
        self._replica = None          # (version, dtype, device) -> 16-bit weight copies
        self._packed = None           # (version, dtype, device) -> fused-kernel weight image
        self._workspace = None        # scratch of the pruned fused route (grown on demand, then reused)
        # fused route, small batches (B <= 4 x CUs): one persistent launch, one env per wave, the weight image streamed
        # straight into a deep LDS ring - the lowest latency per forward (B = 1: 33 us against 52); same output bits as
        # the throughput forms, so it is on by default.  False: the throughput forms at every batch size
        self.latency_form = True
        # final-block query pruning on the fused and per-op routes (the reference's n_queries path,
        # python/policy.py:533-539): exact; False = every token of the final block computed (fused: one persistent kernel)
        self.prune_final = True
        # fused route, pruned form, key counts given: envs of at most 8 tokens share 16-row tiles in twos, of at most 4 tokens ride behind a 9..12-token env or in fours (same bits)
        self.pack_short = True
        # per-op route: a block's output projection + LN2 + FFN as one kernel where the shape has one (d = 384), and the
        # next block's LN1 + packed q|k|v projection behind it in the same launch
        self.fuse_block_tail = True
        self.fuse_next_proj = True
        self.arch = {"n_layers": n_layers, "d": d, "n_heads": n_heads, "ffn": ffn, "T": T, "n_gears": n_gears,
                     "act": act, "final_ln": bool(final_ln), "prop_dim": prop_dim, "obj_dim": obj_dim}

    # ---- weights ------------------------------------------------------------------
    def bump_weights_version(self):
        """Call after every in-place weight update (optimizer step, load):
        the 16-bit replicas and the packed image are rebuilt on next use
        (the reference's fp16_linear.bump_weights_version)."""
        self._version += 1

    def load_state_dict(self, *a, **k):
        r = super().load_state_dict(*a, **k)
        self.bump_weights_version()
        return r

    def _apply(self, fn, *a, **k):
        r = super()._apply(fn, *a, **k)
        self._replica = self._packed = None
        return r

    def _replicas(self, dt, device):
        """Weights cast to the stream dtype (q|k|v concatenated), biases fp32."""
        key = (self._version, dt, str(device))
        if self._replica is not None and self._replica[0] == key:
            return self._replica[1]
        c = lambda w: w.detach().to(dt).contiguous()
        f = lambda b: b.detach().float().contiguous()
        r = {"prop_w": c(self.prop_embed.weight), "prop_b": f(self.prop_embed.bias),
             "obj_w": c(self.obj_embed.weight), "obj_b": f(self.obj_embed.bias),
             "heads_w": c(self.heads.weight), "heads_b": f(self.heads.bias), "blk": []}
        for blk in self.blocks:
            r["blk"].append({
                "qkv_w": c(torch.cat([blk.q_proj.weight, blk.k_proj.weight, blk.v_proj.weight])),
                "qkv_b": f(torch.cat([blk.q_proj.bias, blk.k_proj.bias, blk.v_proj.bias])),
                "out_w": c(blk.out_proj.weight), "out_b": f(blk.out_proj.bias),
                "w0": c(blk.ffn[0].weight), "b0": f(blk.ffn[0].bias),
                "w2": c(blk.ffn[2].weight), "b2": f(blk.ffn[2].bias)})
            w = r["blk"][-1]
            # the packed fused FFN's weight image lives with the replicas it was built from (one per weights version)
            w["ffn_img"] = (ops.ffn_pack_into(None, w["w0"], w["b0"], w["w2"], w["b2"])
                            if ops.ffn_pack_supported(self.d, self.ffn_dim, dt) else None)
            # ... and the images of the one-kernel block tail (output projection + LN2 + FFN + the next block's
            # projection), built on first use per width of that projection
            w["tail_img"] = {}
        self._replica = (key, r)
        return r

    def _desc(self, dt):
        return _lib.CfgDesc(self.n_layers, self.d, self.n_heads, self.ffn_dim, self.T, self.n_gears,
                            _lib.ACT_GELU if self.act == "gelu" else _lib.ACT_RELU,
                            int(self.final_ln is not None), self.prop_dim, self.obj_dim, ops.dt_code(dt),
                            (0 if self.pack_short else _lib.CFG_NO_PACK) | (0 if self.latency_form else _lib.CFG_NO_LATENCY))

    def fused_supported(self, dt=None) -> bool:
        dt = dt or _DTYPES[self.dtype]
        if dt is torch.float32:
            return False
        return _lib.load().bsrl_cfg_pack_size(ctypes.byref(self._desc(dt))) > 0

    def _blocks_shape(self, dt):
        return dict(d=self.d, n_heads=self.n_heads, ffn=self.ffn_dim, T=self.T, act=self.act, n_queries=1, dtype=dt)

    def blocks_supported(self, dt=None) -> bool:
        dt = dt or _DTYPES[self.dtype]
        if dt is torch.float32:
            return False
        return ops.blocks_pack_size(self.n_layers, **self._blocks_shape(dt)) > 0

    def blocks_image(self, dt, device):
        """Weight image of the fused block stack for the current weights version."""
        key = (self._version, dt, str(device))
        if self._blocks_image is not None and self._blocks_image[0] == key:
            return self._blocks_image[1]
        shape = self._blocks_shape(dt)
        img = torch.empty(ops.blocks_pack_size(self.n_layers, **shape), dtype=torch.uint8, device=device)
        params = [[b.ln_attn.weight, b.ln_attn.bias, b.q_proj.weight, b.q_proj.bias, b.k_proj.weight, b.k_proj.bias,
                   b.v_proj.weight, b.v_proj.bias, b.out_proj.weight, b.out_proj.bias, b.ln_ffn.weight, b.ln_ffn.bias,
                   b.ffn[0].weight, b.ffn[0].bias, b.ffn[2].weight, b.ffn[2].bias] for b in self.blocks]
        ops.blocks_pack(params, img, **shape)
        self._blocks_image = (key, img)
        return img

    def packed_image(self, dt, device):
        """The fused kernel's weight image for the current weights version
        (one cast+permute kernel over the fp32 masters)."""
        key = (self._version, dt, str(device))
        if self._packed is not None and self._packed[0] == key:
            return self._packed[1]
        lib = _lib.load()
        desc = self._desc(dt)
        size = lib.bsrl_cfg_pack_size(ctypes.byref(desc))
        if size <= 0:
            raise ops.Unsupported("fused forward does not support this shape/dtype")
        for p in self.parameters():
            if p.dtype is not torch.float32 or not p.is_contiguous() or p.device != device:
                raise RuntimeError("fused forward needs contiguous fp32 master parameters on the obs device")
        prm = _lib.CfgParams()
        dp = lambda t: t.data_ptr()
        prm.prop_w, prm.prop_b = dp(self.prop_embed.weight), dp(self.prop_embed.bias)
        prm.obj_w, prm.obj_b = dp(self.obj_embed.weight), dp(self.obj_embed.bias)
        for i, blk in enumerate(self.blocks):
            b = prm.blk[i]
            b.ln_attn_w, b.ln_attn_b = dp(blk.ln_attn.weight), dp(blk.ln_attn.bias)
            b.q_w, b.q_b = dp(blk.q_proj.weight), dp(blk.q_proj.bias)
            b.k_w, b.k_b = dp(blk.k_proj.weight), dp(blk.k_proj.bias)
            b.v_w, b.v_b = dp(blk.v_proj.weight), dp(blk.v_proj.bias)
            b.out_w, b.out_b = dp(blk.out_proj.weight), dp(blk.out_proj.bias)
            b.ln_ffn_w, b.ln_ffn_b = dp(blk.ln_ffn.weight), dp(blk.ln_ffn.bias)
            b.ffn0_w, b.ffn0_b = dp(blk.ffn[0].weight), dp(blk.ffn[0].bias)
            b.ffn2_w, b.ffn2_b = dp(blk.ffn[2].weight), dp(blk.ffn[2].bias)
        if self.final_ln is not None:
            prm.final_ln_w, prm.final_ln_b = dp(self.final_ln.weight), dp(self.final_ln.bias)
        prm.heads_w, prm.heads_b = dp(self.heads.weight), dp(self.heads.bias)
        if self._packed is not None and self._packed[1].numel() == size and self._packed[1].device == device:
            img = self._packed[1]          # refresh in place: the address must not move under a captured graph
        else:
            img = torch.empty(size, device=device, dtype=torch.uint8)
        with torch.cuda.device(device):
            rc = lib.bsrl_cfg_pack(ctypes.byref(desc), ctypes.byref(prm), img.data_ptr(),
                                   torch.cuda.current_stream(device).cuda_stream)
        if not _lib.check(rc, "bsrl_cfg_pack"):
            raise ops.Unsupported("bsrl_cfg_pack")
        self._packed = (key, img)
        return img

    # ---- forward ------------------------------------------------------------------
    @torch.no_grad()
    def forward_stacked(self, obs, n_valid=None, route=None):
        """obs (B, obs_dim) fp32 (or the stream dtype) on the GPU; n_valid (B,)
        int32 = attendable object tokens per env (None = all).  Returns
        logits (B, 29, n_gears) fp32 and value (B,) fp32."""
        if not obs.is_cuda:
            raise RuntimeError("ConfigPolicy.forward_stacked runs on the GPU only (no CPU path)")
        if obs.dim() != 2 or obs.shape[1] != self.obs_dim:
            raise RuntimeError(f"obs must be (B, {self.obs_dim}), got {tuple(obs.shape)}")
        if n_valid is not None:
            if n_valid.dtype is not torch.int32 or n_valid.shape != (obs.shape[0],) or not n_valid.is_cuda:
                raise RuntimeError("n_valid must be an int32 (B,) device tensor")
            n_valid = n_valid.contiguous()
        dt = _DTYPES[self.dtype]
        route = route or self.route
        if route == "auto":
            route = "fused" if self.fused_supported(dt) else "blocks" if self.blocks_supported(dt) else "ops"
        if route == "fused":
            return self._forward_fused(obs, n_valid, dt)
        if route == "blocks":
            return self._forward_blocks(obs, n_valid, dt)
        if route != "ops":
            raise ValueError(f"route must be auto/ops/fused/blocks, got {route!r}")
        return self._forward_ops(obs, n_valid, dt)

    def forward(self, obs, n_valid=None):
        logits, value = self.forward_stacked(obs, n_valid)
        return list(logits.unbind(1)), value

    def _forward_fused(self, obs, n_valid, dt):
        B = obs.shape[0]
        img = self.packed_image(dt, obs.device)
        if obs.stride(1) != 1:
            obs = obs.contiguous()
        n_log = N_ACTION_HEADS * self.n_gears
        logits = torch.empty(B, n_log, device=obs.device, dtype=torch.float32)
        value = torch.empty(B, device=obs.device, dtype=torch.float32)
        desc = self._desc(dt)
        lib = _lib.load()
        ws_ptr, ws_bytes = None, 0
        if self.prune_final:
            ws_bytes = lib.bsrl_cfg_workspace_size(ctypes.byref(desc), B)
            ws = self._workspace
            if ws is None or ws.numel() < ws_bytes or ws.device != obs.device:
                ws = self._workspace = torch.empty(ws_bytes, device=obs.device, dtype=torch.uint8)
            ws_ptr = ws.data_ptr()
        with torch.cuda.device(obs.device):
            rc = lib.bsrl_cfg_forward(ctypes.byref(desc), img.data_ptr(), obs.data_ptr(), obs.stride(0),
                                      ops.dt_code(obs.dtype), None if n_valid is None else n_valid.data_ptr(),
                                      logits.data_ptr(), value.data_ptr(), B, ws_ptr, ws_bytes,
                                      torch.cuda.current_stream(obs.device).cuda_stream)
        if not _lib.check(rc, "bsrl_cfg_forward"):
            raise ops.Unsupported("bsrl_cfg_forward")
        return logits.view(B, N_ACTION_HEADS, self.n_gears), value

    def _tokens(self, obs, r, dt):
        """Tokenizer on the GEMM kernels: the obs is rounded once to the stream dtype
        (python/policy.py:1200-1209), then one Linear per token type writes its rows of the
        (B, T, d) stream directly (ops.cfg_embed is the same op as one VALU kernel)."""
        B, T = obs.shape[0], self.T
        o = obs.to(dt)
        x = torch.empty(B, T, self.d, device=obs.device, dtype=dt)
        ops.linear(o[:, :self.prop_dim], r["prop_w"], r["prop_b"], out=x[:, 0:1])
        ops.linear(o[:, self.prop_dim:].reshape(B * (T - 1), self.obj_dim), r["obj_w"], r["obj_b"], out=x[:, 1:])
        return x

    def _forward_blocks(self, obs, n_valid, dt):
        B, T = obs.shape[0], self.T
        r = self._replicas(dt, obs.device)
        if obs.dtype not in (torch.float32, dt):
            obs = obs.float()
        x = self._tokens(obs, r, dt)                                                          # (B, T, d)
        # additive key bias of the padding mask: tokens 0..n_valid attendable (exp(-16384) == 0 in fp32)
        if n_valid is None:
            bias = torch.zeros(B, T, device=obs.device, dtype=dt)
        else:
            pos = torch.arange(T, device=obs.device, dtype=torch.int32)
            bias = ((pos[None, :] > n_valid[:, None]).to(dt) * -16384.0).contiguous()
        h, _ = ops.blocks_forward(self.blocks_image(dt, obs.device), x, bias, self.n_layers, self.n_heads, self.ffn_dim,
                                  self.act, 1, want_res=False)                                 # (B, 1, d)
        h = h.view(B, self.d)
        if self.final_ln is not None:
            h = ops.ln_fwd(h, self.final_ln.weight, self.final_ln.bias, self.final_ln.eps)
        n_log = N_ACTION_HEADS * self.n_gears
        logits, value = ops.linear(h, r["heads_w"], r["heads_b"], out_dtype=torch.float32, split=n_log)
        return logits.view(B, N_ACTION_HEADS, self.n_gears), value.view(B)

    def _forward_ops(self, obs, n_valid, dt):
        B, T, d = obs.shape[0], self.T, self.d
        r = self._replicas(dt, obs.device)
        if obs.dtype not in (torch.float32, dt):
            obs = obs.float()
        x = self._tokens(obs, r, dt)                                                          # (B, T, d)
        h = None                # LN1 of the block, when the previous block's kernel wrote it
        proj = None             # the block's packed projection of h (q|k|v, or k|v for the pruned final block), likewise
        L = len(self.blocks)
        for i, (blk, w) in enumerate(zip(self.blocks, r["blk"])):
            pruned = self.prune_final and i + 1 == L
            if proj is None:
                # Row slices of the packed q|k|v weight are contiguous views: keys and values only for a pruned block
                lo = d if pruned else 0
                if h is None and self.fuse_block_tail and self.fuse_next_proj and ops.ln_proj_supported(d, 3 * d - lo, dt):
                    # LN1 + the packed projection in one kernel (LN1 itself written only for the pruned block's query row)
                    img = w["tail_img"].get(("lead", lo))
                    if img is None:
                        img = w["tail_img"][("lead", lo)] = ops.ln_proj_pack(w["qkv_w"][lo:], w["qkv_b"][lo:])
                    h, proj = ops.ln_proj_fused(x, img, 3 * d - lo, blk.ln_attn.weight.detach(), blk.ln_attn.bias.detach(),
                                                blk.ln_attn.eps, want_ho=pruned)
                else:
                    if h is None:
                        h = ops.ln_fwd(x, blk.ln_attn.weight, blk.ln_attn.bias, blk.ln_attn.eps)
                    proj = ops.linear(h, w["qkv_w"][lo:], w["qkv_b"][lo:])
            if pruned:
                # Only token 0 of the final block is read (the reference's n_queries path, python/policy.py:533-539:
                # exact, masking is key-side only): keys and values of every token, the query, the output projection,
                # LN2 and the FFN of token 0 alone.
                q0 = ops.linear(h[:, 0], w["qkv_w"][:d], w["qkv_b"][:d])                      # (B, d), rows T*d apart
                att = ops.attn_fwd(q0.view(B, 1, d), proj[..., :d], proj[..., d:], self.n_heads, n_valid=n_valid)
                x = ops.linear(att.view(B, d), w["out_w"], w["out_b"], residual=x[:, 0]).view(B, 1, d)
                proj = None
            else:
                att = ops.attn_fwd(proj[..., :d], proj[..., d:2 * d], proj[..., 2 * d:], self.n_heads, n_valid=n_valid)
                proj = None
                if self.fuse_block_tail and ops.proj_ffn_supported(d, self.ffn_dim, dt):
                    # output projection + residual, LN2, FFN, the next block's LN1 and its packed projection in one
                    # kernel (k|v only, and LN1 written for the query row, when that block is the pruned final one)
                    nblk = self.blocks[i + 1] if i + 1 < L else None
                    nxt_pruned = self.prune_final and i + 2 == L
                    lo = d if nxt_pruned else 0
                    n_next = (3 * d - lo) if nblk is not None and self.fuse_next_proj else 0
                    img = w["tail_img"].get(n_next)
                    if img is None:
                        wn = r["blk"][i + 1] if n_next else None
                        img = w["tail_img"][n_next] = ops.proj_ffn_pack(
                            w["out_w"], w["out_b"], w["w0"], w["b0"], w["w2"], w["b2"],
                            wn["qkv_w"][lo:] if wn else None, wn["qkv_b"][lo:] if wn else None)
                    res = ops.proj_ffn_fused(att, x, img, self.ffn_dim, blk.ln_ffn.weight.detach(), blk.ln_ffn.bias.detach(),
                                             blk.ln_ffn.eps, act=self.act,
                                             ln_w=nblk.ln_attn.weight.detach() if nblk is not None else None,
                                             ln_b=nblk.ln_attn.bias.detach() if nblk is not None else None,
                                             eps=nblk.ln_attn.eps if nblk is not None else 1e-5, n_next=n_next,
                                             want_ho=nxt_pruned or n_next == 0)
                    x, h = res[0], res[1]
                    proj = res[2] if n_next else None
                    continue
                x = ops.linear(att, w["out_w"], w["out_b"], residual=x)                       # x + out(att)
            h2 = ops.ln_fwd(x, blk.ln_ffn.weight, blk.ln_ffn.bias, blk.ln_ffn.eps)
            fused = h = None
            if dt is not torch.float32 and ops.ffn_fused_profitable(d, self.ffn_dim, dt):
                # the fused kernel also writes the next block's LN1 (same arithmetic as ln_fwd on the rounded stream)
                nxt = self.blocks[i + 1].ln_attn if i + 1 < len(self.blocks) else None
                fused = ops.ffn_fused(x, h2, w["w0"], w["b0"], w["w2"], w["b2"], act=self.act,
                                      ln_w=nxt.weight.detach() if nxt is not None else None,
                                      ln_b=nxt.bias.detach() if nxt is not None else None,
                                      eps=nxt.eps if nxt is not None else 1e-5, image=w["ffn_img"])
            if fused is not None:
                x, h = fused
            else:
                hid = ops.linear(h2, w["w0"], w["b0"], act=self.act)                          # (B, T, ffn)
                x = ops.linear(hid, w["w2"], w["b2"], residual=x)
        h = x[:, 0]                                                                           # (B, d), row stride T*d
        if self.final_ln is not None:
            h = ops.ln_fwd(h.contiguous(), self.final_ln.weight, self.final_ln.bias, self.final_ln.eps)
        n_log = N_ACTION_HEADS * self.n_gears
        logits, value = ops.linear(h, r["heads_w"], r["heads_b"], out_dtype=torch.float32, split=n_log)
        return logits.view(B, N_ACTION_HEADS, self.n_gears), value.view(B)

    # ---- construction helpers --------------------------------------------------------
    @classmethod
    def from_spec(cls, spec, **kw):
        """spec: any object with the fields of the config description
        (n_layers, d, n_heads, ffn, T, n_gears, act, final_ln, prop_dim, obj_dim)."""
        return cls(spec.n_layers, spec.d, spec.n_heads, spec.ffn, spec.T, spec.n_gears, spec.act, spec.final_ln,
                   spec.prop_dim, spec.obj_dim, **kw)
