"""ctypes binding of libbsrl_hip.so (the only route from Python to the kernels).

There is no fallback: if the library has not been built, load() raises."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libbsrl_hip.so")
ABI_VERSION = 17
CFG_NO_PACK = 1                 # bsrl_cfg_desc.flags: one env per tile in the fused forward
CFG_NO_LATENCY = 2              # bsrl_cfg_desc.flags: small batches take the throughput forms too
CFG_STATIC_MAX_ENVS = 16384     # BSRL_CFG_STATIC_MAX_ENVS: batch limit of bsrl_cfg_forward_static

F32, F16, BF16 = 0, 1, 2
ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2
MAX_LAYERS = 8

_p, _i64, _i32, _f = C.c_void_p, C.c_int64, C.c_int, C.c_float


class CfgDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "d", "n_heads", "ffn", "T", "n_gears", "act", "final_ln",
                                         "prop_dim", "obj_dim", "dtype", "flags")]


class _Blk(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("ln_attn_w", "ln_attn_b", "q_w", "q_b", "k_w", "k_b", "v_w", "v_b",
                                          "out_w", "out_b", "ln_ffn_w", "ln_ffn_b", "ffn0_w", "ffn0_b",
                                          "ffn2_w", "ffn2_b")]


class CfgParams(C.Structure):
    _fields_ = ([(n, C.c_void_p) for n in ("prop_w", "prop_b", "obj_w", "obj_b")]
                + [("blk", _Blk * MAX_LAYERS)]
                + [(n, C.c_void_p) for n in ("final_ln_w", "final_ln_b", "heads_w", "heads_b")])


class BlocksDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "d", "n_heads", "ffn", "T", "act", "n_queries", "dtype")]


class BlocksParams(C.Structure):
    _fields_ = [("blk", _Blk * MAX_LAYERS)]


# name -> (restype, argtypes); must list every symbol include/bsrl.h declares
SIGNATURES = {
    "bsrl_version": (_i32, []),
    "bsrl_last_error": (C.c_char_p, []),
    "bsrl_ln_fwd": (_i32, [_p, _p, _p, _p, _p, _p, _i64, _i64, _f, _i32, _p]),
    "bsrl_ln_fwd_add": (_i32, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _f, _i32, _p]),
    "bsrl_linear": (_i32, [_p, _i64, _p, _p, _p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i64, _i64,
                           _i32, _i32, _i32, _p]),
    "bsrl_linear_grouped": (_i32, [_p, _i64, _p, _p, _p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i64, _i64,
                                   _i32, _i32, _i32, _i64, _i64, _p]),
    "bsrl_mlp2": (_i32, [_p, _i64, _p, _p, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, _i64, _i64, _p]),
    "bsrl_attn_fwd": (_i32, [_p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _p, _p,
                             _i64, _i64, _i64, _i64, _i64, _i32, _p]),
    "bsrl_ffn_fused": (_i32, [_p, _p, _p, _p, _p, _p, _p, _p, _f, _p, _p, _i64, _i64, _i64, _i32, _i32, _p]),
    "bsrl_ffn_fused_supported": (_i32, [_i64, _i64, _i32]),
    "bsrl_ffn_pack_size": (_i64, [_i64, _i64, _i32]),
    "bsrl_ffn_pack": (_i32, [_p, _p, _p, _p, _i64, _i64, _i32, _p, _p]),
    "bsrl_ffn_packed": (_i32, [_p, _p, _p, _p, _p, _f, _p, _p, _p, _i64, _i64, _i64, _i32, _i32, _p]),
    "bsrl_ln_proj_pack_size": (_i64, [_i64, _i64, _i32]),
    "bsrl_ln_proj_pack": (_i32, [_p, _p, _i64, _i64, _i32, _p, _p]),
    "bsrl_ln_proj_packed": (_i32, [_p, _p, _p, _p, _f, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "bsrl_proj_ffn_pack_size": (_i64, [_i64, _i64, _i64, _i32]),
    "bsrl_proj_ffn_pack": (_i32, [_p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i32, _p, _p]),
    "bsrl_proj_ffn_packed": (_i32, [_p, _p, _p, _p, _p, _f, _p, _p, _f, _p, _p, _p, _i64, _i64, _i64, _i64, _i32, _i32, _p]),
    "bsrl_cfg_embed": (_i32, [_p, _i64, _i32, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i32, _p]),
    "bsrl_cfg_pack_size": (_i64, [C.POINTER(CfgDesc)]),
    "bsrl_cfg_pack": (_i32, [C.POINTER(CfgDesc), C.POINTER(CfgParams), _p, _p]),
    "bsrl_cfg_workspace_size": (_i64, [C.POINTER(CfgDesc), _i64]),
    "bsrl_cfg_forward": (_i32, [C.POINTER(CfgDesc), _p, _p, _i64, _i32, _p, _p, _p, _i64, _p, _i64, _p]),
    "bsrl_cfg_forward_static": (_i32, [C.POINTER(CfgDesc), _p, _p, _i64, _i32, _p, _p, _p, _i64, _p]),
    "bsrl_blocks_pack_size": (_i64, [C.POINTER(BlocksDesc)]),
    "bsrl_blocks_pack": (_i32, [C.POINTER(BlocksDesc), C.POINTER(BlocksParams), _p, _p]),
    "bsrl_blocks_forward": (_i32, [C.POINTER(BlocksDesc), _p, _p, _p, _p, _p, _i64, _p]),
    "bsrl_note_frontend": (_i32, [_p, _i64, _i32, _p, _p, _i32, _i32, _f, _p, _p, _p, _p, _p, _i64, _i32, _p]),
    "bsrl_note_frontend_padded": (_i32, [_p, _i64, _i32, _p, _p, _i32, _i32, _f, _p, _p, _p, _p, _p, _i64, _i32, _p]),
    "bsrl_counter_add": (_i32, [_p, C.c_uint64, _p]),
    "bsrl_sample_heads": (_i32, [_p, _i64, _i64, _i64, _p, _p, C.c_uint64, C.c_uint64, _p, _p, _i32,
                                 _p, _p, _p, _p, _p, _p]),
    "bsrl_critic_pool": (_i32, [_p, _p, _p, C.c_float, _p, _p, _p, _i64, _i64, _i64, _i64, _i32, _p]),
    "bsrl_ln_bwd_workspace_size": (_i64, [_i64]),
    "bsrl_ln_bwd": (_i32, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i32, _p]),
    "bsrl_attn_bwd": (_i32, [_p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _p, _p, _i64, _i64,
                             _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _p]),
    "bsrl_linear_gated": (_i32, [_p, _i64, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _i32, _p]),
    "bsrl_relu_bwd": (_i32, [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i32, _p]),
    "bsrl_wgrad_workspace_size": (_i64, [_i64, _i64]),
    "bsrl_wgrad": (_i32, [_p, _i64, _p, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "bsrl_vres_mix": (_i32, [_p, _i64, _p, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "bsrl_hsphere": (_i32, [_i32, _p, _p, C.c_float, _p, _p, _p, _i64, _i64, _i32, _p]),
    "bsrl_softmax_expect": (_i32, [_p, _p, _p, _i64, _i64, _p]),
}

_lib = None


def load():
    """Load the library once; raise (never fall back) when it is missing or stale."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} not found: the HIP kernels are not built. Run `python -m beatsaberrl_amd.build` "
            "(there is no CPU or torch fallback for the kernel path).")
    # torch first: it ships its own HIP runtime, and the library must bind to THAT copy (the one that owns torch's
    # device memory and streams).  Loaded the other way round, the system runtime comes in with the library, torch
    # brings a second one, and launches fail with "no ROCm-capable device is detected".
    import torch  # noqa: F401
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)        # AttributeError here = a symbol the header declares is missing
        fn.restype, fn.argtypes = res, args
    v = lib.bsrl_version()
    if v != ABI_VERSION:
        raise RuntimeError(f"libbsrl_hip.so ABI version {v}, Python binding expects {ABI_VERSION}: rebuild")
    _lib = lib
    return lib


def check(rc: int, name: str) -> bool:
    """True = enqueued, False = shape unsupported by the kernel set; raises on errors."""
    if rc == 0:
        return True
    if rc > 0:
        return False
    raise RuntimeError(f"{name} failed ({rc}): {load().bsrl_last_error().decode()}")
