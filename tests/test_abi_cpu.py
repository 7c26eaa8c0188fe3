"""No-GPU checks of the C-ABI boundary: the library loads, exports every symbol
include/bsrl.h declares, and rejects bad arguments before touching the device."""
import ctypes
import os
import re

import pytest

from beatsaberrl_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "bsrl.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bsrl_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    names = _declared()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/bsrl.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "Python binding table and header disagree"


def test_version_and_error_string(lib):
    assert lib.bsrl_version() == _lib.ABI_VERSION
    assert isinstance(lib.bsrl_last_error(), bytes)


def test_argument_errors_are_reported_without_a_device(lib):
    rc = lib.bsrl_ln_fwd(None, None, None, None, None, None, 4, 128, 1e-5, _lib.F16, None)
    assert rc == -1 and b"null" in lib.bsrl_last_error()
    rc = lib.bsrl_linear(1, 8, 1, None, None, 0, 1, 8, None, 0, 0, 4, 0, 8, 0, _lib.F16, _lib.F16, None)
    assert rc == -1 and b"shape" in lib.bsrl_last_error()
    rc = lib.bsrl_linear(1, 4, 1, None, None, 0, 1, 8, None, 0, 0, 4, 8, 8, 0, _lib.F16, _lib.F16, None)
    assert rc == -1 and b"stride" in lib.bsrl_last_error()
    rc = lib.bsrl_attn_fwd(1, 0, 0, 1, 0, 0, 1, 0, 0, None, None, 1, 2, 16, 17, 4, 32, _lib.F16, None)
    assert rc == -1
    # zero rows: nothing to do, no launch
    assert lib.bsrl_ln_fwd(16, 16, 16, 16, None, None, 0, 128, 1e-5, _lib.F16, None) == 0
    # unsupported shapes are > 0, not errors
    assert lib.bsrl_ln_fwd(16, 16, 16, 16, None, None, 4, 129, 1e-5, _lib.F16, None) > 0
    assert lib.bsrl_attn_fwd(16, 8, 8, 16, 8, 8, 16, 8, 8, None, None, 16, 2, 64, 64, 4, 32, _lib.F16, None) > 0


def test_new_entry_points_reject_bad_arguments_without_a_device(lib):
    C = ctypes
    # front end: null pointers, short rows, obs dtype that is neither fp32 nor the stream dtype, bad z scale
    args = [16, 630, _lib.F32, 16, 16, 1, 0, C.c_float(8.0), 16, 16, 16, 16, 16, 4, _lib.F16, None]
    for entry in (lib.bsrl_note_frontend, lib.bsrl_note_frontend_padded):
        bad = list(args); bad[0] = None
        assert entry(*bad) == -1 and b"null" in lib.bsrl_last_error()
        bad = list(args); bad[1] = 629
        assert entry(*bad) == -1
        bad = list(args); bad[2] = _lib.BF16
        assert entry(*bad) == -1 and b"stream dtype" in lib.bsrl_last_error()
        bad = list(args); bad[7] = C.c_float(0.0)
        assert entry(*bad) == -1
        ok = list(args); ok[13] = 0
        assert entry(*ok) == 0                                  # B == 0: nothing to do
    # action epilogue: K and head-count limits, sampling without an output
    assert lib.bsrl_sample_heads(16, 4, 29, 9, None, None, 0, 0, None, None, 0, 16, 16, None, None, None, None) == -1
    assert lib.bsrl_sample_heads(16, 4, 33, 7, None, None, 0, 0, None, None, 0, 16, 16, None, None, None, None) == -1
    assert lib.bsrl_sample_heads(16, 4, 29, 7, None, None, 0, 0, None, None, 0, None, 16, None, None, None, None) == -1
    assert lib.bsrl_sample_heads(16, 0, 29, 7, None, None, 0, 0, None, None, 0, 16, 16, None, None, None, None) == 0
    assert lib.bsrl_counter_add(None, 1, None) == -1
    # value-residual mix and SimBaV2 row stages: null pointers, pitches below the row width, unknown op
    assert lib.bsrl_vres_mix(16, 8, 16, 8, None, 16, 16, 8, 4, 8, _lib.F16, None) == -1
    assert lib.bsrl_vres_mix(16, 4, 16, 8, 16, 16, 16, 8, 4, 8, _lib.F16, None) == -1 and b"pitches" in lib.bsrl_last_error()
    assert lib.bsrl_vres_mix(16, 8, 16, 8, 16, 16, 16, 8, 0, 8, _lib.F16, None) == 0
    assert lib.bsrl_hsphere(7, 16, 16, 1.0, None, 16, 16, 4, 8, _lib.F32, None) == -1 and b"unknown op" in lib.bsrl_last_error()
    assert lib.bsrl_hsphere(0, 16, 16, 1.0, None, None, 16, 4, 8, _lib.F32, None) == -1
    assert lib.bsrl_hsphere(2, 16, 16, 1.0, None, None, 16, 4, 8, _lib.F32, None) == -1
    assert lib.bsrl_hsphere(1, 16, 16, 1.0, None, None, 16, 0, 8, _lib.F32, None) == 0
    # backward entry points: null pointers, bad shapes and dtypes are refused before any launch
    assert lib.bsrl_ln_bwd_workspace_size(192) == 2048 * 3 * 192 * 4 and lib.bsrl_ln_bwd_workspace_size(0) == 0
    assert lib.bsrl_ln_bwd(16, 16, 16, 16, 16, None, 16, 16, 16, None, None, 4, 128, _lib.F16, None) == -1
    assert lib.bsrl_ln_bwd(16, 16, 16, 16, 16, None, 16, 16, 16, None, 16, 4, 0, _lib.F16, None) == -1
    assert lib.bsrl_ln_bwd(16, 16, 16, 16, 16, None, 16, 16, 16, None, 16, 4, 100, _lib.F16, None) == 1      # d % 8 != 0: unsupported
    assert lib.bsrl_wgrad_workspace_size(768, 192) == 128 * (768 * 192 + 768) * 4
    assert lib.bsrl_wgrad(16, 8, 16, 8, 16, None, 16, 4, 8, 8, _lib.F32, None) == -1 and b"F16 or BF16" in lib.bsrl_last_error()
    assert lib.bsrl_wgrad(16, 4, 16, 8, 16, None, 16, 4, 8, 8, _lib.F16, None) == -1
    assert lib.bsrl_wgrad(16, 8, 16, 8, 16, None, None, 4, 8, 8, _lib.F16, None) == -1
    assert lib.bsrl_linear_gated(16, 8, 16, None, 8, 16, 8, 4, 8, 8, _lib.F16, None) == -1
    assert lib.bsrl_linear_gated(16, 8, 16, 16, 4, 16, 8, 4, 8, 8, _lib.F16, None) == -1
    assert lib.bsrl_linear_gated(16, 8, 16, 16, 8, 16, 8, 0, 8, 8, _lib.F16, None) == 0
    assert lib.bsrl_relu_bwd(16, 8, None, 8, 16, 8, 4, 8, _lib.F16, None) == -1
    assert lib.bsrl_relu_bwd(16, 8, 16, 8, 16, 8, 0, 8, _lib.F16, None) == 0
    ab = lambda T, TQ, dh, dt, q=16: lib.bsrl_attn_bwd(q, 96, 96, 16, 96, 96, 16, 96, 96, None, None, 16, 96, 96,
                                                      16, 96, 96, 16, 96, 96, 16, 96, 96, 4, T, TQ, 1, dh, dt, None)
    assert ab(29, 30, 32, _lib.F16) == -1 and ab(29, 29, 32, _lib.F16, q=None) == -1
    assert ab(49, 5, 32, _lib.F16) == 1 and ab(29, 5, 40, _lib.F16) == 1 and ab(29, 5, 64, _lib.F32) == 1      # unsupported shapes
    # critic pool: null pointers, heads that do not divide d, shapes outside the MFMA form (reported as unsupported)
    cp = lambda T, d, H, dt, x=16, B=4: lib.bsrl_critic_pool(x, 16, 16, C.c_float(1e-5), 16, None, 16, B, T, d, H, dt, None)
    assert cp(29, 192, 4, _lib.F16, x=None) == -1 and b"null" in lib.bsrl_last_error()
    assert cp(29, 192, 5, _lib.F16) == -1 and cp(0, 192, 4, _lib.F16) == -1 and cp(29, 192, 4, 9) == -1
    assert cp(29, 192, 4, _lib.F32) == 1 and cp(33, 192, 4, _lib.F16) == 1 and cp(29, 96, 3, _lib.F16) == 1
    assert cp(29, 192, 4, _lib.F16, B=0) == 0
    # grouped linear: the group must divide the rows, fit its stride and exclude a split output
    g = lambda rows, grp, gs, y2=None, split=0: lib.bsrl_linear_grouped(
        16, 8, 16, None, None, 0, 16, 8, y2, 8 if y2 else 0, split, rows, 8, 8, 0, _lib.F16, _lib.F16, grp, gs, None)
    assert g(6, 4, 64) == -1 and b"group" in lib.bsrl_last_error()
    assert g(8, 4, 16) == -1
    assert g(8, 4, 64, y2=16, split=4) == -1
    assert g(0, 4, 64) == 0


def test_block_stack_shape_support_table(lib):
    d = lambda **k: _lib.BlocksDesc(**{**dict(n_layers=6, d=192, n_heads=4, ffn=768, T=29, act=_lib.ACT_RELU,
                                              n_queries=5, dtype=_lib.F16), **k})
    size = lib.bsrl_blocks_pack_size(ctypes.byref(d()))
    # 6 blocks x 72 stages x 12 KB of fragments + 6 x (9 * 192 + 768) fp32 vector entries
    assert size == 6 * 72 * 12 * 1024 + 6 * (9 * 192 + 768) * 4
    assert lib.bsrl_blocks_pack_size(ctypes.byref(d(d=128, ffn=512, n_layers=3))) == 3 * 48 * 8 * 1024 + 3 * (9 * 128 + 512) * 4
    assert lib.bsrl_blocks_pack_size(ctypes.byref(d(d=256, n_heads=8, ffn=1024, T=32, n_layers=4, dtype=_lib.BF16))) > 0
    for bad in (d(dtype=_lib.F32), d(T=33), d(d=384, n_heads=12), d(n_heads=6), d(ffn=100), d(n_queries=17),
                d(n_layers=9), d(act=_lib.ACT_NONE), d(n_layers=8, ffn=4096)):       # the last: vectors exceed the LDS budget
        assert lib.bsrl_blocks_pack_size(ctypes.byref(bad)) == 0
    rc = lib.bsrl_blocks_forward(ctypes.byref(d(T=33)), 16, 16, 16, None, 16, 4, None)
    assert rc > 0                                                # unsupported shape: a return code, not an error
    rc = lib.bsrl_blocks_forward(ctypes.byref(d()), None, 16, 16, None, 16, 4, None)
    assert rc == -1 and b"null" in lib.bsrl_last_error()
    assert lib.bsrl_blocks_forward(ctypes.byref(d()), 16, 16, 16, None, 16, 0, None) == 0


def test_host_modules_refuse_cpu_tensors():
    import torch
    from beatsaberrl_amd.config_policy import ConfigPolicy
    from beatsaberrl_amd.fused_ln import FusedLayerNorm
    m = ConfigPolicy(dtype="f16")
    with pytest.raises(RuntimeError, match="GPU only"):
        m.forward_stacked(torch.zeros(2, m.obs_dim))
    with pytest.raises(RuntimeError, match="GPU only"):
        FusedLayerNorm(128)(torch.zeros(2, 128))


def test_config_policy_state_dict_layout_matches_oracle():
    from beatsaberrl_amd.config_policy import ConfigPolicy
    from oracle import config_model as cm
    for ci in (1, 2, 3):
        spec = cm.CONFIGS[ci]["spec"]
        m = ConfigPolicy.from_spec(spec)
        want = cm.param_shapes(spec)
        got = [(k, tuple(v.shape)) for k, v in m.state_dict().items()]
        assert got == want
