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
