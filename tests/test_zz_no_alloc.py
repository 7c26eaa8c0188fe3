"""bsrl_cfg_forward_static (the forward that allocates nothing: its scratch is a
device array built into the library) against bsrl_cfg_forward with a caller
workspace, through the C ABI.

Both run the same kernels on the same launch shapes, so the gate is bit
equality of logits and values.  Two calls in a row share the GPU's one array:
the second call is smaller, so it runs over what the first one left behind.
"Allocates nothing" is checked on the device's own free-memory figure across a
warm call, and one call is replayed from a captured graph.
The file sorts last on purpose: a failure here must not hide the other tests
under `pytest -x`.
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

from beatsaberrl_amd import _lib, ops  # noqa: E402
from beatsaberrl_amd.config_policy import ConfigPolicy, N_ACTION_HEADS  # noqa: E402
from oracle import config_model as cm  # noqa: E402

DEV = "cuda"


def _model(dtype):
    c = cm.CONFIGS[1]
    p = cm.init_params(c["spec"], c["w_seed"])
    m = ConfigPolicy.from_spec(c["spec"], dtype=dtype, route="fused")
    m.load_state_dict(p)
    return c, p, m.to(DEV)


def _outputs(B, n_log):
    # prefilled with a marker so that an env the call never wrote shows up
    return (torch.full((B, n_log), 7.0, device=DEV, dtype=torch.float32),
            torch.full((B,), 7.0, device=DEV, dtype=torch.float32))


def _run_workspace(lib, m, desc, img, obs, k):
    B, n_log = obs.shape[0], N_ACTION_HEADS * m.n_gears
    lg, v = _outputs(B, n_log)
    ws_bytes = lib.bsrl_cfg_workspace_size(ctypes.byref(desc), B)
    ws = torch.empty(ws_bytes, device=DEV, dtype=torch.uint8)
    rc = lib.bsrl_cfg_forward(ctypes.byref(desc), img.data_ptr(), obs.data_ptr(), obs.stride(0), ops.dt_code(obs.dtype),
                              k.data_ptr(), lg.data_ptr(), v.data_ptr(), B, ws.data_ptr(), ws_bytes,
                              torch.cuda.current_stream().cuda_stream)
    assert _lib.check(rc, "bsrl_cfg_forward")
    torch.cuda.synchronize()
    return lg, v


def _call_static(lib, m, desc, img, obs, k, lg, v):
    rc = lib.bsrl_cfg_forward_static(ctypes.byref(desc), img.data_ptr(), obs.data_ptr(), obs.stride(0),
                                     ops.dt_code(obs.dtype), k.data_ptr(), lg.data_ptr(), v.data_ptr(), obs.shape[0],
                                     torch.cuda.current_stream().cuda_stream)
    assert _lib.check(rc, "bsrl_cfg_forward_static")


def _run_static(lib, m, desc, img, obs, k, warm):
    """warm: this (shape of) call has run before on the device, so the runtime's one-time work - the code object load
    behind hipGetSymbolAddress, a kernel's raised LDS limit - is done: the DEVICE's free memory as the driver reports it
    (hipMemGetInfo, which sees every hipMalloc / hipFree of the process, the library's included - torch's own counters
    see only torch's allocator) must not move across the call."""
    B, n_log = obs.shape[0], N_ACTION_HEADS * m.n_gears
    lg, v = _outputs(B, n_log)
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    _call_static(lib, m, desc, img, obs, k, lg, v)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before          # nothing went through torch's allocator either
    if warm:
        assert torch.cuda.mem_get_info()[0] == free_before, (free_before, torch.cuda.mem_get_info()[0])
    return lg, v


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_static_forward_matches_workspace_forward_twice(lib, dtype):
    c, p, m = _model(dtype)
    dt = torch.float16 if dtype == "f16" else torch.bfloat16
    desc, img = m._desc(dt), m.packed_image(dt, next(m.parameters()).device)
    torch.cuda.synchronize()
    # first call: the largest batch the built-in scratch takes; second call: a smaller, odd batch with another mask
    # mix, over the array the first call left behind
    for B, seed, mask in ((_lib.CFG_STATIC_MAX_ENVS, c["obs_seed"], c["mask"]), (1237, 11, "uniform")):
        obs, k = cm.make_inputs(c["spec"], B, seed, mask)
        obs, k = obs.to(DEV), k.to(DEV)
        print(f"\nstatic forward: dtype={dtype} B={B} seed={seed}", flush=True)
        _run_static(lib, m, desc, img, obs, k, warm=False)           # the runtime's one-time work for this launch shape
        lg_s, v_s = _run_static(lib, m, desc, img, obs, k, warm=True)
        lg_w, v_w = _run_workspace(lib, m, desc, img, obs, k)
        assert torch.equal(lg_s, lg_w) and torch.equal(v_s, v_w)
        assert bool((lg_s != 7.0).any(-1).all()) and bool((v_s != 7.0).all())
    # and against the oracle at a size it finishes quickly (the gate every fused-route test uses is in
    # tests/test_config_policy_gpu.py; here a coarse bound is enough, bit equality above carries the parity)
    ref_lg, _ = cm.forward(p, c["spec"], obs[:256].cpu(), k[:256].cpu())
    assert (lg_s[:256].cpu().view_as(ref_lg) - ref_lg).abs().max().item() < (2e-2 if dtype == "f16" else 2e-1)


def test_static_forward_replays_from_a_captured_graph(lib):
    """After one eager call on the device (the symbol address, the kernels' attributes), the entry point is a pure
    launch: captured into a graph it replays with new observations and key counts in the static buffers and returns
    the bits of the workspace form, replay after replay, with the program's own eager work in between."""
    c, _, m = _model("f16")
    desc, img = m._desc(torch.float16), m.packed_image(torch.float16, next(m.parameters()).device)
    B, n_log = 5000, N_ACTION_HEADS * m.n_gears
    obs0, k0 = cm.make_inputs(c["spec"], B, 21, "uniform")
    s_obs, s_k = obs0.to(DEV), k0.to(DEV)
    lg, v = _outputs(B, n_log)
    _call_static(lib, m, desc, img, s_obs, s_k, lg, v)               # eager warm call, outside capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        _call_static(lib, m, desc, img, s_obs, s_k, lg, v)
    for seed, mask in ((31, "uniform"), (32, "quarter_empty"), (33, "none")):
        obs, k = cm.make_inputs(c["spec"], B, seed, mask)
        s_obs.copy_(obs.to(DEV)); s_k.copy_(k.to(DEV))
        lg.fill_(7.0); v.fill_(7.0)
        g.replay()
        got_lg, got_v = lg.clone(), v.clone()
        x = torch.randn(300, 300, device=DEV)
        (x @ x).sum().item()                                         # unrelated eager work and a sync between replays
        lg_w, v_w = _run_workspace(lib, m, desc, img, obs.to(DEV), k.to(DEV))
        assert torch.equal(got_lg, lg_w) and torch.equal(got_v, v_w), seed


def test_static_forward_rejects_oversize_batch(lib):
    c, _, m = _model("f16")
    desc, img = m._desc(torch.float16), m.packed_image(torch.float16, next(m.parameters()).device)
    B = _lib.CFG_STATIC_MAX_ENVS + 1
    obs, k = cm.make_inputs(c["spec"], B, 3, "uniform")
    obs, k = obs.to(DEV), k.to(DEV)
    lg, v = _outputs(B, N_ACTION_HEADS * m.n_gears)
    rc = lib.bsrl_cfg_forward_static(ctypes.byref(desc), img.data_ptr(), obs.data_ptr(), obs.stride(0),
                                     ops.dt_code(obs.dtype), k.data_ptr(), lg.data_ptr(), v.data_ptr(), B,
                                     torch.cuda.current_stream().cuda_stream)
    assert rc == -1 and b"exceeds" in lib.bsrl_last_error()
    torch.cuda.synchronize()
    assert bool((lg == 7.0).all())       # nothing was launched
