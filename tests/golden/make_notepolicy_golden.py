"""Writes tests/golden/notepolicy_*.npz: (arch, state_dict, obs) -> (logits, value) of the
reference's NotePolicy on CPU fp32.

Run ONCE in the build container, where the reference checkout is mounted read-only:

    python tests/golden/make_notepolicy_golden.py [/root/reference/python [case ...]]

The composition of the full forward (token order, one-hot placement, the 40-lane note
input order, trunk wiring, the critic's use of token 2 and of the pre-final-block stream)
is the one thing closed forms and library routines cannot pin, so these vectors come
from the reference module itself (python/policy.py:784-1403, fp32 record path).  Only
the vectors travel: the fixtures hold numbers, no reference code.  Inputs follow the
reference bench's make_obs (python/bench_policy_forward.py:86-92): randn * 0.7 with the
24 slot-mask lanes set to 0/1.
"""
import json
import os
import sys

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/python"
ONLY = set(sys.argv[2:])          # optional: write just these cases
sys.path.insert(0, REF)
import policy as ref_policy  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = {
    # name: (ctor kwargs, B, seed)
    "notepolicy_geo": (dict(embed=64, trunk_dim=96, n_blocks=2, n_heads=2, n_gears=5, ffn_mult=4, note_geo=True,
                            head_gears=(5,) * 29), 8, 0),
    "notepolicy_ragged_ln": (dict(embed=64, trunk_dim=96, n_blocks=3, n_heads=2, n_gears=5, ffn_mult=2,
                                  note_geo=False, emb_ln=True, final_ln=True, trunk_hidden=128,
                                  head_gears=tuple(7 if j in (8, 15) else 5 for j in range(29))), 6, 1),
    "notepolicy_flux": (dict(embed=64, trunk_dim=64, n_blocks=1, n_heads=2, n_gears=3, ffn_mult=4, note_geo=True,
                             game="flux", z_asinh=4.0, value_bins=51, value_vmax=4.0,
                             head_gears=(3,) * 29), 5, 2),
    # the value-residual mix (blocks 1.. read block 0's values) and the SimBaV2 readout trunk
    "notepolicy_vres_v2": (dict(embed=64, trunk_dim=96, n_blocks=3, n_heads=2, n_gears=5, ffn_mult=2, note_geo=True,
                                value_residual=True, trunk_arch="simbav2", trunk_hidden=128,
                                head_gears=(5,) * 29), 6, 3),
}


def make_obs(n, seed):
    g = torch.Generator().manual_seed(seed)
    obs = torch.randn(n, ref_policy.OBS_DIM, generator=g) * 0.7
    lo = ref_policy.OFF_NOTE_MASK
    obs[:, lo:lo + ref_policy.N_NOTE_SLOTS] = (torch.rand(n, ref_policy.N_NOTE_SLOTS, generator=g) < 0.6).float()
    obs[0, lo:lo + ref_policy.N_NOTE_SLOTS] = 0.0          # an env with no entity at all
    obs[1, lo:lo + ref_policy.N_NOTE_SLOTS] = 1.0          # and one with every slot live
    # is_wall / is_bar lanes as 0/1 like the env writes them
    notes = obs[:, ref_policy.OFF_NOTES:lo].view(n, ref_policy.N_NOTE_SLOTS, ref_policy.NOTE_FEAT)
    notes[..., 14] = (torch.rand(n, ref_policy.N_NOTE_SLOTS, generator=g) < 0.3).float()
    notes[..., 9] = (torch.rand(n, ref_policy.N_NOTE_SLOTS, generator=g) < 0.3).float()
    return obs


def main():
    for name, (kw, B, seed) in CASES.items():
        if ONLY and name not in ONLY:
            continue
        torch.manual_seed(100 + seed)
        m = ref_policy.NotePolicy(**kw).eval()
        with torch.no_grad():
            for p in m.parameters():          # biases / LN affine away from their trivial init
                if p.dim() == 1:
                    p.add_(0.1 * torch.randn_like(p))
        obs = make_obs(B, seed)
        with torch.no_grad():
            logits, value = m.forward_stacked(obs)
        out = {"obs": obs.numpy(), "logits": logits.numpy(), "value": value.numpy(),
               "arch_json": np.frombuffer(json.dumps(m.arch).encode(), dtype=np.uint8)}
        keys = []
        for k, v in m.state_dict().items():
            out["sd." + k] = v.numpy()
            keys.append(k)
        out["sd_keys_json"] = np.frombuffer(json.dumps(keys).encode(), dtype=np.uint8)
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **out)
        print(name, "params", sum(v.numel() for v in m.state_dict().values()), "->", path,
              os.path.getsize(path) // 1024, "KiB", "logits", tuple(logits.shape))


if __name__ == "__main__":
    main()
