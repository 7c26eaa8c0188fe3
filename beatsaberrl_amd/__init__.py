"""MI355X-native policy forward for BeatSaberRL (hand-written HIP behind a C ABI).

Public surface:
  * beatsaberrl_amd.ops            - tensor-level wrappers of the C-ABI entry points
  * beatsaberrl_amd.fused_ln       - FusedLayerNorm (mirrors the reference's fused_ln.py)
  * beatsaberrl_amd.fp16_linear    - fp16-stream op layer (mirrors fp16_linear.py, forward paths)
  * beatsaberrl_amd.config_policy  - ConfigPolicy: the benchmark-config transformer policy
  * beatsaberrl_amd.policy         - NotePolicy drop-in (same state_dict layout / forward_stacked)
"""
__all__ = ["ops", "config_policy"]
