"""MI355X-native tile-level attention forward for NNTile: host-side mirror.

Only what the hot path needs: the C-ABI library (csrc/), its binding
(hip_sdpa), the tensor-level driver that mirrors the reference's tile loop
(sdpa), and seeded synthetic inputs (synth).
"""
__all__ = ["hip_sdpa", "synth"]
