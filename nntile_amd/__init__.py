"""MI355X-native tile-level attention forward for NNTile: host-side mirror.

Only what the hot path needs: the C-ABI library (csrc/) and its ctypes
binding (hip_sdpa), the C++ mirror of the reference's codelet / tile / tensor
layers for this operation (host/, driven from Python through host_mirror),
the key/value cache of the decode path (kv_cache), the benchmark shapes
(configs) and seeded synthetic inputs (synth).
"""
__all__ = ["hip_sdpa", "host_mirror", "kv_cache", "configs", "synth"]
