"""The five workload shapes the path is measured and checked on.

Tensor layout in NNTile terms: Q/A ``[head, seq, n_batch, kv_group,
n_head_kv]``, K/V the same (prefill) or without the kv_group axis (decode).
``batch_flat`` below is the product of the three trailing axes.
"""
from dataclasses import dataclass


@dataclass(frozen=True)
class Workload:
    name: str
    dtype: str          # "fp32" | "bf16"
    head: int
    q_seq: int
    k_seq: int
    n_batch: int
    kv_group: int
    n_head_kv: int
    seq_tile: int       # rows per tile along the sequence axes
    calls: int          # independent slabs the tensor-level loop splits batch_flat into
    seed: int
    decode: bool = False
    outlier_frac: float = 0.0
    outlier_scale: float = 1.0

    @property
    def batch_flat(self):
        return self.n_batch * self.kv_group * self.n_head_kv

    @property
    def causal_offset(self):
        return self.k_seq - self.q_seq

    def visible_pairs(self):
        """Number of (query, key) pairs the causal mask leaves visible, per
        flattened batch entry."""
        off = self.causal_offset
        return sum(min(self.k_seq, q + off + 1) for q in range(self.q_seq)
                   if q + off >= 0)

    def flops(self, causal_exact=True):
        pairs = self.visible_pairs() if causal_exact else self.q_seq * self.k_seq
        return 4.0 * pairs * self.head * self.batch_flat

    def algorithmic_bytes(self):
        """HBM bytes one pass must move: K and V once (un-repeated), Q in, A
        out, lse out; the mask is analytic."""
        e = 2 if self.dtype != "fp32" else 4
        kv = 2 * self.head * self.k_seq * self.n_batch * self.n_head_kv * e
        qa = 2 * self.head * self.q_seq * self.batch_flat * e
        return kv + qa + 4 * self.q_seq * self.batch_flat


CONFIGS = [
    Workload("cfg1_single_head_fp32", "fp32", 64, 256, 256, 1, 1, 1, 256, 1, 42),
    Workload("cfg2_gpt2_small_fp32", "fp32", 64, 1024, 1024, 4, 1, 12, 1024, 4, 43),
    Workload("cfg3_llama_prefill_bf16", "bf16", 128, 4096, 4096, 1, 1, 32, 1024, 1, 44),
    Workload("cfg4_gqa_decode_bf16", "bf16", 128, 16, 8192, 8, 4, 8, 8192, 1, 45,
             decode=True),
    Workload("cfg5_long_seq_bf16", "bf16", 128, 16384, 16384, 1, 1, 8, 1024, 1, 46,
             outlier_frac=0.01, outlier_scale=8.0),
]

BY_NAME = {c.name: c for c in CONFIGS}
