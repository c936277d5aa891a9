#!/usr/bin/env python3
"""Writes tests/golden/sdpa_preset.npz: expected attention outputs for the
input formulas of the reference's own kernel test, computed here in float64
with plain numpy (einsum + logsumexp).  The reference stores no output vectors
for this path, only these input formulas and a float64 loop of its own
(tests/kernel/flash_sdpa_fwd_cudnn.cc:83-175, 211-219, 243-268); this file
restates that loop with library routines, independently of the C++ checker
under oracle/, so the two can be compared.

    python tests/golden/make_golden.py

Cases (all with scale 1/sqrt(head), key j visible to query i iff mask[i, j]):
  preset_causal   K=(i%20-10)*0.1, Q=0.8*K, V=1.2*K; seq 64, head 32, batch 2; j <= i
  preset_full     same data, every key visible
  preset_window   K=0.1*(i%10-5), Q=0.05*(i%7-3), V=0.01*(i%13-6) (tests/tile/
                  flash_sdpa_fwd_cudnn.cc:57-86); seq 96, head 64, batch 1; |i-j| <= 32
  hidden_rows     preset_causal data with the keys of query rows 3 and 40 all hidden
Inputs are rounded to bf16 first (the values every implementation is fed);
the arrays stored are the rounded inputs' outputs A [batch, seq, head] and
lse [batch, seq] in float32.
"""
import os

import numpy as np


def round_bf16(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(x))


def attention(q, k, v, visible):
    """q, k, v: [batch, seq, head] float64; visible: [q_seq, k_seq] bool."""
    head = q.shape[-1]
    s = np.einsum("bqh,bkh->bqk", q, k) / np.sqrt(np.float64(head))
    s = np.where(visible[None], s, -np.inf)
    m = np.max(s, axis=-1, keepdims=True)
    m_safe = np.where(np.isfinite(m), m, 0.0)
    e = np.exp(s - m_safe)
    l = e.sum(-1, keepdims=True)
    with np.errstate(divide="ignore", invalid="ignore"):
        lse = np.where(l > 0, m_safe + np.log(l), -np.inf)[..., 0]
        p = np.where(l > 0, e / l, 0.0)
    return np.einsum("bqk,bkh->bqh", p, v), lse


def preset_kernel_test(seq, head, batch):
    i = np.arange(batch * seq * head)
    k = ((i % 20 - 10) * 0.1).astype(np.float32).reshape(batch, seq, head)
    return k * np.float32(0.8), k, k * np.float32(1.2)


def preset_tile_test(seq, head, batch):
    i = np.arange(batch * seq * head)
    k = (0.1 * (i % 10 - 5)).astype(np.float32).reshape(batch, seq, head)
    q = (0.05 * (i % 7 - 3)).astype(np.float32).reshape(batch, seq, head)
    v = (0.01 * (i % 13 - 6)).astype(np.float32).reshape(batch, seq, head)
    return q, k, v


def main():
    out = {}

    def case(name, qkv, visible):
        q, k, v = (round_bf16(x).astype(np.float64) for x in qkv)
        a, lse = attention(q, k, v, visible)
        out[name + "_A"] = a.astype(np.float32)
        out[name + "_lse"] = lse.astype(np.float32)
        out[name + "_visible"] = visible

    idx = np.arange(64)
    causal = idx[None, :] <= idx[:, None]
    case("preset_causal", preset_kernel_test(64, 32, 2), causal)
    case("preset_full", preset_kernel_test(64, 32, 2), np.ones((64, 64), bool))
    idx = np.arange(96)
    case("preset_window", preset_tile_test(96, 64, 1), np.abs(idx[None, :] - idx[:, None]) <= 32)
    hidden = causal.copy()
    hidden[3, :] = False
    hidden[40, :] = False
    case("hidden_rows", preset_kernel_test(64, 32, 2), hidden)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sdpa_preset.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
