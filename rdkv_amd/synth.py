"""Seeded synthetic workloads of the five benchmark configurations.

Each configuration fixes shapes, value distributions and the bit-allocation rule; nothing
here needs model weights.  K/V are fp16 ~N(0,1) with 4 outlier K channels per head scaled
by 8; the query is fp16 ~N(0,1) taken as already rotated.  Class fractions apply to the T
context tokens of a head (the allocator of the reference assigns a bit-width to every
context token, obkv_fast.py:986-991); ``token_budget`` is carried as metadata only.

Seeds: data ``1000*config + layer (+ 100000*seq)``, allocations
``7919*config + 31*layer + head (+ 100003*seq)``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import numpy as np
import torch


@dataclass(frozen=True)
class SynthConfig:
    index: int
    name: str
    layers: int
    H_q: int
    H_kv: int
    context: int                      # tokens per head before eviction (mean for ragged batches)
    token_budget: int
    batch: int = 1
    context_range: Optional[Tuple[int, int]] = None
    # V class fractions over (evict, 2, 4, 8, 16) or None for a per-head Dirichlet(1,1,1,1,1) draw
    v_fracs: Optional[Tuple[float, float, float, float, float]] = None
    # kept-channel counts (2-bit, 4-bit, 8-bit) or None for Dirichlet(1,1,1) over 64 kept
    k_counts: Optional[Tuple[int, int, int]] = None
    k_keep: int = 64
    D: int = 128

    @property
    def G(self) -> int:
        return self.H_q // self.H_kv


CONFIGS = {
    0: SynthConfig(0, "C0 llama3.1-8b-shaped 4k, 1 layer", 1, 32, 8, 4096, 1024,
                   v_fracs=(0.2, 0.2, 0.3, 0.2, 0.1), k_counts=(16, 32, 16)),
    1: SynthConfig(1, "C1 llama3.1-8b-shaped 32k, 32 layers", 32, 32, 8, 32768, 2048),
    2: SynthConfig(2, "C2 mistral-7b-shaped 128k, 32 layers", 32, 32, 8, 131072, 4096,
                   v_fracs=(0.15, 0.40, 0.30, 0.10, 0.05), k_counts=(26, 38, 0)),
    3: SynthConfig(3, "C3 qwen2.5-72b-shaped 128k, 80 layers, GQA 8", 80, 64, 8, 131072, 8192),
    4: SynthConfig(4, "C4 llama3.1-8b-shaped batch 32 x ctx U[16k,64k]", 32, 32, 8, 40960, 2048,
                   batch=32, context_range=(16384, 65536)),
}


def scaled(cfg: SynthConfig, *, context: Optional[int] = None, layers: Optional[int] = None,
           batch: Optional[int] = None) -> SynthConfig:
    """Same rule set at a smaller size (parity tests)."""
    kw = dict(cfg.__dict__)
    if context is not None:
        kw["context"] = context
        if cfg.context_range is not None:
            lo, hi = cfg.context_range
            kw["context_range"] = (max(1, context * lo // cfg.context), max(2, context * hi // cfg.context))
    if layers is not None:
        kw["layers"] = layers
    if batch is not None:
        kw["batch"] = batch
    return SynthConfig(**kw)


def seq_context(cfg: SynthConfig, seq: int) -> int:
    if cfg.context_range is None:
        return cfg.context
    lo, hi = cfg.context_range
    rng = np.random.default_rng(4242 + 17 * cfg.index + seq)
    return int(rng.integers(lo, hi + 1))


def _largest_remainder(p: np.ndarray, total: int) -> np.ndarray:
    raw = p * total
    base = np.floor(raw).astype(np.int64)
    rem = total - int(base.sum())
    order = np.argsort(-(raw - base), kind="stable")
    base[order[:rem]] += 1
    return base


def head_allocation(cfg: SynthConfig, layer: int, head: int, seq: int = 0):
    """-> (v_bits [T] int64 in {0,2,4,8,16}, k_bits [D] int64 in {0,2,4,8}, outlier channels [4])."""
    T = seq_context(cfg, seq)
    rng = np.random.default_rng(7919 * cfg.index + 31 * layer + head + 100003 * seq)
    fr = np.asarray(cfg.v_fracs) if cfg.v_fracs is not None else rng.dirichlet(np.ones(5))
    counts = np.floor(fr * T).astype(np.int64)          # (evict, 2, 4, 8, 16)
    counts[0] += T - int(counts.sum())                  # remainder -> evicted
    # membership by a seeded random importance ranking: most important -> fp16 ... least -> evicted
    order = rng.permutation(T)
    v_bits = np.zeros(T, dtype=np.int64)
    o = 0
    for bits, n in ((16, counts[4]), (8, counts[3]), (4, counts[2]), (2, counts[1])):
        v_bits[order[o:o + n]] = bits
        o += int(n)
    D = cfg.D
    outliers = rng.choice(D, size=4, replace=False)
    if cfg.k_counts is not None:
        c2, c4, c8 = cfg.k_counts
    else:
        c2, c4, c8 = (int(v) for v in _largest_remainder(rng.dirichlet(np.ones(3)), cfg.k_keep))
    keep = c2 + c4 + c8
    rest = np.setdiff1d(np.arange(D), outliers)
    kept = np.concatenate([outliers, rng.permutation(rest)[:keep - 4]])
    kept = rng.permutation(kept)
    k_bits = np.zeros(D, dtype=np.int64)
    k_bits[kept[:c2]] = 2
    k_bits[kept[c2:c2 + c4]] = 4
    k_bits[kept[c2 + c4:]] = 8
    return v_bits, k_bits, outliers


def layer_allocation(cfg: SynthConfig, layer: int, seq: int = 0):
    """-> (v_bits [H_kv,T], k_bits [H_kv,D], outliers [H_kv,4]) as CPU int64 tensors."""
    vb, kb, oc = zip(*(head_allocation(cfg, layer, h, seq) for h in range(cfg.H_kv)))
    return (torch.from_numpy(np.stack(vb)), torch.from_numpy(np.stack(kb)),
            torch.from_numpy(np.stack(oc)))


def layer_data(cfg: SynthConfig, layer: int, device="cpu", seq: int = 0, outliers=None):
    """-> (K, V [1,H_kv,T,D] fp16, q [H_q,D] fp16) generated on ``device`` with its own
    seeded generator (CPU and GPU streams differ; parity tests generate on the CPU and copy)."""
    T = seq_context(cfg, seq)
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(1000 * cfg.index + layer + 100000 * seq)
    K = torch.randn(1, cfg.H_kv, T, cfg.D, generator=g, device=dev, dtype=torch.float32)
    if outliers is None:
        outliers = layer_allocation(cfg, layer, seq)[2]
    scale = torch.ones(cfg.H_kv, cfg.D, device=dev)
    scale.scatter_(1, outliers.to(dev), 8.0)
    K = (K * scale.view(1, cfg.H_kv, 1, cfg.D)).half()
    V = torch.randn(1, cfg.H_kv, T, cfg.D, generator=g, device=dev, dtype=torch.float32).half()
    q = torch.randn(cfg.H_q, cfg.D, generator=g, device=dev, dtype=torch.float32).half()
    return K, V, q


def dense_fp16_bytes(cfg: SynthConfig, seq: int = 0) -> int:
    """Bytes of the equivalent dense fp16 K+V cache of one layer (full context)."""
    return seq_context(cfg, seq) * cfg.D * 2 * 2 * cfg.H_kv
