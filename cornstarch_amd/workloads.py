"""Deterministic synthetic inputs for the five benchmark/parity configurations.

Tensors come from ``torch.Generator("cpu").manual_seed(1000 * c)`` drawn in the
order Q, K, V, dO; bitfields follow the reference's format
(cornstarch/kernel/interface.py:13-30): a segment of modality bit ``b`` carries
``1 << b`` and text carries bit 62, bit 0 and every modality bit the
configuration uses.  Segment placement: with lengths ``L_k`` and
``T = S - sum(L)``, ``cuts = sort(rng.integers(0, T + 1, n))`` and segment ``k``
starts at ``cuts[k] + sum(L_j for j < k)`` (non-overlapping, order preserved).
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np
import torch


@dataclass(frozen=True)
class Workload:
    name: str
    index: int
    B: int
    S: int
    Hq: int
    Hkv: int
    D: int
    dtype: torch.dtype
    backward: bool
    description: str


WORKLOADS = {
    "C1": Workload("C1", 1, 1, 1024, 8, 8, 64, torch.float32, False, "plumbing: image 0-255, text 256-1023"),
    "C2": Workload("C2", 2, 1, 8192, 32, 8, 128, torch.bfloat16, True, "llama3-8b vlm: 4x576 image segments"),
    "C3": Workload("C3", 3, 1, 16384, 32, 8, 128, torch.bfloat16, True, "vision+audio+text: 3x1024 + 2x1500"),
    "C4": Workload("C4", 4, 8, 4096, 16, 16, 64, torch.bfloat16, True, "packed encoder batch, 1-6 segments/seq"),
    "C5": Workload("C5", 5, 1, 65536, 32, 8, 128, torch.bfloat16, True, "long context, 200 irregular segments"),
}


def text_bits(modality_bits) -> int:
    t = (1 << 62) | 1
    for b in modality_bits:
        t |= 1 << int(b)
    return t


def place_segments(S: int, lengths, bits, seed: int, text: int) -> np.ndarray:
    """One sequence's int64 bitfields with segments placed at seeded offsets."""
    lengths = [int(x) for x in lengths]
    bf = np.full((S,), text, dtype=np.int64)
    n = len(lengths)
    if n == 0:
        return bf
    T = S - sum(lengths)
    assert T >= 0
    rng = np.random.default_rng(seed)
    cuts = np.sort(rng.integers(0, T + 1, size=n))
    off = 0
    for k in range(n):
        s = int(cuts[k]) + off
        bf[s : s + lengths[k]] = 1 << int(bits[k])
        off += lengths[k]
    return bf


def make_bitfields(name: str) -> torch.Tensor:
    w = WORKLOADS[name]
    if name == "C1":
        bf = np.full((1, w.S), text_bits([1]), dtype=np.int64)
        bf[0, :256] = 1 << 1
    elif name == "C2":
        bf = place_segments(w.S, [576] * 4, [1, 2, 3, 4], 0, text_bits(range(1, 5)))[None]
    elif name == "C3":
        bf = place_segments(w.S, [1024, 1500, 1024, 1500, 1024], [1, 2, 3, 4, 5], 0, text_bits(range(1, 6)))[None]
    elif name == "C4":
        rng = np.random.default_rng(0)
        rows = []
        for b in range(w.B):
            n = int(rng.integers(1, 7))
            L = [int(x) for x in rng.integers(256, 1025, n)]
            bits = [int(x) for x in rng.integers(1, 9, n)]
            while sum(L) > w.S:
                L.pop()
                bits.pop()
            rows.append(place_segments(w.S, L, bits, 100 + b, text_bits(range(1, 9))))
        bf = np.stack(rows)
    elif name == "C5":
        rng = np.random.default_rng(0)
        L = rng.integers(16, 513, 200)
        bits = rng.integers(1, 17, 200)
        bf = place_segments(w.S, L, bits, 1, text_bits(range(1, 17)))[None]
    else:
        raise KeyError(name)
    return torch.from_numpy(np.ascontiguousarray(bf))


def make_tensors(name: str, heads=None):
    """(q, k, v, do) on the CPU in the workload's dtype.  ``heads=(hq0, hq1)``
    keeps only q-heads [hq0, hq1) and the kv-heads they map to (same values as the
    full draw) -- used to bound the CPU work of sampled checks."""
    w = WORKLOADS[name]
    g = torch.Generator("cpu").manual_seed(1000 * w.index)
    q = torch.randn((w.B, w.S, w.Hq, w.D), generator=g, dtype=torch.float32)
    k = torch.randn((w.B, w.S, w.Hkv, w.D), generator=g, dtype=torch.float32)
    v = torch.randn((w.B, w.S, w.Hkv, w.D), generator=g, dtype=torch.float32)
    do = torch.randn((w.B, w.S, w.Hq, w.D), generator=g, dtype=torch.float32)
    if name != "C1":
        s = 1.0 / math.sqrt(w.D)
        q, k, v = q * s, k * s, v * s
    q, k, v, do = (t.to(w.dtype) for t in (q, k, v, do))
    if heads is not None:
        G = w.Hq // w.Hkv
        h0, h1 = heads
        assert h0 % G == 0 and h1 % G == 0
        q, do = q[:, :, h0:h1].contiguous(), do[:, :, h0:h1].contiguous()
        k, v = k[:, :, h0 // G : h1 // G].contiguous(), v[:, :, h0 // G : h1 // G].contiguous()
    return q, k, v, do


def flops(name: str, pairs: int):
    """Algorithmic FLOPs over unmasked pairs: fwd 4*D*Hq*pairs, bwd 10*D*Hq*pairs."""
    w = WORKLOADS[name]
    f = 4 * w.D * w.Hq * pairs
    return f, f * 5 // 2
