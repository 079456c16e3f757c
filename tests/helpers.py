"""Shared builders for the parity tests (no reference code is imported anywhere)."""

from __future__ import annotations

import torch

TEXT_124 = (1 << 62) | 1 | (1 << 1) | (1 << 2)


def reference_test_bitfield(batch_size: int, seqlen: int):
    """Bitfield + closed-form mask of the reference's fwd/bwd tests
    (tests/test_kernel/test_bitfield_attention.py:162-184): text everywhere, modality 1 on
    12:24, modality 2 on 36:56; expected = lower triangle with those rows replaced by the
    segment's square."""
    bf = torch.full((batch_size, seqlen), TEXT_124, dtype=torch.int64)
    bf[:, 12:24] = 1 << 1
    bf[:, 36:56] = 1 << 2
    full = torch.tril(torch.ones((batch_size, seqlen, seqlen), dtype=torch.bool))
    full[:, 12:24, :] = False
    full[:, 12:24, 12:24] = True
    full[:, 36:56, :] = False
    full[:, 36:56, 36:56] = True
    return bf, full


def reference_mask_kat(size: str):
    """Known-answer masks of tests/test_kernel/test_bitfield_attention.py:55-110."""
    S = 64 if size == "small" else 256
    bf = torch.full((2, S), TEXT_124, dtype=torch.int64)
    exp = torch.tril(torch.ones((2, S, S), dtype=torch.bool))
    segs = (
        [(0, 12, 24, 1), (1, 4, 16, 1), (1, 36, 56, 2)]
        if size == "small"
        else [(0, 50, 150, 1), (1, 48, 120, 1), (1, 164, 200, 2)]
    )
    for b, s, e, bit in segs:
        bf[b, s:e] = 1 << bit
        exp[b, s:e, :] = False
        exp[b, s:e, s:e] = True
    return bf, exp


def random_bitfield(B: int, S: int, seed: int, nbits: int = 5, pad: int = 0, wide: bool = False):
    """Irregular layout: random segments of random modality bits inside text, optional
    zero padding at the end, optional use of bits above 31."""
    g = torch.Generator().manual_seed(seed)
    bits = list(range(1, nbits + 1))
    if wide:
        bits = [b + 30 for b in bits]  # bits 31..: exercises the upper 32-bit half
    text = (1 << 62) | 1
    for b in bits:
        text |= 1 << b
    bf = torch.full((B, S), text, dtype=torch.int64)
    for b in range(B):
        pos = 0
        while pos < S:
            run = int(torch.randint(1, max(2, S // 6), (1,), generator=g))
            kind = int(torch.randint(0, 3, (1,), generator=g))
            if kind == 0:
                bit = bits[int(torch.randint(0, len(bits), (1,), generator=g))]
                bf[b, pos : pos + run] = 1 << bit
            pos += run
        if pad:
            bf[b, S - pad :] = 0
    return bf


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))
