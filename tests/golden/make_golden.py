#!/usr/bin/env python3
"""Writes tests/golden/bam_golden.npz: small seeded inputs and the fp32 results the oracle gives for them.

Run from the repository root:  python tests/golden/make_golden.py
The vectors are produced by ``oracle/bam_oracle.py`` (nothing of the reference is imported or read); the
bitfield layouts are the ones of the reference's own tests.  ``tests/test_golden.py`` checks on the CPU that
the oracle still reproduces the file and, on the GPU, that the HIP kernels match it.

Cases (all fp16 inputs so that the file stores them exactly):
  ref57     : B2 S57 Hq2 Hkv2 D32, bitfield of tests/test_kernel/test_bitfield_attention.py:162-184
  gqa_pad   : B1 S96 Hq4 Hkv2 D32, irregular segments, 7 padding tokens (bitfield 0), modality bits above 31
  zigzag    : B1 S160 Hq2 Hkv1 D32 split zigzag over two ranks (index tensors), rank 1 stored
  dense     : B1 Sq70 Sk45 H2 D32, materialized bool mask with a dead row
  bias      : B1 S80 Hq2 Hkv1 D32, bitfield of the reference's test, fp32 matrix bias (1, 2, 80, 80)
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import bam_oracle as O  # noqa: E402
from tests.helpers import random_bitfield, reference_test_bitfield  # noqa: E402


def tensors(B, Sq, Sk, Hq, Hkv, D, seed):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Sq, Hq, D, generator=g) * 0.5).half()
    k = (torch.randn(B, Sk, Hkv, D, generator=g) * 0.5).half()
    v = (torch.randn(B, Sk, Hkv, D, generator=g) * 0.5).half()
    do = torch.randn(B, Sq, Hq, D, generator=g).half()
    return q, k, v, do


def pack(out, name, q, k, v, do, o, lse, grads, **extra):
    for key, t in dict(q=q, k=k, v=v, do=do).items():
        out[f"{name}.{key}"] = t.numpy()
    out[f"{name}.o"] = o.numpy().astype(np.float32)
    out[f"{name}.lse"] = lse.numpy().astype(np.float32)
    for key, t in zip(("dq", "dk", "dv"), grads):
        out[f"{name}.{key}"] = t.numpy().astype(np.float32)
    for key, t in extra.items():
        out[f"{name}.{key}"] = t.numpy()


def build():
    out = {}
    # ref57
    bf, _ = reference_test_bitfield(2, 57)
    q, k, v, do = tensors(2, 57, 57, 2, 2, 32, seed=11)
    o, lse = O.attention_forward(q, k, v, bf)
    pack(out, "ref57", q, k, v, do, o, lse, O.attention_backward(q, k, v, bf, do), bf=bf, flags=O.tile_flags(bf))
    # gqa_pad
    bf = random_bitfield(1, 96, seed=12, pad=7, wide=True)
    q, k, v, do = tensors(1, 96, 96, 4, 2, 32, seed=12)
    o, lse = O.attention_forward(q, k, v, bf)
    pack(out, "gqa_pad", q, k, v, do, o, lse, O.attention_backward(q, k, v, bf, do), bf=bf, flags=O.tile_flags(bf))
    # zigzag (rank 1 of 2)
    S = 160
    bf = random_bitfield(1, S, seed=13)
    c = np.array_split(np.arange(S), 4)
    ranks = [np.concatenate([c[0], c[3]]), np.concatenate([c[1], c[2]])]
    idx_q = torch.from_numpy(ranks[1].astype(np.int64))
    idx_k = torch.from_numpy(np.concatenate(ranks).astype(np.int64))
    q, k, v, do = tensors(1, idx_q.numel(), idx_k.numel(), 2, 1, 32, seed=13)  # local (already gathered) tensors
    o, lse = O.attention_forward(q, k, v, bf, idx_q=idx_q, idx_k=idx_k)
    grads = O.attention_backward(q, k, v, bf, do, idx_q=idx_q, idx_k=idx_k)
    pack(out, "zigzag", q, k, v, do, o, lse, grads, bf=bf, idx_q=idx_q, idx_k=idx_k,
         flags=O.tile_flags_indexed(bf, idx_q, idx_k))
    # dense
    g = torch.Generator().manual_seed(14)
    mask = torch.rand(1, 70, 45, generator=g) < 0.5
    mask[:, 5, :] = False
    q, k, v, do = tensors(1, 70, 45, 2, 2, 32, seed=14)
    o, lse = O.masked_attention_forward(q, k, v, mask)
    pack(out, "dense", q, k, v, do, o, lse, O.masked_attention_backward(q, k, v, mask, do), mask=mask,
         flags=O.mask_tile_flags(mask))
    # bias
    bf, _ = reference_test_bitfield(1, 80)
    q, k, v, do = tensors(1, 80, 80, 2, 1, 32, seed=15)
    bias = torch.randn(1, 2, 80, 80, generator=torch.Generator().manual_seed(16))
    o, lse = O.attention_forward(q, k, v, bf, bias=bias)
    pack(out, "bias", q, k, v, do, o, lse, O.attention_backward(q, k, v, bf, do, bias=bias), bf=bf, bias=bias,
         flags=O.tile_flags(bf))
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bam_golden.npz")
    np.savez_compressed(path, **build())
    print(path, os.path.getsize(path), "bytes")
