"""CPU oracle for bitfield-masked attention (BAM).  TEST INFRASTRUCTURE ONLY.

This module is a restatement, in plain torch tensor ops, of the algorithm of the
reference hot path ``cornstarch/kernel/bitfield_attention.py``.  It is the checker
the parity tests, the smoke test and the CPU-baseline leg of the benchmark compare
the HIP kernels against.  Nothing in the shipped package imports it, and the
shipped package never falls back to it.

What pins each function (the pins live in ``tests/test_oracle.py``):

* ``allow_rows`` / ``materialize_mask`` -- the closed-form masks held by the
  reference's own test (``tests/test_kernel/test_bitfield_attention.py:55-110``:
  lower-triangular with modality rows replaced by same-segment squares), plus the
  degenerate cases all-text == causal and all-one-modality == dense.
* ``tile_flags`` -- its definition over the pinned mask
  (``bitfield_attention.py:118-126,143-153``), the analytic tile histogram of the
  1024-token plumbing layout (124 full / 24 partial / 108 empty, 557440 pairs) and
  the per-row-block non-empty counts the reference's context-parallel test expects
  (``tests/test_shardformer/test_context_parallel.py:30-63,258-272``).
* ``attention_sdpa`` -- is the library routine the reference's tests use as ground
  truth (``tests/test_kernel/test_bitfield_attention.py:188-190,287-293``).
* ``attention_forward`` (explicit softmax, also yields LSE) -- pinned against
  ``attention_sdpa`` and against ``torch.logsumexp``.
* ``attention_backward`` -- ``torch.autograd.grad`` through the explicit forward,
  pinned against autograd through SDPA (``test_bitfield_attention.py:198-204``)
  and against the closed-form C restatement in ``bam_oracle.c``.
* index tensors (``idx_q`` / ``idx_k`` of ``allow_rows``, ``attention_forward``,
  ``attention_backward``, ``tile_flags_indexed``) -- the indexed mask equals a gather of the
  pinned global mask; indexed attention over permuted keys equals the plain result gathered at
  ``idx_q`` (what the reference's context-parallel test asserts,
  ``tests/test_shardformer/test_context_parallel.py:311-376``); for block-aligned index sets the
  flags equal the reference's gather of the global flags (``shardformer/layers/utils.py:331-353``).
* ``masked_attention_forward`` / ``masked_attention_backward`` (materialized bool mask, the
  reference's ``flash_attn_func``) -- library SDPA with the same ``attn_mask`` and autograd through it,
  which is what the reference's test compares against (``tests/test_kernel/test_attention.py``);
  ``mask_tile_flags`` -- brute-force classification of random masks.
* ``bias`` of the four attention functions -- library SDPA with the float ``attn_mask`` = bias, -inf
  where the pair is not allowed (forward and autograd through it); closed forms: a bias that is
  constant along the keys leaves o unchanged and shifts lse by that constant, and bias = log w
  turns the softmax into the w-weighted one.
* ``create_bitfield_attention_mask`` -- golden vectors of
  ``tests/test_models/test_multimodal_merge_outputs.py:94-110``.

All functions are device agnostic torch code: the parity tests run them on the CPU
at small sizes and, for the full-size configurations, on whatever device the
inputs live on (fp32 library math, never the HIP kernels).
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn.functional as F

BLOCK_M = 128  # bitfield_attention.py:53
BLOCK_N = 32  # bitfield_attention.py:54
MODALITY_MASK = (1 << 62) - 1  # bitfield_attention.py:92-93


# --------------------------------------------------------------------------- mask
def _gather_bits(bf_row: torch.Tensor, pos: torch.Tensor) -> torch.Tensor:
    """bitfield at global positions ``pos``; positions >= S read 0
    (bitfield_attention.py:86-87)."""
    S = bf_row.shape[0]
    ok = pos < S
    return torch.where(ok, bf_row[pos.clamp(max=S - 1)], torch.zeros_like(pos))


def allow_rows(
    bf_row: torch.Tensor,
    r0: int,
    r1: int,
    idx_q: Optional[torch.Tensor] = None,
    idx_k: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Allow rule for query rows [r0, r1) of ONE sequence -> bool (r1-r0, Sk).

    ``bf_row``: int64 (S_total,).  Without index tensors the query/key positions
    are the row/column numbers; with them they are ``idx_q[row]`` / ``idx_k[col]``
    (global positions, bitfield_attention.py:71-81).
    Rule (bitfield_attention.py:86-101), M = 2**62 - 1:
        allow(i, j) = (i >= j and text_i and (q & k & M) != 0)
                   or (not text_i and (q & M) == (k & M) and (q & M) != 0)
    """
    S = bf_row.shape[0]
    dev = bf_row.device
    if idx_q is None:
        pos_q = torch.arange(r0, r1, device=dev, dtype=torch.int64)
    else:
        pos_q = idx_q[r0:r1].to(torch.int64)
    if idx_k is None:
        pos_k = torch.arange(0, S, device=dev, dtype=torch.int64)
    else:
        pos_k = idx_k.to(torch.int64)
    qf = _gather_bits(bf_row, pos_q)
    kf = _gather_bits(bf_row, pos_k)
    text = (qf & 1) != 0
    qb = (qf & MODALITY_MASK)[:, None]
    kb = (kf & MODALITY_MASK)[None, :]
    causal = pos_q[:, None] >= pos_k[None, :]
    return (causal & text[:, None] & ((qb & kb) != 0)) | (
        (~text)[:, None] & (qb == kb) & (qb != 0)
    )


def materialize_mask(bitfield: torch.Tensor) -> torch.Tensor:
    """bool (B, S, S) attention mask of a (B, S) int64 bitfield tensor."""
    B, S = bitfield.shape
    return torch.stack([allow_rows(bitfield[b], 0, S) for b in range(B)])


def tile_flags(bitfield: torch.Tensor) -> torch.Tensor:
    """int8 (B, ceil(S/128), ceil(S/32)): 0 empty, 1 partial, 2 full.

    A tile is full when every IN-RANGE cell is allowed; the ragged last row/column
    tile counts ``S % 128`` rows / ``S % 32`` columns
    (bitfield_attention.py:143-153).
    """
    B, S = bitfield.shape
    nm, nn = -(-S // BLOCK_M), -(-S // BLOCK_N)
    out = torch.zeros((B, nm, nn), dtype=torch.int8, device=bitfield.device)
    cols = torch.full((nn,), BLOCK_N, dtype=torch.int64, device=bitfield.device)
    if S % BLOCK_N:
        cols[-1] = S % BLOCK_N
    for b in range(B):
        for m in range(nm):
            r0, r1 = m * BLOCK_M, min((m + 1) * BLOCK_M, S)
            a = allow_rows(bitfield[b], r0, r1)  # (rows, S)
            a = F.pad(a, (0, nn * BLOCK_N - S))
            cnt = a.view(r1 - r0, nn, BLOCK_N).sum(dim=(0, 2))
            full = cnt == (r1 - r0) * cols
            out[b, m] = torch.where(cnt == 0, 0, torch.where(full, 2, 1)).to(torch.int8)
    return out


def tile_flags_indexed(bitfield: torch.Tensor, idx_q: torch.Tensor, idx_k: torch.Tensor) -> torch.Tensor:
    """Flags of the LOCAL tiles of index-tensor attention: int8 (B, ceil(Sq/128), ceil(Sk/32)) over
    the mask whose row i / column j stand for global positions idx_q[i] / idx_k[j].  When the
    index sets are made of whole, aligned blocks this equals the reference's recipe of gathering
    rows and columns of the global flags (shardformer/layers/utils.py:331-353)."""
    B = bitfield.shape[0]
    Sq, Sk = idx_q.numel(), idx_k.numel()
    nm, nn = -(-Sq // BLOCK_M), -(-Sk // BLOCK_N)
    out = torch.zeros((B, nm, nn), dtype=torch.int8, device=bitfield.device)
    cols = torch.full((nn,), BLOCK_N, dtype=torch.int64, device=bitfield.device)
    if Sk % BLOCK_N:
        cols[-1] = Sk % BLOCK_N
    for b in range(B):
        for m in range(nm):
            r0, r1 = m * BLOCK_M, min((m + 1) * BLOCK_M, Sq)
            a = allow_rows(bitfield[b], r0, r1, idx_q, idx_k)
            a = F.pad(a, (0, nn * BLOCK_N - Sk))
            cnt = a.view(r1 - r0, nn, BLOCK_N).sum(dim=(0, 2))
            full = cnt == (r1 - r0) * cols
            out[b, m] = torch.where(cnt == 0, 0, torch.where(full, 2, 1)).to(torch.int8)
    return out


def unmasked_pairs(bitfield: torch.Tensor) -> int:
    """Number of allowed (query, key) pairs over the whole batch."""
    B, S = bitfield.shape
    total = 0
    step = 2048
    for b in range(B):
        for r0 in range(0, S, step):
            total += int(allow_rows(bitfield[b], r0, min(r0 + step, S)).sum())
    return total


def create_bitfield_attention_mask(input_ids: torch.Tensor, token_ids: dict) -> torch.Tensor:
    """Bitfield format (cornstarch/kernel/interface.py:13-30): modality number n in
    ``token_ids`` order gets bit n+1; text gets bit 62, bit 0 and every modality bit."""
    text = (1 << 62) | 1
    bits = {}
    for n, key in enumerate(token_ids):
        bits[key] = 1 << (n + 1)
        text |= bits[key]
    out = torch.full(input_ids.shape, text, dtype=torch.int64, device=input_ids.device)
    for key, tok in token_ids.items():
        out = torch.where(input_ids == tok, torch.full_like(out, bits[key]), out)
    return out


# ---------------------------------------------------------------------- attention
def attention_sdpa(q, k, v, bitfield, softmax_scale=None):
    """Materialized-mask attention exactly as the reference's tests build their
    ground truth (test_bitfield_attention.py:188-190,287-293): library SDPA with the
    bool mask, GQA by ``enable_gqa``.  q (B,S,Hq,D), k/v (B,S,Hkv,D) -> (B,S,Hq,D).
    Rows that allow no key come out as NaN from the library; the reference kernel
    defines them as 0 (bitfield_attention.py:441-444,493-495), so they are zeroed."""
    mask = materialize_mask(bitfield).unsqueeze(1)
    o = F.scaled_dot_product_attention(
        q.transpose(1, 2),
        k.transpose(1, 2),
        v.transpose(1, 2),
        attn_mask=mask,
        scale=softmax_scale,
        enable_gqa=q.shape[2] != k.shape[2],
    ).transpose(1, 2)
    dead = ~mask.any(dim=-1)  # (B,1,S)
    return torch.where(dead.transpose(1, 2).unsqueeze(-1), torch.zeros_like(o), o)


def _chunk_forward(qc, kb, vb, allow, scale, bias=None):
    """qc (rows,Hq,D), kb/vb (S,Hkv,D), allow (rows,S) -> o (rows,Hq,D), lse (Hq,rows).
    s = scale * q.k (+ bias) ; lse = log sum_allowed exp(s) ; o = sum_allowed exp(s-lse) v
    (bitfield_attention.py:389-390,410-434,435-495); GQA h -> h // (Hq//Hkv) (:292-293).
    ``bias`` broadcasts against (Hq, rows, S)."""
    Hq, Hkv = qc.shape[1], kb.shape[1]
    g = Hq // Hkv
    kk = kb.repeat_interleave(g, dim=1) if g > 1 else kb
    vv = vb.repeat_interleave(g, dim=1) if g > 1 else vb
    s = torch.einsum("ihd,jhd->hij", qc, kk) * scale
    if bias is not None:
        s = s + bias.to(s.dtype)
    s = s.masked_fill(~allow[None], float("-inf"))
    lse = torch.logsumexp(s, dim=-1)  # -inf where nothing is allowed
    p = torch.exp(s - torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)[..., None])
    o = torch.einsum("hij,jhd->ihd", p, vv)
    return o, lse


def _bias_rows(bias, b, r0, r1):
    """Rows r0..r1 of batch b of a bias broadcastable to (B, Hq, Sq, Sk) -> broadcastable to (Hq, rows, Sk)
    (indexed by LOCAL row / key like the reference, bitfield_attention.py:321-329)."""
    if bias is None:
        return None
    bb = bias[b if bias.shape[0] > 1 else 0]
    return bb[:, r0:r1] if bb.shape[1] > 1 else bb


def attention_forward(q, k, v, bitfield, softmax_scale=None, row_chunk=1024, dtype=torch.float32,
                      idx_q=None, idx_k=None, bias=None):
    """Explicit masked softmax attention -> (o (B,S,Hq,D), lse (B,Hq,S)) in ``dtype``.
    With index tensors q holds the rows at global positions ``idx_q`` and k/v the keys at
    ``idx_k`` (any order); ``bitfield`` stays indexed by global position
    (bitfield_attention.py:71-87).  ``bias``: 4-d, broadcastable to (B, Hq, S, S), added to the
    scaled scores (bitfield_attention.py:410-434)."""
    B, S, Hq, D = q.shape
    scale = softmax_scale or 1.0 / math.sqrt(D)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    o = torch.empty((B, S, Hq, D), dtype=dtype, device=q.device)
    lse = torch.empty((B, Hq, S), dtype=dtype, device=q.device)
    for b in range(B):
        for r0 in range(0, S, row_chunk):
            r1 = min(r0 + row_chunk, S)
            allow = allow_rows(bitfield[b], r0, r1, idx_q, idx_k)
            oc, lc = _chunk_forward(q[b, r0:r1], k[b], v[b], allow, scale, _bias_rows(bias, b, r0, r1))
            o[b, r0:r1] = oc
            lse[b, :, r0:r1] = lc
    return o, lse


def attention_backward(q, k, v, bitfield, do, softmax_scale=None, row_chunk=1024, dtype=torch.float32,
                       idx_q=None, idx_k=None, bias=None):
    """dq, dk, dv of sum(o * do) by autograd through the explicit forward, one row
    chunk at a time (bounded memory).  Matches the reference's gradient contract
    (bitfield_attention.py:840-886): dk/dv are summed over the q-heads of a group."""
    B, S, Hq, D = q.shape
    scale = softmax_scale or 1.0 / math.sqrt(D)
    q, k, v, do = q.to(dtype), k.to(dtype), v.to(dtype), do.to(dtype)
    dq = torch.zeros_like(q)
    dk = torch.zeros_like(k)
    dv = torch.zeros_like(v)
    for b in range(B):
        for r0 in range(0, S, row_chunk):
            r1 = min(r0 + row_chunk, S)
            allow = allow_rows(bitfield[b], r0, r1, idx_q, idx_k)
            qc = q[b, r0:r1].detach().requires_grad_(True)
            kb = k[b].detach().requires_grad_(True)
            vb = v[b].detach().requires_grad_(True)
            oc, _ = _chunk_forward(qc, kb, vb, allow, scale, _bias_rows(bias, b, r0, r1))
            gq, gk, gv = torch.autograd.grad(oc, (qc, kb, vb), do[b, r0:r1])
            dq[b, r0:r1] = gq
            dk[b] += gk
            dv[b] += gv
    return dq, dk, dv


def masked_attention_forward(q, k, v, mask, softmax_scale=None, dtype=torch.float32, bias=None):
    """Attention with a materialized bool mask (B, Sq, Sk) (None: attend everywhere), the contract of
    the reference's ``flash_attn_func`` (cornstarch/kernel/attention.py:184-232: pairs whose mask
    byte is False get -inf before the softmax) -> (o (B,Sq,Hq,D), lse (B,Hq,Sq))."""
    B, Sq, Hq, D = q.shape
    Sk = k.shape[1]
    scale = softmax_scale or 1.0 / math.sqrt(D)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    o = torch.empty((B, Sq, Hq, D), dtype=dtype, device=q.device)
    lse = torch.empty((B, Hq, Sq), dtype=dtype, device=q.device)
    for b in range(B):
        allow = mask[b] if mask is not None else torch.ones((Sq, Sk), dtype=torch.bool, device=q.device)
        o[b], lse[b] = _chunk_forward(q[b], k[b], v[b], allow, scale, _bias_rows(bias, b, 0, Sq))
    return o, lse


def masked_attention_backward(q, k, v, mask, do, softmax_scale=None, dtype=torch.float32, bias=None):
    """dq, dk, dv of sum(o * do) for ``masked_attention_forward`` by autograd."""
    q, k, v, do = (t.to(dtype) for t in (q, k, v, do))
    qr, kr, vr = (t.detach().requires_grad_(True) for t in (q, k, v))
    o, _ = masked_attention_forward(qr, kr, vr, mask, softmax_scale, dtype, bias)
    return torch.autograd.grad(o, (qr, kr, vr), do)


def mask_tile_flags(mask: torch.Tensor) -> torch.Tensor:
    """int8 (B, ceil(Sq/128), ceil(Sk/32)) classification of a bool mask (B, Sq, Sk): 0 empty,
    2 every in-range cell set, 1 otherwise."""
    B, Sq, Sk = mask.shape
    nm, nn = -(-Sq // BLOCK_M), -(-Sk // BLOCK_N)
    padded = F.pad(mask, (0, nn * BLOCK_N - Sk, 0, nm * BLOCK_M - Sq))
    cnt = padded.view(B, nm, BLOCK_M, nn, BLOCK_N).sum(dim=(2, 4))
    cells = F.pad(torch.ones_like(mask), (0, nn * BLOCK_N - Sk, 0, nm * BLOCK_M - Sq)).view(B, nm, BLOCK_M, nn, BLOCK_N).sum(dim=(2, 4))
    return torch.where(cnt == 0, 0, torch.where(cnt == cells, 2, 1)).to(torch.int8)


def delta(o, do):
    """delta[b,h,i] = sum_d o*do in fp32 (bitfield_attention.py:527-572)."""
    return (o.float() * do.float()).sum(-1).transpose(1, 2).contiguous()


def sdpa_forward_backward(q, k, v, bitfield, do=None, softmax_scale=None, row_chunk=2048):
    """The reference tests' ground truth at scale: bool mask from the bitfields + library
    SDPA (``enable_gqa``), one block of query rows at a time so that the mask and the score
    matrix stay bounded.  Returns o, and (dq, dk, dv) of sum(o * do) when ``do`` is given.
    This is the routine the CPU baseline of the benchmark times."""
    B, S, Hq, D = q.shape
    gqa = Hq != k.shape[2]
    o = torch.empty_like(q)
    grads = None
    if do is not None:
        grads = (torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v))
    for b in range(B):
        kb = k[b : b + 1].transpose(1, 2)
        vb = v[b : b + 1].transpose(1, 2)
        for r0 in range(0, S, row_chunk):
            r1 = min(r0 + row_chunk, S)
            allow = allow_rows(bitfield[b], r0, r1)
            dead = ~allow.any(dim=-1)
            qc = q[b : b + 1, r0:r1].transpose(1, 2)
            if do is not None:
                qc, kc, vc = (t.detach().requires_grad_(True) for t in (qc, kb, vb))
            else:
                kc, vc = kb, vb
            oc = F.scaled_dot_product_attention(
                qc, kc, vc, attn_mask=allow[None, None], scale=softmax_scale, enable_gqa=gqa
            )
            oc = torch.where(dead[None, None, :, None], torch.zeros_like(oc), oc)
            o[b, r0:r1] = oc.detach().transpose(1, 2)[0]
            if do is not None:
                gq, gk, gv = torch.autograd.grad(oc, (qc, kc, vc), do[b : b + 1, r0:r1].transpose(1, 2))
                grads[0][b, r0:r1] = gq.transpose(1, 2)[0]
                grads[1][b] += gk.transpose(1, 2)[0]
                grads[2][b] += gv.transpose(1, 2)[0]
    return (o, *grads) if grads is not None else o


def decode_step(query, key, value, scaling=None, sliding_window=None, softcap=None):
    """Single-token decode step of the HF adapter (cornstarch/kernel/interface.py:71-83): the reference forwards it
    to flash-attn through transformers' ``flash_attention_forward`` with ``attention_mask=None``.  flash-attn is not
    part of the reference tree; its published semantics for ONE query at the last position are restated here in
    fp32: scores ``scaling * q.k`` (default 1/sqrt(D)); ``softcap``: ``softcap * tanh(score / softcap)``;
    ``sliding_window`` w (transformers passes ``window_size=(w - 1, w - 1)`` when the cache is longer than w):
    keys ``j >= Sk - w``; softmax; times V.  Grouped kv heads: kv head of q head h is ``h // (Hq // Hkv)``.

    query (B, Hq, 1, D), key / value (B, Hkv, Sk, D) -> (B, 1, Hq, D) fp32."""
    B, Hq, one, D = query.shape
    Hkv, Sk = key.shape[1], key.shape[2]
    g = Hq // Hkv
    qf = query.float()[:, :, 0]                              # (B, Hq, D)
    kf = key.float().repeat_interleave(g, dim=1)             # (B, Hq, Sk, D)
    vf = value.float().repeat_interleave(g, dim=1)
    scale = scaling if scaling is not None else 1.0 / math.sqrt(D)
    s = torch.einsum("bhd,bhjd->bhj", qf, kf) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    if sliding_window is not None and Sk > sliding_window:
        s[:, :, : Sk - sliding_window] = -math.inf
    p = torch.softmax(s, dim=-1)
    return torch.einsum("bhj,bhjd->bhd", p, vf)[:, None]
