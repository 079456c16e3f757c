"""Pins of the oracle: every check here compares the oracle with something that is NOT the
oracle's own formula -- the closed-form masks and expectations held by the reference's own
tests, library routines (SDPA, logsumexp, autograd), analytic counts, or a second,
independently written restatement (C scalar loops vs vectorized torch)."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import bam_oracle as O
from oracle import c_oracle as C
from tests.helpers import random_bitfield, reference_mask_kat, reference_test_bitfield, rel_l2


# ------------------------------------------------------------------ allow rule / mask
@pytest.mark.parametrize("size", ["small", "large"])
def test_mask_matches_reference_kat(size):
    bf, expected = reference_mask_kat(size)
    assert torch.equal(O.materialize_mask(bf), expected)
    assert np.array_equal(C.mask(bf.numpy()), expected.numpy())


@pytest.mark.parametrize("S", [57, 128, 283])
def test_mask_matches_reference_fwd_test_layout(S):
    bf, expected = reference_test_bitfield(2, S)
    assert torch.equal(O.materialize_mask(bf), expected)
    assert np.array_equal(C.mask(bf.numpy()), expected.numpy())


def test_mask_degenerate_layouts():
    S = 96
    tril = torch.tril(torch.ones((1, S, S), dtype=torch.bool))
    # all text == causal (tests/test_shardformer/utils.py:388-391), with or without the
    # decorative bit 62 and whatever bit 63 holds
    for text in [(1 << 62) | 1, 1, -(1 << 63) | 1, (1 << 62) | 1 | 6]:
        bf = torch.full((1, S), text, dtype=torch.int64)
        assert torch.equal(O.materialize_mask(bf), tril)
        assert np.array_equal(C.mask(bf.numpy()), tril.numpy())
    # one modality everywhere == dense; padding (0) == nothing
    bf = torch.full((1, S), 1 << 1, dtype=torch.int64)
    assert O.materialize_mask(bf).all() and C.mask(bf.numpy()).all()
    bf = torch.zeros((1, S), dtype=torch.int64)
    assert not O.materialize_mask(bf).any() and not C.mask(bf.numpy()).any()
    # bits 62/63 alone carry no modality: such tokens see nothing and are seen by nobody
    bf = torch.full((1, S), 1 << 62, dtype=torch.int64)
    assert not O.materialize_mask(bf).any() and not C.mask(bf.numpy()).any()


def test_mask_text_without_modality_bit_cannot_see_that_modality():
    # text carries bit 1 only; a modality-2 segment is invisible to it, modality-1 visible
    S = 32
    bf = torch.full((1, S), (1 << 62) | 1 | 2, dtype=torch.int64)
    bf[0, 4:8] = 2
    bf[0, 12:16] = 4
    m = O.materialize_mask(bf)[0]
    assert m[20, 4:8].all() and not m[20, 12:16].any()
    assert m[12:16, 12:16].all() and not m[12:16, :12].any() and not m[12:16, 16:].any()


@pytest.mark.parametrize("seed", [0, 1, 2])
@pytest.mark.parametrize("wide", [False, True])
def test_two_restatements_agree_on_random_bitfields(seed, wide):
    bf = random_bitfield(2, 200, seed, pad=7, wide=wide)
    assert np.array_equal(O.materialize_mask(bf).numpy(), C.mask(bf.numpy()))
    assert np.array_equal(O.tile_flags(bf).numpy(), C.tile_flags(bf.numpy()))


def test_indexed_mask_is_a_gather_of_the_global_mask():
    # context-parallel callers evaluate the rule on global positions (reference :71-81)
    bf = random_bitfield(1, 160, 3)
    full = O.materialize_mask(bf)[0]
    g = torch.Generator().manual_seed(0)
    idx_q = torch.randperm(160, generator=g)[:48].sort().values
    idx_k = torch.arange(160)
    got = O.allow_rows(bf[0], 0, 48, idx_q=idx_q, idx_k=idx_k)
    assert torch.equal(got, full[idx_q][:, idx_k])
    c = C.mask_indexed(bf.numpy(), idx_q.numpy(), idx_k.numpy())[0]
    assert np.array_equal(c, got.numpy())
    # an out-of-range index behaves like padding
    idx_k2 = torch.cat([idx_k[:10], torch.tensor([160])])
    got2 = O.allow_rows(bf[0], 0, 48, idx_q=idx_q, idx_k=idx_k2)
    assert not got2[:, -1].any()
    assert np.array_equal(C.mask_indexed(bf.numpy(), idx_q.numpy(), idx_k2.numpy())[0], got2.numpy())


# ------------------------------------------------------------------------- tile flags
def test_flags_plumbing_layout_analytic_histogram():
    # tokens 0-255 one image (bit 1), 256-1023 text: derived by hand -> 124 full, 24 partial,
    # 108 empty tiles of 128x32 and 557440 allowed pairs
    bf = torch.full((1, 1024), (1 << 62) | 1 | 2, dtype=torch.int64)
    bf[0, :256] = 2
    for flags in (O.tile_flags(bf), torch.from_numpy(C.tile_flags(bf.numpy()))):
        assert flags.shape == (1, 8, 32) and flags.dtype == torch.int8
        assert [(flags == v).sum().item() for v in (0, 1, 2)] == [108, 24, 124]
    assert O.unmasked_pairs(bf) == 256 * 256 + sum(range(257, 1025)) == 557440


@pytest.mark.parametrize("S", [57, 256, 335, 684, 1024, 2003, 3712])
def test_flags_rowblock_workloads_of_context_parallel_test(S):
    # tests/test_shardformer/test_context_parallel.py:192-274 relies on these per-row-block
    # counts of non-empty tiles: causal -> 4(m+1) capped at ceil(S/32); dense -> ceil(S/32)
    nn = -(-S // 32)
    causal = O.tile_flags(torch.full((1, S), (1 << 62) | 1, dtype=torch.int64))[0]
    assert [(row > 0).sum().item() for row in causal] == [min(4 * (m + 1), nn) for m in range(causal.shape[0])]
    dense = O.tile_flags(torch.full((1, S), 1 << 1, dtype=torch.int64))[0]
    assert (dense == 2).all()  # ragged edge tiles count only in-range cells (reference :149-153)
    # below the diagonal causal tiles are full, on it partial, above it empty
    m = causal.shape[0] - 1
    if S % 128 == 0:
        assert (causal[m, : 4 * m] == 2).all() and (causal[m, 4 * m :] == 1).all()


def test_flags_classification_vs_mask_bruteforce():
    bf = random_bitfield(2, 300, 5, pad=9)
    mask = O.materialize_mask(bf)
    flags = C.tile_flags(bf.numpy())
    for b in range(2):
        for m in range(3):
            for n in range(10):
                t = mask[b, 128 * m : 128 * m + 128, 32 * n : 32 * n + 32]
                want = 0 if t.sum() == 0 else (2 if t.all() else 1)
                assert flags[b, m, n] == want


# ------------------------------------------------------------------- bitfield format
def test_bitfield_format_golden_vectors():
    # tests/test_models/test_multimodal_merge_outputs.py:94-110: vision -> 1<<1, audio -> 1<<2,
    # text -> (1<<62) | 1 | 2 | 4
    from cornstarch_amd.kernel.interface import create_bitfield_attention_mask as product_fn

    vid, aid = 44, 55
    for vis, aud in [([2, 3, 4, 5], [9, 10, 11]), ([0, 1], []), ([], [13, 14, 15])]:
        ids = torch.arange(16).unsqueeze(0).clone()
        want = torch.full((1, 16), (1 << 62) | 1 | 2 | 4, dtype=torch.int64)
        ids[0, vis] = vid
        want[0, vis] = 1 << 1
        ids[0, aud] = aid
        want[0, aud] = 1 << 2
        tok = {"vision": vid, "audio": aid}
        assert torch.equal(O.create_bitfield_attention_mask(ids, tok), want)
        assert torch.equal(product_fn(ids, tok), want)


# --------------------------------------------------------------- forward / backward
def _rand(B, S, Hq, Hkv, D, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, S, Hq, D, generator=g, dtype=dtype) * 0.5
    k = torch.randn(B, S, Hkv, D, generator=g, dtype=dtype) * 0.5
    v = torch.randn(B, S, Hkv, D, generator=g, dtype=dtype) * 0.5
    do = torch.randn(B, S, Hq, D, generator=g, dtype=dtype)
    return q, k, v, do


@pytest.mark.parametrize("S,Hq,Hkv,D", [(57, 6, 6, 32), (144, 6, 2, 64), (283, 6, 3, 16)])
def test_forward_against_library_sdpa_and_c_loops(S, Hq, Hkv, D):
    # the reference's ground truth: SDPA with the materialized mask, enable_gqa
    bf, full = reference_test_bitfield(2, S)
    q, k, v, _ = _rand(2, S, Hq, Hkv, D, dtype=torch.float64)
    want = F.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), attn_mask=full.unsqueeze(1), enable_gqa=True
    ).transpose(1, 2)
    o, lse = O.attention_forward(q, k, v, bf, dtype=torch.float64)
    assert torch.allclose(o, want, atol=1e-10, rtol=0)
    assert torch.allclose(O.attention_sdpa(q, k, v, bf), want, atol=1e-10, rtol=0)
    # LSE against library logsumexp over independently built (repeat_interleave) scores
    g = Hq // Hkv
    s = torch.einsum("bihd,bjhd->bhij", q, k.repeat_interleave(g, dim=2)) / math.sqrt(D)
    want_lse = torch.logsumexp(s.masked_fill(~full.unsqueeze(1), float("-inf")), dim=-1)
    assert torch.allclose(lse, want_lse, atol=1e-10, rtol=0)
    co, clse = C.attn_fwd(q.float().numpy(), k.float().numpy(), v.float().numpy(), bf.numpy())
    assert np.allclose(co, want.float().numpy(), atol=2e-6) and np.allclose(clse, want_lse.float().numpy(), atol=2e-6)


@pytest.mark.parametrize("S,Hq,Hkv,D", [(57, 6, 6, 32), (144, 6, 2, 64), (130, 4, 1, 16)])
def test_backward_against_autograd_through_sdpa(S, Hq, Hkv, D):
    bf, full = reference_test_bitfield(2, S)
    q, k, v, do = _rand(2, S, Hq, Hkv, D, seed=1, dtype=torch.float64)
    qr, kr, vr = (x.clone().requires_grad_(True) for x in (q, k, v))
    ref = F.scaled_dot_product_attention(
        qr.transpose(1, 2), kr.transpose(1, 2), vr.transpose(1, 2), attn_mask=full.unsqueeze(1), enable_gqa=True
    ).transpose(1, 2)
    wq, wk, wv = torch.autograd.grad(ref, (qr, kr, vr), do)
    dq, dk, dv = O.attention_backward(q, k, v, bf, do, row_chunk=50, dtype=torch.float64)
    for got, want in ((dq, wq), (dk, wk), (dv, wv)):
        assert torch.allclose(got, want, atol=1e-10, rtol=0)
    # closed-form restatement (P, dS formulas of the reference's backward) in C
    o, lse = O.attention_forward(q, k, v, bf, dtype=torch.float64)
    dlt = C.delta(o.float().numpy(), do.float().numpy())
    assert np.allclose(dlt, O.delta(o, do).numpy(), atol=1e-5)
    cq, ck, cv = C.attn_bwd(*(x.float().numpy() for x in (q, k, v, do)), lse.float().numpy(), dlt, bf.numpy())
    for got, want in ((cq, wq), (ck, wk), (cv, wv)):
        assert rel_l2(torch.from_numpy(got), want) < 1e-5
    # delta has a second face the oracle does not compute it from: rowsum(o * do) = rowsum(P * (dO V^T)),
    # with P and dO V^T built here from an explicit masked softmax
    g = Hq // Hkv
    kx, vx = k.repeat_interleave(g, dim=2), v.repeat_interleave(g, dim=2)
    sc = torch.einsum("bihd,bjhd->bhij", q, kx) / math.sqrt(D)
    P = torch.softmax(sc.masked_fill(~full.unsqueeze(1), float("-inf")), dim=-1)
    dP = torch.einsum("bihd,bjhd->bhij", do, vx)
    assert torch.allclose(O.delta(o, do).double(), (P * dP).sum(-1), atol=1e-5)


def test_rows_without_any_allowed_key_give_zero_output_and_minus_inf_lse():
    # right padding = bitfield 0 (reference modeling_multimodal_language_model.py:947-948);
    # the reference kernel defines o = 0, lse = -inf there (bitfield_attention.py:441-444,493-495)
    bf = random_bitfield(1, 90, 2, pad=11)
    q, k, v, do = _rand(1, 90, 2, 2, 16, seed=3)
    o, lse = O.attention_forward(q, k, v, bf)
    assert (o[0, -11:] == 0).all() and torch.isinf(lse[0, :, -11:]).all() and (lse[0, :, -11:] < 0).all()
    assert torch.isfinite(o).all()
    co, clse = C.attn_fwd(q.numpy(), k.numpy(), v.numpy(), bf.numpy())
    assert (co[0, -11:] == 0).all() and np.isneginf(clse[0, :, -11:]).all()
    dq, dk, dv = O.attention_backward(q, k, v, bf, do)
    assert torch.isfinite(dq).all() and (dq[0, -11:] == 0).all() and (dk[0, -11:] == 0).all()
    assert torch.allclose(O.attention_sdpa(q, k, v, bf), o, atol=1e-5)


def test_all_text_bitfield_is_plain_causal_attention():
    S = 77
    bf = torch.full((1, S), (1 << 62) | 1, dtype=torch.int64)
    q, k, v, _ = _rand(1, S, 4, 4, 32, seed=4)
    want = F.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True
    ).transpose(1, 2)
    o, _ = O.attention_forward(q, k, v, bf)
    assert torch.allclose(o, want, atol=1e-5)


# ------------------------------------------------------------------ index tensors (context-parallel shards)
def _cp_splits(S, kind):
    """Index sets of two 'ranks' the way the reference splits a sequence
    (shardformer/layers/utils.py:108-146, 180-197): contiguous, zigzag, whole 128-row blocks."""
    if kind == "uniform":
        chunks = np.array_split(np.arange(S), 2)
    elif kind == "zigzag":
        c = np.array_split(np.arange(S), 4)
        chunks = [np.concatenate([c[0], c[3]]), np.concatenate([c[1], c[2]])]
    else:  # whole 128-row blocks dealt alternately, sorted per rank
        blocks = np.arange(-(-S // 128))
        chunks = [np.concatenate([np.arange(b * 128, min((b + 1) * 128, S)) for b in blocks[r::2]]) for r in range(2)]
    return [torch.from_numpy(c.astype(np.int64)) for c in chunks]


@pytest.mark.parametrize("kind", ["uniform", "zigzag", "blocks"])
def test_indexed_attention_is_the_plain_result_gathered(kind):
    # what the reference's context-parallel test asserts (test_context_parallel.py:311-376): each rank's
    # output / dq equals its rows of the plain result, and dk / dv summed over the ranks equal the plain ones
    S, Hq, Hkv, D = 300, 4, 2, 16
    bf = random_bitfield(1, S, seed=5)
    q, k, v, do = _rand(1, S, Hq, Hkv, D, seed=2, dtype=torch.float64)
    o, lse = O.attention_forward(q, k, v, bf, dtype=torch.float64)
    dq, dk, dv = O.attention_backward(q, k, v, bf, do, dtype=torch.float64)
    ranks = _cp_splits(S, kind)
    idx_k = torch.cat(ranks)
    sum_dk, sum_dv = torch.zeros_like(dk), torch.zeros_like(dv)
    for idx_q in ranks:
        ql, dol = q[:, idx_q], do[:, idx_q]
        kl, vl = k[:, idx_k], v[:, idx_k]
        ol, lsel = O.attention_forward(ql, kl, vl, bf, dtype=torch.float64, idx_q=idx_q, idx_k=idx_k)
        assert torch.allclose(ol, o[:, idx_q], atol=1e-12, rtol=0)
        assert torch.allclose(lsel, lse[:, :, idx_q], atol=1e-12, rtol=0)
        gq, gk, gv = O.attention_backward(ql, kl, vl, bf, dol, dtype=torch.float64, idx_q=idx_q, idx_k=idx_k)
        assert torch.allclose(gq, dq[:, idx_q], atol=1e-12, rtol=0)
        sum_dk[:, idx_k] += gk
        sum_dv[:, idx_k] += gv
    assert torch.allclose(sum_dk, dk, atol=1e-11, rtol=0) and torch.allclose(sum_dv, dv, atol=1e-11, rtol=0)


def test_indexed_flags_equal_the_reference_gather_of_global_flags_for_aligned_blocks():
    # the recipe of ContextParallelBatchSplitUtils.get_local_compressed_mask (utils.py:331-353):
    # rows offsets_q[::128] // 128 and columns cat(offsets[::32]) // 32 of the global flags
    S = 640
    bf = random_bitfield(2, S, seed=9)
    glob = O.tile_flags(bf)
    ranks = _cp_splits(S, "blocks")
    idx_k = torch.cat(ranks)
    cols = torch.cat([r[::32] for r in ranks]) // 32
    for idx_q in ranks:
        want = glob[:, idx_q[::128] // 128][:, :, cols]
        assert torch.equal(O.tile_flags_indexed(bf, idx_q, idx_k), want)


# ------------------------------------------------------------------ materialized bool mask (flash_attn_func)
def _reference_dense_mask(B, Sq, Sk):
    """mask of the reference's test (tests/test_kernel/test_attention.py:80-88)."""
    mask = torch.tril(torch.ones(B, Sq, Sk, dtype=torch.bool))
    mask[:, 12:24, :] = False
    mask[:, 12:24, 12:24] = True
    mask[:, 36:56, :] = False
    mask[:, 36:56, 36:56] = True
    return mask


@pytest.mark.parametrize("Sq,Sk", [(57, 57), (128, 300), (283, 144)])
def test_dense_mask_attention_against_library_sdpa(Sq, Sk):
    # ground truth of the reference's test: SDPA with attn_mask = mask (test_attention.py:93-104)
    B, H, D = 2, 3, 16
    g = torch.Generator().manual_seed(3)
    q = torch.randn(B, Sq, H, D, generator=g, dtype=torch.float64) * 0.5
    k = torch.randn(B, Sk, H, D, generator=g, dtype=torch.float64) * 0.5
    v = torch.randn(B, Sk, H, D, generator=g, dtype=torch.float64) * 0.5
    do = torch.randn(B, Sq, H, D, generator=g, dtype=torch.float64)
    mask = _reference_dense_mask(B, Sq, Sk)
    live = mask.any(-1)  # rows of the square blocks that fall outside Sk see nothing: SDPA gives NaN there
    qr, kr, vr = (t.clone().requires_grad_(True) for t in (q, k, v))
    ref = F.scaled_dot_product_attention(
        qr.transpose(1, 2), kr.transpose(1, 2), vr.transpose(1, 2), attn_mask=mask.unsqueeze(1)
    ).transpose(1, 2)
    ref = torch.where(live[:, :, None, None], ref, torch.zeros_like(ref))
    o, lse = O.masked_attention_forward(q, k, v, mask, dtype=torch.float64)
    assert torch.allclose(o, ref, atol=1e-10, rtol=0)
    s = torch.einsum("bihd,bjhd->bhij", q, k) / math.sqrt(D)
    want_lse = torch.logsumexp(s.masked_fill(~mask.unsqueeze(1), float("-inf")), dim=-1)
    assert torch.equal(torch.isfinite(lse), torch.isfinite(want_lse))
    assert torch.allclose(lse[torch.isfinite(lse)], want_lse[torch.isfinite(want_lse)], atol=1e-10, rtol=0)
    wq, wk, wv = torch.autograd.grad(ref, (qr, kr, vr), do)
    dq, dk, dv = O.masked_attention_backward(q, k, v, mask, do, dtype=torch.float64)
    for got, want in ((dq, wq), (dk, wk), (dv, wv)):
        assert torch.allclose(got, want, atol=1e-10, rtol=0)
    # no mask at all == plain softmax attention
    o2, _ = O.masked_attention_forward(q, k, v, None, dtype=torch.float64)
    ref2 = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)).transpose(1, 2)
    assert torch.allclose(o2, ref2, atol=1e-10, rtol=0)


def test_dense_mask_tile_flags_against_loops():
    g = torch.Generator().manual_seed(4)
    mask = torch.rand(2, 300, 170, generator=g) < 0.5
    mask[:, :128, :64] = True  # full tiles
    mask[:, 128:256, 32:96] = False  # empty tiles
    mask[:, 256:, 160:] = True  # the ragged corner tile, full
    got = O.mask_tile_flags(mask)
    assert got.shape == (2, 3, 6)
    for b in range(2):
        for m in range(3):
            for n in range(6):
                t = mask[b, m * 128 : (m + 1) * 128, n * 32 : (n + 1) * 32]
                want = 0 if not t.any() else 2 if t.all() else 1
                assert got[b, m, n] == want
    assert got[0, 0, 0] == 2 and got[0, 1, 1] == 0 and got[0, 2, 5] == 2


# ------------------------------------------------------------------ additive bias
@pytest.mark.parametrize("kind", ["vector", "matrix", "matrix_per_batch"])
def test_bias_against_library_sdpa_with_float_mask(kind):
    # SDPA adds a float attn_mask to the scaled scores: bias where the pair is allowed, -inf elsewhere
    B, S, Hq, Hkv, D = 2, 150, 4, 2, 16
    g = torch.Generator().manual_seed(11)
    q = torch.randn(B, S, Hq, D, generator=g, dtype=torch.float64) * 0.5
    k = torch.randn(B, S, Hkv, D, generator=g, dtype=torch.float64) * 0.5
    v = torch.randn(B, S, Hkv, D, generator=g, dtype=torch.float64) * 0.5
    do = torch.randn(B, S, Hq, D, generator=g, dtype=torch.float64)
    shape = {"vector": (1, Hq, 1, S), "matrix": (1, Hq, S, S), "matrix_per_batch": (B, 1, S, S)}[kind]
    bias = torch.randn(shape, generator=g, dtype=torch.float64)
    bf, allow = reference_test_bitfield(B, S)
    fmask = torch.where(allow.unsqueeze(1), bias.expand(B, Hq, S, S), torch.full((), float("-inf"), dtype=torch.float64))
    qr, kr, vr = (t.clone().requires_grad_(True) for t in (q, k, v))
    ref = F.scaled_dot_product_attention(
        qr.transpose(1, 2), kr.transpose(1, 2), vr.transpose(1, 2), attn_mask=fmask, enable_gqa=True
    ).transpose(1, 2)
    o, lse = O.attention_forward(q, k, v, bf, dtype=torch.float64, bias=bias, row_chunk=64)
    assert torch.allclose(o, ref, atol=1e-10, rtol=0)
    kk = k.repeat_interleave(Hq // Hkv, dim=2)
    s = torch.einsum("bihd,bjhd->bhij", q, kk) / math.sqrt(D) + fmask
    assert torch.allclose(lse, torch.logsumexp(s, dim=-1), atol=1e-10, rtol=0)
    want = torch.autograd.grad(ref, (qr, kr, vr), do)
    got = O.attention_backward(q, k, v, bf, do, dtype=torch.float64, bias=bias, row_chunk=64)
    for a, b_ in zip(got, want):
        assert torch.allclose(a, b_, atol=1e-10, rtol=0)
    # the materialized-mask functions take the same bias
    o2, lse2 = O.masked_attention_forward(q, k, v, allow, dtype=torch.float64, bias=bias)
    assert torch.allclose(o2, ref, atol=1e-10, rtol=0) and torch.allclose(lse2, lse, atol=1e-10, rtol=0)
    got2 = O.masked_attention_backward(q, k, v, allow, do, dtype=torch.float64, bias=bias)
    for a, b_ in zip(got2, want):
        assert torch.allclose(a, b_, atol=1e-10, rtol=0)


def test_bias_closed_forms():
    B, S, H, D = 1, 96, 2, 8
    g = torch.Generator().manual_seed(12)
    q, k, v = (torch.randn(B, S, H, D, generator=g, dtype=torch.float64) for _ in range(3))
    bf, _ = reference_test_bitfield(B, S)
    o0, lse0 = O.attention_forward(q, k, v, bf, dtype=torch.float64)
    # constant along the keys: softmax unchanged, lse shifted by the constant
    c = torch.randn(B, H, S, 1, generator=g, dtype=torch.float64)
    o1, lse1 = O.attention_forward(q, k, v, bf, dtype=torch.float64, bias=c.expand(B, H, S, S))
    assert torch.allclose(o1, o0, atol=1e-12, rtol=0)
    assert torch.allclose(lse1, lse0 + c[..., 0], atol=1e-12, rtol=0)
    # bias = log w on zero queries: o = sum_j w_j v_j / sum_j w_j over the allowed keys
    w = torch.rand(1, H, 1, S, generator=g, dtype=torch.float64) + 0.1
    o2, _ = O.attention_forward(torch.zeros_like(q), k, v, bf, dtype=torch.float64, bias=w.log())
    allow = O.materialize_mask(bf)[0].to(torch.float64)  # (S, S)
    ww = allow[None] * w[0, :, 0][:, None, :]  # (H, S, S)
    want = torch.einsum("hij,jhd->ihd", ww / ww.sum(-1, keepdim=True), v[0])
    assert torch.allclose(o2[0], want, atol=1e-12, rtol=0)


# ------------------------------------------------------------------ the routine the CPU baseline times
@pytest.mark.parametrize("row_chunk", [128, 77, 4096])
def test_chunked_sdpa_routine_matches_the_attention_oracle(row_chunk):
    # grouped kv heads, padding rows (bitfield 0) and a chunk that does not divide the sequence
    B, S, Hq, Hkv, D = 2, 300, 4, 2, 32
    g = torch.Generator().manual_seed(11)
    q = torch.randn(B, S, Hq, D, generator=g)
    k = torch.randn(B, S, Hkv, D, generator=g)
    v = torch.randn(B, S, Hkv, D, generator=g)
    do = torch.randn(B, S, Hq, D, generator=g)
    bf = random_bitfield(B, S, seed=5, pad=9)
    o, dq, dk, dv = O.sdpa_forward_backward(q, k, v, bf, do, row_chunk=row_chunk)
    o_ref, _ = O.attention_forward(q, k, v, bf)
    assert (o - o_ref).abs().max().item() <= 1e-5
    assert torch.equal(O.sdpa_forward_backward(q, k, v, bf, row_chunk=row_chunk), o)  # forward-only form
    for got, want in zip((dq, dk, dv), O.attention_backward(q, k, v, bf, do)):
        assert rel_l2(got, want) <= 1e-5
    # padding rows: zero output, zero gradient, finite everywhere
    assert (o[:, S - 9 :] == 0).all() and (dq[:, S - 9 :] == 0).all()
    assert all(torch.isfinite(t).all() for t in (o, dq, dk, dv))


# ------------------------------------------------------------------ single-token decode step
def _decode_inputs(B=2, Hq=4, Hkv=2, Sk=37, D=16, seed=3):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(B, Hq, 1, D, generator=g), torch.randn(B, Hkv, Sk, D, generator=g),
            torch.randn(B, Hkv, Sk, D, generator=g))


def test_decode_step_plain_is_library_sdpa():
    q, k, v = _decode_inputs()
    want = F.scaled_dot_product_attention(q, k, v, enable_gqa=True).transpose(1, 2)
    assert torch.allclose(O.decode_step(q, k, v), want, atol=1e-6)
    want = F.scaled_dot_product_attention(q, k, v, enable_gqa=True, scale=0.3).transpose(1, 2)
    assert torch.allclose(O.decode_step(q, k, v, scaling=0.3), want, atol=1e-6)


def test_decode_step_window_and_softcap_closed_forms():
    q, k, v = _decode_inputs()
    Sk = k.shape[2]
    plain = O.decode_step(q, k, v)
    # a window at least as long as the cache, or a cap far above every score, changes nothing
    assert torch.equal(O.decode_step(q, k, v, sliding_window=Sk), plain)
    assert torch.equal(O.decode_step(q, k, v, sliding_window=Sk + 5), plain)
    assert torch.allclose(O.decode_step(q, k, v, softcap=1e6), plain, atol=1e-5)
    # a window of w keys == attention over the last w keys of the cache
    for w in (1, 5, Sk - 1):
        want = F.scaled_dot_product_attention(q, k[:, :, Sk - w :], v[:, :, Sk - w :], enable_gqa=True).transpose(1, 2)
        assert torch.allclose(O.decode_step(q, k, v, sliding_window=w), want, atol=1e-6)
    assert torch.allclose(O.decode_step(q, k, v, sliding_window=1)[:, 0], v[:, :, -1].repeat_interleave(2, 1), atol=1e-6)
    # a tiny cap flattens the scores: softmax of (almost) equal logits is the mean of V
    mean_v = v.mean(dim=2).repeat_interleave(2, 1)
    assert torch.allclose(O.decode_step(q, k, v, softcap=1e-4)[:, 0], mean_v, atol=1e-3)


def test_decode_step_brute_force_with_both():
    q, k, v = _decode_inputs(B=1, Hq=2, Hkv=1, Sk=9, D=4, seed=8)
    cap, w, scale = 0.7, 4, 0.9
    got = O.decode_step(q, k, v, scaling=scale, sliding_window=w, softcap=cap)
    for h in range(2):
        logits = []
        for j in range(9 - w, 9):
            s = scale * sum(float(q[0, h, 0, d]) * float(k[0, 0, j, d]) for d in range(4))
            logits.append(cap * math.tanh(s / cap))
        mx = max(logits)
        e = [math.exp(x - mx) for x in logits]
        for d in range(4):
            want = sum(e[i] * float(v[0, 0, 9 - w + i, d]) for i in range(w)) / sum(e)
            assert abs(float(got[0, 0, h, d]) - want) <= 1e-5
