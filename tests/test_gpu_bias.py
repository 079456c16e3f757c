"""Additive attention bias (``bias`` of ``bitfield_attn_func`` / ``flash_attn_func`` and of the private
forward / backward entry points) on an MI355X, through the C ABI.

The reference accepts a 4-d bias whose last two dimensions are (1, seqlen_k) ("vector") or
(seqlen_q, seqlen_k) ("matrix"), in fp32 or the dtype of q, broadcast over batch and heads
(cornstarch/kernel/bitfield_attention.py:952-972); none of its tests passes one, so the expectations are the
fp32 oracle's (library SDPA with a float mask pins it).  Forward within 1e-2 + 1e-2 |x|, log-sum-exp within
1e-2, gradients within relative L2 5e-2.
"""

import math

import pytest
import torch

from cornstarch_amd.kernel import attention as A
from cornstarch_amd.kernel import bitfield_attention as BA
from oracle import bam_oracle as O
from tests.helpers import random_bitfield, reference_test_bitfield, rel_l2

pytestmark = pytest.mark.gpu

GRAD_REL_L2 = 5e-2


def dev():
    return torch.device("cuda:0")


def inputs(B, Sq, Sk, Hq, Hkv, D, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Sq, Hq, D, generator=g) * 0.5).to(dtype)
    k = (torch.randn(B, Sk, Hkv, D, generator=g) * 0.5).to(dtype)
    v = (torch.randn(B, Sk, Hkv, D, generator=g) * 0.5).to(dtype)
    do = torch.randn(B, Sq, Hq, D, generator=g).to(dtype)
    return q, k, v, do


def make_bias(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * 1.5).to(dtype)


def alibi(Hq, S):
    # ALiBi in its cheap form: slope_h * key position (the per-row shift slope_h * i cancels in the softmax)
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / Hq) for h in range(Hq)])
    return (slopes[None, :, None, None] * torch.arange(S, dtype=torch.float32)[None, None, None, :]).contiguous()


def check_bitfield(q, k, v, do, bf, bias, scale=None):
    d = dev()
    qg, kg, vg = (t.to(d).requires_grad_(True) for t in (q, k, v))
    out = BA.bitfield_attn_func(qg, kg, vg, bf.to(d), bias.to(d), scale)
    gq, gk, gv = torch.autograd.grad(out, (qg, kg, vg), do.to(d))
    torch.cuda.synchronize()
    fb = bias.float()
    o_ref, _ = O.attention_forward(q, k, v, bf, softmax_scale=scale, bias=fb)
    torch.testing.assert_close(out.float().cpu(), o_ref, atol=1e-2, rtol=1e-2)
    want = O.attention_backward(q, k, v, bf, do, softmax_scale=scale, bias=fb)
    for got, w in zip((gq, gk, gv), want):
        assert got.dtype == q.dtype
        assert rel_l2(got.float().cpu(), w) <= GRAD_REL_L2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("head_dim", [32, 64, 128])
@pytest.mark.parametrize("kind", ["vector_f32", "vector_16", "matrix_f32", "matrix_16"])
@pytest.mark.parametrize("S", [57, 256, 283])
def test_bitfield_attention_with_bias(dtype, head_dim, kind, S):
    B, Hq, Hkv = 2, 4, 2
    q, k, v, do = inputs(B, S, S, Hq, Hkv, head_dim, dtype, seed=S)
    bf, _ = reference_test_bitfield(B, S)
    bdtype = torch.float32 if kind.endswith("f32") else dtype
    shape = (1, Hq, 1, S) if kind.startswith("vector") else (B, Hq, S, S)
    check_bitfield(q, k, v, do, bf, make_bias(shape, bdtype, seed=head_dim + S))


def test_alibi_on_a_multimodal_layout_and_lse():
    B, S, Hq, Hkv, D = 1, 1024, 8, 2, 128
    q, k, v, do = inputs(B, S, S, Hq, Hkv, D, torch.bfloat16, seed=5)
    bf = random_bitfield(B, S, seed=9)
    bias = alibi(Hq, S) * 0.01
    check_bitfield(q, k, v, do, bf, bias)
    d = dev()
    bfg = bf.to(d)
    flags = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bfg)
    o, lse, _ = BA._bitfield_attn_forward(q.to(d), k.to(d), v.to(d), bfg, flags, bias=bias.to(d))
    _, lse_ref = O.attention_forward(q, k, v, bf, bias=bias)
    live = torch.isfinite(lse_ref)
    assert torch.equal(torch.isfinite(lse[..., :S].cpu()), live)
    assert (lse[..., :S].cpu()[live] - lse_ref[live]).abs().max().item() <= 1e-2
    BA.BitfieldUtils.clear_cache()


def test_bias_broadcast_over_batch_and_heads_unaligned_views_and_private_backward():
    # (1, 1, S, S) broadcast over batch and heads; a bias that is a slice of a wider tensor (odd row stride,
    # odd first element: the kernels fall back to element loads)
    B, S, Hq, Hkv, D = 2, 200, 4, 4, 64
    q, k, v, do = inputs(B, S, S, Hq, Hkv, D, torch.float16, seed=3)
    bf = random_bitfield(B, S, seed=4)
    wide = make_bias((1, 1, S, S + 3), torch.float32, seed=6)
    bias = wide[..., 1 : S + 1]
    assert bias.stride(-1) == 1 and bias.stride(-2) % 4 != 0
    check_bitfield(q, k, v, do, bf, bias)
    # private entry points: fp32 gradients accumulated into the caller's buffers
    d = dev()
    qg, kg, vg, dg, bg, bfg = (t.to(d) for t in (q, k, v, do, wide, bf))
    bg = bg[..., 1 : S + 1]
    flags = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bfg)
    o, lse, sc = BA._bitfield_attn_forward(qg, kg, vg, bfg, flags, bias=bg)
    acc = [torch.zeros_like(t, dtype=torch.float32) for t in (qg, kg, vg)]
    BA._bitfield_attn_backward(dg, qg, kg, vg, o, bfg, flags, lse, *acc, bias=bg, softmax_scale=sc)
    want = O.attention_backward(q, k, v, bf, do, bias=bias)
    for got, w in zip(acc, want):
        assert rel_l2(got.cpu(), w) <= GRAD_REL_L2
    BA.BitfieldUtils.clear_cache()


def test_bias_constant_along_keys_changes_nothing_but_lse():
    B, S, Hq, Hkv, D = 1, 384, 4, 2, 128
    q, k, v, _ = inputs(B, S, S, Hq, Hkv, D, torch.bfloat16, seed=21)
    d = dev()
    bf = random_bitfield(B, S, seed=22).to(d)
    flags = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf)
    qg, kg, vg = (t.to(d) for t in (q, k, v))
    o0, lse0, _ = BA._bitfield_attn_forward(qg, kg, vg, bf, flags)
    c = torch.full((1, Hq, 1, S), 3.0, device=d)
    o1, lse1, _ = BA._bitfield_attn_forward(qg, kg, vg, bf, flags, bias=c)
    assert (o1.float() - o0.float()).abs().max().item() <= 4e-3
    live = torch.isfinite(lse0)
    assert torch.equal(torch.isfinite(lse1), live)
    assert (lse1[live] - lse0[live] - 3.0).abs().max().item() <= 1e-3
    BA.BitfieldUtils.clear_cache()


@pytest.mark.parametrize("Sq,Sk", [(128, 1024), (300, 170), (57, 57)])
@pytest.mark.parametrize("kind", ["vector", "matrix"])
@pytest.mark.parametrize("with_mask", [True, False], ids=["mask", "nomask"])
def test_materialized_mask_attention_with_bias(Sq, Sk, kind, with_mask):
    B, Hq, Hkv, D = 2, 4, 2, 64
    q, k, v, do = inputs(B, Sq, Sk, Hq, Hkv, D, torch.bfloat16, seed=Sq + Sk)
    mask = None
    if with_mask:
        g = torch.Generator().manual_seed(Sk)
        mask = torch.rand(B, Sq, Sk, generator=g) < 0.5
        mask[:, :, 0] = True
    bias = make_bias((1, Hq, 1, Sk) if kind == "vector" else (B, Hq, Sq, Sk), torch.float32, seed=1)
    d = dev()
    qg, kg, vg = (t.to(d).requires_grad_(True) for t in (q, k, v))
    out = A.flash_attn_func(qg, kg, vg, bias=bias.to(d), mask=mask.to(d) if with_mask else None)
    gq, gk, gv = torch.autograd.grad(out, (qg, kg, vg), do.to(d))
    o_ref, _ = O.masked_attention_forward(q, k, v, mask, bias=bias)
    torch.testing.assert_close(out.float().cpu(), o_ref, atol=1e-2, rtol=1e-2)
    want = O.masked_attention_backward(q, k, v, mask, do, bias=bias)
    for got, w in zip((gq, gk, gv), want):
        assert rel_l2(got.float().cpu(), w) <= GRAD_REL_L2


def test_index_tensors_with_bias():
    # the bias is indexed by LOCAL row / key (reference bitfield_attention.py:321-329 uses offs_m / offs_n)
    B, S, Hq, Hkv, D = 1, 512, 4, 2, 64
    q, k, v, do = inputs(B, 256, S, Hq, Hkv, D, torch.bfloat16, seed=31)
    bf = random_bitfield(B, S, seed=32)
    idx_q = torch.cat([torch.arange(0, 128), torch.arange(384, 512)])
    idx_k = torch.arange(S)
    bias = make_bias((1, Hq, 256, S), torch.float32, seed=33)
    d = dev()
    flags = O.tile_flags_indexed(bf, idx_q, idx_k).to(d)
    o, lse, sc = BA._bitfield_attn_forward(q.to(d), k.to(d), v.to(d), bf.to(d), flags, offsets_q=idx_q.to(d),
                                           offsets_k=idx_k.to(d), bias=bias.to(d))
    o_ref, _ = O.attention_forward(q, k, v, bf, idx_q=idx_q, idx_k=idx_k, bias=bias)
    torch.testing.assert_close(o.float().cpu(), o_ref, atol=1e-2, rtol=1e-2)
    acc = [torch.zeros_like(t, dtype=torch.float32, device=d) for t in (q, k, v)]
    BA._bitfield_attn_backward(do.to(d), q.to(d), k.to(d), v.to(d), o, bf.to(d), flags, lse, *acc,
                               offsets_q=idx_q.to(d), offsets_k=idx_k.to(d), bias=bias.to(d), softmax_scale=sc)
    want = O.attention_backward(q, k, v, bf, do, idx_q=idx_q, idx_k=idx_k, bias=bias)
    for got, w in zip(acc, want):
        assert rel_l2(got.cpu(), w) <= GRAD_REL_L2


def test_bias_argument_checks():
    d = dev()
    q, k, v, _ = (t.to(d) for t in inputs(1, 128, 128, 2, 2, 64, torch.bfloat16))
    bf = torch.full((1, 128), (1 << 62) | 1, dtype=torch.int64, device=d)
    with pytest.raises(RuntimeError):
        BA.bitfield_attn_func(q, k, v, bf, torch.zeros(1, 2, 5, 128, device=d))
    with pytest.raises(AssertionError):
        BA.bitfield_attn_func(q, k, v, bf, torch.zeros(2, 1, 128, device=d))
    with pytest.raises(AssertionError):
        BA.bitfield_attn_func(q, k, v, bf, torch.zeros(1, 2, 1, 128, device=d, dtype=torch.float64))
    # a bias whose last stride is not 1 is copied by the forward, like the reference does
    bt = torch.zeros(1, 2, 128, 128, device=d).transpose(-1, -2)
    out = BA.bitfield_attn_func(q, k, v, bf, bt)
    assert (out.float() - BA.bitfield_attn_func(q, k, v, bf).float()).abs().max().item() <= 4e-3
    BA.BitfieldUtils.clear_cache()
