"""Parity of the HIP kernels (through the C ABI) with the oracle, on an MI355X.

Bars: tile flags and materialized mask bit exact; forward output within max-abs 2e-2 of the
fp32 oracle (1e-2 + 1e-2*|x| elementwise for the reference's own test grid); gradients
within relative L2 5e-2.  The oracle runs on the CPU for the small cases and, for the
full-size workloads, as fp32 library math on the GPU (never the HIP kernels).
"""

import math

import pytest
import torch

from cornstarch_amd import workloads as W
from cornstarch_amd.kernel import bitfield_attention as BA
from cornstarch_amd.kernel import interface
from oracle import bam_oracle as O
from oracle import c_oracle as C
from tests.helpers import random_bitfield, reference_mask_kat, reference_test_bitfield, rel_l2

pytestmark = pytest.mark.gpu

O_MAX_ABS = 2e-2
GRAD_REL_L2 = 5e-2


def dev():
    return torch.device("cuda:0")


def flags_of(bf_gpu):
    BA.BitfieldUtils.clear_cache()
    return BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf_gpu)


def run_hip(q, k, v, bf, do=None, scale=None):
    """q, k, v, do: CPU tensors in the kernel dtype -> (o, lse[:S], dq, dk, dv) on the CPU."""
    d = dev()
    qg, kg, vg = (t.to(d).requires_grad_(do is not None) for t in (q, k, v))
    bfg = bf.to(d)
    BA.BitfieldUtils.clear_cache()
    o = BA.bitfield_attn_func(qg, kg, vg, bfg, softmax_scale=scale)
    grads = (None, None, None)
    if do is not None:
        grads = torch.autograd.grad(o, (qg, kg, vg), do.to(d))
    _, lse, _ = BA._bitfield_attn_forward(qg.detach(), kg.detach(), vg.detach(), bfg, flags_of(bfg), softmax_scale=scale)
    torch.cuda.synchronize()
    S = q.shape[1]
    return (o.detach().cpu(), lse[:, :, :S].cpu(), *(g.cpu() if g is not None else None for g in grads))


def make_inputs(B, S, Hq, Hkv, D, dtype, seed=0, std=0.5):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, S, Hq, D, generator=g) * std).to(dtype)
    k = (torch.randn(B, S, Hkv, D, generator=g) * std).to(dtype)
    v = (torch.randn(B, S, Hkv, D, generator=g) * std).to(dtype)
    do = torch.randn(B, S, Hq, D, generator=g).to(dtype)
    return q, k, v, do


def check_against_oracle(q, k, v, do, bf, scale=None, tight=False):
    o, lse, dq, dk, dv = run_hip(q, k, v, bf, do, scale)
    o_ref, lse_ref = O.attention_forward(q, k, v, bf, softmax_scale=scale)
    gq, gk, gv = O.attention_backward(q, k, v, bf, do, softmax_scale=scale)
    assert torch.isfinite(o).all()
    assert (o.float() - o_ref).abs().max().item() <= O_MAX_ABS
    if tight:  # the reference's own assert_close bar, widened for the bf16 output rounding
        torch.testing.assert_close(o.float(), o_ref, rtol=1e-2, atol=1e-2)
    fin = torch.isfinite(lse_ref)
    assert torch.equal(torch.isfinite(lse), fin)
    assert (lse[fin] - lse_ref[fin]).abs().max().item() <= 1e-2
    for got, want in ((dq, gq), (dk, gk), (dv, gv)):
        assert torch.isfinite(got).all()
        assert rel_l2(got, want) <= GRAD_REL_L2
        if tight:
            torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2)


# ------------------------------------------------------------------ flags and mask
@pytest.mark.parametrize("size", ["small", "large"])
def test_mask_kat_of_the_reference(size):
    bf, expected = reference_mask_kat(size)
    got = BA.materialize_bitfield_mask(bf.to(dev())).cpu()
    assert torch.equal(got, expected)


@pytest.mark.parametrize("S", [1, 31, 57, 128, 144, 283, 1000])
@pytest.mark.parametrize("wide", [False, True])
def test_flags_and_mask_bit_exact_on_irregular_bitfields(S, wide):
    bf = random_bitfield(3, S, seed=S, pad=min(5, S - 1), wide=wide)
    bfg = bf.to(dev())
    assert torch.equal(flags_of(bfg).cpu(), O.tile_flags(bf))
    assert torch.equal(flags_of(bfg).cpu(), torch.from_numpy(C.tile_flags(bf.numpy())))
    assert torch.equal(BA.materialize_bitfield_mask(bfg).cpu(), O.materialize_mask(bf))


@pytest.mark.parametrize("S", [57, 256, 335, 684, 1024, 2003, 3712])
def test_flags_rowblock_workloads_of_the_context_parallel_test(S):
    nn = -(-S // 32)
    causal = flags_of(torch.full((1, S), (1 << 62) | 1, dtype=torch.int64, device=dev()))[0].cpu()
    assert [(r > 0).sum().item() for r in causal] == [min(4 * (m + 1), nn) for m in range(causal.shape[0])]
    dense = flags_of(torch.full((1, S), 1 << 1, dtype=torch.int64, device=dev()))[0].cpu()
    assert (dense == 2).all()


@pytest.mark.parametrize("S", [57, 335, 1024, 3712])
def test_row_block_workloads_for_the_makespan_split(S):
    # torch.sum(compressed_mask > 0, dim=(0, 2)) of shardformer/layers/utils.py:161-166; for an all-text
    # sequence block m sees 4 (m + 1) tiles per sequence (test_context_parallel.py:258-272)
    causal = torch.full((3, S), (1 << 62) | 1, dtype=torch.int64, device=dev())
    got = BA.BitfieldUtils.nonempty_tiles_per_row_block(flags_of(causal))
    nm, nn = -(-S // 128), -(-S // 32)
    want = torch.tensor([3 * min(4 * (m + 1), nn) for m in range(nm)])
    assert got.dtype == torch.int64 and torch.equal(got.cpu(), want)
    bf = random_bitfield(2, S, seed=S).to(dev())
    flags = flags_of(bf)
    assert torch.equal(BA.BitfieldUtils.nonempty_tiles_per_row_block(flags), torch.sum(flags > 0, dim=(0, 2)))


@pytest.mark.parametrize("B,S", [(1, 57), (3, 335), (2, 1024), (2, 3712), (5, 2049)])
def test_row_block_workloads_come_with_the_plan(B, S):
    # the plan builder's numbering launch leaves the same sums in the plan: the flags tensor the cache holds gets them
    # from there (no launch), any other flags tensor -- a copy, a re-indexed one, one written since -- from the kernel
    bf = random_bitfield(B, S, seed=S + B, pad=min(5, S - 1)).to(dev())
    BA.BitfieldUtils.clear_cache()
    flags = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf)
    plan = BA.BitfieldUtils.plan_for(flags, bf)
    assert plan is not None and plan.struct.row_workloads
    want = torch.sum(flags > 0, dim=(0, 2))
    from_plan = BA.BitfieldUtils.nonempty_tiles_per_row_block(flags)
    assert from_plan.dtype == torch.int64 and from_plan.data_ptr() == plan.row_workloads().data_ptr()
    assert torch.equal(from_plan, want)
    copy = flags.clone()
    from_kernel = BA.BitfieldUtils.nonempty_tiles_per_row_block(copy)
    assert from_kernel.data_ptr() != plan.row_workloads().data_ptr() and torch.equal(from_kernel, want)
    flags[:, 0, 0] = 0  # written since the plan was built: counted again
    assert torch.equal(BA.BitfieldUtils.nonempty_tiles_per_row_block(flags), torch.sum(flags > 0, dim=(0, 2)))
    BA.BitfieldUtils.clear_cache()


def test_flags_of_a_strided_bitfield_row_view():
    base = random_bitfield(4, 600, seed=11)
    big = torch.zeros((4, 1000), dtype=torch.int64)
    big[:, :600] = base
    view = big.to(dev())[:, :600]  # row stride 1000
    assert not view.is_contiguous()
    assert torch.equal(flags_of(view).cpu(), O.tile_flags(base))


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_flags_bit_exact_on_the_benchmark_workloads(name):
    bf = W.make_bitfields(name)
    bfg = bf.to(dev())
    got = flags_of(bfg)
    want = O.tile_flags(bfg)  # oracle as torch library ops on the device (4.3e9 cells for C5)
    assert torch.equal(got, want)
    if name != "C5":
        assert torch.equal(got.cpu(), O.tile_flags(bf))
    if name == "C1":
        assert [(got == v).sum().item() for v in (0, 1, 2)] == [108, 24, 124]


def test_flag_cache_semantics():
    d = dev()
    a = random_bitfield(1, 256, 1).to(d)
    b = random_bitfield(1, 256, 2).to(d)
    BA.BitfieldUtils.clear_cache()
    fa = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(a)
    assert BA.BitfieldUtils.compressed_mask_cache is fa
    assert BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(a) is fa  # cached across layers
    fb = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(b)  # different mask: never stale
    assert torch.equal(fb.cpu(), O.tile_flags(b.cpu()))
    a[0, 5] = 0  # in-place edit bumps the version -> recomputed
    fa2 = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(a)
    assert torch.equal(fa2.cpu(), O.tile_flags(a.cpu()))
    BA.BitfieldUtils.clear_cache()
    assert BA.BitfieldUtils.compressed_mask_cache is None


def test_flag_cache_survives_a_mask_rebuilt_at_the_same_address():
    # A caller that never clears the cache builds a fresh mask every step by the same recipe (full_like + in-place
    # writes, as create_bitfield_attention_mask does): same shape, same version counter, and the caching allocator
    # likes to hand the freed block back.  The cache keeps its mask alive, so the new one cannot alias it.
    d = dev()
    S = 384

    def build(lo, hi):
        m = torch.full((1, S), (1 << 62) | 1 | 2, dtype=torch.int64, device=d)
        m[0, lo:hi] = 2
        return m

    BA.BitfieldUtils.clear_cache()
    a = build(10, 200)
    ptr_a, ver_a = a.data_ptr(), a._version
    fa = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(a).clone()
    del a  # the step is over; without the cache's reference the block would return to the allocator
    b = build(250, 380)
    assert b._version == ver_a
    assert b.data_ptr() != ptr_a  # the cached mask still owns its address
    fb = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(b)
    assert torch.equal(fb.cpu(), O.tile_flags(b.cpu()))
    assert not torch.equal(fb, fa)
    # after clear_cache() the address is free again; whatever the allocator does then, the flags are b2's
    BA.BitfieldUtils.clear_cache()
    del b
    b2 = build(100, 300)
    f2 = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(b2)
    assert torch.equal(f2.cpu(), O.tile_flags(b2.cpu()))
    BA.BitfieldUtils.clear_cache()


# ----------------------------------------------------------------------- delta pre-pass
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("S", [57, 128, 300])
def test_delta_prepass_against_both_oracles(D, dtype, S):
    # bam_bwd_preprocess (reference _bwd_preprocess_do_o_dot, bitfield_attention.py:527-572) called through the C
    # ABI on strided views: o as the transposed (B, H, S, D) buffer the HF adapter produces, do as a slice of a
    # wider buffer.  delta is (B, Hq, ceil(S/128)*128); entries at rows >= S must be left alone.
    from cornstarch_amd.kernel import _bam_hip

    d = dev()
    B, Hq = 2, 3
    g = torch.Generator().manual_seed(100 + D + S)
    o_base = (torch.randn(B, Hq, S, D, generator=g) * 0.7).to(dtype).to(d)
    do_base = torch.randn(B, S, Hq, D + 8, generator=g).to(dtype).to(d)
    o = o_base.transpose(1, 2)      # (B, S, Hq, D) view, head stride S * D
    do = do_base[..., 8:]           # row stride D + 8
    assert not o.is_contiguous() and not do.is_contiguous()
    S_r = -(-S // 128) * 128
    delta = torch.full((B, Hq, S_r), -777.0, dtype=torch.float32, device=d)
    _bam_hip.call(
        "bam_bwd_preprocess", o.data_ptr(), do.data_ptr(), delta.data_ptr(), *BA._strides3(o, do),
        B, S, Hq, D, BA._dtype_code(dtype), BA._stream_ptr(d),
    )
    torch.cuda.synchronize()
    assert (delta[:, :, S:] == -777.0).all()
    want = O.delta(o.cpu(), do.cpu())  # (B, Hq, S) fp32
    got = delta[:, :, :S].cpu()
    scale = want.abs().max().item()
    assert (got - want).abs().max().item() <= 1e-5 * max(scale, 1.0)
    want_c = torch.from_numpy(C.delta(o.float().cpu().contiguous().numpy(), do.float().cpu().contiguous().numpy()))
    assert (got - want_c.reshape(want.shape)).abs().max().item() <= 1e-5 * max(scale, 1.0)


# ------------------------------------------------- the reference's fwd/bwd test grids
REF_TOL = 5e-3  # rtol = atol of the reference's own assert_close (test_bitfield_attention.py:196-204, 299-307)
# dV in bf16 gets twice that bar.  dV = P^T dO with P rounded to bf16 before the product, exactly where the
# reference kernel rounds it (bitfield_attention.py:861), while the library SDPA it is compared with keeps P in
# fp32: the measured distance is up to 1.9 bars from the library result and 1.8 from the fp32 oracle (the
# library's own bf16 result sits 0.6 bars from the oracle, i.e. output rounding only).  O, dQ and dK stay inside
# one bar, and so does everything in fp16.
REF_TOL_DV_BF16 = 1e-2


def check_reference_case(batch_size, seqlen, Hq, Hkv, head_dim, dtype):
    """One case of the reference's test: seed 0, q/k/v ~ N(0, 0.5^2) drawn on the device, its bitfield, and its
    ground truth -- library SDPA in the SAME low precision with the closed-form mask, forward and autograd --
    at its own tolerance; next to it the fp32 oracle (run as library math on the device) at this repository's
    bars."""
    d = dev()
    torch.manual_seed(0)
    q, k, v = (
        torch.empty(batch_size, seqlen, h, head_dim, device=d, dtype=dtype).normal_(mean=0, std=0.5).requires_grad_(True)
        for h in (Hq, Hkv, Hkv)
    )
    bf, full_mask = (t.to(d) for t in reference_test_bitfield(batch_size, seqlen))
    want = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), full_mask.unsqueeze(1), enable_gqa=Hq != Hkv
    ).transpose(1, 2)
    BA.BitfieldUtils.clear_cache()
    got = BA.bitfield_attn_func(q, k, v, bitfield_mask=bf)
    torch.testing.assert_close(want, got, rtol=REF_TOL, atol=REF_TOL)
    g = torch.randn_like(want)
    grads_want = torch.autograd.grad(want, (q, k, v), g)
    grads_got = torch.autograd.grad(got, (q, k, v), g)
    for name, a, b in zip(("dq", "dk", "dv"), grads_want, grads_got):
        tol = REF_TOL_DV_BF16 if (name == "dv" and dtype == torch.bfloat16) else REF_TOL
        torch.testing.assert_close(a, b, rtol=tol, atol=tol, msg=lambda m, name=name: f"{name}: {m}")
    # fp32 oracle
    qd, kd, vd = q.detach(), k.detach(), v.detach()
    o_ref, lse_ref = O.attention_forward(qd, kd, vd, bf)
    assert (got.detach().float() - o_ref).abs().max().item() <= O_MAX_ABS
    _, lse, _ = BA._bitfield_attn_forward(qd, kd, vd, bf, flags_of(bf))
    assert (lse[:, :, :seqlen] - lse_ref).abs().max().item() <= 1e-2
    for a, b in zip(grads_got, O.attention_backward(qd, kd, vd, bf, g)):
        assert rel_l2(a.float(), b) <= GRAD_REL_L2


@pytest.mark.parametrize("head_dim", [32, 64, 128])
@pytest.mark.parametrize("seqlen", [57, 128, 144, 256, 283, 512, 1024])
@pytest.mark.parametrize("batch_size", [1, 2, 4])
def test_reference_grid_mha_fp16(head_dim, seqlen, batch_size):
    # tests/test_kernel/test_bitfield_attention.py:113-204 (H = 6, fp16, N(0, 0.5^2)): all 63 cases
    check_reference_case(batch_size, seqlen, 6, 6, head_dim, torch.float16)


@pytest.mark.parametrize("head_dim", [32, 64, 128])
@pytest.mark.parametrize("seqlen", [57, 128, 144, 256, 283, 512, 1024])
@pytest.mark.parametrize("batch_size", [1, 2])
@pytest.mark.parametrize("num_kv_heads", [1, 2, 3])
def test_reference_grid_gqa_bf16(head_dim, seqlen, batch_size, num_kv_heads):
    # tests/test_kernel/test_bitfield_attention.py:207-307 (Hq = 6, bf16): all 126 cases
    check_reference_case(batch_size, seqlen, 6, num_kv_heads, head_dim, torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_case_against_the_cpu_oracle(dtype):
    # the same layout checked against the oracle run on the CPU (the grids above run it on the device)
    bf, _ = reference_test_bitfield(2, 283)
    q, k, v, do = make_inputs(2, 283, 6, 2, 64, dtype)
    check_against_oracle(q, k, v, do, bf, tight=True)


@pytest.mark.parametrize("S,D,Hq,Hkv", [(200, 128, 4, 2), (517, 64, 4, 4), (96, 32, 2, 1)])
@pytest.mark.parametrize("wide", [False, True])
def test_irregular_bitfields_with_padding(S, D, Hq, Hkv, wide):
    bf = random_bitfield(2, S, seed=S + D, pad=9, wide=wide)
    q, k, v, do = make_inputs(2, S, Hq, Hkv, D, torch.bfloat16, seed=1)
    o, lse, dq, dk, dv = run_hip(q, k, v, bf, do)
    # padded rows (bitfield 0): o = 0, lse = -inf, no gradient flows in or out
    assert (o[:, -9:] == 0).all() and torch.isneginf(lse[:, :, -9:]).all()
    assert (dq[:, -9:] == 0).all() and (dk[:, -9:] == 0).all() and (dv[:, -9:] == 0).all()
    check_against_oracle(q, k, v, do, bf)


@pytest.mark.parametrize("S", [2, 3, 17, 31, 33, 65, 97])
@pytest.mark.parametrize("D", [32, 64, 128])
def test_very_short_sequences(S, D):
    # one ragged slice, one slice and a ragged one, odd slice counts: the corner cases of the slice pairs of dK/dV
    bf = random_bitfield(2, S, seed=S + D)
    q, k, v, do = make_inputs(2, S, 4, 2, D, torch.bfloat16, seed=S)
    check_against_oracle(q, k, v, do, bf)


@pytest.mark.parametrize("D", [32, 64, 128])
def test_single_token_sequence(D):
    # a token that sees only itself: o = v, lse = scale * q.k, dv = do, and dq = dk = 0 up to the rounding of o
    bf = torch.full((2, 1), (1 << 62) | 1 | 2, dtype=torch.int64)
    q, k, v, do = make_inputs(2, 1, 4, 2, D, torch.bfloat16, seed=D)
    o, lse, dq, dk, dv = run_hip(q, k, v, bf, do)
    kv_of_head = torch.arange(4) // 2
    assert torch.equal(o.cpu(), v[:, :, kv_of_head])
    want_lse = (q.float() * k.float()[:, :, kv_of_head]).sum(-1).transpose(1, 2) / math.sqrt(D)
    assert (lse[:, :, :1].cpu() - want_lse).abs().max().item() <= 1e-2
    want_dv = do.float().view(2, 1, 2, 2, D).sum(3)
    assert (dv.float().cpu() - want_dv).abs().max().item() <= 4e-2
    assert dq.float().abs().max().item() <= 1e-2 and dk.float().abs().max().item() <= 1e-2


def test_all_text_bitfield_is_causal_attention():
    # tests/test_shardformer/utils.py:388-391
    S = 300
    bf = torch.full((1, S), (1 << 62) | 1, dtype=torch.int64)
    q, k, v, do = make_inputs(1, S, 4, 4, 64, torch.float16, seed=3)
    o, *_ = run_hip(q, k, v, bf)
    want = torch.nn.functional.scaled_dot_product_attention(
        q.float().transpose(1, 2), k.float().transpose(1, 2), v.float().transpose(1, 2), is_causal=True
    ).transpose(1, 2)
    assert (o.float() - want).abs().max().item() <= 5e-3


def test_custom_softmax_scale_and_cross_check_with_c_oracle():
    bf = random_bitfield(1, 150, seed=8)
    q, k, v, do = make_inputs(1, 150, 2, 1, 32, torch.float16, seed=5)
    check_against_oracle(q, k, v, do, bf, scale=0.3)
    o, lse, dq, dk, dv = run_hip(q, k, v, bf, do, scale=0.3)
    co, clse = C.attn_fwd(q.float().numpy(), k.float().numpy(), v.float().numpy(), bf.numpy(), scale=0.3)
    assert (o.float() - torch.from_numpy(co)).abs().max().item() <= 5e-3
    cq, ck, cv = C.attn_bwd(*(x.float().numpy() for x in (q, k, v, do)), clse,
                            C.delta(co, do.float().numpy()), bf.numpy(), scale=0.3)
    for got, want in ((dq, cq), (dk, ck), (dv, cv)):
        assert rel_l2(got, torch.from_numpy(want)) <= 2e-2


@pytest.mark.parametrize("D", [16, 40, 80, 96])
def test_head_dims_between_the_native_ones(D):
    bf, _ = reference_test_bitfield(1, 144)
    q, k, v, do = make_inputs(1, 144, 4, 2, D, torch.bfloat16, seed=D)
    check_against_oracle(q, k, v, do, bf)


# ------------------------------------------------------------------------ properties
def test_gqa_equals_mha_with_repeated_kv_heads_bit_exactly():
    bf = random_bitfield(2, 400, seed=21)
    q, k, v, do = make_inputs(2, 400, 8, 2, 128, torch.bfloat16, seed=2)
    o_g, lse_g, dq_g, dk_g, dv_g = run_hip(q, k, v, bf, do)
    kr, vr = k.repeat_interleave(4, dim=2), v.repeat_interleave(4, dim=2)
    o_m, lse_m, dq_m, dk_m, dv_m = run_hip(q, kr, vr, bf, do)
    assert torch.equal(o_g, o_m) and torch.equal(lse_g, lse_m) and torch.equal(dq_g, dq_m)
    # dk of a kv head = sum of the dk of its q heads (fp32 sums in another order)
    assert rel_l2(dk_g, dk_m.float().view(2, 400, 2, 4, 128).sum(3)) <= 1e-2
    assert rel_l2(dv_g, dv_m.float().view(2, 400, 2, 4, 128).sum(3)) <= 1e-2


def test_masked_keys_do_not_influence_anything_bit_exactly():
    S = 384
    bf = torch.full((1, S), (1 << 62) | 1 | 2, dtype=torch.int64)
    bf[0, 100:228] = 4  # a modality the text does not carry: invisible to text, sees only itself
    q, k, v, do = make_inputs(1, S, 2, 2, 64, torch.bfloat16, seed=4)
    o1, lse1, dq1, dk1, dv1 = run_hip(q, k, v, bf, do)
    k2, v2 = k.clone(), v.clone()
    k2[0, 100:228] = 7.0
    v2[0, 100:228] = -9.0
    o2, lse2, dq2, dk2, dv2 = run_hip(q, k2, v2, bf, do)
    text = torch.ones(S, dtype=torch.bool)
    text[100:228] = False
    assert torch.equal(o1[0, text], o2[0, text]) and torch.equal(lse1[0][:, text], lse2[0][:, text])
    assert torch.equal(dq1[0, text], dq2[0, text])
    assert torch.equal(dk1[0, text], dk2[0, text]) and torch.equal(dv1[0, text], dv2[0, text])


def test_output_is_linear_in_v_and_runs_are_deterministic():
    bf = random_bitfield(1, 500, seed=31)
    q, k, v, do = make_inputs(1, 500, 4, 1, 128, torch.bfloat16, seed=6)
    a = run_hip(q, k, v, bf, do)
    b = run_hip(q, k, v, bf, do)
    for x, y in zip(a, b):
        assert torch.equal(x, y)  # no atomics anywhere: bit-identical reruns
    o2, lse2, *_ = run_hip(q, k, v * 2, bf)
    assert torch.equal(o2, a[0] * 2) and torch.equal(lse2, a[1])  # power-of-two scaling is exact


def test_strided_views_as_the_hf_adapter_passes_them():
    class M(torch.nn.Module):
        pass

    B, H, Hkv, S, D = 2, 4, 2, 200, 64
    bf = random_bitfield(B, S, seed=41)
    g = torch.Generator().manual_seed(0)
    q = (torch.randn(B, H, S, D, generator=g) * 0.5).bfloat16()  # (B, H, S, D) as HF modules hold them
    k = (torch.randn(B, Hkv, S, D, generator=g) * 0.5).bfloat16()
    v = (torch.randn(B, Hkv, S, D, generator=g) * 0.5).bfloat16()
    BA.BitfieldUtils.clear_cache()
    out, w = interface.bitfield_attention_forward(M(), q.to(dev()), k.to(dev()), v.to(dev()), bf.to(dev()),
                                                  scaling=123.0)  # ignored, as in the reference
    assert w is None and out.shape == (B, S, H, D)
    o_ref, _ = O.attention_forward(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), bf)
    assert (out.float().cpu() - o_ref).abs().max().item() <= O_MAX_ABS


def test_backward_accumulates_into_caller_buffers():
    # the private backward ADDS into fp32 dq/dk/dv (reference :1248-1250 zeroes them first)
    d = dev()
    bf = random_bitfield(1, 256, seed=51)
    q, k, v, do = (t.to(d) for t in make_inputs(1, 256, 2, 2, 64, torch.bfloat16, seed=7))
    bfg = bf.to(d)
    flags = flags_of(bfg)
    o, lse, sc = BA._bitfield_attn_forward(q, k, v, bfg, flags)
    assert sc == 1 / math.sqrt(64) and lse.shape == (1, 2, 256) and lse.dtype == torch.float32
    z = [torch.zeros_like(t, dtype=torch.float32) for t in (q, k, v)]
    BA._bitfield_attn_backward(do, q, k, v, o, bfg, flags, lse, *z)
    ones = [torch.ones_like(t, dtype=torch.float32) for t in (q, k, v)]
    BA._bitfield_attn_backward(do, q, k, v, o, bfg, flags, lse, *ones)
    for a, b in zip(z, ones):
        assert torch.allclose(a + 1, b, atol=1e-6)
    # a bias of the wrong shape is the reference's RuntimeError (bitfield_attention.py:964-968)
    with pytest.raises(RuntimeError):
        BA._bitfield_attn_forward(q, k, v, bfg, flags, bias=torch.zeros(1, 2, 2, 256, device=d))
    # identity index tensors change nothing
    ar = torch.arange(256, device=d)
    o2, lse2, _ = BA._bitfield_attn_forward(q, k, v, bfg, flags, offsets_q=ar, offsets_k=ar)
    assert torch.equal(o2, o) and torch.equal(lse2, lse)


@pytest.mark.parametrize("accumulate", [1, 0], ids=["fp32_accumulate", "typed_overwrite"])
def test_combined_backward_entry_point(accumulate):
    # bam_bwd = dK/dV and dQ in one call; the host functions use the two separate entry points, so this one is
    # called here directly, with and without a bias descriptor, and compared with them bit for bit
    import ctypes

    from cornstarch_amd.kernel import _bam_hip

    d = dev()
    B, S, Hq, Hkv, D = 2, 200, 4, 2, 64
    bf = random_bitfield(B, S, seed=61).to(d)
    q, k, v, do = (t.to(d) for t in make_inputs(B, S, Hq, Hkv, D, torch.bfloat16, seed=62))
    flags = flags_of(bf)
    bias = torch.randn(1, Hq, 1, S, device=d)
    for bias_t in (None, bias):
        o, lse, sc = BA._bitfield_attn_forward(q, k, v, bf, flags, bias=bias_t)
        delta = torch.empty_like(lse)
        BA._launch_bwd_preprocess(o, do, delta)
        gdt = torch.float32 if accumulate else q.dtype
        want = [torch.zeros(t.shape, dtype=gdt, device=d) for t in (q, k, v)]
        bview = BA._BiasView(bias_t, q, B, Hq, S, S) if bias_t is not None else None
        BA._launch_bwd_dkdv(q, k, v, do, lse, delta, want[1], want[2], bf, flags, sc, accumulate=bool(accumulate), bias=bview)
        BA._launch_bwd_dq(q, k, v, do, lse, delta, want[0], bf, flags, sc, accumulate=bool(accumulate), bias=bview)
        got = [torch.zeros(t.shape, dtype=gdt, device=d) for t in (q, k, v)]
        _bam_hip.call(
            "bam_bwd", q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            got[0].data_ptr(), got[1].data_ptr(), got[2].data_ptr(), bf.data_ptr(), flags.data_ptr(),
            *BA._strides3(q, k, v, do, *got), bf.stride(0), flags.stride(0), flags.stride(1),
            B, S, Hq, Hkv, D, float(sc), BA._dtype_code(q.dtype), accumulate,
            bview.byref() if bview is not None else None, None, BA._stream_ptr(d),
        )
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b)
        wq, wk, wv = O.attention_backward(q.cpu(), k.cpu(), v.cpu(), bf.cpu(), do.cpu(),
                                          bias=bias_t.cpu() if bias_t is not None else None)
        for a, w in zip(got, (wq, wk, wv)):
            assert rel_l2(a.float().cpu(), w) <= GRAD_REL_L2


# -------------------------------------------------- the five benchmark configurations
def _oracle_on_device(q, k, v, do, bf, row_chunk):
    o, lse = O.attention_forward(q, k, v, bf, row_chunk=row_chunk)
    grads = O.attention_backward(q, k, v, bf, do, row_chunk=row_chunk) if do is not None else (None,) * 3
    return (o, lse, *grads)


def test_config1_plumbing_fp32_reference_on_cpu():
    # forward only, fp32 N(0,1) inputs; the oracle runs in fp32 on the CPU, the kernels get the
    # same values rounded to their 16-bit input types (the oracle consumes the rounded values)
    q, k, v, _ = W.make_tensors("C1")
    bf = W.make_bitfields("C1")
    for dt in (torch.float16, torch.bfloat16):
        qr, kr, vr = (t.to(dt) for t in (q, k, v))
        o, lse, *_ = run_hip(qr, kr, vr, bf)
        o_ref, lse_ref = O.attention_forward(qr, kr, vr, bf)
        assert (o.float() - o_ref).abs().max().item() <= O_MAX_ABS
        assert (lse - lse_ref).abs().max().item() <= 1e-2
        assert (o.float() - O.attention_sdpa(qr.float(), kr.float(), vr.float(), bf)).abs().max().item() <= O_MAX_ABS


@pytest.mark.parametrize("name,row_chunk", [("C2", 1024), ("C3", 1024), ("C4", 1024), ("C5", 256)])
def test_full_size_configs_against_fp32_library_math(name, row_chunk):
    d = dev()
    q, k, v, do = (t.to(d) for t in W.make_tensors(name))
    bf = W.make_bitfields(name).to(d)
    w = W.WORKLOADS[name]
    qg, kg, vg = (t.requires_grad_(True) for t in (q, k, v))
    BA.BitfieldUtils.clear_cache()
    o = BA.bitfield_attn_func(qg, kg, vg, bf)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do)
    _, lse, _ = BA._bitfield_attn_forward(q.detach(), k.detach(), v.detach(), bf, flags_of(bf))
    o = o.detach()
    # fp32 oracle on the device, one KV group at a time to bound memory
    G = w.Hq // w.Hkv
    worst_o, worst_lse = 0.0, 0.0
    num = {"dq": 0.0, "dk": 0.0, "dv": 0.0}
    den = {"dq": 0.0, "dk": 0.0, "dv": 0.0}
    groups = range(w.Hkv)
    for hk in groups:
        hs = slice(hk * G, (hk + 1) * G)
        ks = slice(hk, hk + 1)
        o_r, lse_r, gq, gk, gv = _oracle_on_device(
            q.detach()[:, :, hs], k.detach()[:, :, ks], v.detach()[:, :, ks], do[:, :, hs], bf, row_chunk)
        worst_o = max(worst_o, (o[:, :, hs].float() - o_r).abs().max().item())
        worst_lse = max(worst_lse, (lse[:, hs, : w.S] - lse_r).abs().max().item())
        for key, got, want in (("dq", dq[:, :, hs], gq), ("dk", dk[:, :, ks], gk), ("dv", dv[:, :, ks], gv)):
            num[key] += float((got.double() - want.double()).pow(2).sum())
            den[key] += float(want.double().pow(2).sum())
    assert worst_o <= O_MAX_ABS, worst_o
    assert worst_lse <= 1e-2, worst_lse
    for key in num:
        assert math.sqrt(num[key] / den[key]) <= GRAD_REL_L2, (key, math.sqrt(num[key] / den[key]))


@pytest.mark.parametrize("S", [131072, 131072 + 4096 + 57])
def test_long_sequences_single_pass_and_several_passes(S):
    # Up to 131072 tokens a workgroup lists its tiles / slices once; beyond that the kernels walk the sequence in
    # several passes (and no plan is built: the flags alone drive them).  The second length needs two passes in all
    # three attention kernels and is ragged in every tile size.  The oracle runs as fp32 library math on the device.
    Hq, Hkv, D = 2, 1, 32
    d = dev()
    g = torch.Generator().manual_seed(77)
    q = (torch.randn(1, S, Hq, D, generator=g) * 0.5).to(torch.bfloat16).to(d)
    k = (torch.randn(1, S, Hkv, D, generator=g) * 0.5).to(torch.bfloat16).to(d)
    v = (torch.randn(1, S, Hkv, D, generator=g) * 0.5).to(torch.bfloat16).to(d)
    do = torch.randn(1, S, Hq, D, generator=g).to(torch.bfloat16).to(d)
    text = (1 << 62) | 1 | 2 | 4
    bf = torch.full((1, S), text, dtype=torch.int64)
    bf[0, 1000:5000] = 2        # two modality segments, the second one ends with the sequence
    bf[0, S - 3000:] = 4
    bf = bf.to(d)
    flags = flags_of(bf)
    assert torch.equal(flags.cpu(), O.tile_flags(bf.cpu()))
    assert (BA.BitfieldUtils.plan_for(flags, bf) is not None) == (S <= 131072)
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    o = BA.bitfield_attn_func(qg, kg, vg, bf)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do)
    o_r, lse_r, gq, gk, gv = _oracle_on_device(q, k, v, do, bf, 512)
    assert (o.detach().float() - o_r).abs().max().item() <= O_MAX_ABS
    for got, want in ((dq, gq), (dk, gk), (dv, gv)):
        assert rel_l2(got.float(), want) <= GRAD_REL_L2
    BA.BitfieldUtils.clear_cache()


@pytest.mark.parametrize("std,D,dtype", [(2.0, 128, torch.bfloat16), (3.0, 64, torch.float16), (4.0, 128, torch.bfloat16)])
def test_large_score_magnitudes(std, D, dtype):
    # log-sum-exp up to ~80: the deferred rescale of the online softmax (probabilities may exceed 1 by up to
    # 2^8 before the running maximum moves) must stay finite and accurate, also in fp16
    g = torch.Generator().manual_seed(5)
    B, S, Hq, Hkv = 1, 700, 4, 2
    q = (torch.randn(B, S, Hq, D, generator=g) * std).to(dtype)
    k = (torch.randn(B, S, Hkv, D, generator=g) * std).to(dtype)
    v = torch.randn(B, S, Hkv, D, generator=g).to(dtype)
    do = torch.randn(B, S, Hq, D, generator=g).to(dtype)
    bf = random_bitfield(B, S, seed=3)
    o, lse, dq, dk, dv = run_hip(q, k, v, bf, do)
    o_ref, lse_ref = O.attention_forward(q, k, v, bf)
    assert lse_ref.abs().max().item() > 15
    assert torch.isfinite(o).all()
    assert (o.float() - o_ref).abs().max().item() <= O_MAX_ABS
    assert (lse - lse_ref).abs().max().item() <= 3e-2
    for got, want in zip((dq, dk, dv), O.attention_backward(q, k, v, bf, do)):
        assert rel_l2(got.float(), want) <= GRAD_REL_L2


# ------------------------------------------------- what the wider dV bar of the bf16 grid consists of
def _dv_models(q, k, v, do, allow, scale, lse=None):
    """dV of the reference's arithmetic, built from fp32 library ops on the device
    (bitfield_attention.py:842-861): P = exp(scale * q.k - lse) in fp32, then P^T dO accumulated in fp32 and summed
    over the q heads of a kv head -- once with P rounded to the input dtype before the product (what the reference
    kernel and these kernels do), once with P kept in fp32 (what library SDPA does).  lse: (B, Hq, S) to use, or
    None for the exact fp32 log-sum-exp.  allow: bool (B, S, S).
    Returns (rounded, unrounded, exact lse), dV fp32 (B, S, Hkv, D)."""
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    G = Hq // Hkv
    qf, kf, gf = q.float(), k.float(), do.float()
    s = torch.einsum("bihd,bjhd->bhij", qf, kf.repeat_interleave(G, dim=2)) * scale
    s = s.masked_fill(~allow[:, None], -math.inf)
    exact = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - (exact if lse is None else lse)[..., None])
    out = []
    for pp in (p.to(q.dtype).float(), p):
        dv_h = torch.einsum("bhij,bihd->bjhd", pp, gf)                    # per q head
        out.append(dv_h.view(B, S, Hkv, G, D).sum(dim=3))
    return out[0], out[1], exact


@pytest.mark.parametrize("seqlen,head_dim,num_kv_heads,batch_size",
                         [(1024, 128, 1, 2), (1024, 64, 1, 2), (1024, 32, 1, 1), (512, 128, 2, 2), (283, 64, 3, 1),
                          (1024, 128, 3, 2)])
def test_the_dv_excess_over_library_sdpa_is_where_p_is_rounded(seqlen, head_dim, num_kv_heads, batch_size):
    # Cases of the reference's GQA bf16 grid (seed 0, N(0, 0.5^2), Hq = 6) with the largest dV distance from library
    # SDPA.  The kernels' dV is taken in fp32 from the accumulating entry point and decomposed:
    #  (1) given the lse the forward returned, it IS the reference arithmetic -- P = exp(scale s - lse) rounded to
    #      bf16, P^T dO accumulated in fp32 -- to a small fraction of the reference's 5e-3 bar;
    #  (2) that lse differs from the exact fp32 log-sum-exp by at most log(1 + 2^-9): the forward sums the
    #      probabilities as the P V product sees them, rounded to bf16 (so that the weights of O add up to one),
    #      where the reference sums them before rounding (bitfield_attention.py:470-481).  A shift of a row's lse
    #      by a fraction of a bf16 ulp moves P across rounding boundaries in rows with few keys, which is why
    #  (3) against the same arithmetic with the EXACT lse the distance is 1.4 to 2.5 bars (inside 3);
    #  (4) the reference arithmetic itself sits 0.6 to 1.5 bars from the same sums with P kept in fp32, i.e. from
    #      library SDPA's arithmetic: rounding P where the reference rounds it uses up most or all of a 5e-3 bar
    #      against SDPA on these cases before any other difference counts.
    d = dev()
    torch.manual_seed(0)
    q, k, v = (
        torch.empty(batch_size, seqlen, h, head_dim, device=d, dtype=torch.bfloat16).normal_(mean=0, std=0.5)
        for h in (6, num_kv_heads, num_kv_heads)
    )
    bf, full_mask = (t.to(d) for t in reference_test_bitfield(batch_size, seqlen))
    do = torch.randn_like(q)
    scale = 1.0 / math.sqrt(head_dim)
    BA.BitfieldUtils.clear_cache()
    flags = flags_of(bf)
    o, lse, _ = BA._bitfield_attn_forward(q, k, v, bf, flags)
    dq32, dk32, dv32 = (torch.zeros_like(t, dtype=torch.float32) for t in (q, k, v))
    BA._bitfield_attn_backward(do, q, k, v, o, bf, flags, lse, dq32, dk32, dv32)
    lse_k = lse[:, :, :seqlen]
    same_lse, _, exact = _dv_models(q, k, v, do, full_mask, scale, lse=lse_k)
    rounded, unrounded, _ = _dv_models(q, k, v, do, full_mask, scale)

    def bars(a, b):
        return ((a - b).abs() / (REF_TOL + REF_TOL * b.abs())).max().item()

    assert bars(dv32, same_lse) <= 0.25                                   # (1)
    assert (lse_k - exact).abs().max().item() <= math.log1p(2.0 ** -9) + 1e-5   # (2)
    assert bars(dv32, rounded) <= 3.0                                     # (3)
    assert bars(unrounded, rounded) > 0.5                                 # (4)
    # and the typed backward (what autograd returns) is the fp32 result rounded once
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = BA.bitfield_attn_func(qg, kg, vg, bitfield_mask=bf)
    dv_typed = torch.autograd.grad(out, vg, do)[0]
    assert torch.equal(dv_typed, dv32.to(torch.bfloat16))
    BA.BitfieldUtils.clear_cache()
