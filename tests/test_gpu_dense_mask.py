"""Materialized-mask attention (``flash_attn_func(q, k, v, mask=...)``) on an MI355X, through the C ABI.

The grid follows the reference's test of this entry point (tests/test_kernel/test_attention.py:10-111:
fp16 / bf16, head dims 32 / 64 / 128, query / key lengths incl. 128x1024 and 1024x128, the tril +
modality-squares mask, batch 1, 12 heads).  Checked against the fp32 oracle: flags bit exact, forward within
1e-2 + 1e-2 |x|, gradients within relative L2 5e-2.
"""

import pytest
import torch

from cornstarch_amd.kernel import attention as A
from cornstarch_amd.kernel import interface
from oracle import bam_oracle as O
from tests.helpers import rel_l2

pytestmark = pytest.mark.gpu

GRAD_REL_L2 = 5e-2


def dev():
    return torch.device("cuda:0")


def reference_mask(B, Sq, Sk):
    mask = torch.tril(torch.ones(B, Sq, Sk, dtype=torch.bool))
    mask[:, 12:24, :] = False
    mask[:, 12:24, 12:24] = True
    mask[:, 36:56, :] = False
    mask[:, 36:56, 36:56] = True
    return mask


def inputs(B, Sq, Sk, Hq, Hkv, D, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Sq, Hq, D, generator=g) * 0.5).to(dtype)
    k = (torch.randn(B, Sk, Hkv, D, generator=g) * 0.5).to(dtype)
    v = (torch.randn(B, Sk, Hkv, D, generator=g) * 0.5).to(dtype)
    do = torch.randn(B, Sq, Hq, D, generator=g).to(dtype)
    return q, k, v, do


def check(q, k, v, do, mask, scale=None):
    d = dev()
    qg, kg, vg = (t.to(d).requires_grad_(True) for t in (q, k, v))
    mg = mask.to(d) if mask is not None else None
    out = A.flash_attn_func(qg, kg, vg, mask=mg, softmax_scale=scale)
    gq, gk, gv = torch.autograd.grad(out, (qg, kg, vg), do.to(d))
    torch.cuda.synchronize()
    o_ref, _ = O.masked_attention_forward(q, k, v, mask, softmax_scale=scale)
    assert out.dtype == q.dtype and out.shape == q.shape
    torch.testing.assert_close(out.float().cpu(), o_ref, atol=1e-2, rtol=1e-2)
    wq, wk, wv = O.masked_attention_backward(q, k, v, mask, do, softmax_scale=scale)
    for got, want in ((gq, wq), (gk, wk), (gv, wv)):
        assert got.dtype == q.dtype
        assert rel_l2(got.float().cpu(), want) <= GRAD_REL_L2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("head_dim", [32, 64, 128])
@pytest.mark.parametrize(
    "seqlen", [(128, 128), (128, 1024), (1024, 128), (1024, 1024), (57, 57), (144, 144), (283, 283)],
    ids=["128x128", "128x1024", "1024x128", "1024x1024", "57x57", "144x144", "283x283"],
)
def test_reference_grid(dtype, head_dim, seqlen):
    Sq, Sk = seqlen
    q, k, v, do = inputs(1, Sq, Sk, 12, 12, head_dim, dtype)
    check(q, k, v, do, reference_mask(1, Sq, Sk))


@pytest.mark.parametrize("Sq,Sk", [(300, 170), (64, 515), (1, 33)])
def test_mask_flags_bit_exact_and_random_masks_with_dead_rows(Sq, Sk):
    g = torch.Generator().manual_seed(Sq)
    mask = torch.rand(2, Sq, Sk, generator=g) < 0.4
    mask[:, : Sq // 2, : Sk // 3] = True
    mask[:, Sq // 2 :, Sk // 2 :] = False
    mask[:, -1, :] = False  # a row that sees nothing: o = 0, gradients 0
    flags = A.mask_tile_flags(mask.to(dev()), 2, Sq, Sk, dev())
    assert torch.equal(flags.cpu(), O.mask_tile_flags(mask))
    q, k, v, do = inputs(2, Sq, Sk, 4, 2, 64, torch.bfloat16, seed=Sk)  # grouped kv heads as well
    check(q, k, v, do, mask)


def test_no_mask_head_dim_40_custom_scale():
    q, k, v, do = inputs(2, 200, 333, 4, 4, 40, torch.float16, seed=8)
    check(q, k, v, do, None, scale=0.2)


def test_private_entry_points_and_hf_adapter():
    d = dev()
    q, k, v, do = (t.to(d) for t in inputs(1, 144, 144, 4, 4, 64, torch.bfloat16, seed=2))
    mask = reference_mask(1, 144, 144).to(d)
    o, lse, scale = A._flash_attn_forward(q, k, v, mask=mask)
    assert lse.shape == (1, 4, 256) and lse.dtype == torch.float32 and scale == 64 ** -0.5
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    A._flash_attn_backward(do, q, k, v, o, lse, dq, dk, dv, mask=mask, softmax_scale=scale)
    want = O.masked_attention_backward(q.cpu(), k.cpu(), v.cpu(), mask.cpu(), do.cpu())
    for got, w in zip((dq, dk, dv), want):
        assert rel_l2(got.float().cpu(), w) <= GRAD_REL_L2
    out, none = interface.cornstarch_attention_forward(None, q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), mask)
    assert none is None and torch.equal(out, o)
    with pytest.raises(RuntimeError):  # reference attention.py:886-890
        A.flash_attn_func(q, k, v, bias=torch.zeros(1, 4, 3, 144, device=d))


def test_full_size_mask_materialized_from_bitfields_gives_the_bitfield_result_bit_for_bit():
    # C2 (S = 8192, GQA 32/8, D = 128): the same kernels with the allow decision read from the materialized mask
    # instead of derived from the bitfields must produce identical bits, forward and backward
    from cornstarch_amd import workloads as W
    from cornstarch_amd.kernel import bitfield_attention as BA

    d = dev()
    q, k, v, do = (t.to(d) for t in W.make_tensors("C2"))
    bf = W.make_bitfields("C2").to(d)
    mask = BA.materialize_bitfield_mask(bf)
    assert mask.dtype == torch.bool and mask.shape == (1, 8192, 8192)
    BA.BitfieldUtils.clear_cache()
    flags_b = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf)
    assert torch.equal(A.mask_tile_flags(mask, 1, 8192, 8192, d), flags_b)
    outs = []
    for fn in (lambda a, b, c: BA.bitfield_attn_func(a, b, c, bf), lambda a, b, c: A.flash_attn_func(a, b, c, mask=mask)):
        qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
        o = fn(qg, kg, vg)
        outs.append((o.detach(), *torch.autograd.grad(o, (qg, kg, vg), do)))
    # o and dq: every query row sees the same key tiles in the same order on both paths -> identical bits.
    # dk, dv: the bitfield path pairs up the row slices that have work (its plan), the mask path walks whole
    # 128-row blocks, so the fp32 partial sums of the two row streams meet in another order.
    names = ("o", "dq", "dk", "dv")
    for name, a, b in zip(names, *outs):
        if name in ("o", "dq"):
            assert torch.equal(a, b), name
        else:
            assert rel_l2(a.float(), b.float()) <= 2e-3, name
    BA.BitfieldUtils.clear_cache()


# ------------------------------------------------- flags + plan of a mask in one pass
@pytest.mark.parametrize("Sq,Sk,D", [(300, 170, 64), (517, 517, 128), (517, 516, 128), (1024, 2000, 32), (33, 700, 64)])
def test_mask_plan_classes_and_results_do_not_depend_on_the_plan(Sq, Sk, D, monkeypatch):
    d = dev()
    g = torch.Generator().manual_seed(Sq + Sk)
    mask = torch.rand(2, Sq, Sk, generator=g) < 0.5
    mask[:, : Sq // 2, : Sk // 3] = True           # full tiles
    mask[:, Sq // 3 :, Sk // 2 :] = False          # empty tiles
    mask[0, 40:70, :] = False                      # one empty and two partly empty row slices
    mask[:, -1, :] = False
    mg = mask.to(d)
    A._MaskPlan.forget()
    flags, plan = A._MaskPlan.get(mg, 2, Sq, Sk, d)
    assert plan is not None and torch.equal(flags.cpu(), O.mask_tile_flags(mask))
    assert A._MaskPlan.get(mg, 2, Sq, Sk, d)[1] is plan          # kept for the backward of the same mask
    n_q, n_k = -(-Sq // 32), -(-Sk // 32)
    pad = torch.nn.functional.pad(mask, (0, n_k * 32 - Sk, 0, n_q * 32 - Sq))
    cells = torch.nn.functional.pad(torch.ones_like(mask), (0, n_k * 32 - Sk, 0, n_q * 32 - Sq))
    cnt = pad.view(2, n_q, 32, n_k, 32).sum(dim=(2, 4))
    tot = cells.view(2, n_q, 32, n_k, 32).sum(dim=(2, 4))
    want = torch.where(cnt == 0, 0, torch.where(cnt == tot, 2, 1)).to(torch.uint8)
    fine = plan.fine_classes().cpu()
    assert torch.equal(fine[:, :n_q], want) and (fine[:, n_q:] == 0).all()
    assert torch.equal(plan.row_workloads().cpu(), torch.sum(flags.cpu() > 0, dim=(0, 2)))  # per 128-row block
    for b in range(2):
        order = plan.slice_order()[b].cpu().tolist()
        assert order[:n_q] == list(range(n_q - 1, -1, -1)) and all(x == -1 for x in order[n_q:])

    # the mask packed to bits, both orientations, zero outside the mask
    st, ws = plan.struct, plan.workspace

    def words(ptr, count):
        off = ptr - ws.data_ptr()
        return ws[off : off + 4 * count].view(torch.int32).cpu().to(torch.int64) & 0xFFFFFFFF

    rows_pad, keys_pad, n_blocks = 128 * -(-Sq // 128), 128 * -(-Sk // 128), 2 * -(-n_k // 2)
    assert (st.row_bits_stride_n, st.row_bits_stride_b) == (rows_pad, n_blocks * rows_pad)
    assert (st.col_bits_stride_s, st.col_bits_stride_b) == (keys_pad, (rows_pad // 32) * keys_pad)
    big = torch.zeros(2, rows_pad, max(keys_pad, 32 * n_blocks), dtype=torch.int64)
    big[:, :Sq, :Sk] = mask
    weights = 1 << torch.arange(32, dtype=torch.int64)
    want_rows = (big[:, :, : 32 * n_blocks].view(2, rows_pad, n_blocks, 32) * weights).sum(-1).permute(0, 2, 1)
    got_rows = words(st.row_bits, 2 * n_blocks * rows_pad).view(2, n_blocks, rows_pad)
    assert torch.equal(got_rows, want_rows)
    want_cols = (big[:, :, :keys_pad].view(2, rows_pad // 32, 32, keys_pad) * weights[None, None, :, None]).sum(2)
    got_cols = words(st.col_bits, 2 * (rows_pad // 32) * keys_pad).view(2, rows_pad // 32, keys_pad)
    assert torch.equal(got_cols, want_cols)

    q, k, v, do = (t.to(d) for t in inputs(2, Sq, Sk, 4, 2, D, torch.bfloat16, seed=Sq))

    def run():
        o, lse, scale = A._flash_attn_forward(q, k, v, mask=mg)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        A._flash_attn_backward(do, q, k, v, o, lse, dq, dk, dv, mask=mg, softmax_scale=scale)
        torch.cuda.synchronize()
        return o, lse[:, :, :Sq], dq, dk, dv

    with_plan = run()
    real_get = A._MaskPlan.get.__func__
    monkeypatch.setattr(A._MaskPlan, "get", classmethod(lambda cls, *a: (real_get(cls, *a)[0], None)))
    without = run()
    for name, a, b in zip(("o", "lse", "dq", "dk", "dv"), with_plan, without):
        # dk, dv: fp32 partial sums of the two row streams meet in another order.  dq at head dim 128: with a plan
        # the backward hands dS from dK/dV to the dQ kernel, without one dQ recomputes it.
        if name in ("dk", "dv") or (name == "dq" and D == 128):
            assert rel_l2(a.float(), b.float()) <= 2e-3, name
        else:
            assert torch.equal(a, b), name
    o_ref, _ = O.masked_attention_forward(q.cpu(), k.cpu(), v.cpu(), mask)
    torch.testing.assert_close(with_plan[0].float().cpu(), o_ref, atol=1e-2, rtol=1e-2)
    A._MaskPlan.forget()
