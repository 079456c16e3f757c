"""The backward that hands dS from the dK/dV kernel to the dQ kernel through a workspace (head dim 128) against the
backward that recomputes S and dP for dQ: same dk / dv bit for bit, dq to rounding (both sum the same rounded dS
values, in another order), both within the gradient bar of the fp32 oracle.  The reference computes dS once per tile
as well (bitfield_attention.py:877-898) and adds ds k to dq with atomics; here the sum has one owner per row."""

import math

import pytest
import torch

from cornstarch_amd.kernel import attention as A
from cornstarch_amd.kernel import bitfield_attention as BA
from oracle import bam_oracle as O
from tests.helpers import random_bitfield, rel_l2

pytestmark = pytest.mark.gpu

GRAD_REL_L2 = 5e-2


def dev():
    return torch.device("cuda:0")


def inputs(B, S, Hq, Hkv, D, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, S, Hq, D, generator=g) * 0.5).to(dtype)
    k = (torch.randn(B, S, Hkv, D, generator=g) * 0.5).to(dtype)
    v = (torch.randn(B, S, Hkv, D, generator=g) * 0.5).to(dtype)
    do = torch.randn(B, S, Hq, D, generator=g).to(dtype)
    return q, k, v, do


def build(bf):
    BA.BitfieldUtils.clear_cache()
    flags = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf)
    plan = BA.BitfieldUtils.plan_for(flags, bf)
    assert plan is not None
    return flags, plan


@pytest.mark.parametrize("S", [1, 57, 283, 1000])
def test_pair_numbering_against_the_fine_classes(S):
    bf = random_bitfield(3, S, seed=S, pad=min(5, S - 1)).to(dev())
    flags, plan = build(bf)
    st, ws = plan.struct, plan.workspace
    slots, nkt, num_n = 4 * flags.shape[1], -(-S // 128), -(-S // 32)
    fine = torch.nn.functional.pad(plan.fine_classes().cpu(), (0, 4 * nkt - num_n))
    has = (fine.view(3, slots, nkt, 4) != 0).any(dim=3)                          # (B, slots, nkt)
    i32 = ws.view(torch.int32)
    entry = torch.as_strided(i32, (3, slots, nkt), (st.ds_entry_stride_b, nkt, 1), (st.ds_entry - ws.data_ptr()) // 4).cpu()
    base = torch.as_strided(i32, (3, nkt), (nkt, 1), (st.ds_tile_base - ws.data_ptr()) // 4).cpu()
    # the pairs of a key tile carry consecutive numbers from the tile's base, by ascending slice; the tiles' blocks of
    # numbers tile [0, total) without gaps or overlaps (which tile gets which block is not specified)
    blocks = []
    for bb in range(3):
        for t in range(nkt):
            col = has[bb, :, t]
            n_t = int(col.sum())
            start = int(base[bb, t])
            assert entry[bb, :, t][col].tolist() == list(range(start, start + n_t))
            assert (entry[bb, :, t][~col] == -1).all()
            if n_t:
                blocks.append((start, n_t))
    blocks.sort()
    assert all(blocks[i][0] + blocks[i][1] == blocks[i + 1][0] for i in range(len(blocks) - 1))
    assert not blocks or (blocks[0][0] == 0 and blocks[-1][0] + blocks[-1][1] == int(has.sum()))
    assert plan.ds_pairs() == int(has.sum())
    # the order in which the dK/dV kernel takes the key tiles: every (batch, tile) once, most pairs first, ties by code
    order = torch.as_strided(i32, (3 * nkt,), (1,), (st.ds_tile_order - ws.data_ptr()) // 4).cpu().tolist()
    counts = has.sum(dim=1).reshape(-1).tolist()                                 # by code b * nkt + t
    assert order == sorted(range(3 * nkt), key=lambda c: (-counts[c], c))
    BA.BitfieldUtils.clear_cache()


def run_backward(q, k, v, do, bf, handover, monkeypatch, accumulate=False):
    monkeypatch.setattr(BA, "_ds_workspace_limit", (lambda device: 1 << 40) if handover else (lambda device: 0))
    flags, plan = build(bf)
    o, lse, scale = BA._bitfield_attn_forward(q, k, v, bf, flags)
    if accumulate:
        grads = [torch.zeros_like(t, dtype=torch.float32) for t in (q, k, v)]
        BA._bitfield_attn_backward(do, q, k, v, o, bf, flags, lse, *grads, softmax_scale=scale)
    else:
        grads = BA._bitfield_attn_backward_overwrite(do, q, k, v, o, bf, flags, lse, scale)
    torch.cuda.synchronize()
    assert plan.struct.ds_workspace is None  # detached after the launches
    return [g.clone() for g in grads]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,S,Hq,Hkv", [(2, 57, 2, 1), (1, 283, 4, 4), (2, 517, 4, 2), (1, 1000, 8, 2), (1, 2048, 4, 1)])
@pytest.mark.parametrize("accumulate", [False, True], ids=["typed", "fp32"])
def test_handover_equals_recomputation(dtype, B, S, Hq, Hkv, accumulate, monkeypatch):
    d = dev()
    bf = random_bitfield(B, S, seed=S, pad=3).to(d)
    q, k, v, do = (t.to(d) for t in inputs(B, S, Hq, Hkv, 128, dtype, seed=S))
    with_ds = run_backward(q, k, v, do, bf, True, monkeypatch, accumulate)
    recomputed = run_backward(q, k, v, do, bf, False, monkeypatch, accumulate)
    assert torch.equal(with_ds[1], recomputed[1]) and torch.equal(with_ds[2], recomputed[2])  # dk, dv: same kernel
    assert rel_l2(with_ds[0].float(), recomputed[0].float()) <= 2e-3
    again = run_backward(q, k, v, do, bf, True, monkeypatch, accumulate)
    assert all(torch.equal(a, b) for a, b in zip(with_ds, again))                            # no atomics: reruns agree
    for got, want in zip(with_ds, O.attention_backward(q, k, v, bf, do)):
        assert torch.isfinite(got).all() and rel_l2(got.float(), want) <= GRAD_REL_L2
    BA.BitfieldUtils.clear_cache()


def test_every_block_the_dq_kernel_reads_was_written(monkeypatch):
    # the workspace starts as NaN bit patterns: a block read but never written would show up in dq
    d = dev()
    B, S, Hq, Hkv = 2, 777, 4, 2
    bf = random_bitfield(B, S, seed=12, pad=9).to(d)
    q, k, v, do = (t.to(d) for t in inputs(B, S, Hq, Hkv, 128, torch.bfloat16, seed=5))
    flags, plan = build(bf)
    o, lse, scale = BA._bitfield_attn_forward(q, k, v, bf, flags)
    delta = torch.empty_like(lse)
    BA._launch_bwd_preprocess(o, do, delta)
    ws = plan.attach_ds_workspace(Hq, 128, S)
    assert ws is not None and ws.numel() == plan.ds_pairs() * Hq * 8192
    ws.fill_(0xFF)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    BA._launch_bwd_dkdv(q, k, v, do, lse, delta, dk, dv, bf, flags, scale, accumulate=False, plan=plan)
    BA._launch_bwd_dq(q, k, v, do, lse, delta, dq, bf, flags, scale, accumulate=False, plan=plan)
    plan.detach_ds_workspace()
    torch.cuda.synchronize()
    assert torch.isfinite(dq).all()
    dq2 = torch.empty_like(q)
    BA._launch_bwd_dq(q, k, v, do, lse, delta, dq2, bf, flags, scale, accumulate=False, plan=plan)  # recomputing kernel
    assert rel_l2(dq.float(), dq2.float()) <= 2e-3
    BA.BitfieldUtils.clear_cache()


def test_handover_with_index_tensors_dense_masks_and_bias(monkeypatch):
    d = dev()
    B, S, Hq, Hkv = 2, 640, 4, 2
    bf_cpu = random_bitfield(B, S, seed=3, pad=4)
    q, k, v, do = inputs(B, S, Hq, Hkv, 128, torch.bfloat16, seed=9)

    # index tensors: one zigzag "rank" (rows of chunks 0 and 3 of 4, keys of all chunks rank by rank)
    chunks = torch.arange(S).chunk(4)
    idx_q = torch.cat([chunks[0], chunks[3]])
    idx_k = torch.cat([chunks[0], chunks[3], chunks[1], chunks[2]])
    flags = O.tile_flags_indexed(bf_cpu, idx_q, idx_k).to(d)
    results = []
    for handover in (True, False):
        monkeypatch.setattr(BA, "_ds_workspace_limit", (lambda device: 1 << 40) if handover else (lambda device: 0))
        BA.BitfieldUtils.clear_cache()
        ql, dol = q[:, idx_q].contiguous().to(d), do[:, idx_q].contiguous().to(d)
        kl, vl = k[:, idx_k].contiguous().to(d), v[:, idx_k].contiguous().to(d)
        bfg, oq, ok = bf_cpu.to(d), idx_q.to(d), idx_k.to(d)
        o, lse, scale = BA._bitfield_attn_forward(ql, kl, vl, bfg, flags, oq, ok)
        grads = [torch.zeros_like(t, dtype=torch.float32) for t in (ql, kl, vl)]
        BA._bitfield_attn_backward(dol, ql, kl, vl, o, bfg, flags, lse, *grads, offsets_q=oq, offsets_k=ok, softmax_scale=scale)
        torch.cuda.synchronize()
        results.append(grads)
    assert torch.equal(results[0][1], results[1][1]) and torch.equal(results[0][2], results[1][2])
    assert rel_l2(results[0][0], results[1][0]) <= 2e-3
    want = O.attention_backward(q[:, idx_q], k[:, idx_k], v[:, idx_k], bf_cpu, do[:, idx_q], idx_q=idx_q, idx_k=idx_k)
    for got, w in zip(results[0], want):
        assert rel_l2(got.cpu(), w) <= GRAD_REL_L2

    # a materialized mask plus an ALiBi-like bias vector
    mask = O.materialize_mask(bf_cpu).to(d)
    bias = (-(torch.arange(S, dtype=torch.float32)[None, None, None, :]) * torch.tensor([0.01, 0.02, 0.04, 0.08])[None, :, None, None]).to(d)
    qd, kd, vd, dod = (t.to(d) for t in (q, k, v, do))
    results = []
    for handover in (True, False):
        monkeypatch.setattr(BA, "_ds_workspace_limit", (lambda device: 1 << 40) if handover else (lambda device: 0))
        A._MaskPlan.forget()
        o, lse, scale = A._flash_attn_forward(qd, kd, vd, bias=bias, mask=mask)
        grads = [torch.empty_like(t) for t in (qd, kd, vd)]
        A._flash_attn_backward(dod, qd, kd, vd, o, lse, *grads, bias=bias, mask=mask, softmax_scale=scale)
        torch.cuda.synchronize()
        results.append(grads)
    assert torch.equal(results[0][1], results[1][1]) and torch.equal(results[0][2], results[1][2])
    assert rel_l2(results[0][0].float(), results[1][0].float()) <= 2e-3
    want = O.masked_attention_backward(q, k, v, mask.cpu(), do, bias=bias.cpu())
    for got, w in zip(results[0], want):
        assert rel_l2(got.float().cpu(), w) <= GRAD_REL_L2
    A._MaskPlan.forget()
    BA.BitfieldUtils.clear_cache()


def test_head_dim_64_and_a_zero_limit_keep_the_recomputing_backward():
    d = dev()
    bf = random_bitfield(1, 300, seed=1).to(d)
    flags, plan = build(bf)
    assert plan.attach_ds_workspace(4, 64, 300) is None and plan.struct.ds_workspace is None
    ws = plan.attach_ds_workspace(4, 128, 300)
    assert ws is not None and plan.struct.ds_workspace == ws.data_ptr() and plan.struct.ds_capacity == plan.ds_pairs()
    plan.detach_ds_workspace()
    assert plan.struct.ds_workspace is None and plan.struct.ds_capacity == 0
    BA.BitfieldUtils.clear_cache()


def test_a_workspace_that_cannot_be_allocated_means_recomputation(monkeypatch):
    # no room for the dS workspace: the backward runs without it (the dQ kernel recomputes) instead of failing
    d = dev()
    q, k, v, do = (t.to(d) for t in inputs(1, 517, 4, 2, 128, torch.bfloat16, seed=3))
    bf = random_bitfield(1, 517, seed=4, pad=5).to(d)

    def grads():
        BA.BitfieldUtils.clear_cache()
        qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = BA.bitfield_attn_func(qg, kg, vg, bf)
        res = torch.autograd.grad(out, (qg, kg, vg), do)
        torch.cuda.synchronize()
        return res

    with_ws = grads()
    calls = []

    def no_memory(nbytes, device):
        calls.append(nbytes)
        raise torch.cuda.OutOfMemoryError("no room (test)")

    monkeypatch.setattr(BA._TilePlan, "_allocate", staticmethod(no_memory))
    without = grads()
    assert calls and calls[0] == 4 * 8192 * BA.BitfieldUtils.plan_for(
        BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf), bf).ds_pairs()
    want = O.attention_backward(q.cpu(), k.cpu(), v.cpu(), bf.cpu(), do.cpu())
    for a, b, w in zip(with_ws, without, want):
        assert rel_l2(a.float(), b.float()) <= 2e-3
        assert rel_l2(b.float().cpu(), w) <= GRAD_REL_L2
    BA.BitfieldUtils.clear_cache()


@pytest.mark.parametrize("runs", [2, 4])
@pytest.mark.parametrize("accumulate", [False, True], ids=["typed", "fp32"])
def test_heads_in_runs_under_a_small_workspace_limit(runs, accumulate, monkeypatch):
    # a limit that holds the dS of Hq / runs heads only: the backward takes the kv heads in `runs` runs through one
    # workspace of that size, and every gradient comes out bit for bit as with one launch pair for all heads
    from cornstarch_amd.kernel import _bam_hip

    d = dev()
    B, S, Hq, Hkv = 2, 640, 8, 4
    bf = random_bitfield(B, S, seed=21, pad=6).to(d)
    q, k, v, do = (t.to(d) for t in inputs(B, S, Hq, Hkv, 128, torch.bfloat16, seed=8))
    whole = run_backward(q, k, v, do, bf, True, monkeypatch, accumulate)

    flags, plan = build(bf)
    limit = _bam_hip.load().bam_ds_workspace_bytes(Hq // runs, plan.ds_pairs())
    monkeypatch.setattr(BA, "_ds_workspace_limit", lambda device: limit)
    assert plan.ds_head_runs(B, Hq, Hkv, 128, S) == runs
    assert plan.ds_head_runs(B, Hq, Hkv, 64, S) == 1  # no hand-over at head dim 64: nothing to split for
    allocated = []
    real = BA._TilePlan._allocate
    monkeypatch.setattr(BA._TilePlan, "_allocate",
                        staticmethod(lambda nbytes, device: allocated.append(nbytes) or real(nbytes, device)))
    o, lse, scale = BA._bitfield_attn_forward(q, k, v, bf, flags)
    if accumulate:
        grads = [torch.zeros_like(t, dtype=torch.float32) for t in (q, k, v)]
        BA._bitfield_attn_backward(do, q, k, v, o, bf, flags, lse, *grads, softmax_scale=scale)
    else:
        grads = BA._bitfield_attn_backward_overwrite(do, q, k, v, o, bf, flags, lse, scale)
    torch.cuda.synchronize()
    assert allocated == [limit] and plan.struct.ds_workspace is None
    for got, want in zip(grads, whole):
        assert torch.equal(got, want)
    BA.BitfieldUtils.clear_cache()


def test_heads_in_runs_with_index_tensors_and_dense_masks(monkeypatch):
    d = dev()
    B, S, Hq, Hkv = 1, 512, 4, 2
    bf_cpu = random_bitfield(B, S, seed=5, pad=4)
    q, k, v, do = inputs(B, S, Hq, Hkv, 128, torch.bfloat16, seed=2)
    chunks = torch.arange(S).chunk(4)
    idx_q = torch.cat([chunks[1], chunks[2]])
    idx_k = torch.cat([chunks[1], chunks[2], chunks[0], chunks[3]])
    flags = O.tile_flags_indexed(bf_cpu, idx_q, idx_k).to(d)
    ql, dol = q[:, idx_q].contiguous().to(d), do[:, idx_q].contiguous().to(d)
    kl, vl = k[:, idx_k].contiguous().to(d), v[:, idx_k].contiguous().to(d)
    bfg, oq, ok = bf_cpu.to(d), idx_q.to(d), idx_k.to(d)
    mask = O.materialize_mask(bf_cpu).to(d)
    qd, kd, vd, dod = (t.to(d) for t in (q, k, v, do))
    results = {}
    for limit in (1 << 40, None):  # None: room for one kv head's q heads
        if limit is None:
            per_run = []
            # the limit follows the plan in use: the dS of Hq / Hkv heads
            monkeypatch.setattr(BA, "_ds_workspace_limit", lambda device: per_run[-1])
            real_runs = BA._TilePlan.ds_head_runs

            def runs_with_limit(self, batch, nheads, nheads_k, head_dim, seqlen_k):
                from cornstarch_amd.kernel import _bam_hip
                per_run.append(_bam_hip.load().bam_ds_workspace_bytes(nheads // nheads_k, self.ds_pairs()))
                n = real_runs(self, batch, nheads, nheads_k, head_dim, seqlen_k)
                assert n == nheads_k
                return n

            monkeypatch.setattr(BA._TilePlan, "ds_head_runs", runs_with_limit)
        else:
            monkeypatch.setattr(BA, "_ds_workspace_limit", lambda device: limit)
        BA.BitfieldUtils.clear_cache()
        A._MaskPlan.forget()
        o, lse, scale = BA._bitfield_attn_forward(ql, kl, vl, bfg, flags, oq, ok)
        g1 = [torch.zeros_like(t, dtype=torch.float32) for t in (ql, kl, vl)]
        BA._bitfield_attn_backward(dol, ql, kl, vl, o, bfg, flags, lse, *g1, offsets_q=oq, offsets_k=ok, softmax_scale=scale)
        o, lse, scale = A._flash_attn_forward(qd, kd, vd, mask=mask)
        g2 = [torch.empty_like(t) for t in (qd, kd, vd)]
        A._flash_attn_backward(dod, qd, kd, vd, o, lse, *g2, mask=mask, softmax_scale=scale)
        torch.cuda.synchronize()
        results[limit] = g1 + g2
    for a, b in zip(results[1 << 40], results[None]):
        assert torch.equal(a, b)
    A._MaskPlan.forget()
    BA.BitfieldUtils.clear_cache()


def test_runs_of_heads_below_the_limit_when_the_workspace_is_large(monkeypatch):
    # within the limit, a workspace above the preferred size is still split while a run keeps enough workgroups
    d = dev()
    B, S, Hq, Hkv = 2, 640, 16, 8
    bf = random_bitfield(B, S, seed=2, pad=3).to(d)
    flags, plan = build(bf)
    key_tiles = B * 5
    monkeypatch.setattr(BA, "_ds_workspace_limit", lambda device: 1 << 40)
    assert plan.ds_head_runs(B, Hq, Hkv, 128, S) == 1                    # small workspace: one run
    monkeypatch.setattr(BA, "_DS_RUN_TARGET", 1)
    monkeypatch.setattr(BA, "_DS_RUN_MIN_WORKGROUPS", 2 * key_tiles)     # a run keeps at least two kv heads
    assert plan.ds_head_runs(B, Hq, Hkv, 128, S) == 4
    monkeypatch.setattr(BA, "_DS_RUN_MIN_WORKGROUPS", 8 * key_tiles + 1)  # no run is large enough: not split
    assert plan.ds_head_runs(B, Hq, Hkv, 128, S) == 1
    BA.BitfieldUtils.clear_cache()
