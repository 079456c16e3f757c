"""Index-tensor attention (``offsets_q`` / ``offsets_k``) on an MI355X, through the C ABI.

The cases follow the reference's context-parallel test
(tests/test_shardformer/test_context_parallel.py:284-376): a sequence is split over two "ranks", each
rank attends from its own rows to the keys of all ranks (concatenated rank by rank), and the results
must equal the plain attention result restricted to the rank's rows; dk / dv summed over the ranks must
equal the plain ones.  Both ranks run one after the other on the one GPU.  Bars as in
test_gpu_parity.py: flags / gathers bit exact, O max-abs 2e-2, gradients relative L2 5e-2 against the
fp32 oracle.
"""

import numpy as np
import pytest
import torch

from cornstarch_amd.kernel import _bam_hip
from cornstarch_amd.kernel import bitfield_attention as BA
from oracle import bam_oracle as O
from tests.helpers import TEXT_124, random_bitfield, rel_l2

pytestmark = pytest.mark.gpu

O_MAX_ABS = 2e-2
GRAD_REL_L2 = 5e-2


def dev():
    return torch.device("cuda:0")


def splits(S, kind):
    """Index sets of two ranks (reference shardformer/layers/utils.py:108-146, 180-197 and the split of
    test_context_parallel.py:316-319)."""
    if kind == "reference_test":  # first rank: a multiple of 128 rows, second rank: the rest
        base = (S // 2 // 128) * 128
        chunks = [np.arange(0, base), np.arange(base, S)]
    elif kind == "zigzag":
        c = np.array_split(np.arange(S), 4)
        chunks = [np.concatenate([c[0], c[3]]), np.concatenate([c[1], c[2]])]
    elif kind == "blocks":  # whole 128-row blocks dealt alternately (what the makespan split produces)
        blocks = np.arange(-(-S // 128))
        chunks = [np.concatenate([np.arange(b * 128, min((b + 1) * 128, S)) for b in blocks[r::2]]) for r in range(2)]
    else:  # "scattered": a random partition, positions in random order -- nothing is contiguous
        perm = np.random.RandomState(S).permutation(S)
        chunks = [perm[: S // 3], perm[S // 3 :]]
    return [torch.from_numpy(np.asarray(c, dtype=np.int64)) for c in chunks if len(c)]


def inputs(B, S, Hq, Hkv, D, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, S, Hq, D, generator=g) * 0.5).to(dtype)
    k = (torch.randn(B, S, Hkv, D, generator=g) * 0.5).to(dtype)
    v = (torch.randn(B, S, Hkv, D, generator=g) * 0.5).to(dtype)
    do = torch.randn(B, S, Hq, D, generator=g).to(dtype)
    return q, k, v, do


def test_gather_bitfields_bit_exact():
    bf = random_bitfield(3, 500, seed=1, wide=True)
    idx = torch.randint(0, 500, (333,), dtype=torch.int64)
    idx[7], idx[100] = 500, 10_000  # outside the bitfield: reads 0 (bitfield_attention.py:86-87)
    d = dev()
    bits = torch.empty((3, 333), dtype=torch.int64, device=d)
    pos = torch.empty((333,), dtype=torch.int32, device=d)
    bfg, idxg = bf.to(d), idx.to(d)
    _bam_hip.call("bam_gather_bitfields", bfg.data_ptr(), bfg.stride(0), 500, idxg.data_ptr(), 333, bits.data_ptr(),
                  bits.stride(0), pos.data_ptr(), 3, torch.cuda.current_stream().cuda_stream)
    want = torch.where(idx < 500, bf[:, idx.clamp(max=499)], torch.zeros(1, dtype=torch.int64))
    assert torch.equal(bits.cpu(), want)
    assert torch.equal(pos.cpu().to(torch.int64), idx)


def run_rank(q, k, v, do, bf, idx_q, idx_k, flags):
    """One rank's forward + backward through `_bitfield_attn_forward` / `_bitfield_attn_backward`, the entry
    points the reference's context-parallel wrapper calls (context_parallel_bitfield_attention.py:137-147,
    270-294).  CPU tensors in, CPU results out."""
    d = dev()
    ql, dol = q[:, idx_q].contiguous().to(d), do[:, idx_q].contiguous().to(d)
    kl, vl = k[:, idx_k].contiguous().to(d), v[:, idx_k].contiguous().to(d)
    bfg, fl = bf.to(d), flags.to(d)
    oq, ok = idx_q.to(d), idx_k.to(d)
    o, lse, scale = BA._bitfield_attn_forward(ql, kl, vl, bfg, fl, oq, ok)
    dq = torch.zeros_like(ql, dtype=torch.float32)
    dk = torch.zeros_like(kl, dtype=torch.float32)
    dv = torch.zeros_like(vl, dtype=torch.float32)
    BA._bitfield_attn_backward(dol, ql, kl, vl, o, bfg, fl, lse, dq, dk, dv, offsets_q=oq, offsets_k=ok, softmax_scale=scale)
    torch.cuda.synchronize()
    return o.cpu(), lse[:, :, : idx_q.numel()].cpu(), dq.cpu(), dk.cpu(), dv.cpu()


def check_ranks(B, S, Hq, Hkv, D, dtype, kind, bf, flags_from="oracle"):
    q, k, v, do = inputs(B, S, Hq, Hkv, D, dtype, seed=S)
    o, lse = O.attention_forward(q, k, v, bf)
    dq, dk, dv = O.attention_backward(q, k, v, bf, do)
    ranks = splits(S, kind)
    idx_k = torch.cat(ranks)
    sum_dk, sum_dv = torch.zeros_like(dk), torch.zeros_like(dv)
    for idx_q in ranks:
        if flags_from == "oracle":
            flags = O.tile_flags_indexed(bf, idx_q, idx_k)
        else:  # the reference recipe (shardformer/layers/utils.py:331-353) on the library's own global flags
            BA.BitfieldUtils.clear_cache()
            glob = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf.to(dev())).cpu()
            cols = torch.cat([r[::32] for r in ranks]) // 32
            flags = glob[:, idx_q[::128] // 128][:, :, cols].contiguous()
            assert torch.equal(flags, O.tile_flags_indexed(bf, idx_q, idx_k))
        go, glse, gdq, gdk, gdv = run_rank(q, k, v, do, bf, idx_q, idx_k, flags)
        assert (go.float() - o[:, idx_q]).abs().max() <= O_MAX_ABS
        live = torch.isfinite(lse[:, :, idx_q])
        assert torch.equal(torch.isfinite(glse), live)
        assert (glse[live] - lse[:, :, idx_q][live]).abs().max() <= 1e-2
        assert rel_l2(gdq, dq[:, idx_q]) <= GRAD_REL_L2
        sum_dk[:, idx_k] += gdk
        sum_dv[:, idx_k] += gdv
    assert rel_l2(sum_dk, dk) <= GRAD_REL_L2 and rel_l2(sum_dv, dv) <= GRAD_REL_L2


@pytest.mark.parametrize("seq_len", [256, 336, 400, 1024])
@pytest.mark.parametrize("batch_size", [1, 2])
def test_reference_context_parallel_case(batch_size, seq_len):
    # shapes, dtype, bitfield and split of test_context_parallel.py:284-319 (seq 64 gives rank 0 nothing)
    bf = torch.full((batch_size, seq_len), TEXT_124, dtype=torch.int64)
    bf[:, 32:44] = 1 << 1
    check_ranks(batch_size, seq_len, 8, 4, 64, torch.bfloat16, "reference_test", bf)


@pytest.mark.parametrize("kind", ["zigzag", "blocks", "scattered"])
@pytest.mark.parametrize("S,D,Hq,Hkv", [(300, 128, 4, 2), (777, 64, 4, 4), (1024, 32, 2, 1)])
def test_split_kinds_on_irregular_bitfields(kind, S, D, Hq, Hkv):
    bf = random_bitfield(2, S, seed=S + 1, pad=9, wide=(D == 64))
    check_ranks(2, S, Hq, Hkv, D, torch.float16 if D == 32 else torch.bfloat16, kind, bf)


@pytest.mark.parametrize("S", [640, 1024])
def test_local_flags_from_the_reference_recipe(S):
    bf = random_bitfield(2, S, seed=S)
    check_ranks(2, S, 4, 2, 128, torch.bfloat16, "blocks", bf, flags_from="reference_recipe")


def test_one_offset_tensor_without_the_other_is_rejected():
    d = dev()
    q = torch.zeros((1, 128, 2, 64), dtype=torch.bfloat16, device=d)
    bf = torch.full((1, 128), TEXT_124, dtype=torch.int64, device=d)
    flags = torch.zeros((1, 1, 4), dtype=torch.int8, device=d)
    with pytest.raises(ValueError):
        BA._bitfield_attn_forward(q, q, q, bf, flags, offsets_q=torch.arange(128, device=d))


def test_index_view_is_gathered_once_per_forward_backward_pair():
    # the backward of a shard reuses the gathered bitfields / positions of its forward; a changed offset tensor
    # (new tensor, or the same tensor written in place) is gathered again
    d = dev()
    S = 300
    bf = random_bitfield(1, S, seed=4).to(d)
    q, k, v, do = (t.to(d) for t in inputs(1, S, 2, 1, 64, torch.bfloat16, seed=4))
    off = torch.randperm(S, generator=torch.Generator().manual_seed(1)).to(d)
    BA.BitfieldUtils.clear_cache()
    assert BA._IndexView._last is None
    view_flags = O.tile_flags_indexed(bf.cpu(), off.cpu(), off.cpu()).to(d)
    o, lse, sc = BA._bitfield_attn_forward(q, k, v, bf, view_flags, offsets_q=off, offsets_k=off)
    first = BA._IndexView._last[1]
    grads = [torch.zeros_like(t, dtype=torch.float32) for t in (q, k, v)]
    BA._bitfield_attn_backward(do, q, k, v, o, bf, view_flags, lse, *grads, offsets_q=off, offsets_k=off)
    assert BA._IndexView._last[1] is first
    off2 = off.clone()
    BA._bitfield_attn_forward(q, k, v, bf, view_flags, offsets_q=off2, offsets_k=off2)
    assert BA._IndexView._last[1] is not first
    second = BA._IndexView._last[1]
    off2[:2] = off2[:2].flip(0)  # in-place edit: version bump
    fl2 = O.tile_flags_indexed(bf.cpu(), off2.cpu(), off2.cpu()).to(d)
    o2, _, _ = BA._bitfield_attn_forward(q, k, v, bf, fl2, offsets_q=off2, offsets_k=off2)
    assert BA._IndexView._last[1] is not second
    o_ref, _ = O.attention_forward(q.cpu(), k.cpu(), v.cpu(), bf.cpu(), idx_q=off2.cpu(), idx_k=off2.cpu())
    assert (o2.float().cpu() - o_ref).abs().max().item() <= O_MAX_ABS
    BA.BitfieldUtils.clear_cache()
    assert BA._IndexView._last is None


# ------------------------------------------------- the plan of a shard (classes of its 32 x 32 tiles, slice order)
def _rank_with_and_without_plan(q, k, v, do, bf, idx_q, idx_k, flags, use_plan):
    d = dev()
    ql, dol = q[:, idx_q].contiguous().to(d), do[:, idx_q].contiguous().to(d)
    kl, vl = k[:, idx_k].contiguous().to(d), v[:, idx_k].contiguous().to(d)
    bfg, fl = bf.to(d), flags.to(d)
    oq, ok = idx_q.to(d), idx_k.to(d)
    BA.BitfieldUtils.clear_cache()
    view = BA._IndexView.get(bfg, oq, ok)
    assert view.plan is not None
    if not use_plan:
        view.plan = None  # the kernels then work from the caller's 128 x 32 flags alone
    o, lse, scale = BA._bitfield_attn_forward(ql, kl, vl, bfg, fl, oq, ok)
    dq, dk, dv = (torch.zeros_like(t, dtype=torch.float32) for t in (ql, kl, vl))
    BA._bitfield_attn_backward(dol, ql, kl, vl, o, bfg, fl, lse, dq, dk, dv, offsets_q=oq, offsets_k=ok, softmax_scale=scale)
    torch.cuda.synchronize()
    assert BA._IndexView._last[1] is view
    return o.cpu(), lse[:, :, : idx_q.numel()].cpu(), dq.cpu(), dk.cpu(), dv.cpu(), view


@pytest.mark.parametrize("kind", ["zigzag", "blocks", "scattered"])
@pytest.mark.parametrize("S,D,Hq,Hkv", [(777, 64, 4, 2), (1024, 128, 4, 1)])
def test_shard_results_do_not_depend_on_the_plan(kind, S, D, Hq, Hkv):
    bf = random_bitfield(2, S, seed=S + 3, pad=5)
    q, k, v, do = inputs(2, S, Hq, Hkv, D, torch.bfloat16, seed=S)
    ranks = splits(S, kind)
    idx_k = torch.cat(ranks)
    for idx_q in ranks:
        flags = O.tile_flags_indexed(bf, idx_q, idx_k)
        without = _rank_with_and_without_plan(q, k, v, do, bf, idx_q, idx_k, flags, False)
        with_plan = _rank_with_and_without_plan(q, k, v, do, bf, idx_q, idx_k, flags, True)
        for name, a, b in zip(("o", "lse", "dq", "dk", "dv"), with_plan, without):
            # dk, dv: fp32 partial sums of the two row streams meet in another order.  dq at head dim 128: with a
            # plan the backward hands dS from dK/dV to the dQ kernel, without one dQ recomputes it.
            if name in ("dk", "dv") or (name == "dq" and D == 128):
                assert rel_l2(a, b) <= 2e-3, name
            else:
                assert torch.equal(a, b), name
        # the classes are those of the shard's own score matrix, at 32 x 32
        view = with_plan[5]
        n_q, n_k = -(-idx_q.numel() // 32), -(-idx_k.numel() // 32)
        for b in range(2):
            allow = O.allow_rows(bf[b], 0, idx_q.numel(), idx_q, idx_k)
            pad = torch.nn.functional.pad(allow, (0, n_k * 32 - idx_k.numel(), 0, n_q * 32 - idx_q.numel()))
            cells = torch.nn.functional.pad(torch.ones_like(allow), (0, n_k * 32 - idx_k.numel(), 0, n_q * 32 - idx_q.numel()))
            cnt = pad.view(n_q, 32, n_k, 32).sum(dim=(1, 3))
            tot = cells.view(n_q, 32, n_k, 32).sum(dim=(1, 3))
            want = torch.where(cnt == 0, 0, torch.where(cnt == tot, 2, 1)).to(torch.uint8)
            fine = view.plan.fine_classes()[b].cpu()
            assert torch.equal(fine[:n_q], want) and (fine[n_q:] == 0).all()
            order = view.plan.slice_order()[b].cpu().tolist()
            assert sorted(order[:n_q]) == list(range(n_q)) and all(x == -1 for x in order[n_q:])
    BA.BitfieldUtils.clear_cache()
