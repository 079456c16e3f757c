"""Single-token decode step of the HF adapter on an MI355X (reference cornstarch/kernel/interface.py:71-83: eval
mode, one query token, flash-attn called with ``scaling``, ``sliding_window`` and ``softcap``), through the C ABI.

flash-attn itself is not part of the reference tree and not installed: parity with it is unpinned.  What is checked
is the decode kernel against the fp32 restatement of those semantics in ``oracle.decode_step`` (itself pinned by
library SDPA, closed forms and brute force in tests/test_oracle.py), at the forward bar of this repository
(max-abs 2e-2 for 16-bit outputs), plus closed forms on the device."""

import math

import pytest
import torch

from cornstarch_amd.kernel import _bam_hip
from cornstarch_amd.kernel import bitfield_attention as BA
from cornstarch_amd.kernel import interface
from oracle import bam_oracle as O

pytestmark = pytest.mark.gpu

O_MAX_ABS = 2e-2


class _Module(torch.nn.Module):
    pass


def dev():
    return torch.device("cuda:0")


def inputs(B, Hq, Hkv, Sk, D, dtype, seed=0, std=0.5):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Hq, 1, D, generator=g) * std).to(dtype)
    k = (torch.randn(B, Hkv, Sk, D, generator=g) * std).to(dtype)
    v = (torch.randn(B, Hkv, Sk, D, generator=g) * std).to(dtype)
    return q, k, v


def decode(q, k, v, **kw):
    out, w = interface.bitfield_attention_forward(_Module().eval(), q.to(dev()), k.to(dev()), v.to(dev()), None, **kw)
    torch.cuda.synchronize()
    assert w is None and out.shape == (q.shape[0], 1, q.shape[1], q.shape[3]) and out.dtype == q.dtype
    return out.cpu()


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("Sk", [1, 9, 333, 1024, 2500])
@pytest.mark.parametrize("kw", [{}, {"sliding_window": 1}, {"sliding_window": 200}, {"softcap": 30.0}, {"softcap": 0.5},
                                {"sliding_window": 77, "softcap": 2.0, "scaling": 0.31}],
                         ids=["plain", "window1", "window200", "cap30", "cap0.5", "window+cap+scale"])
def test_decode_step_against_the_oracle(D, Sk, kw):
    q, k, v = inputs(2, 8, 2, Sk, D, torch.bfloat16, seed=Sk + D)
    got = decode(q, k, v, **kw)
    want = O.decode_step(q, k, v, **kw)
    assert (got.float() - want).abs().max().item() <= O_MAX_ABS


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D,Hq,Hkv", [(40, 4, 4), (96, 6, 3), (128, 5, 1)])
def test_decode_step_head_dims_between_the_native_ones_and_head_groupings(dtype, D, Hq, Hkv):
    q, k, v = inputs(3, Hq, Hkv, 130, D, dtype, seed=D)
    for kw in ({}, {"sliding_window": 64, "softcap": 5.0}):
        got = decode(q, k, v, **kw)
        assert (got.float() - O.decode_step(q, k, v, **kw)).abs().max().item() <= (1e-2 if dtype == torch.float16 else O_MAX_ABS)


@pytest.mark.parametrize("B,Hq,Hkv,Sk,D", [(1, 32, 8, 8192, 128), (2, 16, 16, 5000, 64), (1, 8, 1, 20001, 128),
                                           (3, 40, 1, 700, 32), (1, 66, 2, 1300, 64)])
def test_decode_step_long_caches_split_over_many_workgroups(B, Hq, Hkv, Sk, D):
    # long caches: many splits and the combine pass; 40 and 33 q heads per kv head: more than one group of 32 heads
    lib = _bam_hip.load()
    assert lib.bam_decode_workspace_bytes(B, Sk, Hq, Hkv, D, 0) > 0
    q, k, v = inputs(B, Hq, Hkv, Sk, D, torch.bfloat16, seed=Sk)
    for kw in ({}, {"sliding_window": Sk // 3, "softcap": 20.0}, {"sliding_window": 33}):
        got = decode(q, k, v, **kw)
        want = O.decode_step(q, k, v, **kw)
        assert (got.float() - want).abs().max().item() <= O_MAX_ABS


def test_decode_step_closed_forms_on_the_device():
    q, k, v = inputs(2, 4, 2, 500, 64, torch.bfloat16, seed=1)
    plain = decode(q, k, v)
    # a window at least as long as the cache changes nothing, bit for bit
    assert torch.equal(decode(q, k, v, sliding_window=500), plain)
    assert torch.equal(decode(q, k, v, sliding_window=10_000), plain)
    # a cap far above every score is the identity up to the rounding of tanh
    assert (decode(q, k, v, softcap=1e4).float() - plain.float()).abs().max().item() <= 1e-2
    # window 1: the output is the last value row
    last = v[:, :, -1].repeat_interleave(2, dim=1)[:, None]
    assert torch.equal(decode(q, k, v, sliding_window=1), last)
    # a tiny cap flattens the scores: the mean of V
    mean_v = v.float().mean(dim=2).repeat_interleave(2, dim=1)[:, None]
    assert (decode(q, k, v, softcap=1e-4).float() - mean_v).abs().max().item() <= 1e-2
    # scaling is honoured on this path (the reference forwards it to flash-attn)
    assert not torch.equal(decode(q, k, v, scaling=1.0), plain)
    assert torch.equal(decode(q, k, v, scaling=1.0 / math.sqrt(64)), plain)


def test_decode_step_large_scores_and_a_cache_view_with_strides():
    # scores of a few hundred before the cap; key / value handed over as strided views of a larger cache buffer
    B, Hq, Hkv, Sk, D = 1, 4, 2, 700, 128
    q, k, v = inputs(B, Hq, Hkv, Sk, D, torch.bfloat16, seed=5, std=4.0)
    cache_k = torch.zeros(B, Hkv, 1024, D, dtype=torch.bfloat16, device=dev())
    cache_v = torch.zeros_like(cache_k)
    cache_k[:, :, :Sk] = k.to(dev())
    cache_v[:, :, :Sk] = v.to(dev())
    for kw in ({}, {"softcap": 50.0}, {"sliding_window": 300}):
        out, _ = interface.bitfield_attention_forward(_Module().eval(), q.to(dev()), cache_k[:, :, :Sk], cache_v[:, :, :Sk],
                                                      None, **kw)
        want = O.decode_step(q, k, v, **kw)
        assert torch.isfinite(out).all()
        assert (out.float().cpu() - want).abs().max().item() <= 4e-2 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("D", [64, 128])
def test_decode_step_with_a_query_view_that_is_only_two_byte_aligned(D):
    # the kernel reads an aligned q with 16-byte loads and any other q element by element: both must agree
    q, k, v = inputs(2, 8, 2, 777, D, torch.bfloat16, seed=D)
    want = O.decode_step(q, k, v)
    wide = torch.zeros(2, 8, 1, D + 1, dtype=q.dtype)
    wide[..., 1:] = q
    view = wide.to(dev())[..., 1:]  # first element at byte offset 2, head stride D + 1
    assert view.data_ptr() % 16 != 0 and view.stride(-1) == 1
    out, _ = interface.bitfield_attention_forward(_Module().eval(), view, k.to(dev()), v.to(dev()), None)
    aligned = decode(q, k, v)
    assert torch.equal(out.cpu(), aligned)
    assert (aligned.float() - want).abs().max().item() <= O_MAX_ABS


def test_training_mode_takes_the_bitfield_path_and_bad_arguments_are_refused():
    q, k, v = (t.to(dev()) for t in inputs(1, 4, 2, 8, 64, torch.bfloat16))
    with pytest.raises(AssertionError, match="int64"):
        interface.bitfield_attention_forward(_Module().train(), q, q, q, None)
    m = _Module().eval()
    with pytest.raises(ValueError):
        interface.bitfield_attention_forward(m, q, k, v, None, sliding_window=0)
    with pytest.raises(NotImplementedError):
        interface.bitfield_attention_forward(m, q, k, v, None, dropout=0.1)
    # the C entry point itself, with its own argument checks
    o = torch.empty(1, 4, 64, dtype=torch.bfloat16, device=dev())
    kt, vt = k.transpose(1, 2), v.transpose(1, 2)
    with pytest.raises(_bam_hip.BamError, match="window"):
        _bam_hip.call("bam_decode", q.data_ptr(), kt.data_ptr(), vt.data_ptr(), o.data_ptr(), q.stride(0), q.stride(1),
                      kt.stride(0), kt.stride(1), kt.stride(2), vt.stride(0), vt.stride(1), vt.stride(2), o.stride(0),
                      o.stride(1), 1, 8, 4, 2, 64, 0.125, BA._dtype_code(q.dtype), -1, 0.0, None, 0, BA._stream_ptr(dev()))
