"""Committed golden vectors (tests/golden/bam_golden.npz, written by tests/golden/make_golden.py).

CPU: the oracle still reproduces the file (guards the checker against drift).  GPU: the HIP kernels, called
through the C ABI, match the stored fp32 results (flags bit exact, O max-abs 2e-2, LSE 1e-2, gradients
relative L2 5e-2) without the oracle being run at all.
"""

import importlib.util
import os

import numpy as np
import pytest
import torch

from tests.helpers import rel_l2

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden", "bam_golden.npz")


def load(case):
    with np.load(GOLDEN, allow_pickle=False) as z:
        return {k.split(".", 1)[1]: torch.from_numpy(z[k]) for k in z.files if k.startswith(case + ".")}


def test_oracle_reproduces_the_golden_file():
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    fresh = mod.build()
    with np.load(GOLDEN, allow_pickle=False) as z:
        assert sorted(z.files) == sorted(fresh)
        for key in z.files:
            a, b = z[key], fresh[key]
            assert a.dtype == b.dtype and a.shape == b.shape, key
            if a.dtype == np.float32:
                fin = np.isfinite(a)
                assert np.array_equal(fin, np.isfinite(b)), key
                assert np.allclose(a[fin], b[fin], atol=1e-5, rtol=1e-5), key
            else:
                assert np.array_equal(a, b), key


def _compare(g, o, lse, dq, dk, dv):
    Sq = g["q"].shape[1]
    assert (o.float().cpu() - g["o"]).abs().max() <= 2e-2
    lse = lse[:, :, :Sq].cpu()
    live = torch.isfinite(g["lse"])
    assert torch.equal(torch.isfinite(lse), live)
    assert (lse[live] - g["lse"][live]).abs().max() <= 1e-2
    for got, key in ((dq, "dq"), (dk, "dk"), (dv, "dv")):
        assert rel_l2(got.float().cpu(), g[key]) <= 5e-2, key


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["ref57", "gqa_pad"])
def test_bitfield_attention_matches_golden(case):
    from cornstarch_amd.kernel import bitfield_attention as BA

    d = torch.device("cuda:0")
    g = load(case)
    bf = g["bf"].to(d)
    BA.BitfieldUtils.clear_cache()
    flags = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf)
    assert torch.equal(flags.cpu(), g["flags"])
    q, k, v = (g[n].to(d).requires_grad_(True) for n in ("q", "k", "v"))
    o = BA.bitfield_attn_func(q, k, v, bf)
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), g["do"].to(d))
    _, lse, _ = BA._bitfield_attn_forward(q.detach(), k.detach(), v.detach(), bf, flags)
    _compare(g, o.detach(), lse, dq, dk, dv)


@pytest.mark.gpu
def test_index_tensor_attention_matches_golden():
    from cornstarch_amd.kernel import bitfield_attention as BA

    d = torch.device("cuda:0")
    g = load("zigzag")
    q, k, v, do, bf, flags, iq, ik = (g[n].to(d) for n in ("q", "k", "v", "do", "bf", "flags", "idx_q", "idx_k"))
    o, lse, scale = BA._bitfield_attn_forward(q, k, v, bf, flags, iq, ik)
    dq, dk, dv = (torch.zeros_like(t, dtype=torch.float32) for t in (q, k, v))
    BA._bitfield_attn_backward(do, q, k, v, o, bf, flags, lse, dq, dk, dv, offsets_q=iq, offsets_k=ik, softmax_scale=scale)
    _compare(g, o, lse, dq, dk, dv)


@pytest.mark.gpu
def test_dense_mask_attention_matches_golden():
    from cornstarch_amd.kernel import attention as A

    d = torch.device("cuda:0")
    g = load("dense")
    mask = g["mask"].to(d)
    assert torch.equal(A.mask_tile_flags(mask, 1, 70, 45, d).cpu(), g["flags"])
    q, k, v = (g[n].to(d).requires_grad_(True) for n in ("q", "k", "v"))
    o = A.flash_attn_func(q, k, v, mask=mask)
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), g["do"].to(d))
    _, lse, _ = A._flash_attn_forward(q.detach(), k.detach(), v.detach(), mask=mask)
    _compare(g, o.detach(), lse, dq, dk, dv)


@pytest.mark.gpu
def test_attention_with_bias_matches_golden():
    from cornstarch_amd.kernel import bitfield_attention as BA

    d = torch.device("cuda:0")
    g = load("bias")
    bf, bias = g["bf"].to(d), g["bias"].to(d)
    BA.BitfieldUtils.clear_cache()
    flags = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf)
    assert torch.equal(flags.cpu(), g["flags"])
    q, k, v = (g[n].to(d).requires_grad_(True) for n in ("q", "k", "v"))
    o = BA.bitfield_attn_func(q, k, v, bf, bias)
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), g["do"].to(d))
    _, lse, _ = BA._bitfield_attn_forward(q.detach(), k.detach(), v.detach(), bf, flags, bias=bias)
    _compare(g, o.detach(), lse, dq, dk, dv)
    BA.BitfieldUtils.clear_cache()
