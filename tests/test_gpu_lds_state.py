"""The kernels must not depend on what earlier kernels left in LDS.

Every launch below runs after the LDS of all compute units was filled with NaN bit patterns and must reproduce,
bit for bit, the result of an undisturbed run.  A read of LDS that the workgroup has not written yet -- or not
visibly: a missing wait between a store and the barrier that publishes it -- shows up as a difference.  (This is how a
missing wait in front of the barrier at the head of the pass loop of the long-sequence kernels was found: the other
waves of a workgroup sometimes read the tile count of the previous pass.)
"""

import ctypes
import math

import pytest
import torch

from cornstarch_amd.kernel import bitfield_attention as BA
from tests import lds_fill
from tests.helpers import random_bitfield

pytestmark = pytest.mark.gpu


def _long_layout(S):
    text = (1 << 62) | 1 | 2 | 4
    bf = torch.full((1, S), text, dtype=torch.int64)
    bf[0, 1000:5000] = 2
    bf[0, S - 3000:] = 4  # these rows see no key of the first pass of a several-pass kernel
    return bf


@pytest.mark.parametrize(
    "S,D,Hq,Hkv,layout,reps",
    [
        (131072 + 4096 + 57, 32, 2, 1, "long", 40),  # two passes in all three attention kernels, ragged
        (131072 + 4096 + 57, 128, 2, 1, "long", 8),
        (2 * 131072 + 4096 + 57, 32, 2, 1, "long", 6),  # three passes
        (131072, 64, 2, 1, "long", 4),               # the longest single-pass sequence, with a plan
        (2000 + 57, 128, 4, 2, "random", 6),
        (517, 64, 4, 4, "random", 6),
        (97, 32, 2, 1, "random", 6),
    ],
)
def test_results_do_not_depend_on_lds_leftovers(S, D, Hq, Hkv, layout, reps):
    d = torch.device("cuda:0")
    fill = lds_fill.load()
    sink = torch.zeros(4, dtype=torch.int32, device=d)

    def poison():
        rc = fill.lds_fill(ctypes.c_void_p(sink.data_ptr()), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0

    g = torch.Generator().manual_seed(S + D)
    q = (torch.randn(1, S, Hq, D, generator=g) * 0.5).to(torch.bfloat16).to(d)
    k = (torch.randn(1, S, Hkv, D, generator=g) * 0.5).to(torch.bfloat16).to(d)
    v = (torch.randn(1, S, Hkv, D, generator=g) * 0.5).to(torch.bfloat16).to(d)
    do = torch.randn(1, S, Hq, D, generator=g).to(torch.bfloat16).to(d)
    bf = (_long_layout(S) if layout == "long" else random_bitfield(1, S, seed=S + D)).to(d)
    scale = 1.0 / math.sqrt(D)
    BA.BitfieldUtils.clear_cache()
    flags = BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf)
    plan = BA.BitfieldUtils.plan_for(flags, bf)

    def run(disturb):
        if disturb:
            poison()
        o, lse, _ = BA._bitfield_attn_forward(q, k, v, bf, flags, softmax_scale=scale)
        # outputs and the delta rows start as NaN: whatever a kernel fails to write stays visible
        dq, dk, dv = (torch.full_like(t, float("nan")) for t in (q, k, v))
        delta = torch.full_like(lse, float("nan"))
        BA._launch_bwd_preprocess(o, do, delta)
        if disturb:
            poison()
        BA._launch_bwd_dkdv(q, k, v, do, lse, delta, dk, dv, bf, flags, scale, accumulate=False, plan=plan)
        if disturb:
            poison()
        BA._launch_bwd_dq(q, k, v, do, lse, delta, dq, bf, flags, scale, accumulate=False, plan=plan)
        torch.cuda.synchronize()
        return {"o": o, "lse": lse[:, :, :S].clone(), "dq": dq, "dk": dk, "dv": dv}

    want = run(False)
    for name, t in want.items():
        if name != "lse":  # (rows that see no key have lse = -inf)
            assert torch.isfinite(t.float()).all(), name
    for rep in range(reps):
        got = run(True)
        for name in want:
            a, b = want[name], got[name]
            same = torch.equal(torch.nan_to_num(a.float(), nan=3e38), torch.nan_to_num(b.float(), nan=3e38))
            assert same, f"{name} of repetition {rep} differs from the undisturbed run"
    BA.BitfieldUtils.clear_cache()
