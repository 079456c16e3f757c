"""The C ABI under HIP graph capture: the library allocates nothing, synchronizes nothing and uses only the stream it
is handed, so a whole step -- flags + plan, forward, delta, dK/dV + dQ with the dS hand-over -- can be recorded once
and replayed.  Every replay is compared, bit for bit, with the same entry points called eagerly on the same inputs;
the replays are separated by eager work and synchronizations of the program itself."""

import ctypes
import math

import pytest
import torch

from cornstarch_amd.kernel import _bam_hip
from cornstarch_amd.kernel import bitfield_attention as BA
from tests.helpers import random_bitfield

pytestmark = pytest.mark.gpu


def dev():
    return torch.device("cuda:0")


def make_inputs(B, S, Hq, Hkv, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, S, Hq, D, generator=g) * 0.5).to(dtype)
    k = (torch.randn(B, S, Hkv, D, generator=g) * 0.5).to(dtype)
    v = (torch.randn(B, S, Hkv, D, generator=g) * 0.5).to(dtype)
    do = torch.randn(B, S, Hq, D, generator=g).to(dtype)
    return q, k, v, do


class _Step:
    """Static buffers of one fwd+bwd step and the five C ABI calls that make it, on a given stream."""

    def __init__(self, B, S, Hq, Hkv, D, dtype, pairs_capacity):
        d = dev()
        self.shape = (B, S, Hq, Hkv, D)
        self.q, self.k, self.v, self.do = (torch.zeros(s, dtype=dtype, device=d)
                                           for s in ((B, S, Hq, D), (B, S, Hkv, D), (B, S, Hkv, D), (B, S, Hq, D)))
        self.bf = torch.zeros((B, S), dtype=torch.int64, device=d)
        self.flags = torch.zeros((B, -(-S // 128), -(-S // 32)), dtype=torch.int8, device=d)
        lib = _bam_hip.load()
        self.plan_ws = torch.zeros((lib.bam_plan_workspace_bytes(B, S),), dtype=torch.uint8, device=d)
        self.plan = _bam_hip.Plan()
        self.o = torch.zeros_like(self.q)
        self.lse = torch.zeros((B, Hq, -(-S // 128) * 128), dtype=torch.float32, device=d)
        self.delta = torch.zeros_like(self.lse)
        self.dq, self.dk, self.dv = torch.zeros_like(self.q), torch.zeros_like(self.k), torch.zeros_like(self.v)
        self.pairs_capacity = pairs_capacity
        nbytes = lib.bam_ds_workspace_bytes(Hq, pairs_capacity) if D == 128 else 0
        self.ds_ws = torch.zeros((max(nbytes, 16),), dtype=torch.uint8, device=d)
        self.use_ds = nbytes > 0

    def load(self, q, k, v, do, bf):
        for dst, src in ((self.q, q), (self.k, k), (self.v, v), (self.do, do), (self.bf, bf)):
            dst.copy_(src)

    def enqueue(self, stream):
        B, S, Hq, Hkv, D = self.shape
        st = stream.cuda_stream
        scale = 1.0 / math.sqrt(D)
        code = BA._dtype_code(self.q.dtype)
        _bam_hip.call("bam_tile_plan", self.bf.data_ptr(), self.bf.stride(0), self.flags.data_ptr(), self.flags.stride(0),
                      self.flags.stride(1), self.plan_ws.data_ptr(), self.plan_ws.numel(), B, S, ctypes.byref(self.plan), st)
        if self.use_ds:  # the caller's part of the plan: where dK/dV leaves dS for dQ
            self.plan.ds_workspace = self.ds_ws.data_ptr()
            self.plan.ds_capacity = self.pairs_capacity
        _bam_hip.call("bam_fwd", self.q.data_ptr(), self.k.data_ptr(), self.v.data_ptr(), self.o.data_ptr(),
                      self.lse.data_ptr(), self.bf.data_ptr(), self.flags.data_ptr(),
                      *BA._strides3(self.q, self.k, self.v, self.o), self.bf.stride(0), self.flags.stride(0),
                      self.flags.stride(1), B, S, Hq, Hkv, D, scale, code, None, ctypes.byref(self.plan), st)
        _bam_hip.call("bam_bwd_preprocess", self.o.data_ptr(), self.do.data_ptr(), self.delta.data_ptr(),
                      *BA._strides3(self.o, self.do), B, S, Hq, D, code, st)
        _bam_hip.call("bam_bwd", self.q.data_ptr(), self.k.data_ptr(), self.v.data_ptr(), self.do.data_ptr(),
                      self.lse.data_ptr(), self.delta.data_ptr(), self.dq.data_ptr(), self.dk.data_ptr(), self.dv.data_ptr(),
                      self.bf.data_ptr(), self.flags.data_ptr(),
                      *BA._strides3(self.q, self.k, self.v, self.do, self.dq, self.dk, self.dv), self.bf.stride(0),
                      self.flags.stride(0), self.flags.stride(1), B, S, Hq, Hkv, D, scale, code, 0, None,
                      ctypes.byref(self.plan), st)

    def results(self):
        return [t.clone() for t in (self.flags, self.o, self.lse, self.dq, self.dk, self.dv)]


@pytest.mark.parametrize("B,S,Hq,Hkv,D", [(2, 640, 8, 2, 128), (3, 333, 4, 4, 64)])
def test_a_recorded_step_replays_bit_for_bit(B, S, Hq, Hkv, D):
    dtype = torch.bfloat16
    # room for every (32-row slice, 128-key tile) pair: the count is device data and cannot be read during capture
    capacity = B * 4 * (-(-S // 128)) * (-(-S // 128))
    step = _Step(B, S, Hq, Hkv, D, dtype, capacity)
    cases = []
    for seed in (1, 2, 3):
        q, k, v, do = (t.to(dev()) for t in make_inputs(B, S, Hq, Hkv, D, dtype, seed=10 * seed + S))
        bf = random_bitfield(B, S, seed=seed + S, pad=7 * seed).to(dev())
        cases.append((q, k, v, do, bf))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # once eagerly on the capture stream (loads the code objects)
        step.load(*cases[0])
        step.enqueue(side)
    side.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step.enqueue(side)

    for case in cases + cases[:1]:
        step.load(*case)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = step.results()
        # eager work of the program between the replays: the same step through the same entry points
        for t in (step.flags, step.o, step.lse, step.dq, step.dk, step.dv):
            t.zero_()
        step.enqueue(torch.cuda.current_stream())
        torch.cuda.synchronize()
        for name, a, b in zip(("flags", "o", "lse", "dq", "dk", "dv"), replayed, step.results()):
            assert torch.equal(a, b), name
        # and the replay is what the public entry point computes
        BA.BitfieldUtils.clear_cache()
        qg, kg, vg = (t.clone().requires_grad_(True) for t in case[:3])
        o = BA.bitfield_attn_func(qg, kg, vg, case[4])
        dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), case[3])
        torch.cuda.synchronize()
        assert torch.equal(replayed[1], o.detach())
        for a, b in zip(replayed[3:], (dq, dk, dv)):
            assert torch.equal(a, b)
