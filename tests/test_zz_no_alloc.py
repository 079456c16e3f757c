"""bam_tile_plan_static -- the plan built in the library's own device array, for callers that cannot allocate --
against bam_tile_plan with a caller workspace: same flags, same fine classes, same slice order, and the same
attention output when the forward kernel is driven by either plan.  Two calls in a row, the second with a smaller
input (the array keeps the first call's contents)."""

import ctypes
import math

import pytest
import torch

from cornstarch_amd.kernel import _bam_hip
from cornstarch_amd.kernel import bitfield_attention as BA
from oracle import bam_oracle as O
from tests.helpers import random_bitfield

pytestmark = pytest.mark.gpu


def _views(struct, B, S):
    """(fine, order) tensors of a bam_plan, copied out of wherever the plan lives"""
    slots, num_n = 4 * -(-S // 128), -(-S // 32)
    fine = torch.empty((B, slots, num_n), dtype=torch.uint8, device="cuda:0")
    order = torch.empty((B, slots), dtype=torch.int32, device="cuda:0")
    # gather row by row through a raw-pointer view (the static array is not a torch allocation)
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpy2D.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t,
                                ctypes.c_size_t, ctypes.c_int]
    hip.hipMemcpy2D.restype = ctypes.c_int
    torch.cuda.synchronize()
    for b in range(B):
        rc = hip.hipMemcpy2D(fine[b].data_ptr(), num_n, struct.fine + b * struct.fine_stride_b, struct.fine_stride_s,
                             num_n, slots, 3)  # hipMemcpyDeviceToDevice
        assert rc == 0
        rc = hip.hipMemcpy2D(order[b].data_ptr(), slots * 4, struct.order + 4 * b * struct.order_stride_b, slots * 4,
                             slots * 4, 1, 3)
        assert rc == 0
    torch.cuda.synchronize()
    return fine, order


def _fwd(q, k, v, bf, flags, plan_ref, scale):
    B, S, Hq, D = q.shape
    o = torch.empty_like(q)
    lse = torch.empty((B, Hq, flags.shape[1] * 128), dtype=torch.float32, device=q.device)
    _bam_hip.call(
        "bam_fwd", q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), bf.data_ptr(),
        flags.data_ptr(), *BA._strides3(q, k, v, o), bf.stride(0), flags.stride(0), flags.stride(1),
        B, S, Hq, k.shape[2], D, float(scale), BA._dtype_code(q.dtype), None, plan_ref, BA._stream_ptr(q.device),
    )
    torch.cuda.synchronize()
    return o, lse[:, :, :S]


def test_plan_in_the_built_in_array_equals_the_plan_in_a_caller_workspace():
    d = torch.device("cuda:0")
    lib = _bam_hip.load()
    stream = BA._stream_ptr(d)
    earlier = []
    for B, S, seed in ((2, 1000, 5), (1, 283, 6)):  # the second call is smaller: stale bytes of the first stay behind it
        bf = random_bitfield(B, S, seed=seed, pad=3).to(d)
        num_m, num_n = -(-S // 128), -(-S // 32)
        # existing entry point, workspace from torch
        need = lib.bam_plan_workspace_bytes(B, S)
        assert 0 < need <= _bam_hip.BAM_STATIC_PLAN_BYTES
        ws = torch.empty((need,), dtype=torch.uint8, device=d)
        flags_a = torch.empty((B, num_m, num_n), dtype=torch.int8, device=d)
        plan_a = _bam_hip.Plan()
        _bam_hip.call("bam_tile_plan", bf.data_ptr(), bf.stride(0), flags_a.data_ptr(), flags_a.stride(0),
                      flags_a.stride(1), ws.data_ptr(), need, B, S, ctypes.byref(plan_a), stream)
        # the entry point that allocates nothing
        flags_b = torch.empty_like(flags_a)
        plan_b = _bam_hip.Plan()
        _bam_hip.call("bam_tile_plan_static", bf.data_ptr(), bf.stride(0), flags_b.data_ptr(), flags_b.stride(0),
                      flags_b.stride(1), B, S, ctypes.byref(plan_b), stream)
        assert plan_b.fine != plan_a.fine and (plan_b.B, plan_b.Sq, plan_b.Sk) == (B, S, S)
        assert plan_a.generation == 0 and plan_b.generation > 0
        assert torch.equal(flags_a, flags_b) and torch.equal(flags_a.cpu(), O.tile_flags(bf.cpu()))
        fine_a, order_a = _views(plan_a, B, S)
        fine_b, order_b = _views(plan_b, B, S)
        assert torch.equal(fine_a, fine_b) and torch.equal(order_a, order_b)
        # and the forward kernel produces the same bits from either plan
        g = torch.Generator().manual_seed(seed)
        q = (torch.randn(B, S, 4, 64, generator=g) * 0.5).bfloat16().to(d)
        k = (torch.randn(B, S, 2, 64, generator=g) * 0.5).bfloat16().to(d)
        v = (torch.randn(B, S, 2, 64, generator=g) * 0.5).bfloat16().to(d)
        o_a, lse_a = _fwd(q, k, v, bf, flags_a, ctypes.byref(plan_a), 1 / math.sqrt(64))
        o_b, lse_b = _fwd(q, k, v, bf, flags_b, ctypes.byref(plan_b), 1 / math.sqrt(64))
        assert torch.equal(o_a, o_b) and torch.equal(lse_a, lse_b)
        o_ref, _ = O.attention_forward(q, k, v, bf)
        assert (o_b.float() - o_ref).abs().max().item() <= 2e-2
        earlier.append((q, k, v, bf, flags_b, plan_b))
    # the plan of the first call lives in the array the second call has rewritten: it is refused, not used
    q, k, v, bf, flags_b, plan_b = earlier[0]
    with pytest.raises(_bam_hip.BamError, match="stale"):
        _fwd(q, k, v, bf, flags_b, ctypes.byref(plan_b), 0.125)


def test_the_static_entry_point_allocates_no_device_memory():
    # after one warm-up call (which resolves the array's address on this GPU), a call changes neither the
    # free device memory the driver reports nor what torch's allocator holds
    d = torch.device("cuda:0")
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemGetInfo.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
    hip.hipMemGetInfo.restype = ctypes.c_int
    B, S = 2, 777
    bf = random_bitfield(B, S, seed=2).to(d)
    flags = torch.empty((B, -(-S // 128), -(-S // 32)), dtype=torch.int8, device=d)
    plan = _bam_hip.Plan()

    def call():
        _bam_hip.call("bam_tile_plan_static", bf.data_ptr(), bf.stride(0), flags.data_ptr(), flags.stride(0),
                      flags.stride(1), B, S, ctypes.byref(plan), BA._stream_ptr(d))

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    call()
    torch.cuda.synchronize()
    before = (free_bytes(), torch.cuda.memory_allocated(d), torch.cuda.memory_reserved(d))
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    assert (free_bytes(), torch.cuda.memory_allocated(d), torch.cuda.memory_reserved(d)) == before
    assert torch.equal(flags.cpu(), O.tile_flags(bf.cpu()))


def test_sizes_beyond_the_built_in_array_are_refused():
    d = torch.device("cuda:0")
    lib = _bam_hip.load()
    B, S = 1, 131072  # 4096 slices: a 16 MiB class matrix
    assert lib.bam_plan_workspace_bytes(B, S) > _bam_hip.BAM_STATIC_PLAN_BYTES
    bf = torch.zeros((B, S), dtype=torch.int64, device=d)
    flags = torch.empty((B, S // 128, S // 32), dtype=torch.int8, device=d)
    plan = _bam_hip.Plan()
    with pytest.raises(_bam_hip.BamError, match="built-in"):
        _bam_hip.call("bam_tile_plan_static", bf.data_ptr(), bf.stride(0), flags.data_ptr(), flags.stride(0),
                      flags.stride(1), B, S, ctypes.byref(plan), BA._stream_ptr(d))
