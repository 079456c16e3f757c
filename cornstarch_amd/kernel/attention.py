"""Materialized-mask attention on MI355X: host side of the reference's
``cornstarch/kernel/attention.py`` (``flash_attn_func``, ``FlashAttnFunc``, ``_flash_attn_forward``,
``_flash_attn_backward``) with the same names, argument order and defaults.

The reference has a second set of Triton kernels for this entry point.  Here it is served by the same
forward / dK,dV / dQ kernels as bitfield attention: a small kernel classifies the 128 x 32 tiles of the
bool mask (empty / partial / full), empty tiles are skipped, and only partial tiles read the mask.

``BLOCK_M`` / ``BLOCK_N`` are also what the reference's context-parallel split code imports from this
module (cornstarch/kernel/attention.py:51-52, cornstarch/shardformer/layers/utils.py:11).
"""

from __future__ import annotations

import atexit
import math
from typing import Optional

import torch
import torch.nn.functional as F

from . import _bam_hip
from .bitfield_attention import (
    _CACHE_LOCK,
    _bias_arg,
    _BiasView,
    _plan_arg,
    _TilePlan,
    _backward_in_head_runs,
    _dtype_code,
    _is_kernel_ready,
    _kernel_ready,
    _launch_bwd_preprocess,
    _padded_head_dim,
    _stream_ptr,
    _strides3,
)

BLOCK_M = 128
BLOCK_N = 32


def mask_tile_flags(mask: Optional[torch.Tensor], batch: int, seqlen_q: int, seqlen_k: int, device) -> torch.Tensor:
    """int8 (B, ceil(Sq/128), ceil(Sk/32)): 0 = no pair of the tile is allowed, 2 = every in-range pair is,
    1 = mixed.  ``mask`` None means "attend everywhere"."""
    num_m, num_n = -(-seqlen_q // BLOCK_M), -(-seqlen_k // BLOCK_N)
    if mask is None:
        return torch.full((batch, num_m, num_n), 2, dtype=torch.int8, device=device)
    flags = torch.empty((batch, num_m, num_n), dtype=torch.int8, device=device)
    with torch.cuda.device(device):
        _bam_hip.call(
            "bam_mask_tile_flags", mask.data_ptr(), flags.data_ptr(), flags.stride(0), flags.stride(1),
            batch, seqlen_q, seqlen_k, _stream_ptr(device),
        )
    return flags


class _MaskPlan:
    """Flags and plan (classes of the 32 x 32 tiles, slice order, the mask packed to bits for the kernels: a quarter
    of the mask's size in all) of a bool mask, from one pass over it.  The forward
    and, later, the backward of one call bring the same mask tensor: the last result is kept, together with the mask
    it was computed from (so its address cannot be handed to another tensor meanwhile), and reused while that is
    unchanged."""

    _last = None

    @classmethod
    def get(cls, mask: Optional[torch.Tensor], batch: int, seqlen_q: int, seqlen_k: int, device):
        """-> (flags int8 (B, ceil(Sq/128), ceil(Sk/32)), plan or None)"""
        if mask is None:
            return mask_tile_flags(None, batch, seqlen_q, seqlen_k, device), None
        with _CACHE_LOCK:
            return cls._get_locked(mask, batch, seqlen_q, seqlen_k, device)

    @classmethod
    def _get_locked(cls, mask: torch.Tensor, batch: int, seqlen_q: int, seqlen_k: int, device):
        key = (mask.data_ptr(), tuple(mask.shape), tuple(mask.stride()), mask._version, mask.device)
        if cls._last is not None and cls._last[0] == key:
            return cls._last[1], cls._last[2]
        import ctypes

        num_m, num_n = -(-seqlen_q // BLOCK_M), -(-seqlen_k // BLOCK_N)
        with torch.cuda.device(device):
            ws_bytes = _bam_hip.load().bam_mask_plan_workspace_bytes(batch, seqlen_q, seqlen_k)
            workspace = None
            if ws_bytes > 0:
                try:
                    workspace = torch.empty((ws_bytes,), dtype=torch.uint8, device=device)
                except torch.cuda.OutOfMemoryError:
                    workspace = None  # no room for a quarter of the mask: flags only, the kernels read the mask bytes
            if workspace is not None:
                flags = torch.empty((batch, num_m, num_n), dtype=torch.int8, device=device)
                struct = _bam_hip.Plan()
                _bam_hip.call(
                    "bam_mask_tile_plan", mask.data_ptr(), flags.data_ptr(), flags.stride(0), flags.stride(1),
                    workspace.data_ptr(), ws_bytes, batch, seqlen_q, seqlen_k, ctypes.byref(struct), _stream_ptr(device),
                )
                plan = _TilePlan(workspace, struct, flags)
            else:
                flags, plan = mask_tile_flags(mask, batch, seqlen_q, seqlen_k, device), None
        cls._last = (key, flags, plan, mask)
        return flags, plan

    @classmethod
    def forget(cls):
        cls._last = None


atexit.register(_MaskPlan.forget)  # (runs before the release of the bitfield module's state, registered earlier)


def _checked_mask(mask, batch, seqlen_q, seqlen_k):
    if mask is None:
        return None
    assert mask.dtype is torch.bool
    assert mask.is_cuda
    assert mask.shape == (batch, seqlen_q, seqlen_k), (
        f"Expected mask shape ({batch, seqlen_q, seqlen_k}), got {mask.shape}"
    )
    if not mask.is_contiguous() or mask.data_ptr() % 4:
        mask = mask.clone(memory_format=torch.contiguous_format)
    return mask


def _flash_attn_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    mask: Optional[torch.Tensor] = None,
    softmax_scale: Optional[float] = None,
):
    """q (B, Sq, H, D), k/v (B, Sk, H, D), mask bool (B, Sq, Sk) -> (o like q, lse fp32
    (B, H, ceil(Sq/128)*128), softmax_scale).  Contract of the reference's ``_flash_attn_forward``
    (attention.py:855-949); grouped kv heads (H_kv dividing H) are accepted as well."""
    batch, seqlen_q, nheads, d = q.shape
    _, seqlen_k, nheads_k, _ = k.shape
    assert k.shape == (batch, seqlen_k, nheads_k, d) and v.shape == k.shape and nheads % nheads_k == 0
    assert d <= 128, "FlashAttention only support head dimensions up to 128"
    assert q.dtype == k.dtype == v.dtype, "All tensors must have the same type"
    assert q.dtype in [torch.float16, torch.bfloat16], "Only support fp16 and bf16"
    assert q.is_cuda and k.is_cuda and v.is_cuda
    softmax_scale = softmax_scale or 1.0 / math.sqrt(d)
    # reference attention.py:874-895
    bias_view = _BiasView(bias, q, batch, nheads, seqlen_q, seqlen_k) if bias is not None else None
    mask = _checked_mask(mask, batch, seqlen_q, seqlen_k)

    dp = _padded_head_dim(d)
    if dp != d:  # zero columns change neither q.k nor the first d columns of p.v
        q, k, v = (F.pad(x, (0, dp - d)) for x in (q, k, v))
    qk, kk, vk = (_kernel_ready(x, 8) for x in (q, k, v))
    flags, plan = _MaskPlan.get(mask, batch, seqlen_q, seqlen_k, q.device)
    lse = torch.empty((batch, nheads, flags.shape[1] * BLOCK_M), device=q.device, dtype=torch.float32)
    o = torch.empty_like(qk)
    with torch.cuda.device(q.device):
        _bam_hip.call(
            "bam_fwd_masked",
            qk.data_ptr(), kk.data_ptr(), vk.data_ptr(), o.data_ptr(), lse.data_ptr(),
            mask.data_ptr() if mask is not None else None, flags.data_ptr(),
            *_strides3(qk, kk, vk, o), flags.stride(0), flags.stride(1),
            batch, seqlen_q, seqlen_k, nheads, nheads_k, dp, float(softmax_scale), _dtype_code(q.dtype),
            _bias_arg(bias_view), _plan_arg(plan), _stream_ptr(q.device),
        )
    if dp != d:
        o = o[..., :d].contiguous()
    return o, lse, softmax_scale


def _flash_attn_backward(
    do: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    o: torch.Tensor,
    lse: torch.Tensor,
    dq: torch.Tensor,
    dk: torch.Tensor,
    dv: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    mask: Optional[torch.Tensor] = None,
    softmax_scale: Optional[float] = None,
):
    """Writes the gradients into the caller's ``dq``, ``dk``, ``dv`` (same dtype as q; the reference
    passes ``torch.empty_like`` buffers, attention.py:1098-1101).  Contract of the reference's
    ``_flash_attn_backward`` (attention.py:952-1069)."""
    if do.stride(-1) != 1:
        do = do.contiguous()
    batch, seqlen_q, nheads, d = q.shape
    _, seqlen_k, nheads_k, _ = k.shape
    assert d <= 128
    seqlen_q_rounded = math.ceil(seqlen_q / BLOCK_M) * BLOCK_M
    assert lse.shape == (batch, nheads, seqlen_q_rounded)
    assert q.stride(-1) == k.stride(-1) == v.stride(-1) == o.stride(-1) == 1
    assert dq.stride(-1) == dk.stride(-1) == dv.stride(-1) == 1
    softmax_scale = softmax_scale or 1.0 / math.sqrt(d)
    # the reference asserts the unit stride here instead of copying (attention.py:1002-1019)
    bias_view = _BiasView(bias, q, batch, nheads, seqlen_q, seqlen_k, may_copy=False) if bias is not None else None
    mask = _checked_mask(mask, batch, seqlen_q, seqlen_k)
    flags, plan = _MaskPlan.get(mask, batch, seqlen_q, seqlen_k, q.device)

    dp = _padded_head_dim(d)
    outs = (dq, dk, dv)
    direct = dp == d and all(x.dtype == q.dtype and _is_kernel_ready(x) for x in outs)
    if dp != d:
        q, k, v, o, do = (F.pad(x, (0, dp - d)) for x in (q, k, v, o, do))
    qk, kk, vk, ok, gk = (_kernel_ready(x, 8) for x in (q, k, v, o, do))
    work = outs if direct else tuple(torch.empty_like(x) for x in (qk, kk, vk))
    lse = lse.contiguous()
    delta = torch.empty_like(lse)
    _launch_bwd_preprocess(ok, gk, delta)
    mask_ptr = mask.data_ptr() if mask is not None else None
    wq, wk, wv = work

    def launch(q, k, v, do, lse, delta, dq, dk, dv):
        heads, heads_k = q.shape[2], k.shape[2]
        with torch.cuda.device(q.device):
            _bam_hip.call(
                "bam_bwd_dkdv_masked",
                q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), lse.data_ptr(), delta.data_ptr(),
                dk.data_ptr(), dv.data_ptr(), mask_ptr, flags.data_ptr(),
                *_strides3(q, k, v, do, dk, dv), flags.stride(0), flags.stride(1),
                batch, seqlen_q, seqlen_k, heads, heads_k, dp, float(softmax_scale), _dtype_code(q.dtype), 0,
                _bias_arg(bias_view), _plan_arg(plan), _stream_ptr(q.device),
            )
            _bam_hip.call(
                "bam_bwd_dq_masked",
                q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), lse.data_ptr(), delta.data_ptr(),
                dq.data_ptr(), mask_ptr, flags.data_ptr(),
                *_strides3(q, k, v, do, dq), flags.stride(0), flags.stride(1),
                batch, seqlen_q, seqlen_k, heads, heads_k, dp, float(softmax_scale), _dtype_code(q.dtype), 0,
                _bias_arg(bias_view), _plan_arg(plan), _stream_ptr(q.device),
            )

    # (a bias is indexed by absolute head: with one, the heads stay in one run)
    _backward_in_head_runs(plan, launch, qk, kk, vk, gk, lse, delta, wq, wk, wv, dp, splittable=bias_view is None)
    if not direct:
        for dst, w in zip(outs, work):
            dst.copy_(w[..., :d])


class FlashAttnFunc(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        q: torch.Tensor,
        k: torch.Tensor,
        v: torch.Tensor,
        bias: Optional[torch.Tensor] = None,
        mask: Optional[torch.Tensor] = None,
        softmax_scale: Optional[float] = None,
    ):
        """
        q: (batch_size, seqlen_q, nheads, headdim)
        k, v: (batch_size, seqlen_k, nheads, headdim)
        mask: optional bool (batch_size, seqlen_q, seqlen_k), True = attend
        """
        q, k, v = [x if x.stride(-1) == 1 else x.contiguous() for x in [q, k, v]]
        if bias is not None and bias.stride(-1) != 1:
            bias = bias.contiguous()
        o, lse, ctx.softmax_scale = _flash_attn_forward(q, k, v, bias=bias, mask=mask, softmax_scale=softmax_scale)
        ctx.save_for_backward(q, k, v, o, lse, bias, mask)
        return o

    @staticmethod
    def backward(ctx, do: torch.Tensor):
        q, k, v, o, lse, bias, mask = ctx.saved_tensors
        assert not ctx.needs_input_grad[3], "FlashAttention does not support bias gradient yet"
        with torch.no_grad():
            dq = torch.empty_like(q)
            dk = torch.empty_like(k)
            dv = torch.empty_like(v)
            _flash_attn_backward(do, q, k, v, o, lse, dq, dk, dv, bias=bias, mask=mask, softmax_scale=ctx.softmax_scale)
        return dq, dk, dv, None, None, None


def flash_attn_func(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    mask: Optional[torch.Tensor] = None,
    softmax_scale: Optional[float] = None,
):
    """Attention with an optional materialized bool mask (reference attention.py:1126-1146)."""
    return FlashAttnFunc.apply(q, k, v, bias, mask, softmax_scale)

