"""Bitfield-masked attention on MI355X: host side of the reference's
``cornstarch/kernel/bitfield_attention.py`` with the same names, argument order and
defaults, backed by hand-written gfx950 HIP kernels reached through ``libbam_hip.so``.

Every token carries an int64 bitfield; the attention mask is derived from those bitfields
inside the kernels (text tokens: causal over tokens sharing a bit; modality tokens:
bidirectional inside their own modality).  There is no PyTorch/CPU fallback: tensors must
live on the GPU and the HIP library must be built.
"""

from __future__ import annotations

import atexit
import contextlib
import math
import os
import threading
from typing import Optional

import torch
import torch.nn.functional as F

from . import _bam_hip

BLOCK_M = 128  # rows of a flag tile (reference bitfield_attention.py:53)
BLOCK_N = 32  # columns of a flag tile (reference bitfield_attention.py:54)
NUM_TOKENS_TO_COMPUTE_PER_BLOCK = 4096  # kept for importers; the HIP forward is single pass
NUM_KV_BLOCKS_PER_BLOCK = NUM_TOKENS_TO_COMPUTE_PER_BLOCK // BLOCK_N

_SUPPORTED_HEAD_DIMS = (32, 64, 128)


def _stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _dtype_code(dtype: torch.dtype) -> int:
    return _bam_hip.BAM_DTYPE_BF16 if dtype == torch.bfloat16 else _bam_hip.BAM_DTYPE_F16


def _kernel_ready(x: torch.Tensor, elems_per_16b: int) -> torch.Tensor:
    """Kernels read 16 bytes at a time: unit last stride, 16-byte aligned rows."""
    ok = (
        x.stride(-1) == 1
        and x.data_ptr() % 16 == 0
        and all(s % elems_per_16b == 0 for s in x.stride()[:-1])
    )
    return x if ok else x.contiguous()


def _padded_head_dim(d: int) -> int:
    for cand in _SUPPORTED_HEAD_DIMS:
        if d <= cand:
            return cand
    raise AssertionError("FlashAttention only support head dimensions up to 128")


def materialize_bitfield_mask(bitfield_mask: torch.Tensor) -> torch.Tensor:
    """bool (B, S, S): the allow rule for every (query, key) pair, evaluated on the GPU.

    Host-callable counterpart of the reference's Triton device function
    ``_materialize_bitfield_mask_block`` (bitfield_attention.py:60-101), which its test
    wraps in a kernel (tests/test_kernel/test_bitfield_attention.py:16-52)."""
    assert bitfield_mask.is_cuda and bitfield_mask.dtype == torch.int64 and bitfield_mask.dim() == 2
    if bitfield_mask.stride(1) != 1:
        bitfield_mask = bitfield_mask.contiguous()
    B, S = bitfield_mask.shape
    out = torch.empty((B, S, S), dtype=torch.uint8, device=bitfield_mask.device)
    with torch.cuda.device(bitfield_mask.device):
        _bam_hip.call(
            "bam_materialize_mask", bitfield_mask.data_ptr(), bitfield_mask.stride(0), out.data_ptr(), B, S,
            _stream_ptr(bitfield_mask.device),
        )
    return out.bool()


# Largest dS workspace the backward allocates for the hand-over of dS from the dK/dV kernel to the dQ kernel.  Where
# the workspace for all heads would be larger, the backward takes the heads in runs of whole kv heads, one launch pair
# per run through the same, smaller workspace; where even one kv head's q heads need more, the dQ kernel recomputes S
# and dP instead.  BAM_DS_WORKSPACE_LIMIT_GB overrides the default (a quarter of the device's memory, at most
# 64 GiB); 0 switches the hand-over off.
_DS_LIMIT_ENV = os.environ.get("BAM_DS_WORKSPACE_LIMIT_GB")


# Below the limit, a backward whose dS workspace for all heads would exceed this size still prefers runs of kv heads
# as long as the dK/dV launch of a run keeps this many workgroups (128-key tiles x batch x kv heads of the run: four
# rounds of the chip's 256 compute units).  One sequence of 65536 tokens with 32 q heads and 8 kv heads: 47 GiB in
# one run, 12 GiB in four runs, the same 41.9 ms either way (and 46.6 ms in eight runs of one kv head each).
# BAM_DS_WORKSPACE_TARGET_GB overrides the size (a value at or above the limit means: one run whenever it fits).
_DS_RUN_TARGET = int(float(os.environ.get("BAM_DS_WORKSPACE_TARGET_GB", "16")) * (1 << 30))
_DS_RUN_MIN_WORKGROUPS = 1024


def _ds_workspace_limit(device) -> int:
    if _DS_LIMIT_ENV is not None:
        return int(float(_DS_LIMIT_ENV) * (1 << 30))
    return min(64 << 30, torch.cuda.get_device_properties(device).total_memory // 4)


class _PinnedInts:
    """A small pool of pinned host ints for asynchronous device-to-host copies of single counters."""

    _buf: Optional[torch.Tensor] = None
    _next = 0
    _SLOTS = 256

    @classmethod
    def slot(cls) -> torch.Tensor:
        if cls._buf is None:
            cls._buf = torch.empty((cls._SLOTS,), dtype=torch.int32, pin_memory=True)
        i = cls._next
        cls._next = (i + 1) % cls._SLOTS
        return cls._buf[i : i + 1]

    _streams: dict = {}

    @classmethod
    def copy_stream(cls, device) -> "torch.cuda.Stream":
        """One side stream per device for these copies, so that they never sit between two kernels of the caller's
        stream."""
        key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
        if key not in cls._streams:
            cls._streams[key] = torch.cuda.Stream(device=device)
        return cls._streams[key]


# The caches below (flags + plan of the last bitfield mask, index view, mask plan) are per process, as in the
# reference; host threads that share them take this lock while they look an entry up or replace it.
_CACHE_LOCK = threading.RLock()


def _release_device_state() -> None:
    """Drops what this module keeps alive between calls (cached flags and plans, the pinned counter slots, the side
    stream) while the GPU runtime is still up: left to interpreter shutdown, pinned memory and streams would be
    released in no particular order after it."""
    try:
        if torch.cuda.is_available() and torch.cuda.is_initialized():
            torch.cuda.synchronize()
    except Exception:  # the runtime is already gone: nothing left to wait for
        pass
    BitfieldUtils.clear_cache()
    _IndexView.forget()
    _PinnedInts._buf = None
    _PinnedInts._streams.clear()


atexit.register(_release_device_state)


class _TilePlan:
    """What the kernels use beyond the 128 x 32 flags to skip masked work (``bam_plan`` of include/bam_hip.h):
    the class of every 32-row x 32-key tile and an order of the 32-row slices in which neighbours need the same
    keys.  Built together with the flags, lives in one workspace tensor, and belongs to exactly one flags tensor."""

    def __init__(self, workspace: torch.Tensor, struct: "_bam_hip.Plan", flags: Optional[torch.Tensor]):
        self.workspace = workspace  # keeps the device memory alive
        self.struct = struct
        self.flags = flags  # None for plans that are not tied to a flags tensor (index-tensor attention)
        self.flags_version = flags._version if flags is not None else -1  # (the builder wrote through raw pointers)
        # The number of (slice, 128-key tile) pairs that have work is device data; it sizes the dS workspace of the
        # backward.  Its copy to the host is enqueued here, right behind the kernels that compute it, and awaited
        # only when a backward asks for it -- by then it has long arrived.
        self._lock = threading.Lock()  # held while a backward has its dS workspace named in the struct
        self._pairs: Optional[int] = None
        self._pairs_host = _PinnedInts.slot()
        count = torch.as_strided(workspace.view(torch.int32), (1,), (1,), (struct.ds_count - workspace.data_ptr()) // 4)
        main = torch.cuda.current_stream(workspace.device)
        side = _PinnedInts.copy_stream(workspace.device)
        built = torch.cuda.Event()
        built.record(main)
        side.wait_event(built)
        with torch.cuda.stream(side):
            self._pairs_host.copy_(count, non_blocking=True)
        workspace.record_stream(side)
        self._pairs_event = torch.cuda.Event()
        self._pairs_event.record(side)

    def row_workloads(self) -> torch.Tensor:
        """int64 (ceil(Sq/128),): non-empty 128 x 32 tiles of each row block, summed over the batch; a view into the
        plan's workspace, written by the plan builder's numbering launch."""
        num_m = -(-self.struct.Sq // 128)
        ws = self.workspace
        return torch.as_strided(ws.view(torch.int64), (num_m,), (1,), (self.struct.row_workloads - ws.data_ptr()) // 8)

    def ds_pairs(self) -> int:
        """How many (32-row slice, 128-key tile) pairs have work (waits for the asynchronous copy on first use)."""
        if self._pairs is None:
            self._pairs_event.synchronize()
            self._pairs = int(self._pairs_host[0])
        return self._pairs

    def attach_ds_workspace(self, nheads: int, head_dim: int, seqlen_k: int) -> Optional[torch.Tensor]:
        """Allocates the dS workspace of one backward call and names it in the plan struct; None (and nothing
        attached) where the hand-over does not apply.  The caller detaches it after its launches."""
        self.detach_ds_workspace()
        if head_dim != 128 or seqlen_k > 131072:
            return None
        pairs = self.ds_pairs()
        nbytes = _bam_hip.load().bam_ds_workspace_bytes(nheads, pairs)
        if nbytes <= 0 or nbytes > _ds_workspace_limit(self.workspace.device) or nheads * pairs >= 1 << 31:
            return None
        try:
            ws = self._allocate(nbytes, self.workspace.device)
        except torch.cuda.OutOfMemoryError:
            return None  # no room for it right now: the dQ kernel recomputes what it needs, as without a workspace
        self.struct.ds_workspace = ws.data_ptr()
        self.struct.ds_capacity = pairs
        return ws

    def ds_head_runs(self, batch: int, nheads: int, nheads_k: int, head_dim: int, seqlen_k: int) -> int:
        """Into how many runs of whole kv heads a backward splits: the smallest divisor of ``nheads_k`` for which the
        dS workspace of one run stays within the limit, and beyond that more runs while a run's workspace is above
        ``_DS_RUN_TARGET`` and its dK/dV launch keeps ``_DS_RUN_MIN_WORKGROUPS`` workgroups.  1: all heads at once
        (also where the hand-over does not apply or no split helps: ``attach_ds_workspace`` then decides)."""
        if head_dim != 128 or seqlen_k > 131072 or nheads % nheads_k != 0:
            return 1
        pairs = self.ds_pairs()
        limit = _ds_workspace_limit(self.workspace.device)
        lib = _bam_hip.load()
        nbytes = {r: lib.bam_ds_workspace_bytes(nheads // r, pairs) for r in range(1, nheads_k + 1) if nheads_k % r == 0}
        fits = [r for r, n in nbytes.items() if 0 < n <= limit and (nheads // r) * pairs < 1 << 31]
        if not fits:
            return 1
        runs = fits[0]
        key_tiles = batch * ((seqlen_k + 127) // 128)
        for r in fits[1:]:
            if nbytes[runs] <= _DS_RUN_TARGET or key_tiles * (nheads_k // r) < _DS_RUN_MIN_WORKGROUPS:
                break
            runs = r
        return runs

    @staticmethod
    def _allocate(nbytes: int, device) -> torch.Tensor:
        return torch.empty((nbytes,), dtype=torch.uint8, device=device)

    def detach_ds_workspace(self) -> None:
        self.struct.ds_workspace = None
        self.struct.ds_capacity = 0

    @contextlib.contextmanager
    def ds_handover(self, nheads: int, head_dim: int, seqlen_k: int):
        """The launches of one backward: the dS workspace (if any) is attached on entry and detached on exit, and
        other host threads that run a backward with the same plan wait meanwhile (the struct is shared; the
        launches only enqueue work, so the wait is short)."""
        with self._lock:
            ws = self.attach_ds_workspace(nheads, head_dim, seqlen_k)
            try:
                yield ws
            finally:
                self.detach_ds_workspace()

    def byref(self):
        import ctypes

        return ctypes.byref(self.struct)

    def fine_classes(self) -> torch.Tensor:
        """uint8 (B, 4 * ceil(S/128), ceil(S/32)) view: class 0 / 1 / 2 of every 32-row x 32-key tile."""
        st, ws = self.struct, self.workspace
        slots, num_n = 4 * (-(-st.Sq // BLOCK_M)), -(-st.Sk // BLOCK_N)
        return torch.as_strided(ws, (st.B, slots, num_n), (st.fine_stride_b, st.fine_stride_s, 1), st.fine - ws.data_ptr())

    def slice_order(self) -> torch.Tensor:
        """int32 (B, 4 * ceil(S/128)) view: the 32-row slices in the order the forward / dQ kernels take them."""
        st, ws = self.struct, self.workspace
        return torch.as_strided(ws.view(torch.int32), (st.B, 4 * (-(-st.Sq // BLOCK_M))), (st.order_stride_b, 1),
                                (st.order - ws.data_ptr()) // 4)


    def group_order(self) -> Optional[torch.Tensor]:
        """int32 (B * ceil(S/128),) view, or None (more than 8192 groups): the groups of four slices of
        ``slice_order()``, as codes ``b * ceil(S/128) + group``, by falling number of 64-key tiles they visit -- the
        order in which the forward / dQ kernels take their workgroups."""
        st, ws = self.struct, self.workspace
        if not st.group_order:
            return None
        return torch.as_strided(ws.view(torch.int32), (st.B * (-(-st.Sq // BLOCK_M)),), (1,),
                                (st.group_order - ws.data_ptr()) // 4)


def _plan_arg(plan: Optional["_TilePlan"]):
    return plan.byref() if plan is not None else None


class BitfieldUtils:
    """Cache of the tile flags ("compressed mask") of the current bitfield mask.

    compressed_mask_cache: int8 (batch, ceil(S / BLOCK_M), ceil(S / BLOCK_N));
        0: every pair of the tile is masked, the tile is skipped
        1: some pairs are allowed, the mask is evaluated
        2: every in-range pair is allowed, the mask is not evaluated
    Same API as the reference (bitfield_attention.py:159-212).  The reference returns
    whatever the cache holds until ``clear_cache()``; here a hit additionally requires the
    argument to be the very memory the flags were computed from, unchanged: the cache holds a
    reference to that tensor (so its address cannot be handed to another tensor while the
    entry lives) and compares address, shape, strides and version counter.
    """

    compressed_mask_cache: Optional[torch.Tensor] = None
    _cache_key = None
    _cache_owner: Optional[torch.Tensor] = None  # the bitfield tensor the cached flags belong to
    _plan: Optional[_TilePlan] = None            # built with the cached flags; None for very long sequences

    @classmethod
    def clear_cache(cls):
        with _CACHE_LOCK:
            cls.compressed_mask_cache = None
            cls._cache_key = None
            cls._cache_owner = None
            cls._plan = None
            _IndexView.forget()

    @classmethod
    def plan_for(cls, compressed_mask: torch.Tensor, bitfield_mask: torch.Tensor) -> Optional[_TilePlan]:
        """The plan that was built together with ``compressed_mask``: only when that is the cached flags tensor
        itself and ``bitfield_mask`` is still the (unchanged) mask they were computed from.  Callers that bring
        their own flags (re-indexed context-parallel shards, for instance) get None and the kernels work from
        the flags alone."""
        with _CACHE_LOCK:
            plan, cached, key = cls._plan, cls.compressed_mask_cache, cls._cache_key
        if plan is None or plan.flags is not cached:
            return None
        # the cache keeps its flags tensor alive, so equal address and shape mean "that tensor" (autograd may hand
        # saved tensors back as new Python objects)
        if compressed_mask.data_ptr() != plan.flags.data_ptr() or compressed_mask.shape != plan.flags.shape:
            return None
        if key != cls._key_of(bitfield_mask):
            return None
        return plan

    @staticmethod
    def _key_of(bitfield_mask: torch.Tensor):
        return (
            bitfield_mask.data_ptr(),
            tuple(bitfield_mask.shape),
            tuple(bitfield_mask.stride()),
            bitfield_mask._version,
            bitfield_mask.device,
        )

    @classmethod
    def materialize_compressed_mask_from_bitfield_mask(cls, bitfield_mask: torch.Tensor) -> torch.Tensor:
        with _CACHE_LOCK:
            return cls._materialize_locked(bitfield_mask)

    @classmethod
    def _materialize_locked(cls, bitfield_mask: torch.Tensor) -> torch.Tensor:
        key = cls._key_of(bitfield_mask)
        if cls.compressed_mask_cache is not None and cls._cache_key == key:
            # _cache_owner is alive, so this address still belongs to the tensor (or a view of the
            # tensor) the flags were computed from, and its version says it has not been written since
            return cls.compressed_mask_cache

        assert bitfield_mask.is_cuda, "bitfield attention runs on the GPU only"
        assert bitfield_mask.dtype == torch.int64 and bitfield_mask.dim() == 2
        bf = bitfield_mask if bitfield_mask.stride(1) == 1 else bitfield_mask.contiguous()
        batch_size, seq_len = bf.shape
        out = torch.empty(
            (batch_size, -(-seq_len // BLOCK_M), -(-seq_len // BLOCK_N)),
            dtype=torch.int8,
            device=bf.device,
        )
        plan = None
        with torch.cuda.device(bf.device):
            ws_bytes = _bam_hip.load().bam_plan_workspace_bytes(batch_size, seq_len)
            if ws_bytes > 0:
                workspace = torch.empty((ws_bytes,), dtype=torch.uint8, device=bf.device)
                struct = _bam_hip.Plan()
                import ctypes

                _bam_hip.call(
                    "bam_tile_plan", bf.data_ptr(), bf.stride(0), out.data_ptr(), out.stride(0), out.stride(1),
                    workspace.data_ptr(), ws_bytes, batch_size, seq_len, ctypes.byref(struct), _stream_ptr(bf.device),
                )
                plan = _TilePlan(workspace, struct, out)
            else:
                _bam_hip.call(
                    "bam_tile_flags", bf.data_ptr(), bf.stride(0), out.data_ptr(), out.stride(0), out.stride(1),
                    batch_size, seq_len, _stream_ptr(bf.device),
                )
        cls.compressed_mask_cache = out
        cls._cache_key = key
        cls._cache_owner = bitfield_mask
        cls._plan = plan
        return out

    @classmethod
    def nonempty_tiles_per_row_block(cls, compressed_mask: torch.Tensor) -> torch.Tensor:
        """int64 (ceil(S/128),): non-empty 128x32 tiles of each row block, summed over the batch --
        ``torch.sum(compressed_mask > 0, dim=(0, 2))``, the per-block workload the makespan-minimizing
        sequence split sorts by (reference shardformer/layers/utils.py:161-171), computed on the GPU so that
        only this small vector has to travel to the host."""
        assert compressed_mask.is_cuda and compressed_mask.dtype == torch.int8 and compressed_mask.dim() == 3
        with _CACHE_LOCK:
            plan, cached = cls._plan, cls.compressed_mask_cache
        # the cached flags tensor itself, unwritten since it was built: its plan already holds the sums, so nothing is
        # launched; the result is a view into the plan's workspace (read it, do not write it)
        if (plan is not None and cached is not None and plan.flags is cached and plan.struct.row_workloads
                and compressed_mask.data_ptr() == cached.data_ptr() and compressed_mask.shape == cached.shape
                and compressed_mask.stride() == cached.stride() and compressed_mask._version == plan.flags_version):
            return plan.row_workloads()
        flags = compressed_mask if compressed_mask.stride(-1) == 1 else compressed_mask.contiguous()
        batch_size, num_m, num_n = flags.shape
        out = torch.empty((num_m,), dtype=torch.int32, device=flags.device)
        with torch.cuda.device(flags.device):
            _bam_hip.call(
                "bam_flag_row_workloads", flags.data_ptr(), flags.stride(0), flags.stride(1), batch_size, num_m, num_n,
                out.data_ptr(), _stream_ptr(flags.device),
            )
        return out.to(torch.int64)


class _BiasView:
    """Additive attention bias as the kernels take it: the checks and the broadcast of the reference host
    functions (bitfield_attention.py:952-972, 1124-1143) and the ``bam_bias`` struct built from the expanded
    view.  ``bias`` is 4-dimensional, broadcastable to (batch, nheads, seqlen_q, seqlen_k), its last two
    dimensions are (1, seqlen_k) ("vector", e.g. ALiBi slopes times key position) or (seqlen_q, seqlen_k)
    ("matrix"); fp32 or the dtype of q.  Nothing is copied unless the last stride is not 1."""

    def __init__(self, bias: torch.Tensor, q: torch.Tensor, batch: int, nheads: int, seqlen_q: int, seqlen_k: int,
                 may_copy: bool = True):
        assert bias.dtype in [q.dtype, torch.float]
        assert bias.is_cuda
        assert bias.dim() == 4
        if bias.stride(-1) != 1:
            assert may_copy, "bias must have unit stride along the keys"
            bias = bias.contiguous()
        if bias.shape[2:] == (1, seqlen_k):
            self.bias_type = "vector"
        elif bias.shape[2:] == (seqlen_q, seqlen_k):
            self.bias_type = "matrix"
        else:
            raise RuntimeError("Last 2 dimensions of bias must be (1, seqlen_k) or (seqlen_q, seqlen_k)")
        bias = bias.expand(batch, nheads, seqlen_q, seqlen_k)
        self.tensor = bias  # keeps the memory alive while launches are in flight on the host side
        self.struct = _bam_hip.Bias(
            bias.data_ptr(), bias.stride(0), bias.stride(1), bias.stride(2), int(bias.dtype == torch.float)
        )

    def byref(self):
        import ctypes

        return ctypes.byref(self.struct)


def _bias_arg(view: Optional["_BiasView"]):
    return view.byref() if view is not None else None


class _IndexView:
    """Index-tensor attention (``offsets_q`` / ``offsets_k`` of the reference entry points,
    bitfield_attention.py:938-939, 1085-1086): local row i of q sits at global position
    ``offsets_q[i]``, local key j at ``offsets_k[j]``, and ``bitfield_mask`` is indexed by global
    position (bitfield_attention.py:71-87).  The gather bitfield[offsets] is done once, by a kernel of
    the library, and the attention kernels read the gathered arrays with unit stride."""

    def __init__(self, bitfield_mask: torch.Tensor, offsets_q: torch.Tensor, offsets_k: torch.Tensor):
        if offsets_q is None or offsets_k is None:
            raise ValueError("offsets_q and offsets_k must be given together")
        dev = bitfield_mask.device
        bf = bitfield_mask if bitfield_mask.stride(1) == 1 else bitfield_mask.contiguous()
        batch, length = bf.shape
        self.seqlen_q, self.seqlen_k = int(offsets_q.numel()), int(offsets_k.numel())
        assert offsets_q.dim() == 1 and offsets_k.dim() == 1
        self._keep = []
        arrays = []
        with torch.cuda.device(dev):
            for off in (offsets_q, offsets_k):
                idx = off.to(device=dev, dtype=torch.int64).contiguous()
                bits = torch.empty((batch, idx.numel()), dtype=torch.int64, device=dev)
                pos = torch.empty((idx.numel(),), dtype=torch.int32, device=dev)
                _bam_hip.call(
                    "bam_gather_bitfields", bf.data_ptr(), bf.stride(0), length, idx.data_ptr(), idx.numel(),
                    bits.data_ptr(), bits.stride(0), pos.data_ptr(), batch, _stream_ptr(dev),
                )
                arrays.append((bits, pos))
                self._keep.append(idx)
        (self.q_bits, self.q_pos), (self.k_bits, self.k_pos) = arrays
        self.struct = _bam_hip.IndexView(
            self.q_bits.data_ptr(), self.k_bits.data_ptr(), self.q_pos.data_ptr(), self.k_pos.data_ptr(),
            self.q_bits.stride(0), self.k_bits.stride(0), self.seqlen_q, self.seqlen_k,
        )
        # the plan of the shard (classes of its 32 x 32 tiles, slice order), from the gathered arrays
        self.plan = None
        with torch.cuda.device(dev):
            ws_bytes = _bam_hip.load().bam_plan_workspace_bytes_rect(batch, self.seqlen_q, self.seqlen_k)
            if ws_bytes > 0:
                import ctypes

                workspace = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
                struct = _bam_hip.Plan()
                _bam_hip.call(
                    "bam_plan_indexed", ctypes.byref(self.struct), workspace.data_ptr(), ws_bytes, batch,
                    ctypes.byref(struct), _stream_ptr(dev),
                )
                self.plan = _TilePlan(workspace, struct, None)

    def byref(self):
        import ctypes

        return ctypes.byref(self.struct)

    # The context-parallel caller runs the forward and, later, the backward of one shard with the same three
    # tensors (context_parallel_bitfield_attention.py:137-147, 270-294): the last view is kept, together with the
    # tensors it was gathered from (so their addresses cannot be handed to other tensors meanwhile), and reused
    # while those are unchanged.
    _last = None

    @staticmethod
    def _tensor_key(t: torch.Tensor):
        return (t.data_ptr(), tuple(t.shape), tuple(t.stride()), t._version, t.device, t.dtype)

    @classmethod
    def get(cls, bitfield_mask: torch.Tensor, offsets_q: torch.Tensor, offsets_k: torch.Tensor) -> "_IndexView":
        if offsets_q is None or offsets_k is None:
            raise ValueError("offsets_q and offsets_k must be given together")
        key = tuple(cls._tensor_key(t) for t in (bitfield_mask, offsets_q, offsets_k))
        with _CACHE_LOCK:
            if cls._last is not None and cls._last[0] == key:
                return cls._last[1]
            view = cls(bitfield_mask, offsets_q, offsets_k)
            cls._last = (key, view, (bitfield_mask, offsets_q, offsets_k))
            return view

    @classmethod
    def forget(cls):
        cls._last = None


def _bitfield_attn_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    bitfield_mask: torch.Tensor,
    compressed_mask: torch.Tensor,
    offsets_q: Optional[torch.Tensor] = None,
    offsets_k: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
    softmax_scale: Optional[float] = None,
):
    """q (B, S, Hq, D), k/v (B, S, Hkv, D) -> (o like q, lse fp32 (B, Hq, ceil(S/128)*128),
    softmax_scale).  Contract of the reference's ``_bitfield_attn_forward``
    (bitfield_attention.py:932-1069)."""
    batch, seqlen_q, nheads, d = q.shape
    _, seqlen_k, nheads_k, _ = k.shape
    assert d <= 128, "FlashAttention only support head dimensions up to 128"
    assert q.dtype == k.dtype == v.dtype, "All tensors must have the same type"
    assert q.dtype in [torch.float16, torch.bfloat16], "Only support fp16 and bf16"
    assert q.is_cuda and k.is_cuda and v.is_cuda
    assert k.shape == v.shape and k.shape[0] == batch and k.shape[3] == d
    assert nheads % nheads_k == 0
    assert bitfield_mask.dtype == torch.int64 and bitfield_mask.dim() == 2 and bitfield_mask.shape[0] == batch
    bias_view = _BiasView(bias, q, batch, nheads, seqlen_q, seqlen_k) if bias is not None else None
    view = None
    if offsets_q is not None or offsets_k is not None:
        view = _IndexView.get(bitfield_mask, offsets_q, offsets_k)
        assert (view.seqlen_q, view.seqlen_k) == (seqlen_q, seqlen_k), "one offset per local query row / key"
    else:
        assert seqlen_q == seqlen_k, "without index tensors query and key sequence lengths must match"
        assert bitfield_mask.shape[1] == seqlen_k
    softmax_scale = softmax_scale or 1.0 / math.sqrt(d)

    dp = _padded_head_dim(d)
    if dp != d:  # zero columns change neither q.k nor the first d columns of p.v
        q, k, v = (F.pad(x, (0, dp - d)) for x in (q, k, v))
    qk, kk, vk = (_kernel_ready(x, 8) for x in (q, k, v))
    bf = bitfield_mask if bitfield_mask.stride(1) == 1 else bitfield_mask.contiguous()
    flags = compressed_mask if compressed_mask.stride(-1) == 1 else compressed_mask.contiguous()
    num_m, num_n = -(-seqlen_q // BLOCK_M), -(-seqlen_k // BLOCK_N)
    assert flags.dtype == torch.int8 and flags.shape == (batch, num_m, num_n)
    plan = BitfieldUtils.plan_for(compressed_mask, bitfield_mask) if view is None else None

    seqlen_q_rounded = num_m * BLOCK_M
    lse = torch.empty((batch, nheads, seqlen_q_rounded), device=q.device, dtype=torch.float32)
    o = torch.empty_like(qk)
    with torch.cuda.device(q.device):
        if view is None:
            _bam_hip.call(
                "bam_fwd",
                qk.data_ptr(), kk.data_ptr(), vk.data_ptr(), o.data_ptr(), lse.data_ptr(), bf.data_ptr(),
                flags.data_ptr(), *_strides3(qk, kk, vk, o),
                bf.stride(0), flags.stride(0), flags.stride(1),
                batch, seqlen_q, nheads, nheads_k, dp, float(softmax_scale), _dtype_code(q.dtype),
                _bias_arg(bias_view), _plan_arg(plan), _stream_ptr(q.device),
            )
        else:
            _bam_hip.call(
                "bam_fwd_indexed",
                qk.data_ptr(), kk.data_ptr(), vk.data_ptr(), o.data_ptr(), lse.data_ptr(), view.byref(),
                flags.data_ptr(), *_strides3(qk, kk, vk, o),
                flags.stride(0), flags.stride(1),
                batch, nheads, nheads_k, dp, float(softmax_scale), _dtype_code(q.dtype),
                _bias_arg(bias_view), _plan_arg(view.plan), _stream_ptr(q.device),
            )
    if dp != d:
        o = o[..., :d].contiguous()
    return o, lse, softmax_scale


def _strides3(*tensors):
    out = []
    for t in tensors:
        out += [t.stride(0), t.stride(1), t.stride(2)]
    return out


def _launch_bwd_preprocess(o, do, delta):
    """delta = rowsum(o * do); tensors must already satisfy the kernels' layout rules."""
    B, S, Hq, D = o.shape
    with torch.cuda.device(o.device):
        _bam_hip.call(
            "bam_bwd_preprocess", o.data_ptr(), do.data_ptr(), delta.data_ptr(), *_strides3(o, do),
            B, S, Hq, D, _dtype_code(o.dtype), _stream_ptr(o.device),
        )


def _launch_bwd_dkdv(q, k, v, do, lse, delta, dk, dv, bf, flags, softmax_scale, accumulate=True, bias=None, plan=None):
    """accumulate=True: dk/dv are fp32 and added to; False: dk/dv have q's dtype and are overwritten.
    ``bf``: the (B, S) bitfield tensor, or an ``_IndexView`` for index-tensor attention.  ``bias``: a
    ``_BiasView`` or None."""
    B, S, Hq, D = q.shape
    with torch.cuda.device(q.device):
        if isinstance(bf, _IndexView):
            _bam_hip.call(
                "bam_bwd_dkdv_indexed",
                q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), lse.data_ptr(), delta.data_ptr(),
                dk.data_ptr(), dv.data_ptr(), bf.byref(), flags.data_ptr(),
                *_strides3(q, k, v, do, dk, dv), flags.stride(0), flags.stride(1),
                B, Hq, k.shape[2], D, float(softmax_scale), _dtype_code(q.dtype), int(accumulate),
                _bias_arg(bias), _plan_arg(bf.plan), _stream_ptr(q.device),
            )
            return
        _bam_hip.call(
            "bam_bwd_dkdv",
            q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            dk.data_ptr(), dv.data_ptr(), bf.data_ptr(), flags.data_ptr(),
            *_strides3(q, k, v, do, dk, dv), bf.stride(0), flags.stride(0), flags.stride(1),
            B, S, Hq, k.shape[2], D, float(softmax_scale), _dtype_code(q.dtype), int(accumulate),
            _bias_arg(bias), _plan_arg(plan), _stream_ptr(q.device),
        )


def _launch_bwd_dq(q, k, v, do, lse, delta, dq, bf, flags, softmax_scale, accumulate=True, bias=None, plan=None):
    B, S, Hq, D = q.shape
    with torch.cuda.device(q.device):
        if isinstance(bf, _IndexView):
            _bam_hip.call(
                "bam_bwd_dq_indexed",
                q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), lse.data_ptr(), delta.data_ptr(),
                dq.data_ptr(), bf.byref(), flags.data_ptr(),
                *_strides3(q, k, v, do, dq), flags.stride(0), flags.stride(1),
                B, Hq, k.shape[2], D, float(softmax_scale), _dtype_code(q.dtype), int(accumulate),
                _bias_arg(bias), _plan_arg(bf.plan), _stream_ptr(q.device),
            )
            return
        _bam_hip.call(
            "bam_bwd_dq",
            q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            dq.data_ptr(), bf.data_ptr(), flags.data_ptr(),
            *_strides3(q, k, v, do, dq), bf.stride(0), flags.stride(0), flags.stride(1),
            B, S, Hq, k.shape[2], D, float(softmax_scale), _dtype_code(q.dtype), int(accumulate),
            _bias_arg(bias), _plan_arg(plan), _stream_ptr(q.device),
        )


def _is_kernel_ready(x: torch.Tensor, elems_per_16b: int = 8) -> bool:
    return _kernel_ready(x, elems_per_16b) is x


def _backward_in_head_runs(plan, launch, q, k, v, do, lse, delta, dq, dk, dv, head_dim, splittable=True):
    """The dK/dV and dQ launches of a backward, ``launch(q, k, v, do, lse, delta, dq, dk, dv)``, under the plan's
    dS hand-over.  When the dS workspace for all heads exceeds the limit, the heads are taken in runs of whole kv
    heads (views of the tensors along the head dimension; lse and delta of a run are made contiguous), every run
    through the same workspace: the launches of a stream run in order, so a run's dQ kernel has read the workspace
    before the next run's dK/dV kernel writes it.  Per head the arithmetic is that of a single launch pair."""
    if plan is None:
        launch(q, k, v, do, lse, delta, dq, dk, dv)
        return
    nheads, nheads_k, seqlen_k = q.shape[2], k.shape[2], k.shape[1]
    runs = plan.ds_head_runs(q.shape[0], nheads, nheads_k, head_dim, seqlen_k) if splittable else 1
    hq, hk = nheads // runs, nheads_k // runs
    with plan.ds_handover(hq, head_dim, seqlen_k):
        if runs == 1:
            launch(q, k, v, do, lse, delta, dq, dk, dv)
            return
        for r in range(runs):
            qs, ks = slice(r * hq, (r + 1) * hq), slice(r * hk, (r + 1) * hk)
            launch(q[:, :, qs], k[:, :, ks], v[:, :, ks], do[:, :, qs], lse[:, qs].contiguous(),
                   delta[:, qs].contiguous(), dq[:, :, qs], dk[:, :, ks], dv[:, :, ks])


def _bitfield_attn_backward_overwrite(do, q, k, v, o, bitfield_mask, compressed_mask, lse, softmax_scale, bias=None):
    """Gradients in the input dtype, written (not accumulated) by the kernels: what
    ``BitfieldAttentionFunction.backward`` needs, without the reference's zero-filled fp32
    staging buffers and the final cast (bitfield_attention.py:1248-1266).  Returns None when the
    layout needs the general path (padded head dimension, unaligned views)."""
    d = q.shape[-1]
    if d not in _SUPPORTED_HEAD_DIMS:
        return None
    if do.stride(-1) != 1 or not _is_kernel_ready(do):
        do = do.contiguous()
    if not all(_is_kernel_ready(x) for x in (q, k, v, o)):
        return None
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    if not all(_is_kernel_ready(x) for x in (dq, dk, dv)):
        return None
    lse = lse.contiguous()
    bf = bitfield_mask if bitfield_mask.stride(1) == 1 else bitfield_mask.contiguous()
    flags = compressed_mask if compressed_mask.stride(-1) == 1 else compressed_mask.contiguous()
    plan = BitfieldUtils.plan_for(compressed_mask, bitfield_mask)
    delta = torch.empty_like(lse)
    batch, seqlen_q, nheads, _ = q.shape
    bias_view = _BiasView(bias, q, batch, nheads, seqlen_q, k.shape[1], may_copy=False) if bias is not None else None
    _launch_bwd_preprocess(o, do, delta)

    def launch(q, k, v, do, lse, delta, dq, dk, dv):
        _launch_bwd_dkdv(q, k, v, do, lse, delta, dk, dv, bf, flags, softmax_scale, accumulate=False, bias=bias_view, plan=plan)
        _launch_bwd_dq(q, k, v, do, lse, delta, dq, bf, flags, softmax_scale, accumulate=False, bias=bias_view, plan=plan)

    # (a bias is indexed by absolute head: with one, the heads stay in one run)
    _backward_in_head_runs(plan, launch, q, k, v, do, lse, delta, dq, dk, dv, d, splittable=bias_view is None)
    return dq, dk, dv


def _bitfield_attn_backward(
    do: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    o: torch.Tensor,
    bitfield_mask: torch.Tensor,
    compressed_mask: torch.Tensor,
    lse: torch.Tensor,
    dq: torch.Tensor,
    dk: torch.Tensor,
    dv: torch.Tensor,
    offsets_q: Optional[torch.Tensor] = None,
    offsets_k: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
    softmax_scale: Optional[float] = None,
):
    """Accumulates the gradients into the caller's fp32 ``dq``, ``dk``, ``dv``.  Contract of
    the reference's ``_bitfield_attn_backward`` (bitfield_attention.py:1073-1199)."""
    if do.stride(-1) != 1:
        do = do.contiguous()
    batch, seqlen_q, nheads, d = q.shape
    _, seqlen_k, nheads_k, _ = k.shape
    assert d <= 128
    seqlen_q_rounded = math.ceil(seqlen_q / BLOCK_M) * BLOCK_M
    assert lse.shape == (batch, nheads, seqlen_q_rounded)
    assert q.stride(-1) == k.stride(-1) == v.stride(-1) == o.stride(-1) == 1
    assert dq.stride(-1) == dk.stride(-1) == dv.stride(-1) == 1
    assert dq.dtype == dk.dtype == dv.dtype == torch.float32
    assert q.is_cuda
    # the reference asserts the unit stride here instead of copying (bitfield_attention.py:1130)
    bias_view = _BiasView(bias, q, batch, nheads, seqlen_q, seqlen_k, may_copy=False) if bias is not None else None
    view = None
    if offsets_q is not None or offsets_k is not None:
        view = _IndexView.get(bitfield_mask, offsets_q, offsets_k)
        assert (view.seqlen_q, view.seqlen_k) == (seqlen_q, seqlen_k), "one offset per local query row / key"
    else:
        assert seqlen_q == seqlen_k, "without index tensors query and key sequence lengths must match"
    softmax_scale = softmax_scale or 1.0 / math.sqrt(d)

    dp = _padded_head_dim(d)
    acc = (dq, dk, dv)
    if dp != d:
        q, k, v, o, do = (F.pad(x, (0, dp - d)) for x in (q, k, v, o, do))
        acc = tuple(torch.zeros(x.shape[:-1] + (dp,), dtype=torch.float32, device=x.device) for x in (dq, dk, dv))
    qk, kk, vk, ok, gk = (_kernel_ready(x, 8) for x in (q, k, v, o, do))
    work = tuple(_kernel_ready(x, 4) for x in acc)
    lse = lse.contiguous()
    bf = bitfield_mask if bitfield_mask.stride(1) == 1 else bitfield_mask.contiguous()
    if view is not None:
        bf = view
    flags = compressed_mask if compressed_mask.stride(-1) == 1 else compressed_mask.contiguous()
    assert flags.shape == (batch, -(-seqlen_q // BLOCK_M), -(-seqlen_k // BLOCK_N))
    plan = BitfieldUtils.plan_for(compressed_mask, bitfield_mask) if view is None else None
    delta = torch.empty_like(lse)
    wq, wk, wv = work
    _launch_bwd_preprocess(ok, gk, delta)
    the_plan = plan if view is None else view.plan

    def launch(q, k, v, do, lse, delta, dq, dk, dv):
        _launch_bwd_dkdv(q, k, v, do, lse, delta, dk, dv, bf, flags, softmax_scale, bias=bias_view, plan=plan)
        _launch_bwd_dq(q, k, v, do, lse, delta, dq, bf, flags, softmax_scale, bias=bias_view, plan=plan)

    # (a bias is indexed by absolute head: with one, the heads stay in one run)
    _backward_in_head_runs(the_plan, launch, qk, kk, vk, gk, lse, delta, wq, wk, wv, dp, splittable=bias_view is None)
    # the kernels accumulated into `work`; hand the sums back if those were copies
    for dst, mid, w in zip((dq, dk, dv), acc, work):
        if dp != d:
            dst += w[..., :d]
        elif w is not mid:
            dst.copy_(w)


class BitfieldAttentionFunction(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        q: torch.Tensor,
        k: torch.Tensor,
        v: torch.Tensor,
        bitfield_mask: torch.Tensor,
        bias: Optional[torch.Tensor] = None,
        softmax_scale: Optional[float] = None,
    ):
        """
        q: (batch_size, seqlen_q, nheads, headdim)
        k, v: (batch_size, seqlen_k, nheads_k, headdim)
        bitfield_mask: (batch_size, seqlen) int64
        """
        q, k, v = [x if x.stride(-1) == 1 else x.contiguous() for x in [q, k, v]]
        if bias is not None and bias.stride(-1) != 1:
            bias = bias.contiguous()

        compressed_mask = BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bitfield_mask)

        o, lse, ctx.softmax_scale = _bitfield_attn_forward(
            q, k, v, bitfield_mask, compressed_mask, bias=bias, softmax_scale=softmax_scale
        )
        ctx.save_for_backward(q, k, v, o, lse, bias, bitfield_mask, compressed_mask)
        return o

    @staticmethod
    def backward(ctx, do: torch.Tensor):
        q, k, v, o, lse, bias, bitfield_mask, compressed_mask = ctx.saved_tensors
        assert not ctx.needs_input_grad[3], "the bitfield mask is not differentiable"
        assert not ctx.needs_input_grad[4], "FlashAttention does not support bias gradient yet"
        with torch.no_grad():
            direct = _bitfield_attn_backward_overwrite(
                do, q, k, v, o, bitfield_mask, compressed_mask, lse, ctx.softmax_scale, bias=bias
            )
            if direct is not None:
                return (*direct, None, None, None)
            dq = torch.zeros_like(q, dtype=torch.float32)
            dk = torch.zeros_like(k, dtype=torch.float32)
            dv = torch.zeros_like(v, dtype=torch.float32)
            _bitfield_attn_backward(
                do, q, k, v, o, bitfield_mask, compressed_mask, lse, dq, dk, dv,
                bias=bias, softmax_scale=ctx.softmax_scale,
            )
        return dq.to(dtype=q.dtype), dk.to(dtype=k.dtype), dv.to(dtype=v.dtype), None, None, None


def bitfield_attn_func(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    bitfield_mask: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    softmax_scale: Optional[float] = None,
) -> torch.Tensor:
    return BitfieldAttentionFunction.apply(q, k, v, bitfield_mask, bias, softmax_scale)
