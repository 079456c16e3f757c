"""CPU-only checks of the host side: the C-ABI library loads and exports what the header
declares, host logic mirrors the reference's interface, the product path refuses to run
without the GPU / the HIP library (no fallback), and the synthetic workloads are the ones
the baseline document describes."""

import ctypes
import os
import re

import pytest
import torch

from cornstarch_amd import workloads as W
from cornstarch_amd.kernel import _bam_hip
from cornstarch_amd.kernel import attention as sibling
from cornstarch_amd.kernel import bitfield_attention as BA
from cornstarch_amd.kernel import interface
from oracle import bam_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "bam_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bam_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_bam_hip.LIB_PATH):
        from cornstarch_amd import build

        build.build_library(force=True)
    lib = ctypes.CDLL(_bam_hip.LIB_PATH)
    names = _declared_symbols()
    assert {"bam_tile_flags", "bam_fwd", "bam_bwd", "bam_bwd_preprocess", "bam_materialize_mask",
            "bam_bwd_dkdv", "bam_bwd_dq", "bam_last_error", "bam_abi_version"} <= set(names)
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/bam_hip.h but not exported"
    assert _bam_hip.load().bam_abi_version() == _bam_hip.ABI_VERSION
    # the binding's prototypes cover every compute entry point of the header
    assert set(_bam_hip.SIGNATURES) == set(names) - {
        "bam_last_error", "bam_abi_version", "bam_plan_workspace_bytes", "bam_plan_workspace_bytes_rect",
        "bam_ds_workspace_bytes", "bam_mask_plan_workspace_bytes", "bam_decode_workspace_bytes"}
    # plan workspace: sized without a GPU; no plan beyond 4096 row slices
    lib2 = _bam_hip.load()
    assert lib2.bam_plan_workspace_bytes(1, 8192) >= 256 * 256 + 256 * 4 and lib2.bam_plan_workspace_bytes(1, 8192) % 256 == 0
    assert lib2.bam_plan_workspace_bytes(2, 131072) > 0 and lib2.bam_plan_workspace_bytes(1, 131073) == 0
    # rectangular problems (context-parallel shards, materialized masks): rows bound the plan, keys only size it
    assert lib2.bam_plan_workspace_bytes_rect(1, 8192, 8192) == lib2.bam_plan_workspace_bytes(1, 8192)
    assert lib2.bam_plan_workspace_bytes_rect(1, 4096, 8192) >= 128 * 256 + 128 * 4
    assert lib2.bam_plan_workspace_bytes_rect(1, 131073, 64) == 0 and lib2.bam_plan_workspace_bytes_rect(1, 64, 262144) > 0
    # a mask plan also holds the mask packed to bits, once per orientation: a quarter of the mask's bytes
    extra = lib2.bam_mask_plan_workspace_bytes(1, 8192, 8192) - lib2.bam_plan_workspace_bytes_rect(1, 8192, 8192)
    assert extra == 2 * 8192 * 8192 // 8 and lib2.bam_mask_plan_workspace_bytes(1, 131073, 64) == 0


def test_abi_rejects_bad_arguments_without_touching_the_gpu():
    lib = _bam_hip.load()
    # null pointers / unsupported head dim are refused before any HIP call
    rc = lib.bam_tile_flags(None, 0, None, 0, 0, 1, 128, None)
    assert rc == -1 and b"null" in lib.bam_last_error()
    args = [ctypes.c_void_p(16)] * 7 + [8] * 15 + [1, 128, 4, 4, 48] + [0.125, 1, None, None, None]
    rc = lib.bam_fwd(*args)
    assert rc == -2 and b"head dimension 48" in lib.bam_last_error()
    args = [ctypes.c_void_p(16)] * 7 + [8] * 15 + [1, 128, 6, 4, 64] + [0.125, 1, None, None, None]
    assert lib.bam_fwd(*args) == -1 and b"multiple of Hkv" in lib.bam_last_error()
    args = [ctypes.c_void_p(8)] + [ctypes.c_void_p(16)] * 6 + [8] * 15 + [1, 128, 4, 4, 64] + [0.125, 1, None, None, None]
    assert lib.bam_fwd(*args) == -1 and b"16-byte aligned" in lib.bam_last_error()
    args = [ctypes.c_void_p(16)] * 7 + [8] * 15 + [1, 128, 4, 4, 64] + [-1.0, 1, None, None, None]
    assert lib.bam_fwd(*args) == -1 and b"scale" in lib.bam_last_error()
    # a bias descriptor without a pointer, or with a pointer that is not a multiple of its element size
    bias = _bam_hip.Bias(None, 0, 0, 0, 1)
    args = [ctypes.c_void_p(16)] * 7 + [8] * 15 + [1, 128, 4, 4, 64] + [0.125, 1, ctypes.byref(bias), None, None]
    assert lib.bam_fwd(*args) == -1 and b"bias" in lib.bam_last_error()
    bias = _bam_hip.Bias(18, 0, 0, 0, 1)
    args = [ctypes.c_void_p(16)] * 7 + [8] * 15 + [1, 128, 4, 4, 64] + [0.125, 1, ctypes.byref(bias), None, None]
    assert lib.bam_fwd(*args) == -1 and b"bias" in lib.bam_last_error()
    # a sequence beyond the sanity bound is refused with a clear error, before anything is launched
    args = [ctypes.c_void_p(16)] * 7 + [8] * 15 + [1, _bam_hip.BAM_MAX_SEQLEN + 1, 4, 4, 64] + [0.125, 1, None, None, None]
    assert lib.bam_fwd(*args) == -2 and b"BAM_MAX_SEQLEN" in lib.bam_last_error()
    with pytest.raises(_bam_hip.BamError):
        _bam_hip.call("bam_materialize_mask", None, 0, None, 1, 8, None)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_bam_hip, "_lib", None)
    monkeypatch.setattr(_bam_hip, "LIB_PATH", "/nonexistent/libbam_hip.so")
    with pytest.raises(_bam_hip.BamError, match="no fallback"):
        _bam_hip.load()


def test_product_path_has_no_cpu_fallback():
    q = torch.randn(1, 64, 2, 32, dtype=torch.bfloat16)
    bf = torch.full((1, 64), (1 << 62) | 1, dtype=torch.int64)
    with pytest.raises(AssertionError):
        BA.bitfield_attn_func(q, q, q, bf)
    with pytest.raises(AssertionError):
        BA.BitfieldUtils.materialize_compressed_mask_from_bitfield_mask(bf)
    flags = torch.zeros((1, 1, 2), dtype=torch.int8)
    with pytest.raises(AssertionError, match="fp16 and bf16"):
        BA._bitfield_attn_forward(q.float(), q.float(), q.float(), bf, flags)
    with pytest.raises(AssertionError, match="up to 128"):
        big = torch.randn(1, 64, 2, 256, dtype=torch.bfloat16)
        BA._bitfield_attn_forward(big, big, big, bf, flags)


def test_module_constants_and_signatures_match_the_reference_interface():
    import inspect

    assert (BA.BLOCK_M, BA.BLOCK_N, BA.NUM_TOKENS_TO_COMPUTE_PER_BLOCK) == (128, 32, 4096)
    assert (sibling.BLOCK_M, sibling.BLOCK_N) == (128, 32)
    assert list(inspect.signature(BA.bitfield_attn_func).parameters) == [
        "q", "k", "v", "bitfield_mask", "bias", "softmax_scale"]
    assert list(inspect.signature(BA._bitfield_attn_forward).parameters) == [
        "q", "k", "v", "bitfield_mask", "compressed_mask", "offsets_q", "offsets_k", "bias", "softmax_scale"]
    assert list(inspect.signature(BA._bitfield_attn_backward).parameters) == [
        "do", "q", "k", "v", "o", "bitfield_mask", "compressed_mask", "lse", "dq", "dk", "dv",
        "offsets_q", "offsets_k", "bias", "softmax_scale"]
    assert list(inspect.signature(interface.bitfield_attention_forward).parameters) == [
        "module", "query", "key", "value", "attention_mask", "dropout", "scaling", "sliding_window", "softcap",
        "kwargs"]
    assert hasattr(BA.BitfieldUtils, "compressed_mask_cache") and BA.BitfieldUtils.compressed_mask_cache is None
    BA.BitfieldUtils.clear_cache()


def test_create_bitfield_attention_mask_format():
    ids = torch.tensor([[5, 9, 9, 7, 3, 7, 1]])
    got = interface.create_bitfield_attention_mask(ids, {"vision": 9, "audio": 7})
    text = (1 << 62) | 1 | 2 | 4
    assert got.tolist() == [[text, 2, 2, 4, text, 4, text]] and got.dtype == torch.int64
    assert interface.create_bitfield_attention_mask(ids).tolist() == [[(1 << 62) | 1] * 7]


def test_adapter_requires_int64_mask():
    class M(torch.nn.Module):
        pass

    q = torch.randn(1, 2, 8, 32)
    with pytest.raises(AssertionError, match="int64"):
        interface.bitfield_attention_forward(M(), q, q, q, torch.ones(1, 8, dtype=torch.bool))
    # the single-token decode step of an eval-mode module never looks at the mask, and like the rest of the
    # product path it has no CPU fallback
    m = M().eval()
    q1 = torch.randn(1, 4, 1, 32, dtype=torch.bfloat16)
    kv = torch.randn(1, 2, 9, 32, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="GPU only"):
        interface.bitfield_attention_forward(m, q1, kv, kv, None)


def test_decode_entry_rejects_bad_arguments_without_touching_the_gpu():
    lib = _bam_hip.load()
    P = ctypes.c_void_p
    good = [P(16)] * 4 + [8] * 10 + [1, 64, 4, 2, 64] + [0.125, 1, 0, 0.0, None, 0, None]
    bad_window = list(good)
    bad_window[21] = -3
    assert lib.bam_decode(*bad_window) == -1 and b"window" in lib.bam_last_error()
    bad_cap = list(good)
    bad_cap[22] = -1.0
    assert lib.bam_decode(*bad_cap) == -1 and b"softcap" in lib.bam_last_error()
    bad_heads = list(good)
    bad_heads[16:18] = [4, 3]
    assert lib.bam_decode(*bad_heads) == -1 and b"multiple of Hkv" in lib.bam_last_error()
    assert lib.bam_decode(*([None] + good[1:])) == -1 and b"null" in lib.bam_last_error()
    # long caches are split over many workgroups and need a workspace for the partial results; short ones do not
    assert lib.bam_decode_workspace_bytes(1, 32, 4, 2, 64, 0) == 0
    need = lib.bam_decode_workspace_bytes(1, 8192, 32, 8, 128, 0)
    assert need > 0 and need % (32 * (128 + 2) * 4) == 0
    assert lib.bam_decode_workspace_bytes(1, 8192, 32, 8, 128, 32) == 0  # a window of one tile: one split
    long_cache = list(good)
    long_cache[15] = 8192
    assert lib.bam_decode(*long_cache) == -1 and b"workspace" in lib.bam_last_error()


# The import statements of the reference's callers, verbatim (file:line of /root/reference/cornstarch/...).
REFERENCE_IMPORT_LINES = [
    # shardformer/layers/utils.py:11-12
    "from cornstarch.kernel.attention import BLOCK_M, BLOCK_N",
    "from cornstarch.kernel.bitfield_attention import BitfieldUtils",
    # shardformer/layers/context_parallel_bitfield_attention.py:7-10
    "from cornstarch.kernel.bitfield_attention import (\n    _bitfield_attn_backward,\n    _bitfield_attn_forward,\n)",
    # shardformer/modeling/llama.py:31 (and gemma, gemma2, gemma3, llama4, mistral, mixtral, phi3, qwen2, qwen3, qwen3_moe)
    "from cornstarch.kernel.bitfield_attention import BitfieldUtils",
    # models/multimodal_language_model/modeling_multimodal_language_model.py:37
    "from cornstarch.kernel.interface import bitfield_attention_forward",
    # kernel/interface.py:9-10
    "from cornstarch.kernel.attention import flash_attn_func",
    "from cornstarch.kernel.bitfield_attention import bitfield_attn_func",
    # tests/test_kernel/test_attention.py:5-7, tests/test_shardformer/test_context_parallel.py:16,
    # tests/test_shardformer/utils.py:42-45
    "from cornstarch.kernel.attention import (\n    flash_attn_func as my_flash_attn_func_triton,\n)",
    "from cornstarch.kernel.bitfield_attention import BitfieldUtils, bitfield_attn_func",
    "from cornstarch.kernel.interface import (\n    bitfield_attention_forward,\n    create_bitfield_attention_mask,\n)",
]


@pytest.mark.parametrize("line", REFERENCE_IMPORT_LINES)
def test_import_statements_of_the_reference_callers_resolve_here(line):
    ns = {}
    exec(line, ns)
    impl = {"BitfieldUtils": BA.BitfieldUtils, "_bitfield_attn_forward": BA._bitfield_attn_forward,
            "_bitfield_attn_backward": BA._bitfield_attn_backward, "bitfield_attn_func": BA.bitfield_attn_func,
            "flash_attn_func": sibling.flash_attn_func, "my_flash_attn_func_triton": sibling.flash_attn_func,
            "bitfield_attention_forward": interface.bitfield_attention_forward,
            "create_bitfield_attention_mask": interface.create_bitfield_attention_mask,
            "BLOCK_M": 128, "BLOCK_N": 32}
    got = {k: v for k, v in ns.items() if k != "__builtins__"}
    assert got and all(got[k] is impl[k] or got[k] == impl[k] for k in got)


def test_cornstarch_kernel_modules_are_the_implementation_modules():
    import importlib

    for name, impl in (("bitfield_attention", BA), ("attention", sibling), ("interface", interface)):
        assert importlib.import_module(f"cornstarch.kernel.{name}") is impl
    # the registration the reference performs at import time
    # (models/multimodal_language_model/modeling_multimodal_language_model.py:42) works through either name
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

    from cornstarch.kernel.interface import bitfield_attention_forward

    ALL_ATTENTION_FUNCTIONS.update({"bitfield_attention": bitfield_attention_forward})
    assert ALL_ATTENTION_FUNCTIONS["bitfield_attention"] is interface.bitfield_attention_forward


def test_cornstarch_package_leaves_other_subpackages_to_a_checkout_further_down_the_path(tmp_path):
    # a stand-in for a Cornstarch checkout: a `cornstarch` package with a subpackage of its own and a kernel
    # package that must NOT win
    import subprocess
    import sys

    pkg = tmp_path / "site" / "cornstarch"
    (pkg / "shardformer").mkdir(parents=True)
    (pkg / "kernel").mkdir()
    (pkg / "__init__.py").write_text("")
    (pkg / "shardformer" / "__init__.py").write_text("from cornstarch.kernel.bitfield_attention import BitfieldUtils\n")
    (pkg / "kernel" / "__init__.py").write_text("")
    (pkg / "kernel" / "bitfield_attention.py").write_text("BitfieldUtils = 'theirs'\n")
    code = (
        "import sys; sys.path[:0] = [%r, %r]\n"
        "import cornstarch.shardformer as s, cornstarch_amd.kernel.bitfield_attention as ours\n"
        "assert s.__file__.startswith(%r), s.__file__\n"
        "assert s.BitfieldUtils is ours.BitfieldUtils\n"
    ) % (ROOT, str(tmp_path / "site"), str(tmp_path))
    subprocess.run([sys.executable, "-c", code], check=True)


# histogram / pair counts of the synthetic workloads quoted by the baseline document
EXPECTED = {
    "C1": (557440, [108, 24, 124]),
    "C2": (24536064, [9685, 1334, 5365]),
    "C3": (91592220, [41456, 2998, 21082]),
    "C4": (38492218, [20466, 5287, 7015]),
}


@pytest.mark.parametrize("name", sorted(EXPECTED))
def test_workload_generator_statistics(name):
    bf = W.make_bitfields(name)
    w = W.WORKLOADS[name]
    assert bf.shape == (w.B, w.S) and bf.dtype == torch.int64
    pairs, hist = EXPECTED[name]
    assert O.unmasked_pairs(bf) == pairs
    flags = O.tile_flags(bf)
    assert [(flags == v).sum().item() for v in (0, 1, 2)] == hist
    assert W.flops(name, pairs) == (4 * w.D * w.Hq * pairs, 10 * w.D * w.Hq * pairs)


def test_workload_tensors_are_seeded_and_sliceable():
    q, k, v, do = W.make_tensors("C1")
    q2, *_ = W.make_tensors("C1")
    assert q.dtype == torch.float32 and torch.equal(q, q2) and q.shape == (1, 1024, 8, 64)
    qa, ka, va, doa = W.make_tensors("C4", heads=(2, 4))
    qf, kf, vf, dof = W.make_tensors("C4")
    assert torch.equal(qa, qf[:, :, 2:4]) and torch.equal(ka, kf[:, :, 2:4]) and torch.equal(doa, dof[:, :, 2:4])
    assert qf.dtype == torch.bfloat16


def test_c5_layout_shape():
    bf = W.make_bitfields("C5")
    assert bf.shape == (1, 65536)
    text = W.text_bits(range(1, 17))
    seg = bf[0] != text
    # 200 segments of 16..512 tokens
    assert 200 * 16 <= int(seg.sum()) <= 200 * 512
    assert set(bf[0][seg].tolist()) <= {1 << b for b in range(1, 17)}
