"""CPU-side checks of the boundary: the C-ABI library loads, exports every symbol that
include/trittention_hip.h declares, rejects bad arguments before launching anything, and the
Python host mirrors the reference's error behaviour.  No kernel runs here."""
import ctypes
import os
import re

import pytest
import torch

from flash_trittention import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "trittention_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tritt_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.lib()
    names = declared_symbols()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_lib.exported_symbols()) == names


def test_version_and_status_strings():
    lib = _lib.lib()
    assert lib.tritt_version() >= 100
    assert lib.tritt_status_string(0) == b"ok"
    assert b"head dimension" in lib.tritt_status_string(-2)


def test_workspace_queries_scale_with_problem():
    lib = _lib.lib()
    a = lib.tritt_tdp_bwd_workspace_bytes(1, 2, 64, 32, _lib.TRITT_F32, 1, 64, 64, 64, 64, 1)
    b = lib.tritt_tdp_bwd_workspace_bytes(2, 2, 64, 32, _lib.TRITT_F32, 1, 64, 64, 64, 64, 1)
    assert 0 < a < b
    assert lib.tritt_tdp_fwd_workspace_bytes(1, 2, 64, 24, _lib.TRITT_F32, 1, 64, 64, 64, 64, 0) == 0  # bad D
    assert lib.tritt_dps_fwd_workspace_bytes(1, 2, 64, 32, _lib.TRITT_BF16, 0) > 0


def test_argument_rejection_happens_before_any_launch():
    lib = _lib.lib()
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(256)  # never dereferenced: rejected first
    args7 = [one] * 7
    assert lib.tritt_tdp_fwd(*args7, 1, 1, 16, 24, 0, 0.1, 1, 16, 16, 16, 16, null, 0, 0, null) == -2
    assert lib.tritt_tdp_fwd(*args7, -1, 1, 16, 32, 0, 0.1, 1, 16, 16, 16, 16, null, 0, 0, null) == -1
    assert lib.tritt_tdp_fwd(*args7, 1, 1, 16, 32, 7, 0.1, 1, 16, 16, 16, 16, null, 0, 0, null) == -1
    assert lib.tritt_tdp_fwd(*args7, 256, 256, 16, 32, 0, 0.1, 1, 16, 16, 16, 16, null, 0, 0, null) == -1  # B*H
    assert lib.tritt_dps_fwd(*args7, 128, 256, 1 << 16, 32, 1, 0.1, 1, 16, null, 0, 0, null) == -1  # B*H*T
    assert lib.tritt_tdp_fwd(null, *args7[1:], 1, 1, 16, 32, 0, 0.1, 1, 16, 16, 16, 16, null, 0, 0, null) == -1
    assert lib.tritt_tdp_fwd(*args7, 1, 1, 16, 32, 0, 0.1, 1, -1, 16, 16, 16, null, 0, 0, null) == -1
    assert lib.tritt_tdp_fwd(*args7, 1, 1, 16, 32, 0, 0.1, 1, 16, 16, 16, 16, null, 0, 1, null) == -3  # no workspace
    assert lib.tritt_dps_fwd(*args7, 1, 1, 16, 32, 0, 0.1, 1, 16, null, 0, 0, null) == -3
    assert lib.tritt_dps_fwd(*args7, 1, 1, 16, 32, 0, 0.1, 1, -2, one, 1 << 30, 0, null) == -1
    odd = ctypes.c_void_p(258)  # not on a 16-byte boundary
    assert lib.tritt_tdp_fwd(odd, *args7[1:], 1, 1, 16, 32, 0, 0.1, 1, 16, 16, 16, 16, null, 0, 0, null) == -1
    assert lib.tritt_dps_fwd(*args7[:3], odd, *args7[4:], 1, 1, 16, 32, 0, 0.1, 1, 16, null, 0, 0, null) == -1
    assert b"misaligned" in lib.tritt_status_string(-1)


def test_empty_problem_is_a_successful_no_op():
    """B, H or T equal to 0: nothing is launched, null pointers are accepted, the workspace size is 0; the head
    dimension and the dtype are still checked."""
    lib = _lib.lib()
    null = ctypes.c_void_p(0)
    for B, H, T in [(0, 2, 16), (2, 0, 16), (2, 2, 0)]:
        assert lib.tritt_tdp_fwd_workspace_bytes(B, H, T, 32, 0, 1, 16, 16, 16, 16, 0) == 0
        assert lib.tritt_tdp_fwd(*[null] * 7, B, H, T, 32, 0, 0.1, 1, 16, 16, 16, 16, null, 0, 0, null) == 0
        assert lib.tritt_tdp_bwd(*[null] * 13, B, H, T, 32, 0, 0.1, 1, 16, 16, 16, 16, null, 0, 0, null) == 0
        assert lib.tritt_dps_fwd(*[null] * 7, B, H, T, 32, 0, 0.1, 1, 16, null, 0, 0, null) == 0
        assert lib.tritt_dps_bwd(*[null] * 13, B, H, T, 32, 0, 0.1, 1, 16, null, 0, 0, null) == 0
    assert lib.tritt_tdp_fwd(*[null] * 7, 0, 2, 16, 24, 0, 0.1, 1, 16, 16, 16, 16, null, 0, 0, null) == -2
    assert lib.tritt_dps_fwd(*[null] * 7, 0, 2, 16, 32, 9, 0.1, 1, 16, null, 0, 0, null) == -1
    assert lib.tritt_tdp_fwd(*[null] * 7, 0, -2, 16, 32, 0, 0.1, 1, 16, 16, 16, 16, null, 0, 0, null) == -1


def test_python_host_validation_matches_reference_errors():
    from flash_trittention import TrittentionTriton, flash_trittention

    q, k1, k2, v1, v2 = (torch.randn(2, 2, 32, 32) for _ in range(5))
    with pytest.raises(ValueError):
        flash_trittention(q, k1, k2, v1, v2[:, :, :16])
    with pytest.raises(ValueError):
        flash_trittention(q, k1, k2, v1, v2.double())
    with pytest.raises(ValueError):
        flash_trittention(*(torch.randn(2, 2, 32, 24) for _ in range(5)))
    with pytest.raises(ValueError):
        TrittentionTriton()(q, k1, k2, v1, v2[:, :, :16])
    # well-formed CPU tensors: the product has no CPU path and says so
    with pytest.raises(RuntimeError, match="GPU"):
        flash_trittention(q, k1, k2, v1, v2)
    with pytest.raises(RuntimeError, match="GPU"):
        TrittentionTriton()(q, k1, k2, v1, v2)


def test_window_arguments_are_clamped_before_they_reach_32_bit_ints():
    """ctypes would silently wrap 2**32 to 0 (a window of zero): the host clamps to seq_len first."""
    from flash_trittention.triple_dot_product.utils import clamp_window, process_masking_variables

    assert process_masking_variables(100, None, 2**31, 2**32, 10**12) == (100, 100, 100, 100)
    assert process_masking_variables(100, 0, 5, 99, 100) == (0, 5, 99, 100)
    assert clamp_window(2**32 + 5, 64) == 64
    for bad in (-1, -2**31):
        with pytest.raises(ValueError):
            process_masking_variables(100, bad, None, None, None)
        with pytest.raises(ValueError):
            clamp_window(bad, 100, "k_diff")


def test_implementation_flags_are_class_constants():
    """Pinning an implementation makes a subclass; the public Functions are never mutated."""
    from flash_trittention.dot_product_sum.trittention_triton import TrittentionTritonFunction
    from flash_trittention.triple_dot_product.flash_trittention import FlashTrittention

    for cls in (FlashTrittention, TrittentionTritonFunction):
        forced = cls.with_flags(_lib.FLAG_FORCE_GENERIC)
        assert forced is not cls and issubclass(forced, cls) and forced.IMPL_FLAGS == _lib.FLAG_FORCE_GENERIC
        assert cls.with_flags(_lib.FLAG_FORCE_GENERIC) is forced and cls.with_flags(0) is cls
        assert cls.IMPL_FLAGS == _lib.FLAG_AUTO


def test_module_front_of_triple_dot():
    from flash_trittention import FlashTrittentionModule

    m = FlashTrittentionModule(causal=True, softmax_scale=0.25, n_ctx=16, k1_window=4)
    assert "k1_window" not in dict(m.named_parameters()) and "windows=(4, None, None, None)" in repr(m)
    q = torch.randn(1, 1, 32, 32)
    with pytest.raises(ValueError, match="n_ctx"):
        m(q, q, q, q, q)
    with pytest.raises(RuntimeError, match="GPU"):
        FlashTrittentionModule()(q, q, q, q, q)


def test_lazy_package_exports():
    import flash_trittention as ft

    assert ft.__all__ == ["flash_trittention", "TrittentionTriton", "FlashTrittentionModule"]
    assert callable(ft.flash_trittention) and callable(ft.TrittentionTriton) and callable(ft.FlashTrittentionModule)
    with pytest.raises(AttributeError):
        ft.nope


def test_product_never_imports_oracle():
    pkg = os.path.join(ROOT, "flash-3-way-attention_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, os.path.join(dirpath, f)
