"""The C-ABI library loads without a GPU and exports every symbol include/uvmi.h declares; host-only entry points work."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    src = open(os.path.join(ROOT, "include", "uvmi.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(uvmi_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    from ultraviolet_amd import _lib
    lib = _lib.lib()
    names = _declared()
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/uvmi.h but not exported"
    assert set(_lib.EXPORTS) <= set(names)
    assert lib.uvmi_version() >= 1


def test_host_only_entry_points():
    from oracle import philox
    from ultraviolet_amd import _lib
    lib = _lib.lib()
    assert lib.uvmi_decode_attn_workspace_bytes(256, 8, 1, 64, 1) == 0
    assert lib.uvmi_decode_attn_workspace_bytes(256, 8, 1, 64, 4) >= 256 * 8 * 4 * (64 + 2) * 4
    assert lib.uvmi_default_splits(2048, 2320, 256) == 1
    assert lib.uvmi_default_splits(64, 2048, 256) == 4
    assert lib.uvmi_default_splits(1, 100000, 256) == 64
    c = (C.c_uint32 * 4)(0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344)
    k = (C.c_uint32 * 2)(0xa4093822, 0x299f31d0)
    o = (C.c_uint32 * 4)()
    lib.uvmi_philox4x32_10(c, k, o)
    assert list(o) == [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]
    assert list(o) == [int(v) for v in philox.philox4x32_10(list(c), list(k))]


def test_argument_errors_are_reported_not_thrown():
    from ultraviolet_amd import _lib
    lib = _lib.lib()
    assert lib.uvmi_quantize_rows(None, 0, 4, 64, 64, None, None, None) == -1
    assert b"null" in lib.uvmi_last_error()
    a = _lib.AttnArgs()
    assert lib.uvmi_decode_attn(C.byref(a), None) == -1
    assert lib.uvmi_decode_attn(None, None) == -1


def test_no_cpu_fallback():
    import torch
    from ultraviolet_amd import _lib
    from ultraviolet_amd.kernels import decode_attention, quantize_kv
    from ultraviolet_amd.kernels.fused_sample import fused_sample, fused_sample_ok
    with pytest.raises(_lib.UvmiError):
        quantize_kv(torch.zeros(2, 64))
    with pytest.raises(_lib.UvmiError):
        decode_attention(torch.zeros(1, 8, 64, dtype=torch.float16), torch.zeros(1, 1, 8, 64, dtype=torch.int8),
                         torch.zeros(1, 1, 8, 64, dtype=torch.int8), torch.zeros(1, dtype=torch.long), torch.zeros(1, dtype=torch.long), 0.1,
                         k_scale=torch.zeros(1, 1, 8, dtype=torch.float16), v_scale=torch.zeros(1, 1, 8, dtype=torch.float16), num_splits=1)
    with pytest.raises(_lib.UvmiError):
        fused_sample(torch.zeros(1, 512), torch.zeros(1), (23.0, 5.0, 7.5))
    assert not fused_sample_ok(torch.device("cpu"), 16384, (23.0, 5.0, 7.5), 1.0)   # reference: test_perf_fz.py:74-77


def test_product_code_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "ultraviolet_amd")
    for dp, _, fs in os.walk(pkg):
        for f in fs:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                txt = open(os.path.join(dp, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", txt, flags=re.M), f
