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
    assert lib.uvmi_version() == _lib.ABI_VERSION
    hdr = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "uvmi.h")).read()
    assert int(re.search(r"#define UVMI_ABI_VERSION (\d+)", hdr).group(1)) == _lib.ABI_VERSION


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


def test_gemm_capability_predicate_and_argument_checks():
    """uvmi_gemm_tn_supported is host logic: 16-bit types, K in slabs of 64 up to 8192, N in fragments of 16 (32 for the
    interleaved SwiGLU layout), pitches that keep 16-byte rows, 32-bit operand offsets.  The entry point refuses bad
    arguments before it touches the device."""
    from ultraviolet_amd import _lib
    lib = _lib.lib()
    F16, BF16, F32 = 0, 1, 2
    ok = lambda *a: bool(lib.uvmi_gemm_tn_supported(*a))
    assert ok(BF16, 2048, 656, 640, 640, 640, 656, 0) and ok(F16, 1, 16, 64, 64, 64, 16, 0)
    assert ok(BF16, 33216, 3328, 640, 640, 640, 1664, 1)             # SWIGLU writes N / 2 columns
    assert not ok(F32, 64, 64, 64, 64, 64, 64, 0)                    # 16-bit only
    assert not ok(BF16, 64, 64, 96, 96, 96, 64, 0)                   # K % 64
    assert not ok(BF16, 64, 64, 8256, 8256, 8256, 64, 0)             # K > 8192
    assert not ok(BF16, 64, 24, 64, 64, 64, 24, 0)                   # N % 16
    assert not ok(BF16, 64, 48, 64, 64, 64, 24, 1)                   # SWIGLU needs N % 32
    assert not ok(BF16, 64, 64, 64, 60, 64, 64, 0)                   # lda < K
    assert not ok(BF16, 64, 64, 64, 68, 64, 64, 0)                   # lda % 8
    assert not ok(BF16, 64, 64, 64, 64, 64, 48, 0)                   # ldc < N
    assert not ok(BF16, 65536, 64, 8192, 8192, 8192, 64, 0)          # operand offsets past 2^30 bytes
    assert not ok(BF16, 64, 64, 64, 64, 64, 64, 3)                   # unknown epilogue
    g = _lib.GemmArgs()
    assert lib.uvmi_gemm_tn_ex(C.byref(g), None) == -1               # null pointers
    assert lib.uvmi_gemm_tn_ex(None, None) == -1


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


# ---------------------------------------------------------------------------------------------- header <-> ctypes layout
_STRUCTS = {"uvmi_attn_args": "AttnArgs", "uvmi_attn_qkv_fuse": "AttnQkvFuse", "uvmi_gemm_args": "GemmArgs",
            "uvmi_prefill_attn_args": "PrefillAttnArgs", "uvmi_prefill_attn_bwd_args": "PrefillAttnBwdArgs",
            "uvmi_kv_append_args": "KvAppendArgs", "uvmi_sample_args": "SampleArgs", "uvmi_qkv_post_args": "QkvPostArgs",
            "uvmi_sched_state": "SchedState", "uvmi_sample_commit": "SampleCommit"}
_CTYPE = {"int": C.c_int, "int64_t": C.c_int64, "uint64_t": C.c_uint64, "float": C.c_float, "size_t": C.c_size_t}


def _header_structs():
    """{struct name: [(field, C type or 'ptr')]} parsed from include/uvmi.h, in declaration order."""
    src = open(os.path.join(ROOT, "include", "uvmi.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    out = {}
    for name, body in re.findall(r"typedef\s+struct\s+(\w+)\s*\{(.*?)\}\s*\w+\s*;", src, flags=re.S):
        fields = []
        for decl in body.split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            m = re.match(r"^(?:const\s+)?(?:struct\s+)?(\w+)\s*(.*)$", decl)
            base, rest = m.group(1), m.group(2)
            for d in rest.split(","):
                d = d.strip()
                fields.append((d.lstrip("* ").strip(), "ptr" if "*" in d else base))
        out[name] = fields
    return out


def test_ctypes_structures_follow_the_header_field_for_field():
    """Order, names and types of every argument structure in ultraviolet_amd/_lib.py against include/uvmi.h, and the dtype
    codes: a binding that drifts from the header reads garbage without any error."""
    from ultraviolet_amd import _lib
    hs = _header_structs()
    assert set(hs) == set(_STRUCTS), set(hs) ^ set(_STRUCTS)
    for cname, pyname in _STRUCTS.items():
        cls = getattr(_lib, pyname)
        assert [f for f, _ in hs[cname]] == [f[0] for f in cls._fields_], cname
        for (fname, ctype), (_, pytype) in zip(hs[cname], cls._fields_):
            if ctype == "ptr":
                assert pytype is C.c_void_p or issubclass(pytype, C._Pointer), (cname, fname)
            else:
                assert pytype is _CTYPE[ctype], (cname, fname, ctype, pytype)
    hdr = open(os.path.join(ROOT, "include", "uvmi.h")).read()
    codes = dict(re.findall(r"#define UVMI_(F16|BF16|F32|I8|I32|I64) (\d+)", hdr))
    assert {k: int(v) for k, v in codes.items()} == dict(F16=_lib.F16, BF16=_lib.BF16, F32=_lib.F32, I8=_lib.I8, I32=_lib.I32, I64=_lib.I64)


def test_ctypes_offsets_equal_the_c_compilers(tmp_path):
    """sizeof and every offsetof as gcc lays the header's structures out, against ctypes' layout of the bindings."""
    import subprocess
    from ultraviolet_amd import _lib
    hs = _header_structs()
    lines = ['#include <stddef.h>', '#include <stdio.h>', '#include "uvmi.h"', "int main(void) {"]
    for cname in _STRUCTS:
        lines.append(f'  printf("{cname} %zu\\n", sizeof({cname}));')
        for f, _ in hs[cname]:
            lines.append(f'  printf("{cname}.{f} %zu\\n", offsetof({cname}, {f}));')
    lines += ["  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    got = dict(l.split() for l in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    for cname, pyname in _STRUCTS.items():
        cls = getattr(_lib, pyname)
        assert int(got[cname]) == C.sizeof(cls), cname
        for f, _ in hs[cname]:
            assert int(got[f"{cname}.{f}"]) == getattr(cls, f).offset, (cname, f)


def test_reference_names_are_mirrored():
    """The names the reference's callers import (ultraviolet/kernels/__init__.py:9-10, model.py:867, 886, 942, perf.py:579-625,
    scripts/rl_grpo.py:1091-1094) exist here; decode_attention_ref / fused_sample_ref are deliberately absent from the
    product (they are the oracle)."""
    import torch
    import ultraviolet_amd.kernels as K
    from ultraviolet_amd import perf
    from ultraviolet_amd.kernels import fast_decode, fused_sample, varlen_attn
    for n in ("decode_attention", "default_splits", "dequantize_kv", "kv_write", "kv_write_rows", "quantize_kv"):
        assert callable(getattr(K, n))
    assert not hasattr(K, "decode_attention_ref") and not hasattr(fused_sample, "fused_sample_ref")
    for n in ("KernelDecodeState", "DecodeState", "prefill_fast", "decode_step_fast", "prefill_packed_host", "patch_model", "unpatch_model"):
        assert hasattr(fast_decode, n)
    for n in ("fused_sample", "fused_sample_ok"):
        assert callable(getattr(fused_sample, n))
    assert callable(varlen_attn.varlen_attention)
    for n in ("make_streamgen", "install_fz", "StreamGen", "sync_weights_inplace"):
        assert hasattr(perf, n)
    assert perf.make_streamgen(perf.StreamGen, ["lp", "hv", "rfh", "fz"]) is perf.StreamGen
    from ultraviolet_amd import _lib
    with pytest.raises(_lib.UvmiError):
        perf.make_streamgen(perf.StreamGen, ["lpp"])
    s = str(torch.ops.mathk.decode_attn.default._schema)   # the reference's op name and argument list (decode_attn.py:174-178)
    assert s.startswith("mathk::decode_attn(Tensor q, Tensor k_cache, Tensor v_cache, Tensor pos, Tensor starts, float scale")
    assert "num_splits" in s and "block_n" in s and "num_warps" in s and "str backend" in s
    assert "mathk::varlen_attn_fwd(Tensor q, Tensor k, Tensor v, Tensor cu" in str(torch.ops.mathk.varlen_attn_fwd.default._schema)
    assert "mathk::varlen_attn_bwd(Tensor go" in str(torch.ops.mathk.varlen_attn_bwd.default._schema)
    import inspect
    assert inspect.signature(fast_decode.patch_model).parameters["kv_dtype"].default == "fp16"   # fast_decode.py:341


def test_checkpoint_with_unsupported_layers_is_refused():
    """A reference checkpoint whose cfg switches on MUDD / the bigram table / conv layers / a non-attention local mixer must
    not load into the attention-only engine with those fields dropped."""
    from ultraviolet_amd.engine import UVWeights, as_uvconfig, make_config
    base = make_config("uv-test").to_dict()
    for extra in (dict(mudd=True), dict(bigram_rows=1024), dict(conv_layers=[1]), dict(local_mixer="gdn")):
        with pytest.raises(ValueError):
            UVWeights.from_checkpoint({"model": {}, "cfg": dict(base, **extra)}, device="cpu")
    import types
    with pytest.raises(ValueError):
        as_uvconfig(types.SimpleNamespace(**base, mudd=True))
    assert as_uvconfig(dict(base, mudd=False, local_mixer="attn")).d_model == base["d_model"]


def test_integration_doc_stub_matches_the_binding():
    """The maintainer's stub printed in the integration notes at the repository root is executed as far as its declarations go (ctypes.CDLL replaced by
    the loaded library) and compared with ultraviolet_amd/_lib.py: same dtype codes, same structure, same layout."""
    import torch
    from ultraviolet_amd import _lib
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = doc[doc.index("```python\nimport ctypes as C, torch"):]
    block = block[len("```python\n"):block.index("\n```")]
    block = block.replace('C.CDLL("libuvmi.so")', "LIB")
    ns = {"LIB": _lib.lib()}
    exec(compile(block, "INTEGRATION.md", "exec"), ns)
    assert ns["_DT"] == {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32, torch.int8: _lib.I8,
                         torch.int32: _lib.I32, torch.int64: _lib.I64}
    assert ns["AttnArgs"]._fields_ == _lib.AttnArgs._fields_
    assert C.sizeof(ns["AttnArgs"]) == C.sizeof(_lib.AttnArgs)
    a = ns["_args"](torch.zeros(2, 8, 64, dtype=torch.bfloat16), torch.zeros(2, 1, 32, 64, dtype=torch.int8), torch.zeros(2, 1, 32, 64, dtype=torch.int8),
                    torch.zeros(2, dtype=torch.long), torch.zeros(2, dtype=torch.long), 0.125, 0, False,
                    torch.zeros(2, 1, 32, dtype=torch.float16), torch.zeros(2, 1, 32, dtype=torch.float16), 1, torch.zeros(2, 8, 64), None)
    assert (a.B, a.H, a.KH, a.S, a.hd, a.q_dtype, a.kv_dtype, a.out_dtype, a.idx_dtype) == (2, 8, 1, 32, 64, 1, 3, 2, 5)
    assert _lib.lib().uvmi_decode_attn_path(C.byref(a)) == 1    # CPU pointers are never dereferenced by the path predicate


def test_weight_stamp_is_stable_on_a_real_module():
    """The stamp a patched model's methods compare must not move unless a parameter was written: nn.Module.state_dict()
    returns fresh detached tensors on every call, so the stamp keys on the live parameters (address + version counter)."""
    import torch
    from ultraviolet_amd.kernels import fast_decode as fd

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = torch.nn.Linear(4, 3)
            self.register_buffer("b", torch.zeros(2))

    m = Net()
    assert [id(t) for t in m.state_dict().values()] != [id(t) for t in m.state_dict().values()]   # why ids cannot be used
    s0 = fd._weights_stamp(m)
    assert fd._weights_stamp(m) == s0 and fd._weights_stamp(m) == s0
    fd._remember_stamp(m)
    assert fd._quick_stamp(m) == m.__dict__["_uvmi_quick"]
    with torch.no_grad():
        m.a.weight.mul_(1.5)                      # an optimizer step
    assert fd._weights_stamp(m) != s0 and fd._quick_stamp(m) != m.__dict__["_uvmi_quick"]
    s1 = fd._weights_stamp(m)
    assert fd._weights_stamp(m) == s1
    with torch.no_grad():
        m.b.add_(1.0)                             # buffers count too
    assert fd._weights_stamp(m) != s1
    # an object that only offers state_dict() without arguments (a dict of tensors) is stamped on its own tensors
    class Plain:
        def __init__(self):
            self._sd = {"w": torch.zeros(3)}
        def state_dict(self):
            return self._sd
    p = Plain()
    s2 = fd._weights_stamp(p)
    assert fd._weights_stamp(p) == s2
    p._sd["w"].add_(1)
    assert fd._weights_stamp(p) != s2
