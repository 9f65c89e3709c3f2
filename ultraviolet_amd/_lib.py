"""ctypes binding of libuvmi.so (declarations: include/uvmi.h).  There is no CPU fallback: if the library has not
been built, or a call fails, an exception is raised."""
from __future__ import annotations

import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libuvmi.so")

F16, BF16, F32, I8, I32, I64 = 0, 1, 2, 3, 4, 5
_DT = {torch.float16: F16, torch.bfloat16: BF16, torch.float32: F32, torch.int8: I8, torch.int32: I32,
       torch.int64: I64}


class UvmiError(RuntimeError):
    pass


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DT[dt]
    except KeyError:
        raise UvmiError(f"dtype {dt} is not supported by libuvmi") from None


class AttnArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("q_dtype", C.c_int), ("sqb", C.c_int64), ("sqh", C.c_int64),
                ("k_cache", C.c_void_p), ("v_cache", C.c_void_p), ("kv_dtype", C.c_int),
                ("skb", C.c_int64), ("skh", C.c_int64), ("sks", C.c_int64),
                ("svb", C.c_int64), ("svh", C.c_int64), ("svs", C.c_int64),
                ("k_scale", C.c_void_p), ("v_scale", C.c_void_p),
                ("ssb", C.c_int64), ("ssh", C.c_int64), ("stb", C.c_int64), ("sth", C.c_int64),
                ("pos", C.c_void_p), ("starts", C.c_void_p), ("idx_dtype", C.c_int), ("rows", C.c_void_p),
                ("out", C.c_void_p), ("out_dtype", C.c_int), ("sob", C.c_int64), ("soh", C.c_int64),
                ("B", C.c_int), ("H", C.c_int), ("KH", C.c_int), ("S", C.c_int), ("hd", C.c_int),
                ("scale", C.c_float), ("window", C.c_int), ("ring", C.c_int), ("num_splits", C.c_int),
                ("chunk_keys", C.c_int), ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
                ("post_vhat", C.c_void_p), ("post_gate", C.c_void_p), ("post_xsa", C.c_void_p), ("post_round_dtype", C.c_int),
                ("fuse", C.c_void_p)]


class AttnQkvFuse(C.Structure):
    _fields_ = [("qkv", C.c_void_p), ("row_stride", C.c_int64), ("ext_col", C.c_int), ("has_gate", C.c_int), ("tok", C.c_void_p),
                ("ve_table", C.c_void_p), ("vocab", C.c_int64), ("has_ve", C.c_int), ("rope_table", C.c_void_p), ("rope_positions", C.c_int),
                ("n_pairs", C.c_int), ("rope", C.c_int), ("eps", C.c_float), ("xsa_eps", C.c_float)]


class GemmArgs(C.Structure):
    _fields_ = [("a", C.c_void_p), ("w", C.c_void_p), ("c", C.c_void_p), ("dtype", C.c_int), ("M", C.c_int64), ("N", C.c_int),
                ("K", C.c_int), ("lda", C.c_int64), ("ldw", C.c_int64), ("ldc", C.c_int64), ("epilogue", C.c_int), ("norm_a", C.c_int),
                ("eps", C.c_float), ("resid", C.c_void_p), ("ldr", C.c_int64), ("ca", C.c_float), ("cb", C.c_float), ("config", C.c_int)]


class PrefillAttnArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("q_dtype", C.c_int), ("sqn", C.c_int64), ("sqh", C.c_int64),
                ("k", C.c_void_p), ("v", C.c_void_p), ("kv_dtype", C.c_int),
                ("skn", C.c_int64), ("skh", C.c_int64), ("svn", C.c_int64), ("svh", C.c_int64),
                ("cu_seqlens", C.c_void_p), ("idx_dtype", C.c_int), ("n_seg", C.c_int),
                ("out", C.c_void_p), ("out_dtype", C.c_int), ("son", C.c_int64), ("soh", C.c_int64),
                ("N", C.c_int), ("H", C.c_int), ("KH", C.c_int), ("hd", C.c_int),
                ("scale", C.c_float), ("window", C.c_int), ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
                ("segments_ready", C.c_int), ("post_vhat", C.c_void_p), ("post_gate", C.c_void_p), ("post_xsa", C.c_void_p)]


class PrefillAttnBwdArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p), ("go", C.c_void_p), ("dtype", C.c_int),
                ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p),
                ("cu_seqlens", C.c_void_p), ("idx_dtype", C.c_int), ("n_seg", C.c_int),
                ("N", C.c_int), ("H", C.c_int), ("KH", C.c_int), ("hd", C.c_int), ("scale", C.c_float), ("window", C.c_int),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t)]


class KvAppendArgs(C.Structure):
    _fields_ = [("k", C.c_void_p), ("v", C.c_void_p), ("x_dtype", C.c_int), ("sxb", C.c_int64), ("sxh", C.c_int64),
                ("k_cache", C.c_void_p), ("v_cache", C.c_void_p),
                ("scb", C.c_int64), ("sch", C.c_int64), ("scs", C.c_int64),
                ("k_scale", C.c_void_p), ("v_scale", C.c_void_p), ("ssb", C.c_int64), ("ssh", C.c_int64),
                ("pos", C.c_void_p), ("idx_dtype", C.c_int), ("rows", C.c_void_p),
                ("B", C.c_int), ("KH", C.c_int), ("S", C.c_int), ("hd", C.c_int), ("ring", C.c_int)]


class SampleArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("x_dtype", C.c_int), ("stride", C.c_int64), ("u", C.c_void_p),
                ("seed", C.c_uint64), ("req_id", C.c_void_p), ("tok_idx", C.c_void_p),
                ("tok", C.c_void_p), ("logp", C.c_void_p), ("u_out", C.c_void_p),
                ("B", C.c_int), ("V", C.c_int),
                ("cap_a", C.c_float), ("cap_b", C.c_float), ("cap_c", C.c_float), ("temperature", C.c_float),
                ("top_k", C.c_int), ("top_p", C.c_float), ("thr_out", C.c_void_p), ("commit", C.c_void_p)]


class QkvPostArgs(C.Structure):
    _fields_ = [("qkv", C.c_void_p), ("dtype", C.c_int), ("xn", C.c_void_p), ("ve_table", C.c_void_p),
                ("ve_gate", C.c_void_p), ("tok", C.c_void_p), ("pos", C.c_void_p), ("rows", C.c_void_p),
                ("last_pos", C.c_void_p), ("inv_freq", C.c_void_p), ("q_out", C.c_void_p), ("q_dtype", C.c_int),
                ("k_out", C.c_void_p), ("v_out", C.c_void_p), ("k_cache", C.c_void_p), ("v_cache", C.c_void_p),
                ("k_scale", C.c_void_p), ("v_scale", C.c_void_p),
                ("scb", C.c_int64), ("sch", C.c_int64), ("scs", C.c_int64), ("ssb", C.c_int64), ("ssh", C.c_int64),
                ("n", C.c_int64), ("vocab", C.c_int64),
                ("H", C.c_int), ("KH", C.c_int), ("hd", C.c_int), ("d", C.c_int), ("ve_ch", C.c_int),
                ("n_pairs", C.c_int), ("S", C.c_int), ("ring", C.c_int), ("has_ve", C.c_int), ("rope", C.c_int),
                ("eps", C.c_float), ("gate_w", C.c_void_p), ("gate_ch", C.c_int), ("gate_out", C.c_void_p),
                ("vhat_out", C.c_void_p), ("xsa_eps", C.c_float), ("rope_table", C.c_void_p), ("rope_positions", C.c_int),
                ("qkv_ld", C.c_int64), ("ext_logits", C.c_int)]


class SchedState(C.Structure):
    _fields_ = [("slot_req", C.c_void_p), ("slot_cnt", C.c_void_p), ("slot_limit", C.c_void_p), ("slot_tok", C.c_void_p),
                ("pos", C.c_void_p), ("starts", C.c_void_p), ("out_tok", C.c_void_p), ("out_lp", C.c_void_p),
                ("done_req", C.c_void_p), ("done_slot", C.c_void_p), ("done_cnt", C.c_void_p), ("counters", C.c_void_p),
                ("max_new", C.c_int64), ("eos_id", C.c_int64), ("B", C.c_int), ("done_cap", C.c_int),
                ("slot_hold", C.c_void_p), ("q_buf", C.c_void_p), ("q_ctl", C.c_void_p), ("q_cap", C.c_int), ("q_stride", C.c_int)]


class SampleCommit(C.Structure):
    _fields_ = [("state", C.POINTER(SchedState)), ("act_slot", C.c_void_p), ("tok_c", C.c_void_p), ("pos_c", C.c_void_p),
                ("starts_c", C.c_void_p), ("req_c", C.c_void_p), ("cnt_c", C.c_void_p), ("retire_p", C.c_float), ("seed", C.c_uint64)]


_lib = None
ABI_VERSION = 4   # UVMI_ABI_VERSION of include/uvmi.h


def lib() -> C.CDLL:
    """Load libuvmi.so once.  Raises UvmiError when it is missing (build it with
    `python -m ultraviolet_amd.csrc.build`)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise UvmiError(f"{LIB_PATH} not found: run `python -m ultraviolet_amd.csrc.build` (no CPU fallback)")
        L = C.CDLL(LIB_PATH)
        if L.uvmi_version() != ABI_VERSION:   # the ctypes structs below mirror one revision of include/uvmi.h
            raise UvmiError(f"{LIB_PATH} was built for revision {L.uvmi_version()} of include/uvmi.h, these bindings are for "
                            f"{ABI_VERSION}: rebuild it with `python -m ultraviolet_amd.csrc.build`")
        L.uvmi_last_error.restype = C.c_char_p
        L.uvmi_decode_attn_workspace_bytes.restype = C.c_size_t
        L.uvmi_decode_attn_workspace_bytes.argtypes = [C.c_int] * 5
        L.uvmi_default_splits.argtypes = [C.c_int64, C.c_int, C.c_int]
        L.uvmi_decode_attn.argtypes = [C.POINTER(AttnArgs), C.c_void_p]
        L.uvmi_decode_attn_path.argtypes = [C.POINTER(AttnArgs)]
        L.uvmi_decode_attn_noalloc.argtypes = [C.POINTER(AttnArgs), C.c_void_p]
        L.uvmi_decode_attn_probe.argtypes = [C.POINTER(AttnArgs), C.c_int, C.c_void_p]
        L.uvmi_prefill_attn.argtypes = [C.POINTER(PrefillAttnArgs), C.c_void_p]
        L.uvmi_prefill_attn_path.argtypes = [C.POINTER(PrefillAttnArgs)]
        L.uvmi_prefill_attn_workspace_bytes.restype = C.c_size_t
        L.uvmi_prefill_attn_workspace_bytes.argtypes = [C.c_int]
        L.uvmi_prefill_attn_bwd.argtypes = [C.POINTER(PrefillAttnBwdArgs), C.c_void_p]
        L.uvmi_prefill_attn_bwd_workspace_bytes.restype = C.c_size_t
        L.uvmi_prefill_attn_bwd_workspace_bytes.argtypes = [C.c_int, C.c_int]
        L.uvmi_quantize_rows.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_int64, C.c_void_p, C.c_void_p,
                                         C.c_void_p]
        L.uvmi_dequantize_rows.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_int, C.c_void_p]
        L.uvmi_kv_write.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                                    C.c_int64, C.c_int, C.c_int64, C.c_void_p]
        L.uvmi_kv_append.argtypes = [C.POINTER(KvAppendArgs), C.c_void_p]
        L.uvmi_fused_sample.argtypes = [C.POINTER(SampleArgs), C.c_void_p]
        L.uvmi_philox4x32_10.argtypes = [C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
        L.uvmi_philox4x32_10.restype = None
        L.uvmi_embed_norm.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_void_p, C.c_int64, C.c_int, C.c_float, C.c_void_p,
                                      C.c_void_p, C.c_void_p]
        L.uvmi_add_norm.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_float, C.c_int64, C.c_int, C.c_float,
                                    C.c_void_p, C.c_void_p, C.c_void_p]
        L.uvmi_qkv_post.argtypes = [C.POINTER(QkvPostArgs), C.c_void_p]
        L.uvmi_attn_post.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_float,
                                     C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.uvmi_swiglu.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_void_p, C.c_void_p]
        L.uvmi_swiglu_norm.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_void_p]
        L.uvmi_sched_compact.argtypes = [C.POINTER(SchedState), C.c_int] + [C.c_void_p] * 7
        L.uvmi_sched_commit.argtypes = [C.POINTER(SchedState), C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_uint64,
                                        C.c_void_p]
        L.uvmi_sched_commit_dense.argtypes = [C.POINTER(SchedState), C.c_int] + [C.c_void_p] * 8 + [C.c_float, C.c_uint64, C.c_void_p]
        L.uvmi_sched_admit.argtypes = [C.POINTER(SchedState), C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.c_void_p]
        L.uvmi_sched_expand.argtypes = [C.POINTER(SchedState), C.c_int, C.c_int] + [C.c_void_p] * 8
        L.uvmi_sched_harvest.argtypes = [C.POINTER(SchedState), C.c_int64, C.c_int] + [C.c_void_p] * 4
        L.uvmi_sched_plan_admit.argtypes = [C.POINTER(SchedState), C.c_int, C.c_int, C.c_int] + [C.c_void_p] * 7
        L.uvmi_sched_step_plan.argtypes = ([C.POINTER(SchedState), C.c_int] + [C.c_void_p] * 6 + [C.c_int, C.c_int, C.c_int] +
                                           [C.c_void_p] * 12)
        L.uvmi_rope_table.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_void_p, C.c_void_p]
        L.uvmi_gemm_tn_supported.argtypes = [C.c_int, C.c_int64, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int]
        L.uvmi_gemm_tn_ex.argtypes = [C.POINTER(GemmArgs), C.c_void_p]
        L.uvmi_gemm_tn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_int, C.c_int64, C.c_int64,
                                   C.c_int64, C.c_int, C.c_void_p]
        _lib = L
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().uvmi_last_error().decode(errors="replace")
        raise UvmiError(f"{what} failed ({rc}): {msg}")


def stream_ptr(t: torch.Tensor) -> int:
    """HIP stream torch is currently launching on for t's device."""
    return torch.cuda.current_stream(t.device).cuda_stream


def require_cuda(*ts: torch.Tensor) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise UvmiError("libuvmi kernels need device tensors (there is no CPU path)")


EXPORTS = ["uvmi_version", "uvmi_last_error", "uvmi_device_cus", "uvmi_quantize_rows", "uvmi_dequantize_rows",
           "uvmi_kv_write", "uvmi_kv_append", "uvmi_decode_attn", "uvmi_decode_attn_workspace_bytes",
           "uvmi_default_splits", "uvmi_decode_attn_path", "uvmi_decode_attn_noalloc", "uvmi_decode_attn_probe", "uvmi_prefill_attn", "uvmi_prefill_attn_workspace_bytes",
           "uvmi_prefill_attn_path", "uvmi_fused_sample", "uvmi_philox4x32_10",
           "uvmi_embed_norm", "uvmi_add_norm", "uvmi_qkv_post", "uvmi_attn_post", "uvmi_swiglu", "uvmi_swiglu_norm",
           "uvmi_prefill_attn_bwd", "uvmi_prefill_attn_bwd_workspace_bytes", "uvmi_sched_compact", "uvmi_sched_commit", "uvmi_sched_commit_dense", "uvmi_sched_admit", "uvmi_sched_expand", "uvmi_sched_harvest", "uvmi_sched_plan_admit", "uvmi_sched_step_plan", "uvmi_rope_table", "uvmi_gemm_tn_supported", "uvmi_gemm_tn", "uvmi_gemm_tn_ex"]
