"""ctypes binding of ``libviewattn.so`` (declarations: ``include/viewattn.h``).

The library is the only compute path of this package: if it is missing the
import of this module raises, there is no fallback.
"""

from __future__ import annotations

import ctypes as C
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# VIEWATTN_LIB selects another build of the same library (e.g. an instrumented one)
LIB_PATH = os.environ.get("VIEWATTN_LIB") or os.path.join(_HERE, "libviewattn.so")

VA_F32, VA_F16, VA_BF16 = 0, 1, 2
VA_ROPE_TABLE, VA_ROPE_MROPE = 0, 1
VA_KERNEL_AUTO, VA_KERNEL_GENERIC, VA_KERNEL_MFMA = 0, 1, 2
VA_SUB_CAUSAL, VA_SUB_SLOTS = 1, 2
PLAN_HEADER_WORDS = 24
VA_ERR_ARG, VA_ERR_CAPACITY = -1, -2
STATIC_SCRATCH_BYTES = 32 << 20  # VA_STATIC_SCRATCH_BYTES: the array va_attention_static keeps on every GPU

_DTYPES = {torch.float32: VA_F32, torch.float16: VA_F16, torch.bfloat16: VA_BF16}

EXPORTED_SYMBOLS = (
    "va_last_error",
    "va_version",
    "va_rope",
    "va_store_kv_rope",
    "va_plan_count",
    "va_plan_build",
    "va_copy_shift_kv",
    "va_plan_capacity",
    "va_plan_fixed_words",
    "va_plan_build_fixed",
    "va_attention",
    "va_attention_static",
)


class VaShape(C.Structure):
    _fields_ = [
        ("num_q_heads", C.c_int32),
        ("num_kv_heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("page_size", C.c_int32),
        ("dtype", C.c_int32),
    ]


class VaRope(C.Structure):
    _fields_ = [
        ("mode", C.c_int32),
        ("rotary_dim", C.c_int32),
        ("cos_sin_dev", C.c_void_p),
        ("max_pos", C.c_int32),
        ("section_h", C.c_int32),
        ("section_w", C.c_int32),
        ("inv_freq_dev", C.c_void_p),
    ]


class VaSubRequests(C.Structure):
    _fields_ = [
        ("n_sub", C.c_int32),
        ("n_subrows", C.c_int32),
        ("n_rows", C.c_int32),
        ("qo_indptr", C.c_void_p),
        ("kv_indptr", C.c_void_p),
        ("kv_indices", C.c_void_p),
        ("seq_lens", C.c_void_p),
        ("flags", C.c_void_p),
        ("chain", C.c_void_p),
        ("sub_worker", C.c_void_p),
    ]


class VaPlanParams(C.Structure):
    _fields_ = [
        ("kernel", C.c_int32),
        ("q_tile", C.c_int32),
        ("kv_chunk", C.c_int32),
        ("target_items", C.c_int32),
        ("wide_tile", C.c_int32),
    ]


class VaPlanCounts(C.Structure):
    _fields_ = [
        ("kernel", C.c_int32),
        ("q_tile", C.c_int32),
        ("kv_chunk", C.c_int32),
        ("n_items", C.c_int32),
        ("n_links", C.c_int32),
        ("n_qrefs", C.c_int32),
        ("n_partials", C.c_int32),
        ("n_row_parts", C.c_int32),
        ("plan_words", C.c_int32),
        ("wide_tile", C.c_int32),
        ("n_wide_items", C.c_int32),
        ("workspace_bytes", C.c_int64),
        ("n_wide_slots", C.c_int32),
    ]


class VaPlanLimits(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("max_sub_requests", "max_sub_rows", "max_chains", "max_chain_members",
                                         "max_chain_rows", "max_rows")]


class VaPlanCapacity(C.Structure):
    _fields_ = [
        ("max_items", C.c_int32),
        ("max_wide_items", C.c_int32),
        ("max_links", C.c_int32),
        ("max_qrefs", C.c_int32),
        ("max_partials", C.c_int32),
        ("max_row_parts", C.c_int32),
        ("max_rows", C.c_int32),
    ]


def _load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python async_llm_amd/build.py` "
            "(hipcc, --offload-arch=gfx950); this package has no other compute path"
        )
    lib = C.CDLL(LIB_PATH)
    lib.va_last_error.restype = C.c_char_p
    lib.va_version.restype = C.c_int
    i64, i32, vp = C.c_int64, C.c_int32, C.c_void_p
    lib.va_rope.restype = C.c_int
    lib.va_rope.argtypes = [vp, vp, vp, i64, i64, i32, i32, i32, i64, i64, C.POINTER(VaRope), vp]
    lib.va_store_kv_rope.restype = C.c_int
    lib.va_store_kv_rope.argtypes = [vp, vp, i64, i64, vp, vp, i64, vp, i32, vp, i64, i64,
                                     C.POINTER(VaShape), C.POINTER(VaRope), vp]
    lib.va_copy_shift_kv.restype = C.c_int
    lib.va_copy_shift_kv.argtypes = [vp, vp, i64, i64, i32, vp, vp, i64, i64, C.POINTER(VaShape), C.POINTER(VaRope), vp]
    lib.va_plan_count.restype = C.c_int
    lib.va_plan_count.argtypes = [C.POINTER(VaSubRequests), C.POINTER(VaShape), C.POINTER(VaPlanParams),
                                  C.POINTER(VaPlanCounts)]
    lib.va_plan_capacity.restype = C.c_int
    lib.va_plan_capacity.argtypes = [C.POINTER(VaShape), C.POINTER(VaPlanParams), C.POINTER(VaPlanLimits),
                                     C.POINTER(VaPlanCapacity)]
    lib.va_plan_fixed_words.restype = C.c_int64
    lib.va_plan_fixed_words.argtypes = [C.POINTER(VaPlanCapacity)]
    lib.va_plan_build_fixed.restype = C.c_int
    lib.va_plan_build_fixed.argtypes = [C.POINTER(VaSubRequests), C.POINTER(VaShape), C.POINTER(VaPlanParams),
                                        C.POINTER(VaPlanCapacity), C.c_void_p, C.c_int64, C.POINTER(VaPlanCounts)]
    lib.va_plan_build.restype = C.c_int
    lib.va_plan_build.argtypes = [C.POINTER(VaSubRequests), C.POINTER(VaShape), C.POINTER(VaPlanParams),
                                  vp, i64, C.POINTER(VaPlanCounts)]
    lib.va_attention.restype = C.c_int
    lib.va_attention.argtypes = [vp, i64, vp, vp, i64, vp, vp, vp, vp, vp, i64, vp, vp, i32, vp, i64,
                                 C.POINTER(VaShape), C.POINTER(VaRope), vp]
    lib.va_attention_static.restype = C.c_int
    lib.va_attention_static.argtypes = [vp, i64, vp, vp, i64, vp, vp, vp, vp, vp, i64, vp, vp, i32,
                                        C.POINTER(VaShape), C.POINTER(VaRope), vp]
    return lib


lib = _load()


class ViewAttnError(RuntimeError):
    pass


def check(rc: int) -> None:
    if rc != 0:
        raise ViewAttnError(f"libviewattn error {rc}: {lib.va_last_error().decode()}")


def dtype_id(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ViewAttnError(f"unsupported element type {dtype}") from None


def require_device(t: torch.Tensor, name: str) -> None:
    if t.device.type != "cuda":
        raise ViewAttnError(
            f"{name} lives on {t.device}: view attention runs on the GPU only (HIP kernels, no CPU path)"
        )


def current_stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def make_shape(hq: int, hkv: int, d: int, page: int, dtype: torch.dtype) -> VaShape:
    return VaShape(hq, hkv, d, page, dtype_id(dtype))


def make_rope(rotary_dim: int, cos_sin: Optional[torch.Tensor], inv_freq: Optional[torch.Tensor],
              mrope_section) -> VaRope:
    """Describe the rotation: interleaved mRoPE when ``mrope_section`` is set
    (cos/sin from ``inv_freq``), else the 1-D fp32 cos|sin table."""
    if mrope_section is not None:
        assert inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.is_contiguous()
        rope = VaRope(VA_ROPE_MROPE, rotary_dim, None, 0, int(mrope_section[1]), int(mrope_section[2]),
                      inv_freq.data_ptr())
        rope._keepalive = inv_freq  # the struct only holds the raw device address
        return rope
    assert cos_sin is not None
    if cos_sin.dtype != torch.float32 or not cos_sin.is_contiguous():
        raise ViewAttnError("cos_sin_cache must be a contiguous fp32 [max_pos, rotary_dim] tensor")
    if rotary_dim and cos_sin.shape[1] != rotary_dim:
        raise ViewAttnError(f"cos_sin_cache has {cos_sin.shape[1]} columns, rotary_dim is {rotary_dim}")
    rope = VaRope(VA_ROPE_TABLE, rotary_dim, cos_sin.data_ptr(), cos_sin.shape[0], 0, 0, None)
    rope._keepalive = cos_sin
    return rope
