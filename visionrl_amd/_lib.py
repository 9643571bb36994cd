"""ctypes binding of ``include/vrl_int4.h``.

The library is loaded from the package tree (``csrc/libvrl_int4.so``); nothing
is compiled at import or call time.  A missing library is an error, never a
reason to fall back to another implementation.
"""

from __future__ import annotations

import ctypes
import os
import threading

from .build import LIB_PATH

ABI_VERSION = 1

SYMBOLS = (
    "vrl_int4_abi_version",
    "vrl_int4_error_string",
    "vrl_int4_gemv_bf16",
    "vrl_int4_dequant_bf16",
    "vrl_int4_gate_up_silu_bf16",
    "vrl_int4_prepacked_bytes",
    "vrl_int4_prepack",
    "vrl_int4_gemv_prepacked_bf16",
    "vrl_int4_gemv_prepacked_norm_bf16",
    "vrl_int4_gemv_prepacked_epilogue_bf16",
    "vrl_int4_grouped_plan_size",
    "vrl_int4_grouped_plan_build",
    "vrl_int4_gemv_grouped_bf16",
    "vrl_cfg_sample_bf16",
    "vrl_int4_head_sample_workspace_bytes",
    "vrl_int4_head_sample_bf16",
    "vrl_int4_head_sample_ex_bf16",
    "vrl_int4_head_sample_static_bf16",
    "vrl_add_rmsnorm_bf16",
    "vrl_rope_attn_decode_bf16",
    "vrl_rope_attn_decode_rows_bf16",
    "vrl_rope_attn_decode_split_workspace_bytes",
    "vrl_rope_attn_decode_split_bf16",
    "vrl_rope_attn_decode_lora_bf16",
    "vrl_lora_down_bf16",
    "vrl_lora_up_add_bf16",
    "vrl_int4_gemv_prepacked_lora_bf16",
    "vrl_int4_gemv_prepacked_lora_up_bf16",
    "vrl_decode_run_calls",
    "vrl_int4_gemv_prepacked_norm_lora_bf16",
)


class StepCall(ctypes.Structure):
    """Mirror of ``vrl_step_call`` (include/vrl_decode.h): one call of a decode step's launch list."""

    _fields_ = [("kind", ctypes.c_int32), ("reserved", ctypes.c_int32), ("p", ctypes.c_void_p * 12),
                ("i", ctypes.c_int64 * 8), ("f", ctypes.c_float * 2)]


# vrl_step_call.kind of the entry points a launch list may hold
STEP_CALL_KINDS = {
    "vrl_int4_gemv_prepacked_bf16": 1, "vrl_int4_gemv_prepacked_norm_bf16": 2,
    "vrl_int4_gemv_prepacked_epilogue_bf16": 3, "vrl_int4_gemv_prepacked_lora_bf16": 4,
    "vrl_int4_gemv_prepacked_lora_up_bf16": 5, "vrl_add_rmsnorm_bf16": 6, "vrl_rope_attn_decode_bf16": 7,
    "vrl_rope_attn_decode_split_bf16": 8, "vrl_rope_attn_decode_rows_bf16": 9,
    "vrl_rope_attn_decode_lora_bf16": 10, "vrl_lora_down_bf16": 11, "vrl_lora_up_add_bf16": 12,
    "vrl_int4_gemv_prepacked_norm_lora_bf16": 13,
}


def step_calls(calls) -> "ctypes.Array":
    """``[(library function, arguments without the stream), ...]`` as an array of ``vrl_step_call`` records:
    every argument goes to the slot list of its declared type, in order (pointers, integers, floats).  The
    objects the arguments refer to must be kept alive by the caller."""
    table = (StepCall * len(calls))()
    for rec, (fn, args) in zip(table, calls):
        if len(args) != len(fn.argtypes) - 1:
            raise ValueError(f"{fn.__name__} takes {len(fn.argtypes) - 1} arguments before the stream")
        rec.kind = STEP_CALL_KINDS[fn.__name__]
        n_p = n_i = n_f = 0
        for kind, value in zip(fn.argtypes[:-1], args):
            if kind is ctypes.c_float:
                rec.f[n_f] = float(value)
                n_f += 1
            elif kind in (ctypes.c_int, ctypes.c_size_t, ctypes.c_int64):
                rec.i[n_i] = int(value)
                n_i += 1
            else:   # c_void_p or a typed pointer: an address, None, a ctypes object or a byref() of one
                if value is None:
                    address = None
                elif isinstance(value, int):
                    address = value
                else:
                    address = ctypes.addressof(getattr(value, "_obj", value))
                rec.p[n_p] = address
                n_p += 1
    return table


class Int4LibraryError(RuntimeError):
    """The HIP library is missing, stale, or returned an error code."""


class Problem(ctypes.Structure):
    """Mirror of ``vrl_int4_problem``."""

    _fields_ = [
        ("x", ctypes.c_void_p),
        ("qweight", ctypes.c_void_p),
        ("scales", ctypes.c_void_p),
        ("qzeros", ctypes.c_void_p),
        ("y", ctypes.c_void_p),
        ("M", ctypes.c_int32),
        ("N", ctypes.c_int32),
        ("K", ctypes.c_int32),
        ("G", ctypes.c_int32),
        ("fused_gate_up", ctypes.c_int32),
        ("prepacked", ctypes.c_int32),
        ("reserved", ctypes.c_int32 * 2),
    ]


class Norm(ctypes.Structure):
    """Mirror of ``vrl_int4_norm``."""

    _fields_ = [
        ("x", ctypes.c_void_p),
        ("residual", ctypes.c_void_p),
        ("weight", ctypes.c_void_p),
        ("h_out", ctypes.c_void_p),
        ("eps", ctypes.c_float),
        ("reserved", ctypes.c_int32),
    ]


class Epilogue(ctypes.Structure):
    """Mirror of ``vrl_int4_epilogue``."""

    _fields_ = [
        ("bias", ctypes.c_void_p),
        ("residual", ctypes.c_void_p),
        ("activation", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


ACT_NONE, ACT_GELU = 0, 1


class HeadExtras(ctypes.Structure):
    """Mirror of ``vrl_int4_head_extras``."""

    _fields_ = [
        ("bias", ctypes.c_void_p),
        ("embed_table", ctypes.c_void_p),
        ("next_embeds", ctypes.c_void_p),
        ("tokens", ctypes.c_void_p),
        ("logprobs", ctypes.c_void_p),
        ("position", ctypes.c_void_p),
        ("slot", ctypes.c_void_p),
        ("embed_dim", ctypes.c_int32),
        ("token_stride", ctypes.c_int32),
        ("active", ctypes.c_void_p),
        ("position_per_row", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


class LoraAdapter(ctypes.Structure):
    """Mirror of ``vrl_lora_adapter``."""

    _fields_ = [
        ("A", ctypes.c_void_p),
        ("B", ctypes.c_void_p),
        ("y", ctypes.c_void_p),
        ("N", ctypes.c_int32),
        ("r", ctypes.c_int32),
        ("scaling", ctypes.c_float),
        ("weights_fp32", ctypes.c_int32),
    ]


class AttnLora(ctypes.Structure):
    """Mirror of ``vrl_attn_lora``."""

    _fields_ = [
        ("t", ctypes.c_void_p),
        ("t_stride", ctypes.c_int32),
        ("weights_fp32", ctypes.c_int32),
        ("q_B", ctypes.c_void_p),
        ("k_B", ctypes.c_void_p),
        ("v_B", ctypes.c_void_p),
        ("r", ctypes.c_int32 * 3),
        ("offset", ctypes.c_int32 * 3),
        ("scaling", ctypes.c_float * 3),
        ("position_per_row", ctypes.c_int32),
        ("o_A", ctypes.c_void_p),
        ("o_t", ctypes.c_void_p),
        ("o_r", ctypes.c_int32),
        ("reserved2", ctypes.c_int32),
    ]


class PlanInfo(ctypes.Structure):
    """Mirror of ``vrl_int4_plan_info``."""

    _fields_ = [
        ("n_problems", ctypes.c_int32),
        ("total_tiles", ctypes.c_int32),
        ("grid", ctypes.c_int32),
        ("block_threads", ctypes.c_int32),
        ("lds_bytes", ctypes.c_int32),
        ("variant", ctypes.c_int32),
        ("reserved", ctypes.c_int32 * 2),
    ]


_lock = threading.Lock()
_lib = None


def _bind(lib):
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.vrl_int4_abi_version.restype = ci
    lib.vrl_int4_abi_version.argtypes = []
    lib.vrl_int4_error_string.restype = ctypes.c_char_p
    lib.vrl_int4_error_string.argtypes = [ci]
    lib.vrl_int4_gemv_bf16.restype = ci
    lib.vrl_int4_gemv_bf16.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, vp]
    lib.vrl_int4_dequant_bf16.restype = ci
    lib.vrl_int4_dequant_bf16.argtypes = [vp, vp, vp, vp, ci, ci, ci, vp]
    lib.vrl_int4_gate_up_silu_bf16.restype = ci
    lib.vrl_int4_gate_up_silu_bf16.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, vp]
    lib.vrl_int4_prepacked_bytes.restype = ctypes.c_size_t
    lib.vrl_int4_prepacked_bytes.argtypes = [ci, ci, ci]
    lib.vrl_int4_prepack.restype = ci
    lib.vrl_int4_prepack.argtypes = [vp, vp, vp, vp, ci, ci, ci, vp]
    lib.vrl_int4_gemv_prepacked_bf16.restype = ci
    lib.vrl_int4_gemv_prepacked_bf16.argtypes = [ctypes.POINTER(Problem), ci, vp]
    lib.vrl_int4_gemv_prepacked_norm_bf16.restype = ci
    lib.vrl_int4_gemv_prepacked_norm_bf16.argtypes = [ctypes.POINTER(Problem), ci, ctypes.POINTER(Norm), vp]
    lib.vrl_int4_grouped_plan_size.restype = ctypes.c_size_t
    lib.vrl_int4_grouped_plan_size.argtypes = [ci]
    lib.vrl_int4_grouped_plan_build.restype = ci
    lib.vrl_int4_grouped_plan_build.argtypes = [
        ctypes.POINTER(Problem), ci, vp, ctypes.c_size_t, ctypes.POINTER(PlanInfo)]
    lib.vrl_int4_gemv_grouped_bf16.restype = ci
    lib.vrl_int4_gemv_grouped_bf16.argtypes = [vp, ctypes.POINTER(PlanInfo), vp]
    lib.vrl_cfg_sample_bf16.restype = ci
    lib.vrl_cfg_sample_bf16.argtypes = [vp, vp, vp, vp, ci, ci, ctypes.c_float, ctypes.c_float, vp]
    lib.vrl_int4_head_sample_workspace_bytes.restype = ctypes.c_size_t
    lib.vrl_int4_head_sample_workspace_bytes.argtypes = [ci, ci]
    lib.vrl_int4_head_sample_bf16.restype = ci
    lib.vrl_int4_head_sample_bf16.argtypes = [ctypes.POINTER(Problem), vp, vp, vp, ci, ctypes.c_float,
                                              ctypes.c_float, vp, ctypes.c_size_t, vp]
    lib.vrl_int4_head_sample_ex_bf16.restype = ci
    lib.vrl_int4_head_sample_ex_bf16.argtypes = [ctypes.POINTER(Problem), ctypes.POINTER(HeadExtras), vp, vp, vp, ci,
                                                 ctypes.c_float, ctypes.c_float, vp, ctypes.c_size_t, vp]
    lib.vrl_int4_gemv_prepacked_epilogue_bf16.restype = ci
    lib.vrl_int4_gemv_prepacked_epilogue_bf16.argtypes = [ctypes.POINTER(Problem), ctypes.POINTER(Norm),
                                                          ctypes.POINTER(Epilogue), vp]
    lib.vrl_int4_head_sample_static_bf16.restype = ci
    lib.vrl_int4_head_sample_static_bf16.argtypes = [ctypes.POINTER(Problem), vp, vp, vp, ci, ctypes.c_float,
                                                     ctypes.c_float, vp]
    lib.vrl_add_rmsnorm_bf16.restype = ci
    lib.vrl_add_rmsnorm_bf16.argtypes = [vp, vp, vp, vp, vp, ci, ci, ctypes.c_float, vp]
    lib.vrl_rope_attn_decode_lora_bf16.restype = ci
    lib.vrl_rope_attn_decode_lora_bf16.argtypes = [vp, vp, vp, ci, ci, vp, vp, vp, vp, vp, vp, vp,
                                                   ci, ci, ci, ci, ci, ctypes.c_float,
                                                   ctypes.POINTER(AttnLora), vp]
    lib.vrl_lora_down_bf16.restype = ci
    lib.vrl_lora_down_bf16.argtypes = [vp, ci, ci, ctypes.POINTER(LoraAdapter), ci, vp, vp]
    lib.vrl_int4_gemv_prepacked_lora_bf16.restype = ci
    lib.vrl_int4_gemv_prepacked_lora_bf16.argtypes = [ctypes.POINTER(Problem), ci, ctypes.POINTER(LoraAdapter), ci, vp, vp]
    lib.vrl_int4_gemv_prepacked_lora_up_bf16.restype = ci
    lib.vrl_int4_gemv_prepacked_lora_up_bf16.argtypes = [ctypes.POINTER(Problem), ctypes.POINTER(LoraAdapter), vp, ci, vp]
    lib.vrl_lora_up_add_bf16.restype = ci
    lib.vrl_lora_up_add_bf16.argtypes = [vp, ci, ci, ctypes.POINTER(LoraAdapter), ci, vp]
    lib.vrl_rope_attn_decode_bf16.restype = ci
    lib.vrl_rope_attn_decode_bf16.argtypes = [vp, vp, vp, ci, ci, vp, vp, vp, vp, vp, vp, vp,
                                              ci, ci, ci, ci, ci, ctypes.c_float, vp]
    lib.vrl_rope_attn_decode_rows_bf16.restype = ci
    lib.vrl_rope_attn_decode_rows_bf16.argtypes = [vp, vp, vp, ci, ci, vp, vp, vp, vp, vp, vp, vp,
                                                   ci, ci, ci, ci, ci, ctypes.c_float, vp, ctypes.c_size_t, vp]
    lib.vrl_rope_attn_decode_split_workspace_bytes.restype = ctypes.c_size_t
    lib.vrl_int4_gemv_prepacked_norm_lora_bf16.restype = ci
    lib.vrl_int4_gemv_prepacked_norm_lora_bf16.argtypes = [ctypes.POINTER(Problem), ci, ctypes.POINTER(Norm),
                                                           ctypes.POINTER(LoraAdapter), ci, vp, vp]
    lib.vrl_decode_run_calls.argtypes = [ctypes.POINTER(StepCall), ci, ctypes.POINTER(ctypes.c_int), vp]
    lib.vrl_decode_run_calls.restype = ci
    lib.vrl_rope_attn_decode_split_workspace_bytes.argtypes = [ci, ci, ci]
    lib.vrl_rope_attn_decode_split_bf16.restype = ci
    lib.vrl_rope_attn_decode_split_bf16.argtypes = [vp, vp, vp, ci, ci, vp, vp, vp, vp, vp, vp, vp,
                                                    ci, ci, ci, ci, ci, ctypes.c_float, vp, ctypes.c_size_t, vp]


def load():
    """Return the loaded library, raising ``Int4LibraryError`` if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise Int4LibraryError(
                    f"{LIB_PATH} is missing: build it with `python -m visionrl_amd.build` "
                    "(there is no CPU or PyTorch fallback for the int4 operators)")
            try:
                lib = ctypes.CDLL(LIB_PATH)
            except OSError as exc:
                raise Int4LibraryError(f"cannot load {LIB_PATH}: {exc}") from exc
            for name in SYMBOLS:
                if not hasattr(lib, name):
                    raise Int4LibraryError(f"{LIB_PATH} does not export {name}")
            _bind(lib)
            got = lib.vrl_int4_abi_version()
            if got != ABI_VERSION:
                raise Int4LibraryError(f"{LIB_PATH} has ABI {got}, this package needs {ABI_VERSION}")
            _lib = lib
    return _lib


def error_string(code: int) -> str:
    return load().vrl_int4_error_string(int(code)).decode()


def check(code: int, what: str) -> None:
    """Turn a non-zero return code into a Python exception.

    Precondition violations (codes >= 1000) are the caller's mistake and raise
    ``ValueError``; HIP launch failures raise ``Int4LibraryError``.
    """
    if code == 0:
        return
    msg = f"{what}: {error_string(code)} (code {code})"
    if code >= 1000:
        raise ValueError(msg)
    raise Int4LibraryError(msg)
