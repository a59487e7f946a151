"""ctypes binding of ``libtybok_hip.so`` (the C ABI declared in ``include/tybok_hip.h``).

The library is loaded from ``tybok_amd/_lib/``; there is no fallback: if it is missing or an
entry point fails, a ``RuntimeError`` is raised (the reference's native helpers raise instead
of exiting too: tybok/policies/fastwam/kernels/coop_grid.h:20-27).
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_longlong, c_size_t, c_void_p

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_lib", "libtybok_hip.so")
_lib: ctypes.CDLL | None = None

# name -> (restype, argtypes); mirrors include/tybok_hip.h one to one
SIGNATURES: dict[str, tuple] = {
    "tk_version": (c_int, []),
    "tk_last_error": (c_char_p, []),
    "tk_device_cus": (c_int, []),
    "tk_workspace_bytes": (c_size_t, []),
    "tk_workspace_init": (c_int, [c_void_p, c_size_t, c_void_p]),
    "tk_fp8w_packed_bytes": (c_size_t, [c_int, c_int]),
    "tk_pack_fp8_weight": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "tk_pack_fp8_gate_up": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "tk_fp8w_gemm": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int,
         c_int, c_void_p, c_size_t, c_void_p],
    ),  # fmt: skip
    "tk_fp8w_gemm_static": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int,
         c_int, c_void_p],
    ),  # fmt: skip
    "tk_static_scratch_bytes": (c_size_t, []),
    "tk_fp8w_gated_ffn": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
         c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),  # fmt: skip
    "tk_fp8w_norm_gated_ffn": (
        c_int,
        [c_void_p, c_int, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),  # fmt: skip
    "tk_set_ffn_fusion": (c_int, [c_int]),
    "tk_set_handoff_spin": (c_int, [c_int]),
    "tk_workspace_handoff_error_offset": (c_size_t, []),
    "tk_quant_act_rows": (c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p]),
    "tk_w8a8_gemm": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
         c_void_p, c_size_t, c_void_p],
    ),  # fmt: skip
    "tk_w8a8_gated_ffn": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
         c_int, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),  # fmt: skip
    "tk_w8a8_ffn_layout": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "tk_bf16w_packed_bytes": (c_size_t, [c_int, c_int]),
    "tk_pack_bf16_weight": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "tk_bf16w_linear": (
        c_int,
        [c_void_p, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
         c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int,
         c_int, c_void_p, c_size_t, c_void_p],
    ),  # fmt: skip
    "tk_bf16w_dense": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
         c_int, c_void_p, c_size_t, c_void_p],
    ),  # fmt: skip
    "tk_f16w_dense": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
         c_int, c_void_p, c_size_t, c_void_p],
    ),  # fmt: skip
    "tk_bf16w_dense_rope": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                    c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "tk_bf16w_dense_vt": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_longlong, c_int, c_int, c_int,
                                  c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "tk_prefix_meta": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "tk_patchify_images": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_float, c_void_p, c_void_p]),
    "tk_patchify_images_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_float, c_void_p, c_void_p]),
    "tk_layer_norm_f16": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_int, c_void_p]),
    "tk_add_layer_norm_f16": (
        c_int,
        [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_int, c_void_p],
    ),
    "tk_attn_prepare_kv": (
        c_int,
        [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
         c_void_p],
    ),  # fmt: skip
    "tk_expert_tail": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float,
         c_int, c_int, c_int, c_void_p],
    ),  # fmt: skip
    "tk_expert_tail_embed": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float,
         c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_void_p],
    ),  # fmt: skip
    "tk_layer_norm": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_float, c_void_p, c_int, c_int, c_int, c_void_p]),
    "tk_expert_kv_project": (
        c_int,
        [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "tk_expert_kv_project_layers": (
        c_int,
        [c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "tk_expert_cross_attn_fused": (
        c_int,
        [c_void_p, c_int, c_void_p, c_float, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int,
         c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    ),  # fmt: skip
    "tk_batched_attn": (
        c_int,
        [c_void_p, c_longlong, c_int, c_int, c_void_p, c_longlong, c_int, c_int, c_void_p, c_longlong, c_int, c_int,
         c_void_p, c_longlong, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p, c_size_t, c_void_p],
    ),  # fmt: skip
    "tk_batched_transpose_v": (
        c_int,
        [c_void_p, c_longlong, c_int, c_int, c_void_p, c_longlong, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    ),  # fmt: skip
    "tk_add_layer_norm": (
        c_int,
        [c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_float, c_void_p, c_int, c_int, c_int, c_void_p],
    ),  # fmt: skip
    "tk_prefix_rows": (
        c_int,
        [c_void_p, c_int, c_int, c_float, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p],
    ),  # fmt: skip
    "tk_add_layer_norm_rows": (
        c_int,
        [c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_float, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    ),  # fmt: skip
    "tk_rms_norm_rows": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_int, c_void_p]),
    "tk_rope_rows": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "tk_expert_attn": (
        c_int,
        [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int,
         c_int, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
         c_int, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),  # fmt: skip
    "tk_debug_decode_fp8": (c_int, [c_void_p, c_void_p]),
    "tk_debug_stream_read": (c_int, [c_void_p, c_size_t, c_int, c_void_p, c_void_p]),
    "tk_debug_fp8w_gemm_cut": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
}


def library_path() -> str:
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    """The loaded library; raises ``RuntimeError`` when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build it with `python -m tybok_amd.csrc.build` "
                "(there is no CPU or torch fallback for the HIP kernels)"
            )
        handle = ctypes.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().tk_last_error()
        raise RuntimeError(f"{what} failed ({rc}): {msg.decode() if msg else 'unknown error'}")
