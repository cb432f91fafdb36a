"""ctypes binding of libmoe_mi355.so (the C ABI declared in include/moe_mi355.h).

The library is the only compute path of this package: if it is missing or cannot
be loaded, every operator raises.  There is no PyTorch or CPU fallback.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmoe_mi355.so")

c_void_p, c_int32, c_size_t, c_float, c_int64 = (ctypes.c_void_p, ctypes.c_int32, ctypes.c_size_t,
                                                 ctypes.c_float, ctypes.c_int64)


class RouterParams(ctypes.Structure):
    """struct moe_router_params."""
    _fields_ = [
        ("n_tokens", c_int32), ("hidden", c_int32), ("n_experts", c_int32), ("top_k", c_int32),
        ("n_group", c_int32), ("topk_group", c_int32), ("scoring", c_int32), ("method", c_int32),
        ("norm_topk_prob", c_int32), ("scale_mode", c_int32), ("logits_bf16", c_int32),
        ("weights_bf16", c_int32), ("norm_eps", c_float), ("routed_scaling_factor", c_float),
    ]


# name -> (restype, argtypes); every symbol include/moe_mi355.h declares
SIGNATURES = {
    "moe_last_error": (ctypes.c_char_p, []),
    "moe_version": (ctypes.c_char_p, []),
    "moe_router": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, ctypes.POINTER(RouterParams), c_void_p,
                                  c_void_p, c_void_p, c_void_p]),
    "moe_router_rmsnorm": (ctypes.c_int, [c_void_p, c_void_p, ctypes.c_float, c_void_p, c_void_p,
                                          ctypes.POINTER(RouterParams), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "moe_dispatch_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32]),
    "moe_dispatch": (ctypes.c_int, [c_void_p, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_size_t, c_void_p]),
    "moe_dispatch_static": (ctypes.c_int, [c_void_p, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p,
                                           c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p]),
    "moe_grouped_workspace_bytes": (c_size_t, [c_int32, c_int32]),
    "moe_grouped_swiglu_bf16": (ctypes.c_int, [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                               c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p,
                                               c_int32, c_void_p, c_size_t, c_void_p]),
    "moe_grouped_swiglu_w8a16": (ctypes.c_int, [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32,
                                                c_int32, c_void_p, c_void_p, c_int32, c_void_p, c_size_t, c_void_p]),
    "moe_dequant_fp8_block128": (ctypes.c_int, [c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_void_p]),
    "moe_combine": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32,
                                   c_int32, c_int32, c_void_p, c_void_p]),
    "moe_combine_residual": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32,
                                            c_int32, c_int32, c_int32, c_void_p, c_void_p]),
    "moe_rmsnorm": (ctypes.c_int, [c_void_p, c_void_p, ctypes.c_float, c_int32, c_int32, c_void_p, c_void_p]),
    "moe_arena_index_create": (ctypes.c_int, [ctypes.POINTER(c_void_p)]),
    "moe_arena_index_destroy": (ctypes.c_int, [c_void_p]),
    "moe_arena_index_add": (ctypes.c_int, [c_void_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int64, ctypes.c_int64,
                                           ctypes.POINTER(ctypes.c_int64), c_int32]),
    "moe_arena_index_parse": (ctypes.c_int, [c_void_p, c_size_t, ctypes.POINTER(c_void_p)]),
    "moe_arena_index_wire_size": (c_size_t, [c_void_p]),
    "moe_arena_index_serialize": (ctypes.c_int, [c_void_p, c_void_p, c_size_t]),
    "moe_arena_index_n_modules": (c_int32, [c_void_p]),
    "moe_arena_index_module": (ctypes.c_int, [c_void_p, c_int32, ctypes.POINTER(ctypes.c_char_p),
                                              ctypes.POINTER(c_int32)]),
    "moe_arena_index_find": (ctypes.c_int, [c_void_p, ctypes.c_char_p]),
    "moe_arena_index_tensor": (ctypes.c_int, [c_void_p, c_int32, c_int32, ctypes.POINTER(ctypes.c_char_p),
                                              ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64),
                                              ctypes.POINTER(c_int32), ctypes.POINTER(ctypes.POINTER(ctypes.c_int64))]),
    "moe_stage_add_module_from_arena": (ctypes.c_int, [c_void_p, c_int32, c_void_p, ctypes.c_char_p, c_void_p, c_size_t,
                                                       c_int32, ctypes.POINTER(ctypes.c_char_p),
                                                       ctypes.POINTER(c_size_t)]),
    "moe_stage_add_module_from_segment": (ctypes.c_int, [c_void_p, c_int32, c_void_p, ctypes.c_char_p, c_void_p, c_size_t,
                                                         c_int32, ctypes.POINTER(ctypes.c_char_p),
                                                         ctypes.POINTER(c_size_t)]),
    "moe_write_words": (ctypes.c_int, [c_void_p, ctypes.POINTER(ctypes.c_uint64), c_int32, c_void_p]),
    "moe_stage_set_bounce": (ctypes.c_int, [c_void_p, c_int32, c_size_t, c_int32]),
    "moe_stage_add_module_pageable": (ctypes.c_int, [c_void_p, c_int32, c_int32, ctypes.POINTER(c_void_p),
                                                     ctypes.POINTER(c_size_t), ctypes.POINTER(c_size_t)]),
    "moe_stage_create": (ctypes.c_int, [ctypes.POINTER(c_void_p), c_int32, ctypes.POINTER(c_size_t),
                                        ctypes.POINTER(c_int32), ctypes.POINTER(c_void_p), c_int32]),
    "moe_stage_set_policy": (ctypes.c_int, [c_void_p, c_int32, c_int32]),
    "moe_stage_fetch": (ctypes.c_int, [c_void_p, ctypes.POINTER(c_int32), c_int32, ctypes.POINTER(c_int32)]),
    "moe_stage_add_module": (ctypes.c_int, [c_void_p, c_int32, c_int32, ctypes.POINTER(c_void_p),
                                            ctypes.POINTER(c_size_t), ctypes.POINTER(c_size_t)]),
    "moe_stage_pump": (ctypes.c_int, [c_void_p]),
    "moe_stage_acquire": (ctypes.c_int, [c_void_p, c_int32, c_void_p, ctypes.POINTER(c_int32)]),
    "moe_stage_release": (ctypes.c_int, [c_void_p, c_int32, c_void_p]),
    "moe_stage_resident": (ctypes.c_int, [c_void_p, c_int32]),
    "moe_stage_set_active_slots": (ctypes.c_int, [c_void_p, c_int32, c_int32, c_int32]),
    "moe_stage_set_model": (ctypes.c_int, [c_void_p, ctypes.c_char_p, c_int32, c_int32]),
    "moe_stage_tag_module": (ctypes.c_int, [c_void_p, c_int32, c_int32, c_int32]),
    "moe_stage_clear_expert_buffer": (ctypes.c_int, [c_void_p, c_int32, c_int32, c_void_p]),
    "moe_stage_set_phase_slots": (ctypes.c_int, [c_void_p, c_int32, c_int32, c_int32]),
    "moe_stage_set_phase": (ctypes.c_int, [c_void_p, ctypes.c_char_p]),
    "moe_stage_reset_prefill_buffer": (ctypes.c_int, [c_void_p]),
    "moe_stage_reset_weight_copy_queue": (ctypes.c_int, [c_void_p]),
    "moe_stage_stats": (ctypes.c_int, [c_void_p, ctypes.POINTER(c_int64), ctypes.POINTER(c_int64)]),
    "moe_stage_sync": (ctypes.c_int, [c_void_p]),
    "moe_stage_destroy": (ctypes.c_int, [c_void_p]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """Load libmoe_mi355.so (built by `make -C moe_gen_amd/csrc` or __graft_entry__.build())."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
                "(hipcc --offload-arch=gfx950). This package has no other compute path.")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error() -> str:
    return lib().moe_last_error().decode()


def check(rc: int, what: str) -> None:
    """Mirror of the reference's convention: native failure -> RuntimeError with the message."""
    if rc != 0:
        raise RuntimeError(f"{what} failed (status {rc}): {last_error()}")
