"""ctypes binding of the C ABI declared in ``include/msa_amd.h``.

There is no fallback: if the HIP library is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("MSA_AMD_LIB", os.path.join(HERE, "libmsa_amd.so"))   # override: an alternative build

MSA_BF16, MSA_F32 = 0, 1
MODE_COSINE, MODE_SCALED_DOT = 0, 1

_vp, _i32, _i64, _f32, _sz = C.c_void_p, C.c_int32, C.c_int64, C.c_float, C.c_size_t

# name -> (restype, argtypes); mirrors include/msa_amd.h one to one
SIGNATURES = {
    "msa_last_error": (C.c_char_p, []),
    "msa_abi_version": (C.c_int, []),
    "msa_chunk_table": (C.c_int, [_vp, _i32, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "msa_pool_chunks": (C.c_int, [_vp, _vp, _vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i32,
                                  _i32, _i32, _vp, _vp, _vp, _vp]),
    "msa_bank_create": (C.c_int, [C.POINTER(_vp), _i32, _i64, _i32, _i32, _i32, _vp, _vp, _i64]),
    "msa_bank_set_layer": (C.c_int, [_vp, _i32, _vp, _vp, _vp]),
    "msa_bank_destroy": (C.c_int, [_vp]),
    "msa_route_workspace_bytes": (_sz, [_i32, _i32, _i32, _i32, _i32, _i64, _i64, _i32]),
    "msa_route_topk_workspace_bytes": (_sz, [_i32, _i32, _i32, _i32, _i32, _i64, _i32]),
    "msa_chunk_scores": (C.c_int, [_vp, _i32, _vp, _vp, _i32, _i32, _i32, _i32, _f32, _vp, _vp, _sz, _vp]),
    "msa_route_topk": (C.c_int, [_vp, _i32, _vp, _vp, _i32, _i32, _i32, _i32, _f32, _i32, _vp, _vp, _vp, _vp, _sz,
                                 _vp]),
    "msa_route_topk_reduce": (C.c_int, [_vp, _i32, _vp, _vp, _i32, _i32, _i32, _i32, _f32, _i32, _i32, _i32, _vp, _vp, _vp,
                                        _vp, _sz, _vp]),
    "msa_route_topk_static": (C.c_int, [_vp, _i32, _vp, _vp, _i32, _i32, _i32, _i32, _f32, _i32, _vp, _vp, _vp, _vp]),
    "msa_profile_enable": (C.c_int, [_i32]),
    "msa_profile_collect": (C.c_int, [_vp, _i32, _vp]),
    "msa_diag_mfma_loop": (C.c_int, [_i32, _i32, _i32, _vp, _vp, _vp]),
    "msa_diag_fill_lds": (C.c_int, [C.c_uint32, _vp, _i32, _vp]),
    "msa_diag_read_stream": (C.c_int, [_vp, C.c_int64, _vp, _i32, _vp]),
    "msa_diag_scan_walk": (C.c_int, [_i32, _i32, _i32, _i32, _i32, _vp]),
    "msa_route_set_tile_pool": (C.c_int, [_i32]),
    "msa_gather_plan": (C.c_int, [_vp, _vp, _i32, _i32, _vp]),
    "msa_gather_kv": (C.c_int, [_vp, _i32, _vp, _i32, _i32, _vp, _vp, _i64, _vp]),
    "msa_gather_device_workspace_bytes": (_sz, [_i32, _i32]),
    "msa_gather_kv_device": (C.c_int, [_vp, _i32, _vp, _i32, _i32, _vp, _vp, _i64, _vp, _vp, _sz, _vp]),
    "msa_route_topk_gather": (C.c_int, [_vp, _i32, _vp, _vp, _i32, _i32, _i32, _i32, _f32, _i32, _vp, _vp, _vp, _vp, _sz,
                                        _i32, _vp, _i32, _i32, _vp, _vp, _i64, _vp, _vp, _sz, _vp]),
    "msa_assemble_context": (C.c_int, [_vp, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp,
                                       _vp, _i32, _vp, _vp]),
    "msa_cache_append": (C.c_int, [_vp, _vp, _i32, _i32, _i32, _i32, _vp, _vp, _i32, _vp, _vp]),
    "msa_cache_append_rows": (C.c_int, [_vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _i32, _vp, _vp]),
    "msa_attn_workspace_bytes": (_sz, [_i32, _i32, _i32, _i32, _i32]),
    "msa_flash_attn": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp, _vp]),
    "msa_flash_set_form": (C.c_int, [_i32]),
    "msa_diag_asm_kernel_resources": (C.c_int, [_i32, _vp, _vp]),
    "msa_flash_attn_hint": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp, _i32, _vp]),
    "msa_qk_norm_rope": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _f32, _vp, _vp, _i32, _i32, _i64, _i32,
                                   _i32, _i32, _vp, _vp, _vp, _vp]),
    "msa_qkv_proj": (C.c_int, [_vp, _i64, _i32, _vp, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _f32, _vp, _vp, _i32, _vp, _vp, _vp,
                               _vp, _vp]),
    "msa_qk_norm_rope_append": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _f32, _vp, _vp, _i32, _i32, _i32,
                                          _i32, _i32, _i32, _vp, _vp, _vp, _i32, _vp, _vp]),
    "msa_rmsnorm": (C.c_int, [_vp, _vp, _vp, _i32, _i64, _i32, _f32, _vp, _vp]),
    "msa_silu_mul": (C.c_int, [_vp, _i32, _i64, _i32, _vp, _vp]),
    "msa_decode_attn_fused": (C.c_int, [_vp, _i64, _vp, _vp, _vp, _f32, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp,
                                        _i32, _vp, _f32, _vp, _vp, _sz, _vp]),
    "msa_greedy_sample": (C.c_int, [_vp, _i32, _i32, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _i32, _vp]),
    "msa_skinny_linear": (C.c_int, [_vp, _vp, _vp, _vp, _f32, _i32, _i32, _i32, _i32, _i32, _vp, _vp]),
    "msa_skinny_linear_workspace_bytes": (_sz, [_i32, _i32, _i32]),
    "msa_skinny_linear_ws": (C.c_int, [_vp, _vp, _vp, _vp, _f32, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _sz, _vp]),
    "msa_sparse_attn": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32,
                                  _i32, _vp, _vp, _sz, _vp]),
}


class MsaError(RuntimeError):
    def __init__(self, code: int, where: str, message: str):
        super().__init__(f"{where} failed with code {code}: {message}")
        self.code = code


_lib: Optional[C.CDLL] = None


def load() -> C.CDLL:
    """Loads the library and declares every entry point; raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `python -m msa_amd.build` "
                          "(there is no CPU or PyTorch fallback for this path)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the library lacks a declared symbol
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


def check(code: int, where: str) -> None:
    if code != 0:
        raise MsaError(code, where, load().msa_last_error().decode("utf-8", "replace"))


def ptr(t) -> Optional[int]:
    """Device/host address of a torch tensor (None passes NULL)."""
    return None if t is None else t.data_ptr()


def dtype_code(torch_dtype) -> int:
    import torch
    if torch_dtype == torch.bfloat16:
        return MSA_BF16
    if torch_dtype == torch.float32:
        return MSA_F32
    raise TypeError(f"unsupported dtype {torch_dtype}: the kernels take bfloat16 or float32")
