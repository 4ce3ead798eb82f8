"""ctypes binding of libanchor_attn_hip.so (the gfx950 kernels behind a C ABI, see
include/anchor_attn_hip.h).  There is no other backend: if the library is missing or a call
fails, this module raises."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_size_t, c_void_p

_LIB_NAME = "libanchor_attn_hip.so"
_lib = None

AA_SCALE_BF16_CHAIN = 0
AA_SCALE_FP32 = 1
AA_GEOMETRY_AS_RUN = 0    # stage-2 candidates [block_size, bb*S - block_size): what the reference's operator does
AA_GEOMETRY_INTENDED = 1  # [S, bb*S): no double-counted keys, no never-attended gap (analysis only)
AA_DTYPE_BF16 = 0
AA_DTYPE_F16 = 1
AA_STATIC_SCRATCH_BYTES = 40 * 1024 * 1024  # capacity of the library's static stage-2 scratch (aa_stage2_select_static)


class AnchorAttnHipError(RuntimeError):
    pass


def library_path() -> str:
    """The in-tree build; ANCHOR_ATTN_HIP_LIB may point at another build of the same library."""
    return os.environ.get("ANCHOR_ATTN_HIP_LIB") or os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)


_T3 = [c_void_p, c_int64, c_int64, c_int64]  # pointer + (batch, head, row) element strides
_DIMS5 = [c_int, c_int, c_int, c_int, c_int]  # batch, n_q_heads, n_kv_heads, n_ctx, head_dim

_SIGNATURES = {
    "aa_version": (c_int, []),
    "aa_last_error": (c_char_p, []),
    "aa_coords_entries_per_head": (c_int64, [c_int, c_int, c_int]),
    "aa_coords_offset": (c_int64, [c_int, c_int, c_int]),
    "aa_mask_words": (c_int64, [c_int, c_int, c_int, c_int, c_int]),
    "aa_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    # (every compute entry point ends with: ..., int dtype, void* stream)
    "aa_stage1_anchor_fwd": (c_int, _T3 * 3 + [c_void_p] * 3 + _DIMS5 + [c_int, c_int, c_float, c_int, c_int, c_void_p]),
    "aa_pool_q_anchor": (c_int, _T3 + [c_void_p] * 3 + [c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "aa_stage2_select": (c_int, [c_void_p, c_void_p] + _T3 + [c_void_p] * 3 + _DIMS5 + [c_int, c_int, c_double, c_float, c_int, c_int, c_void_p]),
    "aa_stage2_select_static": (c_int, [c_void_p, c_void_p] + _T3 + [c_void_p] * 2 + _DIMS5 + [c_int, c_int, c_double, c_float, c_int, c_int, c_void_p]),
    "aa_stage3_sparse_fwd": (c_int, _T3 * 3 + [c_void_p] * 5 + _T3 + _DIMS5 + [c_int, c_int, c_float, c_int, c_void_p]),
    "aa_anchor_attn_fwd": (c_int, _T3 * 4 + [c_void_p, c_size_t, c_void_p] + _DIMS5 + [c_int, c_int, c_double, c_float, c_int, c_int, c_int, c_void_p]),
    "aa_dense_causal_fwd": (c_int, _T3 * 4 + _DIMS5 + [c_float, c_int, c_void_p]),
}

EXPORTS = tuple(_SIGNATURES)


def lib() -> ctypes.CDLL:
    """Load the library once.  Raises if it has not been built (python __graft_entry__.py or
    `make -C anchor-attention_amd/csrc`)."""
    global _lib
    if _lib is None:
        path = library_path()
        if not os.path.exists(path):
            raise AnchorAttnHipError(
                f"{path} is missing: build it with `make -C anchor-attention_amd/csrc` "
                "(there is no fallback implementation)"
            )
        handle = bind(path)
        version = handle.aa_version()
        if version >= 1000:
            raise AnchorAttnHipError(f"{path} is a timing-only build (aa_version() = {version}) that leaves part of a "
                                     "kernel out; it computes wrong results and is not loaded as the operator")
        _lib = handle
    return _lib


def bind(path: str) -> ctypes.CDLL:
    """Open a build of the library and declare the C signatures on it (no check of what kind of build it is)."""
    handle = ctypes.CDLL(path)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(handle, name)
        fn.restype = res
        fn.argtypes = args
    return handle


def check(rc: int) -> None:
    if rc != 0:
        msg = lib().aa_last_error().decode("utf-8", "replace")
        raise AnchorAttnHipError(f"anchor_attn HIP library error {rc}: {msg}")


def dtype_code(t) -> int:
    """AA_DTYPE_* of a tensor; anything but bf16 and fp16 raises (the reference silently treats other types as fp16)."""
    import torch
    if t.dtype == torch.bfloat16:
        return AA_DTYPE_BF16
    if t.dtype == torch.float16:
        return AA_DTYPE_F16
    raise AssertionError(f"anchor_attn kernels take bf16 or fp16 tensors, not {t.dtype}")


def t3(t):
    """(data_ptr, stride_b, stride_h, stride_n) of a [B,H,N,D] tensor whose last stride is 1."""
    assert t.dim() == 4 and t.stride(3) == 1
    return (t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))
