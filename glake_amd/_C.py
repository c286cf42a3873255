"""ctypes binding of ``libvtkv.so`` (declared in ``include/vtkv.h``).

The library is loaded from ``glake_amd/lib``; importing this module never builds anything.
If the shared object is missing, every access raises ``VtkvLibraryMissing`` - there is no
fallback implementation.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# VTKV_LIBRARY_PATH selects another build of the same library (e.g. a tuning variant)
LIB_PATH = os.environ.get("VTKV_LIBRARY_PATH") or os.path.join(_HERE, "lib", "libvtkv.so")

F32, BF16, F16, FP8_E4M3 = 0, 1, 2, 3
D2H, H2D, D2D = 0, 1, 2
OK, EINVAL, EHIP, ENOMEM, ESTATE = 0, -1, -2, -3, -4


class VtkvLibraryMissing(RuntimeError):
    pass


class VtkvError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"vtkv error {code}: {message}")
        self.code = code


class VtkvOutOfChunks(VtkvError):
    """The physical chunk pool (or a caller-provided workspace) is too small."""


_i, _i64, _f, _p, _u64 = C.c_int, C.c_int64, C.c_float, C.c_void_p, C.c_uint64

# name -> (restype, argtypes): mirrors include/vtkv.h one to one
SIGNATURES = {
    "vtkv_last_error": (C.c_char_p, []),
    "vtkv_version": (_i, []),
    "vtkv_chunk_bytes": (_i64, []),
    "vtkv_pool_set_chunk_bytes": (_i, [_i64]),
    "vtkv_pool_init": (_i, [_i, _i64]),
    "vtkv_pool_free_chunks": (_i64, []),
    "vtkv_pool_total_chunks": (_i64, []),
    "vtkv_pool_retired_chunks": (_i64, []),
    "vtkv_pool_recreated_chunks": (_i64, []),
    "vtkv_pool_trim": (_i64, [_i64]),
    "vtkv_pool_destroy": (_i, []),
    "vtkv_seg_create": (_p, [_i, _i64, _i64, _i]),
    "vtkv_seg_destroy": (_i, [_p]),
    "vtkv_seg_key_ptr": (_u64, [_p, _i]),
    "vtkv_seg_value_ptr": (_u64, [_p, _i]),
    "vtkv_seg_value_skew": (_i64, [_p]),
    "vtkv_seg_set_value_skew": (_i, [_p, _i64]),
    "vtkv_seg_get_used": (_i64, [_p]),
    "vtkv_seg_set_used": (_i, [_p, _i64]),
    "vtkv_seg_mapped_bytes": (_i64, [_p]),
    "vtkv_seg_expand": (_i, [_p, _i]),
    "vtkv_seg_reserve": (_i, [_p, _i64, _i64]),
    "vtkv_seg_ensure": (_i, [_p, _i64]),
    "vtkv_seg_preempt": (_i, [_p]),
    "vtkv_seg_release": (_i, [_p]),
    "vtkv_seg_share_prefix": (_i, [_p, _p, _i64, _p]),
    "vtkv_pool_shared_chunks": (_i64, []),
    "vtkv_seg_eager_extend": (_i, [_p, _i]),
    "vtkv_map_ahead_batch": (_i, [_p, _i, _i64]),
    "vtkv_seg_pending": (_i, [_p]),
    "vtkv_map_ahead_wait": (_i, []),
    "vtkv_extend_kv_cache_batch": (_i, [_p, _i, _p, _p, _i64, _i, _p]),
    "vtkv_ptr_table_create": (_u64, [_i]),
    "vtkv_ptr_table_destroy": (_i, [_u64]),
    "vtkv_ptr_table_set": (_i, [_u64, _i, _u64]),
    "vtkv_ptr_table_fill": (_i, [_u64, _p, _i, _i, _i]),
    "vtkv_memcpy_h2d": (_i, [_u64, _p, _i64]),
    "vtkv_memcpy_d2h": (_i, [_p, _u64, _i64]),
    "vtkv_memcpy_h2d_async": (_i, [_u64, _p, _i64, _p]),
    "vtkv_reshape_and_cache": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _i64, _i, _i, _f, _f, _p]),
    "vtkv_reshape_and_cache_paged": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _i64, _i, _p]),
    "vtkv_swap_blocks": (_i, [_p, _p, _i64, _p, _i, _i, _p]),
    "vtkv_swap_ranges": (_i, [_p, _p, _p, _i, _i, _i64, _i, _p]),
    "vtkv_host_alloc": (_p, [_i64]),
    "vtkv_host_free": (_i, [_p]),
    "vtkv_copy_blocks": (_i, [_p, _p, _i, _p, _i, _i64, _p]),
    "vtkv_reshape_and_cache_flash": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _i64, _i64, _i, _p]),
    "vtkv_convert_fp8": (_i, [_p, _p, _i64, _f, _i, _i, _p]),
    "vtkv_decode_attention_workspace_bytes": (_i64, [_i, _i, _i, _i, _i]),
    "vtkv_decode_attention": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _f, _i, _p, _i, _i, _i, _f, _f, _p,
                                    _i64, _i, _p]),
    "vtkv_decode_attention_noalloc_max_bytes": (_i64, []),
    "vtkv_decode_attention_noalloc": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _f, _i, _p, _i, _i, _i, _f, _f,
                                            _p]),
    "vtkv_decode_attention_v2_workspace_bytes": (_i64, [_i, _i, _i, _i]),
    "vtkv_decode_attention_v2": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _f, _i, _i, _p, _i,
                                       _i, _i, _f, _f, _p, _i64, _p]),
    "vtkv_decode_append_attention": (_i, [_p, _p, _p, _p, _i64, _i64, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _f,
                                           _i, _p, _i, _i, _i, _f, _f, _p, _i64, _i, _p]),
    "vtkv_prefill_unit_tokens": (_i, [_i, _i, _i]),
    "vtkv_prefill_unit_tokens_for": (_i, [_i, _i, _i, _i]),
    "vtkv_prefill_attention": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _f, _i, _p, _i, _i, _i, _f, _f, _p]),
    "vtkv_set_fused_merge": (_i, [_i]),
    "vtkv_set_head_major": (_i, [_i]),
    "vtkv_set_kernel_timing": (_i, [_i]),
    "vtkv_attention_kernel_times": (_i, [_p, _p, _i]),
}

_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise VtkvLibraryMissing(
                f"{LIB_PATH} is missing: build it with `python -m glake_amd.build` (needs hipcc). "
                "glake_amd has no fallback implementation.")
        # PyTorch ships its own copy of the HIP runtime.  Loaded after this library, it comes in as a second
        # runtime beside the system's one, and a stream or allocation of the one means nothing to the other;
        # loaded first, the dynamic loader resolves this library's dependency to the copy already there.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def last_error() -> str:
    return lib().vtkv_last_error().decode()


def check(rc: int) -> int:
    """Raise on a negative return code, pass non-negative values through."""
    if rc < 0:
        msg = last_error()
        if rc == ENOMEM:
            raise VtkvOutOfChunks(rc, msg)
        raise VtkvError(rc, msg)
    return rc


def check_ptr(p, what: str):
    if not p:
        raise VtkvError(EINVAL, f"{what}: {last_error()}")
    return p
