"""ctypes bindings of the two compiled libraries.

``hip_lib()`` is the kernel library; it refuses to load without a GPU build and raises
:class:`KernelLibraryError` instead of falling back to anything.  ``host_lib()`` is the
allocator library, which needs no GPU.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import c_char_p, c_float, c_int, c_longlong, c_uint, c_void_p, POINTER

from . import build

_lock = threading.Lock()
_hip = None
_host = None


class KernelLibraryError(RuntimeError):
    """The HIP kernel library is missing or could not be loaded."""


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or failed to launch."""


P = c_void_p
I = c_int
F = c_float
LL = c_longlong
U = c_uint

_HIP_SIGNATURES = {
    "kva_embed_gather": [P, P, P, P, I, I, I, I, I, P],
    "kva_embed_gather_prep": [P, P, P, P, P, P, P, I, I, I, I, P],
    "kva_rmsnorm": [P, P, P, P, P, I, I, F, I, I, P, I, I, P],
    "kva_residual_add": [P, P, LL, I, P],
    "kva_scale_softcap": [P, LL, F, F, I, P],
    "kva_stream_read": [P, LL, I, P, P],
    "kva_stream_reread": [P, LL, I, I, P, P],
    "kva_stream_mixed": [P, LL, P, LL, I, P, P],
    "kva_silu_mul": [P, P, I, I, I, P],
    "kva_cast": [P, P, LL, I, I, P],
    "kva_rope_kv_write": [P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, P],
    "kva_attention_rowwise": [P, P, I, P, P, P, I, P, P, I, I, I, I, I, F, I, I, P],
    "kva_attention_mfma": [P, P, P, P, I, P, P, P, I, P, P, P, I, I, P, P, P, I, I, I, I, I, F, I, I, I, I, I, I, I, P],
    "kva_attention_mfma_rope": [P, P, P, P, I, P, P, P, I, P, I, I, I, I, I, I, F, I, I, I, I, P, P, P, I, P],
    "kva_attention_mfma_rope_supported": [I, I, I],
    "kva_attention_max_splits": [],
    "kva_attention_mfma_row_tiles": [I, I],
    "kva_attention_mfma_supported": [I, I],
    "kva_attention_lds_supported": [I, I],
    "kva_attention_lds": [P, P, P, P, I, P, P, P, I, P, I, I, I, I, I, I, F, I, I, I, I, I, P],
    "kva_gemm_skinny": [P, P, P, I, I, I, I, I, I, P, I, I, F, P, P, I, P, P, I, I, P],
    "kva_gemm_skinny_sumsq_parts": [I],
    "kva_tiled_rows": [I],
    "kva_gemm_skinny_partial_slices": [I, I, I],
    "kva_gemm_skinny_partials": [P, P, P, I, I, I, I, I, P],
    "kva_normed_rows_finish": [P, P, P, I, I, P, I, F, P],
    "kva_gemm_skinny_supported": [I, I, I],
    "kva_gemm_skinny_qkv_rope_supported": [I, I, I],
    "kva_gemm_skinny_qkv_rope": [P, I, P, P, I, I, I, I, I, I, P, I, I, F, P, P, P, P, P, P, I, P],
    "kva_gemv": [P, P, P, I, I, I, I, I, I, P, I, I, F, P, P, I, P, P, P],
    "kva_gemv_supported": [I, I, I],
    "kva_gemv_merged_supported": [I, I, I, I, I],
    "kva_gemv_merge_max_parts": [I],
    "kva_gemv_merged": [P, P, I, I, P, I, I, I, P, P, I, P, P, P],
    "kva_gemv_sumsq_parts": [I, I],
    "kva_gemv_qkv_rope_supported": [I, I, I],
    "kva_gemv_qkv_rope": [P, I, P, P, I, I, I, I, I, I, P, I, I, F, P, P, P, P, P, P, I, P],
    "kva_gemm_nt_f32": [P, P, P, I, I, I, I, I, I, P],
    "kva_gemm_vendor": [P, P, P, I, I, I, I, I, I, P],
    "kva_gemm_vendor_init": [],
    "kva_gemm_vendor_tune": [P, P, P, I, I, I, I, I, I, I, P, P, P, P],
    "kva_gemm_vendor_forget": [I, I, I, I, I, I],
    "kva_host_memory_is_mapped": [P],
    "kva_sample": [P, P, I, I, I, P, P, F, P, U, P, P, I, P, P, P, P, P],
    "kva_mark_tokens": [P, P, P, I, I, P],
}


def hip_lib():
    global _hip
    if _hip is not None:
        return _hip
    with _lock:
        if _hip is not None:
            return _hip
        try:
            path = build.build_hip()
            lib = ctypes.CDLL(path)
        except (build.BuildError, OSError) as e:
            raise KernelLibraryError(
                "the HIP kernel library (libkva_hip.so) is not available and there is no other "
                f"code path: {e}") from e
        for name, argtypes in _HIP_SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError:
                continue  # optional entry points are bound where they are used
            fn.argtypes = argtypes
            fn.restype = c_int
        lib.kva_last_error.restype = c_char_p
        lib.kva_sample_workspace_bytes.argtypes = [I, I]
        lib.kva_sample_workspace_bytes.restype = LL
        lib._path = path
        _hip = lib
        return _hip


def bind(name: str, argtypes) -> None:
    """Declares one more entry point of the kernel library (used by later kernel modules)."""
    _HIP_SIGNATURES[name] = argtypes
    if _hip is not None:
        fn = getattr(_hip, name)
        fn.argtypes = argtypes
        fn.restype = c_int


def check(code: int, what: str) -> None:
    if code != 0:
        msg = hip_lib().kva_last_error()
        raise KernelError(f"{what}: {msg.decode() if msg else 'error ' + str(code)}")


def host_lib():
    global _host
    if _host is not None:
        return _host
    with _lock:
        if _host is not None:
            return _host
        path = build.build_host()
        lib = ctypes.CDLL(path)
        IP = POINTER(c_int)
        sig = {
            "kva_pool_create": ([I], P),
            "kva_pool_destroy": ([P], None),
            "kva_pool_num_pages": ([P], I),
            "kva_pool_free_count": ([P], I),
            "kva_pool_takes": ([P], LL),
            "kva_pool_reuses": ([P], LL),
            "kva_pool_take": ([P, I, IP], I),
            "kva_pool_share": ([P, I], I),
            "kva_pool_drop": ([P, IP, I], I),
            "kva_pool_refcount": ([P, I], I),
            "kva_pool_accounting_holds": ([P], I),
            "kva_buddy_create": ([I], P),
            "kva_buddy_destroy": ([P], None),
            "kva_buddy_round": ([I], I),
            "kva_buddy_alloc": ([P, I], I),
            "kva_buddy_free": ([P, I, I], I),
            "kva_buddy_free_units": ([P], I),
            "kva_buddy_reserved_units": ([P], I),
            "kva_buddy_pool_units": ([P], I),
            "kva_buddy_fragmentation_failures": ([P], LL),
            "kva_buddy_free_runs": ([P, IP, I], I),
        }
        for name, (args, res) in sig.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = res
        _host = lib
        return _host
