"""Loads the HIP kernel libraries and declares their C entry points.

There is no fall-back: when a library is missing it is compiled once (hipcc, a few seconds
per file); when that is impossible the import of an operation fails with the reason.
"""
from __future__ import annotations

import ctypes
import threading
from typing import Dict

from ..csrc import build as _build

c_int = ctypes.c_int
c_long = ctypes.c_long
c_float = ctypes.c_float
c_void_p = ctypes.c_void_p

DTYPE_F32 = 0
DTYPE_BF16 = 1

_SIGNATURES = {
    "mv_last_error": (ctypes.c_char_p, []),
    "mv_built_dtypes": (c_int, []),
    "mv_abi_version": (c_int, []),
    "mv_graph_census": (c_int, [c_void_p, c_void_p]),
    # logits, ld, M, V, temperature, top_k, top_p, rng, out, stream (no workspace: see csrc/mv_noalloc.h)
    "mv_sample_noalloc": (c_int, [c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p]),
    "mv_embedding": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p]),
    "mv_add_rmsnorm": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_float, c_int, c_void_p, c_void_p,
                               c_int, c_int, c_int, c_void_p]),
    "mv_rmsnorm": (c_int, [c_void_p, c_long, c_void_p, c_int, c_float, c_int, c_void_p, c_long, c_int, c_int,
                           c_int, c_void_p]),
    "mv_rope_table": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "mv_qk_norm_rope_store": (c_int, [c_void_p, c_long, c_int, c_int, c_int,            # qkv, stride, offsets
                                      c_void_p, c_void_p, c_void_p, c_int, c_int,      # pos, seq, bt, width, page
                                      c_void_p, c_void_p, c_int, c_int, c_int, c_int,  # k, v pages, n, H, Hkv, D
                                      c_void_p, c_void_p, c_int, c_float, c_int,       # qw, kw, wdtype, eps, unit
                                      c_void_p, c_int, c_int, c_int, c_int, c_void_p]),  # table, rot, inter, store, dtype
    "mv_store_v_pages": (c_int, [c_void_p, c_long, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                 c_int, c_int, c_int, c_int, c_void_p]),
    "mv_swiglu": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "mv_gemm_ref": (c_int, [c_void_p, c_long, c_int, c_void_p, c_long, c_int, c_void_p, c_void_p, c_long, c_int,
                            c_int, c_int, c_int, c_void_p]),
    "mv_attention_ref": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                 c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p]),
    "mv_sample": (c_int, [c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_void_p, c_int, c_void_p]),
    # ... as mv_sample up to chunks, then next_ids, positions, context_lens, stream
    "mv_sample_advance": (c_int, [c_void_p, c_long, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
}

# entry points that only the bfloat16 library has
_OPTIONAL_SIGNATURES = {
    "mv_gemm_skinny": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_long, c_int,
                               c_int, c_int, c_int, c_void_p]),
    "mv_gemm_skinny_swiglu": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_void_p]),
    "mv_gemm_skinny_fold_parts": (c_int, [c_int, c_int, c_int]),
    # A, lda, W, bias, resid, ldr, norm_weight, norm_weight_dtype, unit_offset, weighted, ldw, partial, P, M, N, K, stream
    "mv_gemm_skinny_fold": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_int, c_int,
                                    c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    # A, lda, W, bias, C, ldc, partial, P, eps, M, N, K, swiglu, stream
    "mv_gemm_skinny_scaled": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_int, c_float,
                                      c_int, c_int, c_int, c_int, c_void_p]),
    # weighted, ldw, partial, P, eps, out, ldo, dtype, M, width, stream
    "mv_scale_rows": (c_int, [c_void_p, c_long, c_void_p, c_int, c_float, c_void_p, c_long, c_int, c_int, c_int, c_void_p]),
    "mv_gemm_skinny_norm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_float, c_int, c_void_p, c_void_p,
                                    c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "mv_gemm_lt_workspace": (c_long, []),
    # A, lda, W, bias, C, ldc, c_dtype, M, N, K, workspace, workspace_bytes, stream
    "mv_gemm_lt": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_void_p,
                           c_long, c_void_p]),
    "mv_gemm_mid_workspace": (c_long, [c_int, c_int, c_int]),
    "mv_gemm_mid_splits": (c_int, [c_int, c_int]),
    # A, lda, W, M, N, K, work, work_floats, stream
    "mv_gemm_mid_sums": (c_int, [c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_void_p, c_long, c_void_p]),
    # work, bias, C, ldc, c_dtype, M, N, F, swiglu, stream
    "mv_gemm_mid_reduce": (c_int, [c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    # resid, part, F, plane, bias, weight, weight_dtype, eps, unit_offset, out, rows, n_out, h, dtype, stream
    "mv_add_rmsnorm_split": (c_int, [c_void_p, c_void_p, c_int, c_long, c_void_p, c_void_p, c_int, c_float, c_int,
                                     c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    # A, lda, W, bias, C, ldc, c_dtype, M, N, K, swiglu, work, work_floats, stream
    "mv_gemm_mid": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_int,
                            c_void_p, c_long, c_void_p]),
    "mv_device_compute_units": (c_int, []),
    "mv_gemm_tile_workspace": (c_long, [c_int, c_int, c_int, c_int, c_int]),
    "mv_gemm_tile_splits": (c_int, [c_int, c_int, c_int, c_int, c_int]),
    # A, lda, W, bias, C, ldc, c_dtype, M, N, K, gated, work, work_floats, force, stream
    "mv_gemm_tile": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int, c_int,
                             c_void_p, c_long, c_int, c_void_p]),
    # A, lda, W, M, N, K, work, work_floats, force, stream
    "mv_gemm_tile_sums": (c_int, [c_void_p, c_long, c_void_p, c_int, c_int, c_int, c_void_p, c_long, c_int, c_void_p]),
    # A, lda, W, bias, C, ldc, c_dtype, M, N, K, gated, partial, P, eps, stream
    "mv_gemm_tile_scaled": (c_int, [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_long, c_int, c_int, c_int, c_int,
                                    c_int, c_void_p, c_int, c_float, c_void_p]),
    "mv_attention_decode": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                    c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_int,
                                    c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    # qkv, stride, q_off, k_off, v_off, out, out_stride, k_pages, v_pages, block_table, bt_width, page_size,
    # positions, cu_seqlens, n_seqs, H, Hkv, D, scale, window, q_weight, k_weight, weight_dtype, eps, unit_offset,
    # table, rows, store_kv, partials, counters, nsplit, max_pages, waves, token_seq, stream
    "mv_attention_decode_fused": (c_int, [c_void_p, c_long, c_int, c_int, c_int, c_void_p, c_long, c_void_p, c_void_p,
                                          c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                          c_float, c_int, c_void_p, c_void_p, c_int, c_float, c_int, c_void_p, c_void_p,
                                          c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    # ids, table, table_dtype, resid, n, h, vocab, scale, ids2, table2, out2, h2, rows2, stream
    "mv_embedding_gather": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p, c_void_p,
                                    c_void_p, c_int, c_int, c_void_p]),
    "mv_attention_prefill": (c_int, [c_void_p, c_long, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                     c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                     c_float, c_int, c_void_p]),
    "mv_attention_prefill_unit_tokens": (c_int, [c_int, c_int]),
    "mv_launch_empty": (c_int, [c_int, c_int, c_void_p, c_void_p]),
}


class KernelLibraryError(RuntimeError):
    pass


class KernelLibrary:
    """One loaded ``libmvk_<variant>.so``."""

    def __init__(self, variant: str, path: str):
        self.variant = variant
        self.path = path
        try:
            self.dll = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryError(f"cannot load the HIP kernel library {path}: {e}") from e
        for name, (res, args) in _SIGNATURES.items():
            try:
                fn = getattr(self.dll, name)
            except AttributeError as e:
                raise KernelLibraryError(f"{path} lacks the entry point {name}; rebuild it") from e
            fn.restype = res
            fn.argtypes = args
        self.optional = set()
        for name, (res, args) in _OPTIONAL_SIGNATURES.items():
            fn = getattr(self.dll, name, None)
            if fn is not None:
                fn.restype = res
                fn.argtypes = args
                self.optional.add(name)

    def has(self, name: str) -> bool:
        return name in self.optional or name in _SIGNATURES

    def call(self, name: str, *args) -> None:
        rc = getattr(self.dll, name)(*args)
        if rc != 0:
            msg = self.dll.mv_last_error()
            raise KernelLibraryError(msg.decode("utf-8", "replace") if msg else f"{name} failed")

    def offer(self, name: str, *args) -> bool:
        """Calls an entry point that may decline its arguments (return code 2, nothing done):
        False then, True when it ran; any other failure raises."""
        rc = getattr(self.dll, name)(*args)
        if rc == 0:
            return True
        if rc == 2:
            return False
        msg = self.dll.mv_last_error()
        raise KernelLibraryError(msg.decode("utf-8", "replace") if msg else f"{name} failed")


_LOCK = threading.Lock()
_LOADED: Dict[str, KernelLibrary] = {}


def variant_of(dtype_name: str) -> str:
    if dtype_name in ("float32", "f32"):
        return "f32"
    if dtype_name in ("bfloat16", "bf16"):
        return "bf16"
    raise ValueError(f"no kernel library for dtype {dtype_name!r}")


def load(variant: str) -> KernelLibrary:
    """The library of ``variant`` ("f32" or "bf16"), building it first if it is not there."""
    with _LOCK:
        lib = _LOADED.get(variant)
        if lib is not None:
            return lib
        path = _build.find_library(variant)
        if path is None:
            try:
                path = _build.build(variant)
            except Exception as e:
                stale = _build.find_library(variant, require_fresh=False)
                hint = f" (a library built from other sources is at {stale})" if stale else ""
                raise KernelLibraryError(
                    f"the HIP kernel library '{variant}' is not built and building it failed{hint}: {e}") from e
        lib = KernelLibrary(variant, path)
        _LOADED[variant] = lib
        return lib
