"""Loads the HIP kernel library and declares its entry points for ctypes.

There is no fallback: without the library (and without a way to build it) importing an op
raises, so a GPU run can never silently use something else.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_longlong, c_ulonglong, c_void_p
from typing import Optional

_lib: Optional[ctypes.CDLL] = None
_lib_path: Optional[str] = None

P = c_void_p
I = c_int
F = c_float

_SIGNATURES = {
    "sharpi_embed_gather": [P, P, I, P, I, I, F, P],
    "sharpi_scale_softcap": [P, c_longlong, F, F, P],
    "sharpi_add_rmsnorm": [P, P, I, P, I, P, I, P, I, I, F, I, P, P, P, I, P],
    "sharpi_silu_mul": [P, P, P, I, I, I, I, P],
    "sharpi_moe_combine": [P, P, P, P, P, I, I, I, I, P],
    "sharpi_cast": [P, I, P, I, c_longlong, P],
    "sharpi_add_bias": [P, I, P, I, I, P],
    "sharpi_peak_read": [P, c_longlong, P, P, P],
    "sharpi_peak_mfma": [P, I, I, P],
    "sharpi_random_fill": [P, I, c_longlong, c_ulonglong, I, F, I, I, P],
    "sharpi_rope_kv": [P, P, P, P, I, P, P, P, P, I, F, I, F, F, I, I, I, I, I, I, I, I, P],
    "sharpi_attention_generic": [P, P, P, I, P, P, P, P, I, I, F, I, I, I, I, I, I, I, I, P],
    "sharpi_attention_decode": [P, P, P, P, P, P, P, P, P, P, I, I, F, I, I, I, I, I, I, I, I, P],
    "sharpi_attention_prefill": [P, P, P, P, P, P, P, I, I, I, I, F, I, I, I, I, I, I, P],
    "sharpi_gemm_tiled": [P, P, P, I, I, I, I, I, P, P, I, P],
    "sharpi_gemm_skinny": [P, P, P, I, I, I, I, P, P, I, I, I, I, I, P],
    "sharpi_gemm_skinny_swiglu": [P, P, P, I, I, I, P, P, I, P, I, I, I, I, I, P],
    "sharpi_gemm_skinny_picked": [P, P, P, I, I, I, P, P, I, I, I, I, I, I, I, I, I, P],
    "sharpi_add_rmsnorm_router": [P, P, P, I, P, I, I, F, P, I, P, P, I, I, I, I, P],
    "sharpi_router_topk": [P, I, P, I, P, P, P, I, I, I, I, I, I, P],
    "sharpi_moe_permute": [P, P, P, P, P, P, P, I, I, I, I, I, P],
    "sharpi_gemm_grouped": [P, I, P, P, I, I, I, I, P, P, P, I, I, I, P],
    "sharpi_gemm_grouped_swiglu": [P, I, P, P, I, I, I, P, P, P, I, P, I, I, I, P],
    "sharpi_argmax_rows": [P, P, I, I, P],
    "sharpi_sample_rows": [P, P, P, P, P, P, P, P, I, I, P],
    "sharpi_edit_logits": [P, P, P, P, P, P, P, P, I, I, P],
}

# entry points that newer sources add; bound when present
_OPTIONAL_SIGNATURES: dict = {}

# Sizes that the host code lays work out by and the kernels are compiled for: the library says what
# it was built with, and a build with other sizes is refused at load (it would compute wrong results).
DECODE_RUN_KEYS = 256       # keys per block of the decode attention kernel
PREFILL_TILE_TOKENS = 128   # tokens per block of the prefill attention kernel
PICKED_MAX_PAIRS = 64       # (token, pick) pairs the few-rows product takes straight from the router's picks
FUSED_NORM_ROUTER_MAX_HIDDEN = 8192   # widest row of the norm + router kernel
ROUTER_MAX_EXPERTS = 1024   # experts the routing kernels hold scores for
_BUILT_WITH = {
    "sharpi_attention_decode_split_keys": DECODE_RUN_KEYS,
    "sharpi_attention_prefill_tile_tokens": PREFILL_TILE_TOKENS,
    "sharpi_router_max_experts": ROUTER_MAX_EXPERTS,
    "sharpi_gemm_skinny_max_picked": PICKED_MAX_PAIRS,
    "sharpi_add_rmsnorm_router_max_hidden": FUSED_NORM_ROUTER_MAX_HIDDEN,
}


class KernelLibraryError(RuntimeError):
    pass


def library_path() -> Optional[str]:
    return _lib_path


def load(verbose: bool = True) -> ctypes.CDLL:
    """The kernel library, built first if no up-to-date build exists."""
    global _lib, _lib_path
    if _lib is not None:
        return _lib
    from ..csrc import build as _build

    try:
        path = _build.ensure_built(verbose=verbose)
    except Exception as e:  # noqa: BLE001
        raise KernelLibraryError(f"the HIP kernel library is missing and could not be built: {e}") from e
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise KernelLibraryError(f"cannot load {path}: {e}") from e
    for name, args in {**_SIGNATURES, **_OPTIONAL_SIGNATURES}.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            if name in _SIGNATURES:
                raise KernelLibraryError(f"{path} lacks entry point {name}: rebuild the kernels") from None
            continue
        fn.argtypes = args
        fn.restype = c_int
    for name, want in _BUILT_WITH.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            raise KernelLibraryError(f"{path} lacks entry point {name}: rebuild the kernels") from None
        fn.argtypes, fn.restype = [], c_int
        got = fn()
        if got != want:
            raise KernelLibraryError(f"{path} was built with {name}() = {got}, the host code lays work out for {want}")
    _lib, _lib_path = lib, path
    return lib


_takes: dict = {}


def attention_takes(kind: str, hd: int) -> bool:
    """Whether the matrix-core attention kernel of this kind ('decode' or 'prefill') is compiled for
    head size hd: the library is asked, so that the choice of kernel cannot drift from the build."""
    key = (kind, int(hd))
    if key not in _takes:
        fn = getattr(load(), f"sharpi_attention_{kind}_takes")
        fn.argtypes, fn.restype = [c_int], c_int
        _takes[key] = bool(fn(int(hd)))
    return _takes[key]


def grouped_tile_rows() -> int:
    """Rows of the tallest tile of the grouped product for many rows (an expert with more rows is
    cut into sibling tiles): the library says what it was built with."""
    if "tile_rows" not in _takes:
        fn = load().sharpi_gemm_grouped_tile_rows
        fn.argtypes, fn.restype = [], c_int
        _takes["tile_rows"] = int(fn())
    return _takes["tile_rows"]


def grouped_plan_ints(n_experts: int) -> int:
    """Length of the plan that the routing kernel writes for the grouped product of many rows."""
    fn = load().sharpi_grouped_plan_ints
    fn.argtypes, fn.restype = [c_int], c_int
    return int(fn(int(n_experts)))


def register_signature(name: str, argtypes) -> None:
    """Used by op modules that bind further entry points of the library."""
    _SIGNATURES[name] = list(argtypes)
    if _lib is not None:
        fn = getattr(_lib, name)
        fn.argtypes = list(argtypes)
        fn.restype = c_int
