"""ctypes binding of libnats_hip.so (the C ABI declared in include/nats_hip.h).

The library is loaded from the package directory; it is built by ``python -m neuralattentionsearch_amd.build``
(hipcc, gfx950).  There is no fallback: if the shared object is missing, loading raises.
"""
from __future__ import annotations

import ctypes
import functools
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# (NATS_HIP_LIB names another build of the same library, e.g. to time two builds side by side)
LIB_PATH = os.environ.get("NATS_HIP_LIB") or os.path.join(_PKG_DIR, "libnats_hip.so")

c_i64 = ctypes.c_int64
c_p = ctypes.c_void_p
c_i64p = ctypes.POINTER(ctypes.c_int64)

NATS_DTYPE_BF16 = 0
NATS_DTYPE_F32 = 1

ABI_VERSION = 8


class EvictParams(ctypes.Structure):
    """nats_evict_params"""
    _fields_ = [(n, c_i64) for n in
                ("B", "H_kv", "D", "C", "W", "S", "x_len", "fill", "n_ctx_data", "gmin", "tail", "first", "n_alloc",
                 "seq", "update_chunk")]


class EvictResult(ctypes.Structure):
    """nats_evict_result (64 bytes)"""
    _fields_ = [(n, c_i64) for n in
                ("n_ctx_data", "gmin", "all_sw", "all_local", "max_keep", "max_end", "moved_rows", "seq")]


class PastState(ctypes.Structure):
    """nats_past_state"""
    _fields_ = [(n, c_i64) for n in ("n_ctx_data", "old_fill", "gmin", "tail", "seen", "fill_last", "update_chunk")]


# every symbol include/nats_hip.h declares: name -> (restype, argtypes)
SIGNATURES = {
    "nats_abi_version": (ctypes.c_int, []),
    "nats_last_error": (ctypes.c_char_p, []),
    "nats_roles_from_logits": (ctypes.c_int, [c_p, ctypes.c_int, c_i64, c_i64, c_i64, ctypes.c_float, ctypes.c_int,
                                              ctypes.c_int, c_p, c_p, c_p]),
    "nats_role_step": (ctypes.c_int, [c_p, c_p, c_p, ctypes.c_int, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                      ctypes.c_int, ctypes.c_float, ctypes.c_int, c_i64p, c_p, c_i64, c_p, c_p, c_p, c_p,
                                      c_p, c_p]),
    "nats_role_scan": (ctypes.c_int, [c_p, c_i64, c_i64, c_i64, c_i64, c_i64, c_p, c_p, c_p]),
    "nats_prefill_mask": (ctypes.c_int, [c_p, c_i64, c_i64, c_i64, c_i64, c_i64, c_p, c_p, ctypes.c_size_t, c_p]),
    "nats_prefill_tile_map": (ctypes.c_int, [c_p, c_i64, c_i64, c_i64, c_i64, c_i64, c_p, c_p, ctypes.c_size_t, c_p]),
    "nats_prefill_workspace_bytes": (ctypes.c_size_t, [c_i64] * 6),
    "nats_prefill_sched_workspace_bytes": (ctypes.c_size_t, [c_i64] * 5),
    "nats_prefill_fwd": (ctypes.c_int, [c_p, c_p, c_p, c_p, c_p, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                        c_i64p, c_i64p, c_i64p, c_i64p, ctypes.c_float, ctypes.c_int, c_p,
                                        ctypes.c_size_t, c_p]),
    "nats_prefill_past_workspace_bytes": (ctypes.c_size_t, [c_i64] * 4),
    "nats_prefill_past_fwd": (ctypes.c_int, [c_p] * 8 + [c_i64] * 7 + [ctypes.POINTER(PastState)] + [c_i64p] * 5 +
                              [ctypes.c_float, ctypes.c_int, c_p, ctypes.c_size_t, c_p]),
    "nats_prefill_past_mask": (ctypes.c_int, [c_p] * 4 + [c_i64] * 5 + [ctypes.POINTER(PastState), c_i64p, c_p, c_p,
                                                                         ctypes.c_size_t, c_p]),
    "nats_decode_workspace_bytes": (ctypes.c_size_t, [c_i64] * 5),
    "nats_decode_fwd": (ctypes.c_int, [c_p, c_p, c_p, c_p, c_p, c_i64, c_p, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64p,
                                       c_i64p, ctypes.c_float, ctypes.c_int, c_p, ctypes.c_size_t, c_p]),
    "nats_decode_static_scratch_bytes": (ctypes.c_size_t, []),
    "nats_decode_fwd_static": (ctypes.c_int, [c_p, c_p, c_p, c_p, c_p, c_i64, c_p, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64p,
                                              c_i64p, ctypes.c_float, ctypes.c_int, c_p]),
    "nats_evict_workspace_bytes": (ctypes.c_size_t, [c_i64] * 3),
    "nats_evict_plan": (ctypes.c_int, [c_p, c_p, c_p, ctypes.POINTER(EvictParams), c_p, ctypes.c_size_t, c_p, c_p, c_p]),
    "nats_evict_apply_inplace": (ctypes.c_int, [c_p, c_p, c_p, c_p, c_p, c_p, c_p, ctypes.POINTER(EvictParams), c_i64p,
                                                c_i64p, ctypes.c_int, c_p, c_p, c_p]),
    "nats_evict_apply_first": (ctypes.c_int, [c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, ctypes.POINTER(EvictParams),
                                              c_i64p, c_i64p, c_i64p, ctypes.c_int, c_p, c_p, c_p]),
    "nats_cache_append": (ctypes.c_int, [c_p] * 6 + [c_i64] * 7 + [c_i64p] * 4 + [ctypes.c_int, c_p]),
    "nats_cache_append_plan": (ctypes.c_int, [c_p] * 6 + [c_i64] * 7 + [c_i64p] * 4 + [ctypes.c_int, c_p, c_p, c_p,
                                                                                        ctypes.POINTER(EvictParams), c_p,
                                                                                        ctypes.c_size_t, c_p, c_p, c_p]),
    "nats_add_rms_norm": (ctypes.c_int, [c_p, c_p, c_p, c_p, c_p, c_i64, c_i64, ctypes.c_float, ctypes.c_int, c_i64,
                                         ctypes.c_int, c_p]),
    "nats_silu_mul": (ctypes.c_int, [c_p, c_p, c_i64, c_i64, ctypes.c_int, c_p]),
    "nats_matvec": (ctypes.c_int, [c_p, c_p, c_p] + [c_i64] * 6 + [ctypes.c_int, ctypes.c_int, c_p]),
    "nats_rope_qk": (ctypes.c_int, [c_p] * 6 + [c_i64] * 5 + [c_i64p] * 3 + [ctypes.c_int, c_p]),
    "nats_rope_append": (ctypes.c_int, [c_p] * 10 + [c_i64] * 9 + [c_i64p] * 6 + [ctypes.c_int, c_p]),
}

_lib = None


class NatsError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"libnats_hip error {code}: {message}")
        self.code = code


def load() -> ctypes.CDLL:
    """Loads the shared library once and types every entry point.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m neuralattentionsearch_amd.build` (needs hipcc). "
            "This package has no CPU or PyTorch fallback for its kernels.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.nats_abi_version()
    if got != ABI_VERSION:
        raise ImportError(f"{LIB_PATH}: ABI version {got}, expected {ABI_VERSION}; rebuild the library")
    _lib = lib
    return lib


def check(rc: int) -> None:
    """Maps a negative return code to the exception the reference's asserts would have raised."""
    if rc == 0:
        return
    msg = load().nats_last_error().decode(errors="replace")
    if rc in (-1, -2, -3, -5):  # null pointer, shape, dtype, workspace: caller errors
        raise ValueError(f"libnats_hip error {rc}: {msg}")
    if rc == -4:
        raise NotImplementedError(f"libnats_hip error {rc}: {msg}")
    raise NatsError(rc, msg)


@functools.lru_cache(maxsize=4096)
def _i64_array_of(values: tuple):
    return (ctypes.c_int64 * len(values))(*values)


def i64_array(values):
    """A read-only int64[] argument (strides, sizes); equal tuples share one array."""
    return _i64_array_of(tuple(int(v) for v in values))
