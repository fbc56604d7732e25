"""ctypes binding of the C-ABI library (``include/skyrl_lmhead.h``).

The library is loaded from the source tree (``skyrl_amd/csrc/libskyrl_lmhead.so``).  There is no fallback: if it has not
been built, or the symbol table does not match the header, loading raises.
"""

from __future__ import annotations

import ctypes
import os
import threading

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libskyrl_lmhead.so")
ABI_VERSION = 20

_c_i64 = ctypes.c_int64
_c_p = ctypes.c_void_p

# name -> (restype, argtypes); mirrors include/skyrl_lmhead.h one to one.
SIGNATURES = {
    "skyrl_lmhead_version": (ctypes.c_int, []),
    "skyrl_lmhead_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "skyrl_lmhead_fwd_workspace_bytes": (ctypes.c_size_t, [_c_i64, _c_i64, _c_i64]),
    "skyrl_lmhead_bwd_workspace_bytes": (ctypes.c_size_t, [_c_i64, _c_i64, _c_i64, _c_i64]),
    "skyrl_lmhead_fwd": (
        ctypes.c_int,
        [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_i64, _c_i64, _c_i64, ctypes.c_float, _c_p, _c_p, _c_p, _c_p, _c_p,
         ctypes.c_size_t, _c_p],
    ),
    "skyrl_lmhead_fwd_static_scratch": (
        ctypes.c_int,
        [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_i64, _c_i64, _c_i64, ctypes.c_float, _c_p, _c_p, _c_p, _c_p, _c_p],
    ),
    "skyrl_lmhead_static_scratch_bytes": (ctypes.c_size_t, []),
    "skyrl_lmhead_bwd": (
        ctypes.c_int,
        [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, ctypes.c_float, _c_p, _c_p,
         ctypes.c_int, _c_i64, _c_p, ctypes.c_size_t, _c_p],
    ),
    "skyrl_lmhead_bwd_active_rows_workspace_bytes": (ctypes.c_size_t, [_c_i64, _c_i64, _c_i64, _c_i64]),
    "skyrl_lmhead_bwd_active_rows": (
        ctypes.c_int,
        [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, ctypes.c_float, _c_p, _c_p,
         ctypes.c_int, _c_i64, _c_p, ctypes.c_size_t, _c_p],
    ),
    "skyrl_lmhead_split_operand": (ctypes.c_int, [_c_p, ctypes.c_int, _c_i64, _c_i64, _c_i64, ctypes.c_int, _c_p, _c_i64, _c_p]),
    "skyrl_lmhead_bwd_split_workspace_bytes": (ctypes.c_size_t, [_c_i64, _c_i64, _c_i64, _c_i64, _c_i64, ctypes.c_int]),
    "skyrl_lmhead_bwd_split": (
        ctypes.c_int,
        [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_i64, ctypes.c_float, _c_p, _c_p,
         ctypes.c_int, _c_i64, ctypes.c_int, _c_p, ctypes.c_size_t, _c_p],
    ),
    "skyrl_ppo_policy_loss": (
        ctypes.c_int,
        [_c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_int, _c_p, _c_p, _c_p,
         _c_p],
    ),
    "skyrl_approx_kl": (ctypes.c_int, [_c_p, _c_p, _c_p, _c_i64, _c_i64, ctypes.c_int, _c_p, _c_p, _c_p, ctypes.c_int, _c_p, _c_p]),
    "skyrl_actor_loss": (
        ctypes.c_int,
        [_c_p] * 7 + [_c_i64, _c_i64, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_int,
                      ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float, _c_p, _c_p, _c_p, _c_p, _c_p]),
    "skyrl_masked_mean": (ctypes.c_int, [_c_p, _c_p, _c_i64, _c_i64, _c_p, _c_p, _c_p]),
    "skyrl_packed_next_token_labels": (ctypes.c_int, [_c_p, _c_p, _c_i64, _c_i64, _c_p, _c_p]),
    "skyrl_packed_scatter_logprobs": (
        ctypes.c_int, [_c_p, _c_p, _c_i64, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_p, _c_p]),
    "skyrl_packed_gather_grad": (
        ctypes.c_int, [_c_p, _c_p, _c_i64, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_p, _c_p]),
    "skyrl_softce_fwd_workspace_bytes": (ctypes.c_size_t, [_c_i64, _c_i64, _c_i64]),
    "skyrl_softce_bwd_workspace_bytes": (ctypes.c_size_t, [_c_i64, _c_i64, _c_i64, _c_i64]),
    "skyrl_softce_fwd": (
        ctypes.c_int,
        [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, ctypes.c_float, _c_p, _c_p, _c_p,
         _c_p, ctypes.c_size_t, _c_p],
    ),
    "skyrl_softce_bwd": (
        ctypes.c_int,
        [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, ctypes.c_float,
         _c_p, _c_i64, _c_p, ctypes.c_size_t, _c_p],
    ),
    "skyrl_lmhead_topk_workspace_bytes": (ctypes.c_size_t, [_c_i64, _c_i64, _c_i64, _c_i64]),
    "skyrl_lmhead_topk_logits": (
        ctypes.c_int,
        [_c_p, _c_i64, _c_p, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, ctypes.c_float, _c_p, _c_p, _c_p, ctypes.c_size_t, _c_p],
    ),
    "skyrl_softce_topk_fwd": (
        ctypes.c_int,
        [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, ctypes.c_float, _c_p, _c_p, _c_p,
         _c_p],
    ),
    "skyrl_softce_topk_bwd": (
        ctypes.c_int,
        [_c_p, _c_i64, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_i64, ctypes.c_float, _c_p, _c_i64, _c_p],
    ),
    "skyrl_off_policy_correction": (
        ctypes.c_int,
        [_c_p, _c_p, _c_p, _c_i64, _c_i64, ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_float,
         ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float),
         ctypes.POINTER(ctypes.c_float), _c_p, _c_p, _c_p, _c_p, _c_p, _c_p]),
    "skyrl_logits_fwd": (
        ctypes.c_int, [_c_p, ctypes.c_int, _c_i64, _c_p, _c_i64, _c_i64, ctypes.c_float, _c_p, _c_p, _c_p, _c_p, _c_p]),
    "skyrl_logits_bwd": (
        ctypes.c_int,
        [_c_p, ctypes.c_int, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, ctypes.c_float, _c_p, _c_i64, _c_p]),
    "skyrl_logprob_diff_metrics": (ctypes.c_int, [_c_p, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_p]),
    "skyrl_lmhead_mfma_probe": (ctypes.c_int, [_c_p, ctypes.c_int, ctypes.c_int, _c_p, _c_p]),
    "skyrl_lmhead_atomic_floor_probe": (ctypes.c_int, [_c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_p]),
    "skyrl_lmhead_device_info": (ctypes.c_int, [ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]),
    "skyrl_lmhead_num_kernel_kinds": (ctypes.c_int, []),
    "skyrl_lmhead_kernel_name": (ctypes.c_char_p, [ctypes.c_int]),
    "skyrl_lmhead_profile_begin": (_c_p, []),
    "skyrl_lmhead_profile_end": (ctypes.c_int, [_c_p, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(_c_i64)]),
}

_lock = threading.Lock()
_lib = None


class LmHeadLibraryError(RuntimeError):
    """The HIP library is missing, stale, or returned a non-zero status."""


def lib_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Load (once) and return the library.  Raises LmHeadLibraryError when it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(_LIB_PATH):
            raise LmHeadLibraryError(
                f"{_LIB_PATH} is not built. Run `python -m skyrl_amd.csrc.build` (needs hipcc, targets gfx950). "
                "There is no non-HIP fallback for the fused LM-head path."
            )
        lib = ctypes.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError as exc:
                raise LmHeadLibraryError(f"{_LIB_PATH} does not export {name}; rebuild it") from exc
            fn.restype = restype
            fn.argtypes = argtypes
        got = lib.skyrl_lmhead_version()
        if got != ABI_VERSION:
            raise LmHeadLibraryError(f"{_LIB_PATH} has ABI version {got}, this package expects {ABI_VERSION}; rebuild it")
        _lib = lib
        return lib


def strerror(status: int) -> str:
    return load().skyrl_lmhead_strerror(int(status)).decode("utf-8", "replace")


def check(status: int, what: str) -> None:
    """Turn a non-zero status into an exception (argument errors -> ValueError, HIP errors -> LmHeadLibraryError)."""
    if status == 0:
        return
    msg = f"{what} failed with status {status}: {strerror(status)}"
    if status < 0:
        raise ValueError(msg)
    raise LmHeadLibraryError(msg)


class KernelProfile:
    """Context manager around skyrl_lmhead_profile_begin/end: per-kernel HIP-event times of the calls made inside it.

    ``with KernelProfile() as prof: ...`` then ``prof.results`` is ``{kernel name: (total_ms, launches)}``.
    """

    def __enter__(self):
        self._lib = load()
        self._handle = self._lib.skyrl_lmhead_profile_begin()
        if not self._handle:
            raise LmHeadLibraryError("a kernel profile is already open on this thread")
        self.results = {}
        return self

    def __exit__(self, *exc):
        n = self._lib.skyrl_lmhead_num_kernel_kinds()
        ms = (ctypes.c_double * n)()
        cnt = (_c_i64 * n)()
        st = self._lib.skyrl_lmhead_profile_end(self._handle, ms, cnt)
        if exc[0] is None:
            check(st, "skyrl_lmhead_profile_end")
        self.results = {self._lib.skyrl_lmhead_kernel_name(k).decode(): (float(ms[k]), int(cnt[k])) for k in range(n)}
        return False
