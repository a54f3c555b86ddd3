"""ctypes loader for ``libphyai_fp8.so`` (the gfx950 HIP kernels behind a C ABI).

There is no fallback: if the shared library is missing or does not export the
symbols the header declares, importing the ops fails loudly.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
# PHYAI_FP8_LIBRARY=stamps (set before the first call) makes the whole process use the debug build whose GEMM
# kernels record time stamps of their phases (`make -C phyai_amd/csrc stamps`): same entry points, same results.
STAMPS_LIB_PATH = os.path.join(_PKG, "lib", "libphyai_fp8_stamps.so")
# PHYAI_FP8_LIBRARY=ablate: the time-stamp build with parts of a kernel's main loop left out (`make ablate ABLATE=n`),
# for measurements only - its results are wrong by design.
LIB_PATH = {"stamps": STAMPS_LIB_PATH, "ablate": os.path.join(_PKG, "lib", "libphyai_fp8_ablate.so")}.get(
    os.environ.get("PHYAI_FP8_LIBRARY", ""), os.path.join(_PKG, "lib", "libphyai_fp8.so"))
CSRC_DIR = os.path.join(_PKG, "csrc")
ABI_VERSION = 8

# name -> (restype, argtypes); mirrors include/phyai_fp8.h one to one.
_i64, _vp, _int, _sz = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
SIGNATURES: dict[str, tuple[object, list[object]]] = {
    "phyai_fp8_abi_version": (_int, []),
    "phyai_fp8_last_error": (ctypes.c_char_p, []),
    "phyai_fp8_quant_rowwise": (_int, [_vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "phyai_fp8_quant_static": (_int, [_vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "phyai_fp8_weight_quant_rowwise": (_int, [_vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "phyai_fp8_weight_to_operand_order": (_int, [_vp, _i64, _i64, _int, _vp, _vp]),
    "phyai_fp8_linear_workspace_bytes": (_sz, [_i64, _i64, _i64, _int]),
    "phyai_fp8_gemm": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp]),
    "phyai_fp8_linear": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp]),
    "phyai_fp8_mlp_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _int]),
    "phyai_fp8_mlp": (_int, [_vp, _i64, _vp, _vp, _vp, _int, _vp, _vp, _vp, _int, _vp, _i64, _vp, _i64, _i64, _vp, _i64,
                             _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp]),
    "phyai_fp8_describe_mlp_plan": (_int, [_i64, _i64, _i64, _i64, _int, ctypes.c_char_p, _sz]),
    "phyai_fp8_linear_static": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "phyai_fp8_gemm_addcmul": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i64,
                                      _i64, _int, _vp, _sz, _vp]),
    "phyai_fp8_linear_addcmul": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i64,
                                        _i64, _int, _vp, _sz, _vp]),
    "phyai_fp8_rmsnorm_quant": (_int, [_vp, _i64, _vp, _int, _i64, _i64, ctypes.c_float, _vp, _i64, _vp, _vp, _vp]),
    "phyai_fp8_adarmsnorm_quant": (_int, [_vp, _i64, _vp, _i64, _i64, _i64, _i64, ctypes.c_float, _vp, _i64, _vp,
                                          _i64, _vp, _vp, _vp]),
    "phyai_fp8_describe_plan": (_int, [_i64, _i64, _i64, _int, ctypes.c_char_p, _sz]),
    "phyai_fp8_describe_linear_plan": (_int, [_i64, _i64, _i64, _int, ctypes.c_char_p, _sz]),
    "phyai_fp8_debug_cast_e4m3": (_int, [_vp, _i64, _vp, _vp]),
    "phyai_fp8_debug_stamps": (_int, [_vp, _i64]),
    "phyai_fp8_debug_mfma_rate": (_int, [_int, _int, _vp, _vp, _vp]),
}


class Fp8LibraryError(RuntimeError):
    """The native library is missing, stale, or a call into it failed."""


_lib: ctypes.CDLL | None = None


def build(verbose: bool = False) -> str:
    """Compile the HIP sources for gfx950 with hipcc (``make -C phyai_amd/csrc``)."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.check_call(["make", "-C", CSRC_DIR, "-j8"], stdout=out, stderr=out)
    return LIB_PATH


def open_library(path: str) -> ctypes.CDLL:
    """Open one build of the library and give its entry points their signatures."""
    if not os.path.exists(path):
        raise Fp8LibraryError(
            f"{path} not found: build it with `make -C {CSRC_DIR}` "
            "(or phyai_amd._lib.build()); there is no non-HIP fallback"
        )
    lib = ctypes.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise Fp8LibraryError(f"{path} does not export {name}; rebuild it") from e
        fn.restype = res
        fn.argtypes = args
    got = lib.phyai_fp8_abi_version()
    if got != ABI_VERSION:
        raise Fp8LibraryError(f"{path} has ABI version {got}, expected {ABI_VERSION}; rebuild it")
    return lib


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        _lib = open_library(LIB_PATH)
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().phyai_fp8_last_error()
        raise Fp8LibraryError(f"{what} failed (rc={rc}): {msg.decode() if msg else ''}")
