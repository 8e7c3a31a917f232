"""Loading the built HIP modules through ctypes.

A module is loaded when one of its functions is first asked for and is compiled
then if it is not built. There is no other implementation behind these
functions: without the extension every call raises BackendError.
"""
import ctypes

from ..errors import BackendError
from . import build

_loaded = {}

_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float
_U32 = ctypes.c_uint32
_SZ = ctypes.c_size_t

# module -> function -> argument types (every function returns int, 0 = ok)
SIGNATURES = {
    "elementwise": {
        "hb_embed": [_P, _P, _I, _P, _I, _I, _I, _I, _P],
        "hb_rmsnorm": [_P, _P, _P, _I, _P, _I, _I, _F, _P],
        "hb_qk_norm_rope_write": [_P, _I, _P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _P, _P, _P, _I,
                                  _I, _I, _I, _I, _F, _I, _I, ctypes.c_size_t, _P],
        "hb_swiglu": [_P, _P, _I, _I, _I, _P],
        "hb_fill_u32": [_P, _U32, _SZ, _P],
    },
    "gemm_plain": {
        "hb_gemm_plain": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P],
    },
    "attention_plain": {
        "hb_attention_plain": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P],
    },
    "sampling": {
        "hb_argmax": [_P, _I, _I, _I, _P, _P, _P, _I, _P],
        "hb_argmax_noalloc": [_P, _I, _I, _I, _P, _P],
        "hb_argmax_noalloc_setup": [],
        "hb_sample": [_P, _I, _I, _I, _F, _I, _F, _P, _P, _P, _P, _P, _I, _P, _P, _P],
        "hb_sample_nucleus": [_P, _I, _I, _I, _F, _F, _P, _P, _P, _P, _P, _P, _P],
        "hb_force_tokens": [_P, _I, _I, _I, _P, _P, _I, _P],
        "hb_sample_all": [_P, _I, _I, _I, _F, _P, _P, _P, _P, _P],
    },
}


def register_signatures(module, functions):
    """Add the functions of a further module (used by the MFMA modules)."""
    SIGNATURES.setdefault(module, {}).update(functions)


def load(module):
    """The ctypes library of a module, built first if need be."""
    lib = _loaded.get(module)
    if lib is not None:
        return lib
    path = build.build_module(module)
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise BackendError(f"cannot load {path}: {e}") from None
    lib.hb_last_error.restype = ctypes.c_char_p
    lib.hb_last_error.argtypes = []
    for fname, argtypes in SIGNATURES.get(module, {}).items():
        fn = getattr(lib, fname)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    _loaded[module] = lib
    return lib


def loaded_modules():
    return sorted(_loaded)


_functions = {}


def call(module, fname, *args):
    """Call a C entry point; a non-zero return becomes BackendError with its text."""
    fn = _functions.get((module, fname))
    if fn is None:
        fn = _functions[(module, fname)] = getattr(load(module), fname)
    if fn(*args) != 0:
        raise BackendError(load(module).hb_last_error().decode(errors="replace"))
