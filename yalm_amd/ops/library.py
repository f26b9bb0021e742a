"""Loads the gfx950 kernel library through ctypes and declares its entry points.

There is no fallback: if the library can neither be found nor built, or the GPU
is absent, the call fails with an error that says so."""
import ctypes
import threading

from ..csrc import build as _build

_lock = threading.Lock()
_lib = None

_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float

_SIGNATURES = {
    "yalm_abi_version": (ctypes.c_int, []),
    "yalm_error_string": (ctypes.c_char_p, [_I]),
    "yalm_embed": (_I, [_P, _I, _P, _P, _I, _I, _I, _P]),
    "yalm_rmsnorm": (_I, [_P, _P, _I, _P, _I, _P, _I, _I, _F, _P]),
    "yalm_gemm": (_I, [_P, _P, _P, _P, ctypes.c_long, _I, _I, _I, _I, _I, _I, _I, _P]),
    "yalm_gemm_norm": (_I, [_P, _P, _F, _P, _P, _I, _I, _I, _I, _I, _P]),
    "yalm_gemm_norm_qkv_rope": (_I, [_P, _P, _F, _P, _P, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "yalm_gemm_chain": (_I, [_P, _P, _P, _I, _I, _I, _I, _I, _P, _I, _F, _P, _P, _P, _P]),
    "yalm_gemm_chain_parts": (_I, [_I]),
    "yalm_gemm_chain_qkv_rope": (_I, [_P, _P, _I, _F, _P, _P, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "yalm_rope_kv_write": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "yalm_gemm_partial": (_I, [_P, _P, _P, ctypes.c_long, _I, _I, _I, _P, _P]),
    "yalm_gemm_bf16_dma_workspace": (ctypes.c_long, [_I, _I, _I]),
    "yalm_gemm_add_norm": (_I, [_P, _P, _P, _P, ctypes.c_long, _I, _I, _I, _P, _F, _P, _P]),
    "yalm_rope_kv_write_tiles": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "yalm_attn_prefill": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "yalm_attn_decode": (_I, [_P, _P, _P, _P, _I, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "yalm_attn_decode_workspace": (ctypes.c_long, [_I, _I, _I, _I]),
    "yalm_attn_prefill_lse": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I,
                                   _P, _I, _P]),
    "yalm_attn_decode_lse": (_I, [_P, _P, _P, _P, _I, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P,
                                  _P, _I, _P]),
    "yalm_sink_store": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P]),
    "yalm_attn_sink_mix": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "yalm_attn_decode_sinks": (_I, [_P, _P, _P, _P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P]),
    "yalm_attn_decode_static": (_I, [_P, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "yalm_argmax": (_I, [_P, _P, _I, _I, _P]),
    "yalm_sample": (_I, [_P, _P, _F, _P, _I, _I, _P]),
    "yalm_token_prob": (_I, [_P, _P, _P, _I, _I, _P]),
    "yalm_gemm_add_emit": (_I, [_P, _P, _P, _P, ctypes.c_long, _I, _I, _I, _P, _P, _P, _P]),
    "yalm_gemm_add_emit_parts": (_I, [_I]),
    "yalm_gemm_scaled": (_I, [_P, _P, _P, _P, ctypes.c_long, _I, _I, _I, _I, _I, _P, _I, _F, _P]),
    "yalm_gemm_partial_scaled": (_I, [_P, _P, _P, ctypes.c_long, _I, _I, _I, _P, _P, _I, _F, _P]),
    "yalm_probe_read": (_I, [_P, ctypes.c_long, _P, _I, _P]),
    "yalm_probe_mfma": (_I, [_I, _I, _I, _P, _P, _P]),
}

ABI_VERSION = 24


class KernelError(RuntimeError):
    pass


def lib():
    """The loaded library (built at the first call if it does not exist yet)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = _build.library_path()
        try:
            handle = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError("the HIP kernel library %s cannot be loaded: %s" % (path, e)) from e
        for name, (res, args) in _SIGNATURES.items():
            try:
                fn = getattr(handle, name)
            except AttributeError as e:
                raise KernelError("the HIP kernel library %s lacks %s; rebuild it with "
                                  "`python -m yalm_amd.csrc.build`" % (path, name)) from e
            fn.restype = res
            fn.argtypes = args
        if handle.yalm_abi_version() != ABI_VERSION:
            raise KernelError("the HIP kernel library %s is stale (ABI %d, wanted %d); rebuild it with "
                              "`python -m yalm_amd.csrc.build`" % (path, handle.yalm_abi_version(), ABI_VERSION))
        handle._path = path
        _lib = handle
    return _lib


def check(code, what):
    if code != 0:
        msg = lib().yalm_error_string(code)
        raise KernelError("%s failed: %s (code %d)" % (what, msg.decode() if msg else "?", code))
