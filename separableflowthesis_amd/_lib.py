"""ctypes binding of libsepcorr.so (the C ABI declared in include/sepcorr.h).

There is no fallback: if the library is missing or a symbol is absent, loading raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsepcorr.so")

_P = ctypes.c_void_p
_I = ctypes.c_int
_SZ = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/sepcorr.h one to one
SIGNATURES = {
    "sepcorr_last_error": (ctypes.c_char_p, []),
    "sepcorr_abi_version": (_I, []),
    "sepcorr_set_contraction": (_I, [_I]),
    "sepcorr_set_max_avg_backward": (_I, [_I]),
    "sepcorr_profile_enable": (_I, [_I]),
    "sepcorr_profile_collect": (_I, [ctypes.c_char_p, _SZ, ctypes.POINTER(ctypes.c_float), _I]),
    "sepcorr_max_avg_forward": (_I, [_P, _P, _P, _P] + [_I] * 6 + [_P, _SZ, _P]),
    "sepcorr_forward_workspace_bytes": (_SZ, [_I] * 7),
    "sepcorr_max_argmax_avg_forward": (_I, [_P] * 6 + [_I] * 6 + [_P, _SZ, _P]),
    "sepcorr_compression_forward": (_I, [_P] * 6 + [_I] * 7 + [_P, _SZ, _P]),
    "sepcorr_backward_workspace_bytes": (_SZ, [_I] * 6),
    "sepcorr_max_argmax_avg_backward": (_I, [_P] * 8 + [_I] * 6 + [_P, _SZ, _P]),
    "sepcorr_max_argmax_avg_backward_static": (_I, [_P] * 8 + [_I] * 6 + [_P]),
    "sepcorr_compression_backward": (_I, [_P] * 10 + [_I] * 7 + [_P, _SZ, _P]),
    "sepcorr_compression_forward_from_logits": (_I, [_P] * 8 + [_I] * 8 + [_P, _SZ, _P]),
    "sepcorr_compression_backward_from_logits_workspace_bytes": (_SZ, [_I] * 8),
    "sepcorr_compression_backward_from_logits": (_I, [_P] * 14 + [_I] * 7 + [_P, _SZ, _P]),
    "sepcorr_forward_levels_workspace_bytes": (_SZ, [_P, _P] + [_I] * 6),
    "sepcorr_max_argmax_avg_forward_levels": (_I, [_P] * 4 + [_I] + [_P] * 4 + [_I] * 4 + [_P, _SZ, _P]),
    "sepcorr_compression_forward_from_logits_levels": (_I, [_P] * 4 + [_I] + [_P] * 6 + [_I] * 5 + [_P, _SZ, _P]),
    "sepcorr_compression_backward_from_logits_levels": (_I, [_P] * 4 + [_I] + [_P] * 10 + [_I] * 5 + [_P, _SZ, _P]),
    "sepcorr_softmax_rows": (_I, [_P, _P, _I, _P, ctypes.c_long, _I, _P]),
    "sepcorr_fused_backward": (_I, [_P] * 12 + [_I] * 7 + [_P, _SZ, _P]),
    "sepcorr_fused_backward_add": (_I, [_P] * 12 + [_I] * 7 + [_P, _SZ, _P]),
    "sepcorr_attention_logits_forward": (_I, [_P] * 5 + [_I] * 5 + [_P]),
    "sepcorr_attention_logits_workspace_bytes": (_SZ, [_I] * 5),
    "sepcorr_attention_logits_backward": (_I, [_P] * 6 + [_I] * 5 + [_P, _SZ, _P]),
    "sepcorr_attention_logits_forward_levels": (_I, [_P] * 6 + [_I] * 5 + [_P]),
    "sepcorr_attention_logits_levels_workspace_bytes": (_SZ, [_P] + [_I] * 5),
    "sepcorr_attention_logits_backward_levels": (_I, [_P] * 8 + [_I] * 5 + [_P, _SZ, _P]),
    "sepcorr_attention_forward": (_I, [_P] * 4 + [_I] * 5 + [_P]),
    "sepcorr_attention_workspace_bytes": (_SZ, [_I] * 5),
    "sepcorr_attention_backward": (_I, [_P] * 7 + [_I] * 5 + [_P, _SZ, _P]),
    "sepcorr_assemble_forward": (_I, [_P] * 2 + [_I] * 8 + [_P]),
    "sepcorr_assemble_backward": (_I, [_P] * 2 + [_I] * 8 + [_P]),
    "sepcorr_assemble_forward_multi": (_I, [_P] * 3 + [_I] + [_P] + [_I] * 5 + [_P]),
    "sepcorr_assemble_backward_multi": (_I, [_P] * 4 + [_I] * 6 + [_P]),
    "sepcorr_feature_pyramid_forward": (_I, [_P] * 2 + [_I] * 5 + [ctypes.c_float, _P]),
    "sepcorr_feature_pyramid_backward": (_I, [_P] * 2 + [_I] * 5 + [ctypes.c_float, _P]),
    "sepcorr_lookup_forward": (_I, [_P] * 6 + [_I] * 6 + [ctypes.c_float, _P]),
    "sepcorr_lookup_backward_workspace_bytes": (_SZ, [_P] * 2 + [_I] * 6),
    "sepcorr_lookup_backward": (_I, [_P] * 8 + [_I] * 6 + [ctypes.c_float, _P, _SZ, _P]),
    "sepcorr_lookup1d_forward": (_I, [_P] * 3 + [_I] * 9 + [_P]),
    "sepcorr_lookup1d_backward": (_I, [_P] * 3 + [_I] * 9 + [_P]),
}

_lib = None


def load():
    """Load libsepcorr.so once and attach the prototypes.  Raises if it was not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
                "(or __graft_entry__.build()); there is no CPU fallback for this operator")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the library does not export it
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc):
    if rc != 0:
        raise RuntimeError(load().sepcorr_last_error().decode() or f"sepcorr error {rc}")
