"""ctypes binding of libpbs_hip.so.  There is no fallback: a missing library or a
failing call raises."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libpbs_hip.so")

# name -> (restype, argtypes); mirrors include/pbs_hip.h
_P, _I, _L, _F, _Z = c_void_p, c_int, c_int64, c_float, c_size_t
SIGNATURES = {
    "pbs_abi_version": (c_int, []),
    "pbs_last_error": (c_char_p, []),
    "pbs_score_keys_workspace_bytes": (_Z, [_I, _I, _I, _I, _I]),
    "pbs_score_keys": (c_int, [_P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _L, _L, _L, _L, _L, _L, _P, _Z, _P]),
    "pbs_score_keys_static": (c_int, [_P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _L, _L, _L, _L, _L, _L, _P]),
    "pbs_segment_argsort": (c_int, [_P, _P, _I, _I, _I, _I, _P]),
    "pbs_gather_kv": (c_int, [_P] * 6 + [_I] * 6 + [_L] * 6 + [_I, _P, _P]),
    "pbs_pool_k_permuted": (c_int, [_P] * 4 + [_I] * 6 + [_L] * 3 + [_I, _P]),
    "pbs_pool_blocks": (c_int, [_P] * 6 + [_I] * 6 + [_L] * 6 + [_I, _I, _P]),
    "pbs_pool_q": (c_int, [_P, _P, _I, _I, _I, _I, _I, _L, _L, _L, _I, _P]),
    "pbs_block_logits_softmax": (c_int, [_P, _P, _P, _I, _I, _I, _I, _P]),
    "pbs_block_logits_softmax_candidates_only": (c_int, [_P, _P, _P, _I, _I, _I, _I, _P]),
    "pbs_block_logits_softmax_causal": (c_int, [_P, _P, _P, _I, _I, _I, _P]),
    "pbs_select_blocks_workspace_bytes": (_Z, [_I]),
    "pbs_select_blocks": (c_int, [_P, _P, _F, _I, _I, _I, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "pbs_block_mask_to_csr": (c_int, [_P, _P, _P, _P, _I, _I, _I, _P]),
    "pbs_sparse_attn_workspace_bytes": (c_size_t, [_I] * 4),
    "pbs_sparse_attn_fwd": (c_int, [_P] * 8 + [_I] * 7 + [_L] * 12 + [_F, _P, _P]),
    "pbs_sparse_attn_fwd_optional_diagonal": (c_int, [_P] * 9 + [_I] * 6 + [_L] * 12 + [_F, _P, _P]),
    "pbs_unpermute": (c_int, [_P, _P, _P, _I, _I, _I, _I, _L, _L, _L, _P]),
    "pbs_rope_qk": (c_int, [_P] * 6 + [_I] * 5 + [_L] * 8 + [_P]),
    "pbs_identity_indices": (c_int, [_P, _I, _I, _P]),
    "pbs_prefill_attn_workspace_bytes": (_Z, [_I, _I, _I, _I, _I, _I, _I]),
    "pbs_prefill_attn_fwd": (c_int, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I] + [_L] * 12 +
                             [_F, _P, _I, _I, _I, _I, _F, _P, _Z, _P]),
}

_lib = None


class PbsHipError(RuntimeError):
    pass


def load():
    """Loads the library once.  torch must already be imported so that the HIP
    runtime torch ships is the one the library binds to."""
    global _lib
    if _lib is not None:
        return _lib
    import torch  # noqa: F401  (pulls in libamdhip64 before our library asks for it)
    if not os.path.exists(LIB_PATH):
        raise PbsHipError(
            f"{LIB_PATH} is missing: build it with `python -m pbs_attn_amd.build` "
            "(hipcc, gfx950).  There is no non-HIP implementation of this path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code: int, what: str):
    if code != 0:
        msg = load().pbs_last_error()
        raise PbsHipError(f"{what} failed ({code}): {msg.decode() if msg else ''}")
