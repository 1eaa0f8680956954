"""ctypes binding of libfdattn.so.  There is no fallback: without the built
library every op raises."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfdattn.so")

_vp, _i, _f, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/fdattn.h declaration by declaration
SIGNATURES = {
    "fdattn_version": (ctypes.c_char_p, []),
    "fdattn_last_error": (ctypes.c_char_p, []),
    "fdattn_write_cache_kv": (_i, [_vp] * 13 + [_i] * 11 + [_vp]),
    "fdattn_decode_workspace_bytes": (_sz, [_i] * 5),
    "fdattn_decode_attention": (_i, [_vp] * 10 + [_sz] + [_i] * 8 + [_f, _vp]),
    "fdattn_decode_noalloc_scratch_bytes": (_sz, []),
    "fdattn_decode_attention_noalloc": (_i, [_vp] * 9 + [_i] * 8 + [_f, _vp]),
    "fdattn_decode_uses_mfma": (_i, [_i] * 5),
    "fdattn_decode_chunks_per_sequence": (_i, [_i] * 3),
    "fdattn_sqattn_path": (_i, [_i] * 5),
    "fdattn_decode_attention_stages": (_i, [_vp] * 10 + [_sz] + [_i] * 8 + [_f, _i, _vp]),
    "fdattn_decode_attention_generic": (_i, [_vp] * 10 + [_i] + [_vp] * 2 + [_sz] + [_i] * 8 + [_f, _vp]),
    "fdattn_decode_attention_tiles": (_i, [_vp] * 10 + [_i] + [_vp] * 2 + [_sz] + [_i] * 8 + [_f, _vp]),
    "fdattn_decode_attention_sparse": (_i, [_vp] * 10 + [_i] + [_vp] * 2 + [_sz] + [_i] * 8 + [_f, _vp]),
    "fdattn_splitkv_combine": (_i, [_vp] * 5 + [_i] * 3 + [_vp]),
    "fdattn_sqattn_workspace_bytes": (_sz, [_i] * 3),
    "fdattn_sqattn_select": (_i, [_vp] * 10 + [_sz] + [_i] * 9 + [_vp]),
    "fdattn_sqattn_select_exact": (_i, [_vp] * 10 + [_sz] + [_i] * 9 + [_vp]),
    "fdattn_append_attention_prefill": (_i, [_vp] * 11 + [_i] * 10 + [_f, _vp]),
    "fdattn_append_attention_prefill_generic": (_i, [_vp] * 11 + [_i] * 10 + [_f, _vp]),
    "fdattn_append_attention_prefill_tiles": (_i, [_vp] * 11 + [_i] * 10 + [_f, _vp]),
    "fdattn_append_attention_workspace_bytes": (_sz, [_i] * 6),
    "fdattn_append_attention": (_i, [_vp] * 14 + [_sz] + [_i] * 12 + [_f, _vp]),
    "fdattn_prefill_auto_splits": (_i, [_i] * 3),
    "fdattn_prefill_auto_splits_for": (_i, [_i] * 4),
    "fdattn_append_attention_prefill_split_workspace_bytes": (_sz, [_i] * 3),
    "fdattn_append_attention_prefill_split": (_i, [_vp] * 12 + [_sz] + [_i] * 11 + [_f, _vp]),
    "fdattn_append_attention_workspace_bytes_ex": (_sz, [_i] * 7),
    "fdattn_write_cache_kv_ex": (_i, [_vp] * 13 + [_i] * 11 + [_vp, _vp]),
    "fdattn_append_attention_ex": (_i, [_vp] * 14 + [_sz] + [_i] * 12 + [_f, _vp, _vp]),
    "fdattn_pool_create": (_vp, [_i] * 4),
    "fdattn_pool_destroy": (None, [_vp]),
    "fdattn_pool_reserve": (_i, [_vp, _i, _i]),
    "fdattn_pool_release": (_i, [_vp, _i]),
    "fdattn_pool_fork": (_i, [_vp, _i, _i, _i]),
    "fdattn_pool_free_blocks": (_i, [_vp]),
    "fdattn_pool_seq_blocks": (_i, [_vp, _i]),
    "fdattn_pool_refcount": (_i, [_vp, _i]),
    "fdattn_pool_block_tables": (ctypes.POINTER(ctypes.c_int32), [_vp]),
    "fdattn_kv_wire_bytes": (_sz, [_i] * 4),
    "fdattn_kv_wire_bytes_for": (_sz, [_i] * 5),
    "fdattn_kv_export": (_i, [_vp] * 8 + [_i] * 8 + [_vp]),
    "fdattn_kv_import": (_i, [_vp] * 9 + [_i] * 8 + [_vp]),
}



class StepExtras(ctypes.Structure):
    """fdattn_step_extras of include/fdattn.h"""
    _fields_ = [("qkv_bias", _vp), ("q_norm_weight", _vp), ("k_norm_weight", _vp), ("rms_norm_eps", _f),
                ("prefill_rows", _i), ("sqattn_top_k", _i), ("decode_tokens", _i), ("sqattn_per_token", _i)]


_lib = None


class FdattnError(RuntimeError):
    """An entry point of libfdattn.so returned non-zero (the reference's ops throw, PD_THROW)."""


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FdattnError(
                "libfdattn.so is not built (%s missing): run `python -m fastdeploy_amd.build`; "
                "there is no CPU or PyTorch fallback for this path" % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(rc, what):
    if rc != 0:
        msg = lib().fdattn_last_error().decode()
        kind = ValueError if rc < 0 else FdattnError
        raise kind("%s failed (%d): %s" % (what, rc, msg))
