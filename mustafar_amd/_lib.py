"""ctypes binding of libmustafar_hip.so (the C ABI declared in include/mustafar_hip.h).

The library is the product: if it is missing the loader raises; nothing here falls back to a
CPU or PyTorch implementation.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmustafar_hip.so")

_lib = None

_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_u64 = ctypes.c_uint64
_sz = ctypes.c_size_t



class ProjSource(ctypes.Structure):
    """struct mstf_proj_source of include/mustafar_hip.h."""
    _fields_ = [("x", _vp), ("stride_batch", _i64), ("stride_token", _i64), ("stride_head", _i64),
                ("batch", _i), ("heads", _i), ("rows", _i),
                ("cos", _vp), ("sin", _vp), ("rope_stride_batch", _i64), ("rope_stride_token", _i64),
                ("rot", _vp), ("rot_stride_batch", _i64), ("rot_stride_token", _i64), ("rot_stride_head", _i64)]


_ps = ctypes.POINTER(ProjSource)

# name -> (restype, argtypes); must list every symbol of include/mustafar_hip.h
SIGNATURES = {
    "mstf_strerror": (ctypes.c_char_p, [_i]),
    "mstf_last_hip_error": (_i, []),
    "mstf_version": (_i, []),
    "mstf_probe_read": (_i, [_vp, _vp, _sz, _vp, _i]),
    "mstf_test_set_spin_limit": (None, [_i64]),
    "mstf_prune_rows_f16": (_i, [_vp, _vp, _vp, _i64, _i, _i]),
    "mstf_compress_workspace_bytes": (_sz, [_i, _i, _i]),
    "mstf_compress_key_f16": (_i, [_vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _u64, _vp, _sz]),
    "mstf_compress_value_f16": (_i, [_vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _u64, _vp, _sz]),
    "mstf_scatter_key_f16": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp, _u64]),
    "mstf_scatter_value_f16": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp, _u64]),
    "mstf_append_key_f16": (_i, [_vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz]),
    "mstf_append_value_f16": (_i, [_vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz]),
    "mstf_compress_kv_workspace_bytes": (_sz, [_i, _i, _i]),
    "mstf_compress_kv_f16": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _u64, _vp, _vp, _vp, _vp, _vp,
                                  _u64, _vp, _sz]),
    "mstf_append_kv_f16": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                _vp, _sz]),
    "mstf_compress_proj_f16": (_i, [_vp, _ps, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _u64, _vp, _sz]),
    "mstf_append_proj_f16": (_i, [_vp, _ps, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz]),
    "mstf_key_spmv_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    "mstf_value_spmv_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "mstf_value_spmv_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _sz]),
    "mstf_scale_softmax_f16": (_i, [_vp, _vp, _vp, _i64, _i, _i64, _i64, _i]),
    "mstf_decode_attention_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "mstf_decode_attention_splits": (_i, [_i, _i, _i, _i]),
    "mstf_decode_attention_f16": (_i, [_vp] * 12 + [_i, _i, _i, _i, _vp, _sz]),
    "mstf_decode_attention_static_f16": (_i, [_vp] * 12 + [_i, _i, _i, _i]),
    "mstf_decode_attention_partial_f16": (_i, [_vp] * 10 + [_i, _i, _i, _i, _vp, _sz]),
    "mstf_decode_attention_merge_f16": (_i, [_vp, _vp, _sz, _vp, _vp, _i, _i, _i, _i]),
    "mstf_decode_attention_window_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "mstf_decode_attention_window_f16": (_i, [_vp] * 12 + [_i, _vp, _i, _vp, _vp, _i, _i, _i, _i, _vp, _sz]),
    "mstf_decode_attention_window_pool_f16": (_i, [_vp] * 12 + [_i, _vp, _i, _vp, _vp, _i, _vp, _i64, _i, _i, _i, _vp,
                                                   _sz]),
    "mstf_decode_step_pool_f16": (_i, [_vp] * 9 + [_vp, _i64, _vp, _i64, _vp, _i64, _i, _i, _i, _vp, _vp, _i64, _vp, _vp, _i, _i,
                                       _vp, _vp, _vp, _vp, _i, _vp, _i64, _i, _vp, _sz]),
    "mstf_decode_step_quant_pool": (_i, [_vp] * 11 + [_vp, _i64, _vp, _i64, _vp, _i64, _i, _i, _i, _vp, _vp, _i64, _vp, _vp, _i,
                                         _i, _vp, _vp, _vp, _vp, _i, _vp, _i64, _i, _i, _i, _i, _vp, _sz]),
    "mstf_window_append_f16": (_i, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _i, _i, _i, _i, _vp, _vp, _i64, _vp, _vp, _vp, _i,
                               _i, _vp, _vp]),
    "mstf_compress_quant_workspace_bytes": (_sz, [_i, _i, _i]),
    "mstf_compress_key_quant": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u64, _vp,
                                     _sz]),
    "mstf_compress_value_quant": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u64,
                                       _vp, _sz]),
    "mstf_key_spmv_quant": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i]),
    "mstf_value_spmv_quant_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "mstf_value_spmv_quant": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i,
                                   _vp, _sz]),
    "mstf_decode_attention_quant": (_i, [_vp] * 14 + [_i, _i, _i, _i, _i, _i, _i, _vp, _sz]),
    "mstf_compress_quant_grouped": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u64,
                                         _vp, _sz]),
    "mstf_key_spmv_quant_grouped": (_i, [_vp] * 8 + [_i] * 9),
    "mstf_value_spmv_quant_grouped": (_i, [_vp] * 8 + [_i] * 9 + [_vp, _sz]),
    "mstf_decode_attention_quant_grouped": (_i, [_vp] * 14 + [_i] * 8 + [_vp, _sz]),
    "mstf_decode_attention_window_quant": (_i, [_vp] * 14 + [_i, _vp, _i, _vp, _vp] + [_i] * 7 + [_vp, _sz]),
    "mstf_decode_attention_window_quant_pool": (_i, [_vp] * 14 + [_i, _vp, _i, _vp, _vp, _i, _vp, _i64] + [_i] * 6
                                                + [_vp, _sz]),
}


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libmustafar_hip.so is missing at %s: build it with `python -m mustafar_amd.build` "
                "(there is no fallback implementation)" % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(rc, what):
    if rc != 0:
        l = lib()
        msg = l.mstf_strerror(rc).decode()
        extra = " (hipError %d)" % l.mstf_last_hip_error() if rc == -5 else ""
        raise RuntimeError("%s failed: %s%s" % (what, msg, extra))
