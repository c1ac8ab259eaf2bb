"""ctypes binding of libtqhip.so (declared in include/tqhip.h).

There is no CPU fallback: if the shared library is missing the import of any
kernel wrapper raises, and every wrapper refuses tensors that are not on a GPU.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("TQHIP_LIB", os.path.join(_HERE, "lib", "libtqhip.so"))

TQ_F32, TQ_F16, TQ_BF16 = 0, 1, 2
TQ_ENCODE_MLX, TQ_ENCODE_METAL = 0, 1
TQ_MMA_OFF, TQ_MMA_FP16, TQ_MMA_SPLIT = 0, 1, 2
TQ_OP_SPARSE_V, TQ_OP_FLASH_DECODE, TQ_OP_VONLY_DECODE = 0, 1, 2

_p = C.c_void_p
_i = C.c_int
_l = C.c_int64
_f = C.c_float
_fp = C.POINTER(C.c_float)
_z = C.c_size_t


class DecodeShape(C.Structure):
    """Mirror of struct tq_decode_shape."""
    _fields_ = [
        ("n_seq", C.c_int32), ("n_kv_heads", C.c_int32), ("n_rep", C.c_int32), ("dim", C.c_int32),
        ("bits", C.c_int32), ("block_size", C.c_int32),
        ("seq_len", C.c_int64), ("seq_offsets", C.c_void_p),
        ("k_seq_stride", C.c_int64), ("k_head_stride", C.c_int64),
        ("kn_seq_stride", C.c_int64), ("kn_head_stride", C.c_int64),
        ("v_seq_stride", C.c_int64), ("v_head_stride", C.c_int64),
        ("vn_seq_stride", C.c_int64), ("vn_head_stride", C.c_int64),
        ("mask", C.c_void_p), ("mask_seq_stride", C.c_int64), ("mask_head_stride", C.c_int64),
        ("attn_scale", C.c_float), ("out_dtype", C.c_int32), ("allow_mma", C.c_int32),
    ]


class VOnlyCacheDesc(C.Structure):
    """Mirror of struct tq_vonly_cache_desc."""
    _fields_ = [
        ("k_f16", C.c_void_p), ("v_raw", C.c_void_p), ("v_packed", C.c_void_p), ("v_norms", C.c_void_p),
        ("v_signs", C.c_void_p), ("boundaries", C.c_float * 15), ("centroids", C.c_float * 16),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t), ("t_alloc", C.c_int64),
        ("n_seq", C.c_int32), ("n_kv_heads", C.c_int32), ("n_rep", C.c_int32), ("dim", C.c_int32),
        ("bits", C.c_int32), ("variant", C.c_int32), ("allow_mma", C.c_int32),
    ]


class PackedCacheDesc(C.Structure):
    """Mirror of struct tq_packed_cache_desc."""
    _fields_ = [
        ("k_packed", C.c_void_p), ("k_norms", C.c_void_p), ("v_packed", C.c_void_p), ("v_norms", C.c_void_p),
        ("k_signs", C.c_void_p), ("v_signs", C.c_void_p), ("boundaries", C.c_float * 15), ("centroids", C.c_float * 16),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t), ("t_alloc", C.c_int64),
        ("n_seq", C.c_int32), ("n_kv_heads", C.c_int32), ("n_rep", C.c_int32), ("dim", C.c_int32),
        ("bits", C.c_int32), ("variant", C.c_int32),
    ]


# name -> (restype, argtypes); the authoritative list of exported symbols
PROTOTYPES = {
    "tq_version": (_i, []),
    "tq_last_error": (C.c_char_p, []),
    "tq_status_string": (C.c_char_p, [_i]),
    "tq_encode": (_i, [_p, _i, _p, _fp, _p, _p, _l, _l, _l, _l, _i, _i, _i, _p]),
    "tq_vonly_append": (_i, [_p, _i, _p, _i, _p, _fp, _p, _p, _p, _p, _l, _l, _l, _l, _l, _l, _i, _i, _i, _p]),
    "tq_dequant": (_i, [_p, _p, _fp, _p, _p, _i, _l, _l, _l, _l, _l, _i, _i, _p]),
    "tq_prerotate_query": (_i, [_p, _i, _p, _p, _l, _i, _p]),
    "tq_prerot_qk_scores": (_i, [_p, _p, _p, _fp, _p, _i, _i, _l, _l, _l, _i, _i, _i, _p]),
    "tq_packed_qk_scores": (_i, [_p, _p, _p, _fp, _p, _p, _i, _l, _l, _l, _i, _i, _p]),
    "tq_dense_qk_scores": (_i, [_p, _i, _p, _p, _i, _i, _l, _l, _i, _f, _p]),
    "tq_softmax_rows": (_i, [_p, _p, _l, _p, _l, _l, _f, _p]),
    "tq_sparse_v_matvec": (_i, [_p, _p, _p, _fp, _p, _p, _p, _z, _i, _i, _l, _l, _l, _i, _i, _f, _i, _p]),
    "tq_flash_decode": (_i, [_p, _p, _p, _p, _p, _fp, _fp, _p, _p, _p, _z, C.POINTER(DecodeShape), _p]),
    "tq_flash_decode_plan": (_i, [_i, _i, _l, _i, _i]),
    "tq_vonly_decode_attn": (_i, [_p, _i, _p, _p, _p, _fp, _p, _p, _p, _z, C.POINTER(DecodeShape), _p]),
    "tq_vonly_decode_attn_static": (_i, [_p, _i, _p, _p, _p, _fp, _p, _p, C.POINTER(DecodeShape), _p]),
    "tq_vonly_decode_step": (_i, [C.POINTER(VOnlyCacheDesc), _p, _i, _p, _i, _p, _i, _p, _i, _l, _f, _p]),
    "tq_packed_decode_step": (_i, [C.POINTER(PackedCacheDesc), _p, _i, _p, _i, _p, _i, _p, _i, _l, _f, _p]),
    "tq_vonly_append_at": (_i, [_p, _i, _p, _i, _p, _fp, _p, _p, _p, _p, _l, _l, _l, _i, _i, _i, _p, _p]),
    "tq_vonly_decode_step_at": (_i, [C.POINTER(VOnlyCacheDesc), _p, _i, _p, _i, _p, _i, _p, _i, _p, _f, _p]),
    "tq_packed_decode_step_at": (_i, [C.POINTER(PackedCacheDesc), _p, _i, _p, _i, _p, _i, _p, _i, _p, _f, _p]),
    "tq_vonly_decode_attn_phases": (_i, [_p, _i, _p, _p, _p, _fp, _p, _p, _p, _z, C.POINTER(DecodeShape), _i, _p]),
    "tq_vonly_sparse_decode_attn": (_i, [_p, _i, _p, _p, _p, _fp, _p, _f, _p, _p, _z, C.POINTER(DecodeShape), _p]),
    "tq_vonly_sparse_workspace_bytes": (_z, [_i, _i, _l]),
    "tq_flash_decode_from_q": (_i, [_p, _i, _p, _p, _p, _p, _p, _fp, _fp, _p, _f, _p, _p, _z, C.POINTER(DecodeShape), _p]),
    "tq_flash_sparse_decode": (_i, [_p, _p, _p, _p, _p, _fp, _fp, _p, _f, _p, _p, _z, C.POINTER(DecodeShape), _p]),
    "tq_workspace_bytes": (_z, [_i, _i, _i, _l, _i]),
    "tq_prefill_attn": (_i, [_p, _i, _p, _p, _p, _p, _fp, _fp, _p, _p, _p, _i, _p, _z, _i, _i, _l, _l, _l,
                            _l, _l, _l, _l, _i, _i, _f, _i, _p]),
    "tq_prefill_workspace_bytes": (_z, [_i, _l, _l, _i]),
    "tq_probe_read": (_i, [_p, _z, _p, _i, _z, _p]),
}

_lib = None


def load():
    """Load libtqhip.so once; raises OSError with the build hint if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise OSError(
            f"libtqhip.so not found at {LIB_PATH}; build it with "
            f"`make -C {os.path.join(os.path.dirname(_HERE), 'csrc')}` (needs hipcc, targets gfx950)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


# statuses whose reference counterpart is a ValueError raised before launch
# (sparse_v.py:147-157, flash_attention.py:224-234, metal_kernels_v4.py:138-139,188-191,
#  quantizer.py:37-38)
_VALUE_ERRORS = {-2, -3, -4, -7, -9}
STATIC_SCRATCH_BYTES = 4 << 20     # TQ_STATIC_SCRATCH_BYTES of include/tqhip.h


def check(status: int) -> None:
    if status == 0:
        return
    msg = load().tq_last_error().decode("utf-8", "replace")
    if status in _VALUE_ERRORS:
        raise ValueError(msg)
    raise RuntimeError(f"libtqhip error {status}: {msg}")


def host_floats(values) -> C.Array:
    vals = [float(v) for v in values]
    return (C.c_float * len(vals))(*vals)
