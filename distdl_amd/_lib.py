"""ctypes binding of ``libdistdl_hip.so`` (the C ABI declared in
``include/distdl_hip.h``).

The library is the only compute path of this package: there is no eager or CPU
fallback.  If it has not been built, or a tensor does not live on a GPU, the
callers below raise instead of computing something else.
"""

import ctypes
import os
from ctypes import POINTER
from ctypes import c_char_p
from ctypes import c_double
from ctypes import c_float
from ctypes import c_int
from ctypes import c_int32
from ctypes import c_int64
from ctypes import c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdistdl_hip.so")

DDL_MAX_DIMS = 8

DDL_OP_COPY = 0
DDL_OP_ADD = 1

DDL_DT_BITS = 0
DDL_DT_F32 = 1
DDL_DT_F64 = 2
DDL_DT_BF16 = 3
DDL_DT_F16 = 4
DDL_DT_I32 = 5
DDL_DT_I64 = 6

DDL_HALO_AUTO = 0
DDL_HALO_ROWS = 1
DDL_HALO_LINES = 2

DDL_EMBEDDING_BACKWARD_STATIC_MAX_ELEMS = 1048576


class ddl_box_t(ctypes.Structure):
    _fields_ = [
        ("src", c_void_p),
        ("dst", c_void_p),
        ("ndim", c_int32),
        ("reserved", c_int32),
        ("shape", c_int64 * DDL_MAX_DIMS),
        ("src_stride", c_int64 * DDL_MAX_DIMS),
        ("dst_stride", c_int64 * DDL_MAX_DIMS),
    ]


# name -> (restype, argtypes); every symbol include/distdl_hip.h declares.
SIGNATURES = {
    "ddl_version": (c_char_p, []),
    "ddl_last_error": (c_char_p, []),
    "ddl_copy_boxes": (c_int, [POINTER(ddl_box_t), c_int, c_int, c_int, c_int, c_void_p]),
    "ddl_sum_boxes": (c_int, [POINTER(ddl_box_t), POINTER(c_void_p), c_int, c_int, c_int, c_double, c_void_p]),
    "ddl_pack_boxes": (c_int, [c_void_p, POINTER(c_int64), POINTER(c_int64), c_int, c_int, c_int,
                               POINTER(c_int64), POINTER(c_int64), POINTER(c_void_p), c_void_p]),
    "ddl_unpack_boxes": (c_int, [c_void_p, POINTER(c_int64), POINTER(c_int64), c_int, c_int, c_int,
                                 POINTER(c_int64), POINTER(c_int64), POINTER(c_void_p), c_int, c_int, c_void_p]),
    "ddl_zero_boxes": (c_int, [c_void_p, POINTER(c_int64), POINTER(c_int64), c_int, c_int, c_int,
                               POINTER(c_int64), POINTER(c_int64), c_void_p]),
    "ddl_halo_pad_exchange": (c_int, [c_void_p, c_void_p, POINTER(c_int64), c_int, c_int, POINTER(c_int64),
                                      POINTER(c_int64), POINTER(c_int64), POINTER(c_void_p), POINTER(c_void_p),
                                      c_int, c_void_p]),
    "ddl_ln_partial_stats": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "ddl_ln_normalize_affine": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, POINTER(c_int64),
                                        c_void_p, c_void_p, c_float, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "ddl_layer_norm": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_float, c_void_p, c_int64,
                               c_void_p, c_void_p, c_void_p]),
    "ddl_ln_stats_normalize": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_int, POINTER(c_int64),
                                       c_void_p, c_void_p, c_float, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "ddl_ln_partial_stats_f32": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "ddl_ln_normalize_affine_f32": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int, POINTER(c_int64),
                                            c_void_p, c_void_p, c_float, c_void_p, c_int64, c_void_p, c_void_p,
                                            c_void_p]),
    "ddl_ln_bwd_partial": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_void_p]),
    "ddl_ln_bwd_input": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_int, c_float, c_void_p, c_int64, c_void_p]),
    "ddl_ln_bwd_params": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_int64, c_void_p]),
    "ddl_ln_bwd_partial_params": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                          c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "ddl_ln_bwd_input_params": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_int, c_float, c_void_p, c_int64, c_void_p, c_int64,
                                        c_void_p, c_void_p, c_void_p]),
    "ddl_ln_bwd_one_pass": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_int, c_int, c_float, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p,
                                    c_void_p]),
    "ddl_ln_bwd_partial_f32": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                       c_void_p, c_void_p]),
    "ddl_ln_bwd_input_f32": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_int, c_float, c_void_p, c_int64, c_void_p]),
    "ddl_ln_bwd_params_f32": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_void_p, c_int64, c_void_p]),
    "ddl_ln_bwd_partial_params_f32": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                              c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "ddl_ln_bwd_input_params_f32": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_int, c_float, c_void_p, c_int64, c_void_p, c_int64,
                                            c_void_p, c_void_p, c_void_p]),
    "ddl_embedding_gather": (c_int, [c_void_p, c_int64, c_int64, c_int, c_void_p, c_int, c_int64, c_int64, c_int64,
                                     c_void_p, c_void_p]),
    "ddl_embedding_renorm": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int64, c_int64, c_int64, c_float,
                                     c_float, c_void_p, c_void_p]),
    "ddl_embedding_backward": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64,
                                       c_int, c_void_p, c_int64, c_void_p, c_int64, c_void_p]),
    "ddl_embedding_backward_static": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int64, c_int64, c_int64,
                                              c_int64, c_int, c_void_p, c_int64, c_void_p]),
    "ddl_linear": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int64,
                           c_int64, c_void_p]),
    "ddl_gemm": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int, c_int64, c_int64,
                         c_int64, c_int64, c_void_p]),
    "ddl_gemm_f32": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int64,
                             c_int64, c_int64, c_void_p]),
    "ddl_colsum": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_void_p]),
    "ddl_linear_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                c_int64, c_void_p]),
    "ddl_transpose_2d": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p]),
    "ddl_colsum_bf16": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_void_p]),
}

_lib = None


class HipLibraryMissing(RuntimeError):
    pass


def load():
    """Loads the shared library once and declares every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HipLibraryMissing(
            f"{LIB_PATH} is not built; run `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or __graft_entry__.build()). distdl_amd has no fallback compute path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(rc, what):
    if rc != 0:
        msg = load().ddl_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed with code {rc}: {msg}")


def i64_array(values):
    values = [int(v) for v in values]
    return (c_int64 * max(len(values), 1))(*values)


def ptr_array(values):
    return (c_void_p * max(len(values), 1))(*[None if v in (None, 0) else int(v) for v in values])
