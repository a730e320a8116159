"""ctypes binding of libl3kernels.so (declared in include/l3_kernels.h).

Loading fails loudly: there is no CPU or PyTorch fallback for any operator.
"""

import ctypes
import os

_LIB_NAME = "libl3kernels.so"
_HERE = os.path.dirname(os.path.abspath(__file__))

L3_OK = 0
L3_ERR_NULL_POINTER = -1
L3_ERR_HEAD_SIZE = -2
L3_ERR_HEAD_RATIO = -3
L3_ERR_SHAPE = -4
L3_ERR_STRIDE = -5
L3_ERR_ALIGNMENT = -6
L3_ERR_WORKSPACE = -7
L3_ERR_SPLITS = -8
L3_ERR_HIP = -9
L3_ERR_FLAGS = -10
L3_ERR_SCRATCH = -11
L3_ERR_SCALE = -12
L3_ATTN_MAX_SPLITS = 512
L3_ATTN_STATIC_SCRATCH_BYTES = 16 << 20
L3_LINEAR_MAX_ROWS = 16         # one launch, any matrix shape, optional input norm / SwiGLU / residual / rope epilogue
L3_LINEAR_SPLITK_MAX_ROWS = 64
L3_LINEAR_STAGE_ELEMS = 24576   # activations (rows padded by 8) the fused input norm can stage in LDS
L3_ATTN_FLAG_KERNEL_FMA = 0x1
L3_ATTN_FLAG_WS_COUNTERS = 0x2
L3_ATTN_FLAG_FORM_COOP = 0x4
L3_ATTN_FLAG_FORM_STREAM = 0x8
L3_ATTN_FLAG_FORM_MASK = 0xc
L3_ATTN_FLAG_TWO_LAUNCHES = 0x40
L3_ATTN_COUNTER_BYTES = 128 << 10
L3_ATTN_FLAG_PREFILL_WAVE = 0x10
L3_ATTN_FLAG_PREFILL_TILED = 0x20
L3_ATTN_FLAG_PREFILL_TILED_NO_MAX = 0x30
L3_ATTN_FLAG_PREFILL_MASK = 0x30

# name -> (restype, argtypes); mirrors include/l3_kernels.h line by line
_c_i64p = ctypes.POINTER(ctypes.c_int64)
SIGNATURES = {
    "l3_version": (ctypes.c_int, []),
    "l3_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "l3_attn_choose_splits": (ctypes.c_int, [ctypes.c_int] * 6),
    "l3_attn_decode_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int] * 7),
    "l3_attn_decode": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,  # q k v out
         ctypes.c_void_p, ctypes.c_size_t,                                    # workspace, bytes
         ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,  # B QH KVH S HD
         _c_i64p, _c_i64p, _c_i64p, _c_i64p,                                  # strides
         ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p],        # scale splits flags stream
    ),
    "l3_attn_workspace_init": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "l3_attn_merge_in_launch_available": (ctypes.c_int, []),
    "l3_attn_launches": (ctypes.c_int, [ctypes.c_int] * 7),
    "l3_attn_placement_errors": (ctypes.c_int64, [ctypes.c_void_p]),
    "l3_attn_decode_static": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,  # q k v out
         ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,  # B QH KVH S HD
         _c_i64p, _c_i64p, _c_i64p, _c_i64p,                                  # strides
         ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p],        # scale splits flags stream
    ),
    "l3_attn_decode_devlen": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
         ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
         _c_i64p, _c_i64p, _c_i64p, _c_i64p, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
         ctypes.c_void_p],
    ),
    "l3_rot_embed_append": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64, _c_i64p, ctypes.c_int, ctypes.c_int,
         ctypes.c_void_p],
    ),
    "l3_attn_prefill": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,  # B QH KVH T S HD
         _c_i64p, _c_i64p, _c_i64p, _c_i64p, ctypes.c_float, ctypes.c_int, ctypes.c_void_p],
    ),
    "l3_attn_split": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,  # q k v part_o part_ml
         ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,                   # B QH KVH S HD
         _c_i64p, _c_i64p, _c_i64p, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p],
    ),
    "l3_attn_combine": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
         _c_i64p, ctypes.c_void_p],
    ),
    "l3_rms_norm": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float,
         ctypes.c_void_p],
    ),
    "l3_add_rms_norm": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
         ctypes.c_int, ctypes.c_float, ctypes.c_void_p],
    ),
    "l3_silu_mul": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]),
    "l3_linear_decode": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p],
    ),
    "l3_linear_swiglu_decode": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p],
    ),
    "l3_linear_decode_fused": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
         ctypes.c_void_p],
    ),
    "l3_linear_qkv_rope_append": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
         ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.POINTER(ctypes.c_int64), ctypes.c_int, ctypes.c_int,
         ctypes.c_void_p],
    ),
    "l3_silu_mul_rows": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
         ctypes.c_int64, ctypes.c_void_p],
    ),
    "l3_linear_splitk_plan": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "l3_linear_splitk_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "l3_linear_splitk": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p],
    ),
    "l3_linear_splitk_finish": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
         ctypes.c_void_p],
    ),
    "l3_add_rms_norm_partials": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_void_p],
    ),
    "l3_rot_embed_append_partials": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_int64),
         ctypes.c_int, ctypes.c_int, ctypes.c_void_p],
    ),
    "l3_greedy_step": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p],
    ),
    "l3_argmax_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int]),
    "l3_argmax": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
         ctypes.c_void_p, ctypes.c_void_p],
    ),
    "l3_rot_embed": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
         ctypes.c_int, _c_i64p, ctypes.c_void_p],
    ),
    "l3_hbm_read_stream": (
        ctypes.c_int, [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p],
    ),
    "l3_hbm_rw_stream": (
        ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_void_p],
    ),
}

_lib = None


def library_path() -> str:
    return os.environ.get("L3_KERNELS_LIB", os.path.join(_HERE, _LIB_NAME))


def load():
    """Return the loaded library (cached); raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise ImportError(
            f"{path} not found: build it with `python llama3-custom-inference_amd/build.py` "
            "(hipcc --offload-arch=gfx950). There is no fallback implementation."
        )
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = library/header mismatch
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def strerror(code: int) -> str:
    return load().l3_strerror(int(code)).decode()


_i64_arrays = {}


def i64_array(values):
    """A C array of int64 holding `values` (a sequence of ints).  Stride tuples repeat from call to
    call, so the arrays are kept; callers only ever pass them as read-only arguments."""
    if not isinstance(values, tuple):
        values = tuple(values)
    arr = _i64_arrays.get(values)
    if arr is None:
        arr = (ctypes.c_int64 * len(values))(*[int(v) for v in values])
        if len(_i64_arrays) < 4096:
            _i64_arrays[values] = arr
    return arr
