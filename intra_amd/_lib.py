"""ctypes binding of libintra_hip.so (declared in include/intra_hip.h)."""
import ctypes
import functools
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# INTRA_HIP_LIB overrides the in-tree build (e.g. to try another build of the same ABI)
LIB_PATH = os.environ.get("INTRA_HIP_LIB") or os.path.join(_HERE, "libintra_hip.so")
DIAG_LIB_PATH = os.path.join(_HERE, "libintra_hip_diag.so")  # the -DINTRA_DIAG_TIMERS build (measurement only)

INTRA_OK, INTRA_ERR_INVALID, INTRA_ERR_UNSUPPORTED, INTRA_ERR_HIP = 0, 1, 2, 3

_i64x3 = ctypes.c_int64 * 3


class IntraPlan(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int), ("heads_per_block", ctypes.c_int), ("waves", ctypes.c_int),
                ("pos_per_block", ctypes.c_int), ("n_sets", ctypes.c_int), ("n_mblocks", ctypes.c_int),
                ("work_items", ctypes.c_int), ("grid", ctypes.c_int), ("lds_bytes", ctypes.c_int), ("launches", ctypes.c_int),
                ("pairs_per_head", ctypes.c_int64)]


_FWD_ARGS = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 4 + [ctypes.POINTER(ctypes.c_int64)] * 4 + \
    [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_void_p]

SYMBOLS = {
    "intra_llm_fwd": (ctypes.c_int, _FWD_ARGS),
    "intra_image_fwd": (ctypes.c_int, _FWD_ARGS),
    "intra_llm_fwd_lse": (ctypes.c_int, _FWD_ARGS + [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64)]),
    "intra_image_fwd_lse": (ctypes.c_int, _FWD_ARGS + [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64)]),
    "intra_llm_fwd_ex": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_int] * 4 + [ctypes.POINTER(ctypes.c_int64)] * 4 +
                         [ctypes.c_int] * 6 + [ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p,
                                               ctypes.POINTER(ctypes.c_int64), ctypes.c_uint]),
    "intra_image_fwd_ex": (ctypes.c_int, _FWD_ARGS + [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64), ctypes.c_uint]),
    "intra_llm_bwd": (ctypes.c_int, [ctypes.c_void_p] * 10 + [ctypes.c_int] * 4 + [ctypes.POINTER(ctypes.c_int64)] * 9 +
                      [ctypes.c_int] * 6 + [ctypes.c_float, ctypes.c_void_p]),
    "intra_llm_bwd_noalloc": (ctypes.c_int, [ctypes.c_void_p] * 9 + [ctypes.c_int] * 4 + [ctypes.POINTER(ctypes.c_int64)] * 9 +
                              [ctypes.c_int] * 6 + [ctypes.c_float, ctypes.c_void_p]),
    "intra_image_bwd": (ctypes.c_int, [ctypes.c_void_p] * 10 + [ctypes.c_int] * 4 + [ctypes.POINTER(ctypes.c_int64)] * 9 +
                        [ctypes.c_int] * 3 + [ctypes.c_float, ctypes.c_void_p]),
    "intra_image_bwd_workspace": (ctypes.c_int64, [ctypes.c_int] * 7),
    "intra_llm_bwd_workspace": (ctypes.c_int64, [ctypes.c_int] * 10),
    "intra_model_mask_llm_bwd": (ctypes.c_int, [ctypes.c_int] * 7 + [ctypes.c_void_p]),
    "intra_model_mask_image_bwd": (ctypes.c_int, [ctypes.c_int] * 4 + [ctypes.c_void_p]),
    "intra_plan_llm_ex": (ctypes.c_int, [ctypes.c_int] * 10 + [ctypes.POINTER(IntraPlan)]),
    "intra_model_mask_llm_ex": (ctypes.c_int, [ctypes.c_int] * 8 + [ctypes.c_void_p]),
    "intra_last_error": (ctypes.c_char_p, []),
    "intra_version": (ctypes.c_int, []),
    "intra_set_softmax_mode": (ctypes.c_int, [ctypes.c_int]),
    "intra_get_softmax_mode": (ctypes.c_int, []),
    "intra_diag_set_buffer": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64]),
    "intra_diag_ablation": (ctypes.c_int, []),
    "intra_diag_mfma_ceiling": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_int] * 3 + [ctypes.c_void_p]),
    "intra_plan": (ctypes.c_int, [ctypes.c_int] * 8 + [ctypes.POINTER(IntraPlan)]),
    "intra_model_mask": (ctypes.c_int, [ctypes.c_int] * 7 + [ctypes.c_void_p]),
    "intra_model_deal": (ctypes.c_int, [ctypes.c_int] * 10 + [ctypes.c_void_p, ctypes.c_int64]),
}

_lib = None


def load():
    """Load the shared library once.  Raises ImportError if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is not built; run `python -m intra_amd.build`")
        try:
            lib = ctypes.CDLL(LIB_PATH)
        except OSError as err:
            raise ImportError(f"cannot load {LIB_PATH}: {err}") from err
        for name, (res, args) in SYMBOLS.items():
            try:
                fn = getattr(lib, name)
            except AttributeError as err:  # a library from an older source tree
                raise ImportError(f"{LIB_PATH} is stale (no symbol {name}); run `python -m intra_amd.build`") from err
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def last_error():
    return load().intra_last_error().decode()


@functools.lru_cache(maxsize=256)
def _strides_array(s0, s1, s2):
    return _i64x3(s0, s1, s2)


def strides3(x):
    """The first three element strides of a tensor ((batch, token, head) of a (B, S, H, D) tensor)
    as a C array; the arrays are read-only for the library and cached."""
    st = x.stride()
    return _strides_array(st[0], st[1], st[2])
