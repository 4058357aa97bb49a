"""ctypes binding of the C ABI declared in include/fp6mi.h. There is no CPU fallback: a missing library is an error."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfp6mi.so")
_lib = None


class Fp6miError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        msg = lib().fp6mi_error_string(code).decode()
        super().__init__("%s failed: %s (code %d)" % (where, msg, code))


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("fp6_llm_amd: %s is missing; build it with `python -m fp6_llm_amd.build` (needs hipcc). "
                          "There is no fallback path." % LIB_PATH)
    L = ctypes.CDLL(LIB_PATH)
    vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    sigs = {
        "fp6mi_error_string": (ctypes.c_char_p, [ci]),
        "fp6mi_version": (ci, []),
        "fp6mi_tuning_info": (ctypes.c_char_p, []),
        "fp6mi_prepack_ref": (ci, [ci, ci, vp, vp, sz, sz]),
        "fp6mi_dequant": (ci, [ci, ci, vp, vp, sz, sz, vp]),
        "fp6mi_unpack_ref": (ci, [ci, ci, vp, vp, sz, sz]),
        "fp6mi_native_bytes": (sz, [ci, ci, sz, sz]),
        "fp6mi_prepack_native": (ci, [ci, ci, vp, vp, sz, sz]),
        "fp6mi_relayout_ref_to_native": (ci, [ci, ci, vp, vp, sz, sz]),
        "fp6mi_unpack_native": (ci, [ci, ci, vp, vp, sz, sz]),
        "fp6mi_heuristic_splitk": (ci, [sz, sz, sz, ci]),
        "fp6mi_heuristic_splitk_format": (ci, [ci, ci, sz, sz, sz, ci]),
        "fp6mi_workspace_bytes": (sz, [sz, sz, ci]),
        "fp6mi_linear_native": (ci, [ci, ci, vp, vp, vp, vp, vp, sz, sz, sz, vp, ci]),
        "fp6mi_linear": (ci, [ci, ci, vp, vp, vp, vp, vp, sz, sz, sz, vp, ci]),
        "fp6mi_linear_stateless": (ci, [ci, ci, vp, vp, vp, vp, vp, sz, sz, sz, vp, ci, vp]),
        "fp6mi_linear_native_static": (ci, [ci, ci, vp, vp, vp, vp, vp, sz, sz, sz, ci]),
        "fp6mi_static_workspace_bytes": (sz, []),
        "fp6mi_init": (ci, []),
        "fp6mi_twin_evict": (ci, [vp]),
        "fp6mi_twin_clear": (ci, []),
        "fp6mi_linear_native_cfg": (ci, [ci, ci, vp, vp, vp, vp, vp, sz, sz, sz, vp, ci, ci, ci, ci, ci, ci]),
        "fp6mi_relayout_ref_to_native_gpu": (ci, [ci, ci, vp, vp, vp, sz, sz]),
        "fp6mi_dequant_native_gpu": (ci, [ci, ci, vp, vp, vp, vp, sz, sz]),
        "fp6mi_quantize_native_gpu": (ci, [ci, ci, vp, vp, vp, vp, ci, sz, sz]),
        "fp6mi_query_launch": (ci, [ci, ci, sz, sz, sz, ci, ctypes.POINTER(ci)]),
        "fp6mi_launch_source": (ci, [ci, ci, sz, sz, sz, ci]),
        "fp6mi_group_exps_bytes": (sz, [sz, sz]),
        "fp6mi_pack_group_exps": (ci, [vp, vp, sz, sz]),
        "fp6mi_dequant_grouped": (ci, [ci, ci, vp, vp, sz, sz, vp, vp]),
        "fp6mi_linear_native_grouped": (ci, [ci, ci, vp, vp, vp, vp, vp, vp, sz, sz, sz, vp, ci]),
        "fp6mi_dequant_native_grouped_gpu": (ci, [ci, ci, vp, vp, vp, vp, vp, sz, sz]),
        "fp6mi_linear_native_grouped_cfg": (ci, [ci, ci, vp, vp, vp, vp, vp, vp, sz, sz, sz, vp, ci, ci, ci, ci, ci, ci]),
        "fp6mi_quantize_native_grouped_gpu": (ci, [ci, ci, vp, vp, vp, vp, vp, ci, sz, sz]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


EXPORTED = ["fp6mi_error_string", "fp6mi_version", "fp6mi_tuning_info", "fp6mi_prepack_ref", "fp6mi_dequant", "fp6mi_unpack_ref",
            "fp6mi_native_bytes", "fp6mi_prepack_native", "fp6mi_relayout_ref_to_native", "fp6mi_unpack_native",
            "fp6mi_heuristic_splitk", "fp6mi_heuristic_splitk_format", "fp6mi_workspace_bytes", "fp6mi_linear_native", "fp6mi_linear_native_cfg", "fp6mi_linear", "fp6mi_linear_stateless", "fp6mi_twin_evict", "fp6mi_twin_clear",
            "fp6mi_linear_native_static", "fp6mi_static_workspace_bytes", "fp6mi_init",
            "fp6mi_relayout_ref_to_native_gpu", "fp6mi_dequant_native_gpu", "fp6mi_quantize_native_gpu", "fp6mi_query_launch", "fp6mi_launch_source",
            "fp6mi_group_exps_bytes", "fp6mi_pack_group_exps", "fp6mi_dequant_grouped", "fp6mi_linear_native_grouped", "fp6mi_linear_native_grouped_cfg",
            "fp6mi_dequant_native_grouped_gpu", "fp6mi_quantize_native_grouped_gpu"]


def check(code, where):
    if code != 0:
        raise Fp6miError(code, where)
