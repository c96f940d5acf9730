"""ctypes binding of csrc/libslimk_w2a8.so (the C ABI in include/slimk_w2a8.h).

There is deliberately no fallback: if the shared library is missing or a call
fails, an exception is raised.
"""
import ctypes
import os
import subprocess

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.path.join(_CSRC, "libslimk_w2a8.so")

OK = 0
F16, BF16 = 0, 1
KERNEL_AUTO, KERNEL_SKINNY, KERNEL_TILED, KERNEL_MID = 0, 1, 2, 3
DUMP_NONE, DUMP_GROUPS, DUMP_SUM = 0, 1, 2
QUANT_REF, QUANT_SYM, QUANT_ASYM = 0, 1, 2

# every symbol include/slimk_w2a8.h declares: (restype, argtypes)
_vp, _i, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
SIGNATURES = {
    "slimk_w2a8_version": (_i, []),
    "slimk_w2a8_arch": (ctypes.c_char_p, []),
    "slimk_w2a8_last_error": (ctypes.c_char_p, []),
    "slimk_w2a8_repacked_weight_bytes": (_sz, [_i, _i]),
    "slimk_w2a8_repacked_scale_bytes": (_sz, [_i, _i, _i]),
    "slimk_w2a8_repacked_zp_bytes": (_sz, [_i, _i, _i]),
    "slimk_w2a8_gemm_auto_split_k": (_i, [_i, _i, _i, _i, _i]),
    "slimk_w2a8_gemm_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i]),
    "slimk_w2a8_gemm_auto_route": (_i, [_i, _i, _i, _i]),
    "slimk_w2a8_workspace_init": (_i, [_vp, _sz, _vp]),
    "slimk_w2a8_repack": (_i, [_vp, _i, _vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "slimk_w2a8_quantize_weight": (_i, [_vp, _i, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp, _vp]),
    "slimk_w2a8_quantize_weight4": (_i, [_vp, _i, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp, _vp]),
    "slimk_w2a8_act_quant": (_i, [_vp, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp, _i, _vp]),
    "slimk_w2a8_act_quant_rep": (_i, [_vp, _i, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp, _i, _vp]),
    "slimk_w2a8_gemm": (_i, [_vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i,
                             _vp, _i, _i, _vp, _i, _vp, _sz, _i, _i, _vp]),
    "slimk_w2a8_static_workspace_bytes": (_sz, []),
    "slimk_w2a8_gemm_static": (_i, [_vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _vp]),
    "slimk_w2a8_gemm_fused": (_i, [_vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _i, _i, _vp, _sz, _i, _vp]),
    "slimk_w2a8_gemm_fused_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "slimk_w2a8_set_fused_spin_limit": (_i, [_i]),
    "slimk_w2a8_gemm_grouped": (_i, [_vp, _i, _i, _i, _vp]),
    "slimk_w2a8_gemm_grouped_verify": (_i, [_vp, _i, _i, _i, _vp, _i, _vp]),
    "slimk_w4a8_gemm_auto_split_k": (_i, [_i, _i, _i, _i]),
    "slimk_w4a8_gemm_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "slimk_w4a8_gemm": (_i, [_vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i, _i, _vp, _sz, _i, _vp]),
    "slimk_w2a16_gemm_auto_split_k": (_i, [_i, _i, _i, _i]),
    "slimk_w2a16_gemm_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "slimk_w2a16_gemm": (_i, [_vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _i, _i, _vp, _sz, _i, _vp]),
    "slimk_w2a16_gemm_grouped": (_i, [_vp, _i, _i, _i, _i, _vp]),
    "slimk_w2a8_read_probe": (_i, [_vp, _sz, _vp, _vp]),
}
MAX_GROUP = 24
COUNTER_BLOCK_BYTES = 64 << 10  # SLIMK_W2A8_COUNTER_BLOCK_BYTES


class Problem(ctypes.Structure):
    """struct slimk_w2a8_problem"""
    _fields_ = [("q", _vp), ("s_a", _vp), ("rowsum", _vp), ("w_r", _vp), ("s_r", _vp), ("zp_r", _vp), ("out", _vp),
                ("ldq", _i), ("ldr", _i), ("ldo", _i), ("M", _i), ("N", _i), ("K", _i), ("zp_const", _i)]


class Problem16(ctypes.Structure):
    """struct slimk_w2a16_problem"""
    _fields_ = [("x", _vp), ("w_r", _vp), ("s_r", _vp), ("zp_r", _vp), ("out", _vp),
                ("ldx", _i), ("ldo", _i), ("M", _i), ("N", _i), ("K", _i), ("zp_const", _i)]


class SlimkError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"slimk_w2a8 error {code}: {text}")
        self.code = code


def build(verbose=False):
    """Compile the library in-tree with hipcc for gfx950 (cross-compiles without a GPU)."""
    subprocess.run(["make", "-C", _CSRC, "-B", "-j8", "libslimk_w2a8.so"], check=True,
                   stdout=None if verbose else subprocess.DEVNULL,
                   stderr=None if verbose else subprocess.DEVNULL)
    return LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                f"or `make -C {_CSRC}`; slimkernels_amd has no CPU fallback for the GPU path")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc):
    if rc != OK:
        raise SlimkError(rc, lib().slimk_w2a8_last_error().decode("utf-8", "replace"))
