"""ctypes binding of libbibo_moe.so (declared in include/bibo_moe.h).

The library is the product: there is no Python or CPU fallback.  If it is missing, `lib()` raises."""
from __future__ import annotations

import ctypes
import pathlib
import threading

LIB_PATH = pathlib.Path(__file__).resolve().parent / "libbibo_moe.so"

DTYPE_BF16, DTYPE_F32 = 0, 1
NORM_NONE, NORM_SUM, NORM_SOFTMAX = 0, 1, 2
ALGO_AUTO, ALGO_GENERIC, ALGO_MFMA, ALGO_STREAM, ALGO_FUSED = 0, 1, 2, 3, 4
MAX_EXPERTS, MAX_TOPK = 64, 8
ACT_RADIAL_SIGMOID, ACT_RADIAL_TANH, ACT_SILU = 0, 1, 2
FLAG_ROUND_BLOCK_OUT, FLAG_NO_RESIDUAL = 1, 2
ABI_VERSION = 3

# every symbol include/bibo_moe.h declares
SYMBOLS = (
    "bibo_moe_abi_version", "bibo_moe_strerror", "bibo_moe_workspace_bytes", "bibo_moe_select_algo", "bibo_moe_router_fwd",
    "bibo_moe_permute", "bibo_moe_gateup_fwd", "bibo_moe_down_combine_fwd", "bibo_moe_gateup_down_fwd",
    "bibo_moe_combine_fwd", "bibo_moe_combine_ex_fwd", "bibo_moe_experts_fwd", "bibo_moe_forward", "bibo_moe_rmsnorm_fwd",
    "bibo_moe_ffn_workspace_bytes", "bibo_moe_ffn_forward", "bibo_moe_forward_static", "bibo_moe_backward_workspace_bytes", "bibo_moe_backward", "bibo_moe_experts_backward",
    "bibo_moe_train_state_bytes", "bibo_moe_forward_train", "bibo_moe_backward_saved",
    "bibo_moe_exp_attn_res_fwd",
)
STATIC_SCRATCH_BYTES = 16 << 20


class Shape(ctypes.Structure):
    _fields_ = [("T", ctypes.c_int32), ("H", ctypes.c_int32), ("E", ctypes.c_int32), ("k", ctypes.c_int32),
                ("I", ctypes.c_int32), ("dtype", ctypes.c_int32), ("n_pos", ctypes.c_int32), ("n_neg", ctypes.c_int32),
                ("act", ctypes.c_int32), ("flags", ctypes.c_int32)]


_lock = threading.Lock()
_lib = None


def _declare(l):
    vp, ci, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    l.bibo_moe_abi_version.restype = ci
    l.bibo_moe_abi_version.argtypes = []
    l.bibo_moe_strerror.restype = ctypes.c_char_p
    l.bibo_moe_strerror.argtypes = [ci]
    l.bibo_moe_workspace_bytes.restype = ci
    l.bibo_moe_workspace_bytes.argtypes = [ctypes.POINTER(Shape), ctypes.POINTER(sz)]
    l.bibo_moe_select_algo.restype = ci
    l.bibo_moe_select_algo.argtypes = [ctypes.POINTER(Shape), ci, ctypes.POINTER(ci)]
    l.bibo_moe_router_fwd.restype = ci
    l.bibo_moe_router_fwd.argtypes = [vp, vp, vp, ci, ci, ci, ci, ci, ci, vp, vp, vp, vp, vp]
    l.bibo_moe_permute.restype = ci
    l.bibo_moe_permute.argtypes = [vp, ci, ci, ci, vp, vp, vp, vp, vp, sz, vp]
    l.bibo_moe_gateup_fwd.restype = ci
    l.bibo_moe_gateup_fwd.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, vp, vp]
    l.bibo_moe_down_combine_fwd.restype = ci
    l.bibo_moe_down_combine_fwd.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, vp, vp, sz, vp]
    l.bibo_moe_gateup_down_fwd.restype = ci
    l.bibo_moe_gateup_down_fwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, vp, vp]
    l.bibo_moe_combine_fwd.restype = ci
    l.bibo_moe_combine_fwd.argtypes = [vp, ci, ci, ci, ci, ci, vp, vp]
    l.bibo_moe_combine_ex_fwd.restype = ci
    l.bibo_moe_combine_ex_fwd.argtypes = [vp, ci, vp, vp, vp, ci, ci, ci, vp, ci, ci, ci, ci, vp, vp]
    l.bibo_moe_experts_fwd.restype = ci
    l.bibo_moe_experts_fwd.argtypes = [vp, vp, vp, vp, vp, vp, ctypes.POINTER(Shape), ci, vp, vp, vp, sz, vp]
    l.bibo_moe_rmsnorm_fwd.restype = ci
    l.bibo_moe_rmsnorm_fwd.argtypes = [vp, vp, ctypes.c_float, ci, ci, ci, vp, vp]
    l.bibo_moe_ffn_workspace_bytes.restype = ci
    l.bibo_moe_ffn_workspace_bytes.argtypes = [ctypes.POINTER(Shape), ctypes.POINTER(sz)]
    l.bibo_moe_ffn_forward.restype = ci
    l.bibo_moe_ffn_forward.argtypes = [vp, vp, ctypes.c_float, vp, vp, vp, vp, vp, vp, ctypes.POINTER(Shape), ci, ci, vp, vp,
                                       vp, vp, vp, sz, vp]
    l.bibo_moe_forward_static.restype = ci
    l.bibo_moe_backward_workspace_bytes.restype = ci
    l.bibo_moe_backward_workspace_bytes.argtypes = [ctypes.POINTER(Shape), ctypes.POINTER(sz)]
    l.bibo_moe_backward.restype = ci
    l.bibo_moe_backward.argtypes = [vp, vp, vp, vp, vp, vp, vp, ctypes.POINTER(Shape), ci, vp, vp, vp, vp, vp, vp, vp, sz, vp]
    l.bibo_moe_experts_backward.restype = ci
    l.bibo_moe_experts_backward.argtypes = [vp, vp, vp, vp, vp, vp, vp, ctypes.POINTER(Shape), vp, vp, vp, vp, vp, vp, sz, vp]
    l.bibo_moe_train_state_bytes.restype = ci
    l.bibo_moe_train_state_bytes.argtypes = [ctypes.POINTER(Shape), ctypes.POINTER(sz)]
    l.bibo_moe_forward_train.restype = ci
    l.bibo_moe_forward_train.argtypes = [vp, vp, vp, vp, vp, vp, ctypes.POINTER(Shape), ci, vp, vp, vp, sz, vp, sz, vp]
    l.bibo_moe_backward_saved.restype = ci
    l.bibo_moe_backward_saved.argtypes = [vp, vp, vp, vp, vp, vp, ctypes.POINTER(Shape), ci, vp, sz, vp, vp, vp, vp, vp, vp, vp,
                                          sz, vp]
    l.bibo_moe_exp_attn_res_fwd.restype = ci
    l.bibo_moe_exp_attn_res_fwd.argtypes = [vp, ci, vp, ctypes.c_float, ci, ci, ci, vp, vp]
    l.bibo_moe_forward_static.argtypes = [vp, vp, vp, vp, vp, vp, ctypes.POINTER(Shape), ci, ci, vp, vp, vp, vp, vp, vp]
    l.bibo_moe_forward.restype = ci
    l.bibo_moe_forward.argtypes = [vp, vp, vp, vp, vp, vp, ctypes.POINTER(Shape), ci, ci, vp, vp, vp, vp, vp, vp, sz, vp]


def lib():
    """The loaded library; raises RuntimeError if it has not been built or does not match this binding."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not LIB_PATH.exists():
                raise RuntimeError(
                    f"{LIB_PATH} is missing: the HIP extension is not built (run `python -m bibo_amd.build`). "
                    "bibo_amd has no fallback path.")
            l = ctypes.CDLL(str(LIB_PATH))
            for name in SYMBOLS:
                if not hasattr(l, name):
                    raise RuntimeError(f"{LIB_PATH} does not export {name}; rebuild it")
            _declare(l)
            if l.bibo_moe_abi_version() != ABI_VERSION:
                raise RuntimeError(f"{LIB_PATH} has ABI {l.bibo_moe_abi_version()}, binding expects {ABI_VERSION}")
            _lib = l
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = lib().bibo_moe_strerror(code).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {code})")
