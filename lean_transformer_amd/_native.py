"""ctypes binding of csrc/libleanffn.so and csrc/libleanffn_f16.so (declarations: include/leanffn.h).

The two libraries are the same kernels with the 16-bit element type fixed at compile time (bfloat16 / IEEE binary16);
``lib(dtype)`` picks the one that computes in ``dtype``.  They are the only compute backend of this package: there is no
fallback.  ``lib()`` raises if the shared object has not been built (``python -m lean_transformer_amd._build``), and every
call raises ``RuntimeError`` with the library's own message when it returns a non-zero status.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int32, c_int64, c_size_t, c_uint8, c_uint64, c_void_p
from typing import Optional

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libleanffn.so")
F16_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libleanffn_f16.so")

LT_F32, LT_BF16, LT_F16 = 0, 1, 2
_DTYPES = {torch.float32: LT_F32, torch.bfloat16: LT_BF16, torch.float16: LT_F16}

# every function include/leanffn.h declares; the not-gpu tests check that the built library exports all of them
EXPORTED_SYMBOLS = (
    "lt_version", "lt_last_error",
    "lt_ffn_forward_workspace_bytes", "lt_ffn_backward_workspace_bytes", "lt_ffn_forward", "lt_ffn_backward",
    "lt_linear_backward_workspace_bytes", "lt_linear_forward", "lt_linear_backward", "lt_linear_check_out_group", "lt_linear_check_in_group",
    "lt_blocksparse_forward", "lt_blocksparse_backward",
    "lt_layernorm_forward", "lt_layernorm_backward_workspace_bytes", "lt_layernorm_backward",
    "lt_layernorm_backward_static_scratch_bytes", "lt_layernorm_backward_static",
    "lt_activation_forward", "lt_activation_backward", "lt_dropout_mask", "lt_gemm",
    "lt_profile_enable", "lt_profile_reset", "lt_profile_read",
)


class LtLinear(ctypes.Structure):
    _fields_ = [
        ("weight", c_void_p), ("bias", c_void_p), ("lowrank_first", c_void_p), ("lowrank_second", c_void_p),
        ("forward_indices", c_void_p), ("backward_indices", c_void_p),
        ("in_features", c_int32), ("out_features", c_int32), ("lowrank", c_int32), ("block", c_int32),
        ("blocks_per_out", c_int32), ("blocks_per_in", c_int32), ("out_group", c_int32), ("in_group", c_int32),
    ]


class LtLinearGrads(ctypes.Structure):
    _fields_ = [("weight", c_void_p), ("bias", c_void_p), ("lowrank_first", c_void_p), ("lowrank_second", c_void_p)]


class LtFfnDesc(ctypes.Structure):
    _fields_ = [
        ("tokens", c_int64), ("hidden", c_int32), ("intermediate", c_int32), ("gated", c_int32), ("act", c_int32),
        ("residual", c_int32), ("io_dtype", c_int32), ("compute_dtype", c_int32), ("ln_eps", c_float),
        ("dropout_p", c_float), ("dropout_seed", c_uint64), ("dropout_offset", c_uint64),
        ("ln_weight", c_void_p), ("ln_bias", c_void_p), ("post_ln_weight", c_void_p), ("post_ln_bias", c_void_p),
        ("i2h", LtLinear), ("h2o", LtLinear),
    ]


class LtProfileEntry(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 64), ("launches", c_int64), ("ms", ctypes.c_double), ("flops", ctypes.c_double),
                ("bytes", ctypes.c_double)]


class LtFfnSaved(ctypes.Structure):
    _fields_ = [("pre_activation", c_void_p), ("ln_stats", c_void_p), ("post_ln_input", c_void_p),
                ("i2h_lowrank_hid", c_void_p), ("h2o_lowrank_hid", c_void_p)]


class LtFfnGrads(ctypes.Structure):
    _fields_ = [("dx", c_void_p), ("ln_weight", c_void_p), ("ln_bias", c_void_p), ("post_ln_weight", c_void_p),
                ("post_ln_bias", c_void_p), ("i2h", LtLinearGrads), ("h2o", LtLinearGrads)]


_libs = {}


def _declare(lib):
    lib.lt_version.restype = c_char_p
    lib.lt_last_error.restype = c_char_p
    lib.lt_ffn_forward_workspace_bytes.restype = c_size_t
    lib.lt_ffn_forward_workspace_bytes.argtypes = [POINTER(LtFfnDesc)]
    lib.lt_ffn_backward_workspace_bytes.restype = c_size_t
    lib.lt_ffn_backward_workspace_bytes.argtypes = [POINTER(LtFfnDesc)]
    lib.lt_ffn_forward.argtypes = [POINTER(LtFfnDesc), c_void_p, c_void_p, POINTER(LtFfnSaved), c_void_p, c_size_t, c_void_p]
    lib.lt_ffn_backward.argtypes = [POINTER(LtFfnDesc), c_void_p, c_void_p, POINTER(LtFfnSaved), POINTER(LtFfnGrads),
                                    c_void_p, c_size_t, c_void_p]
    lib.lt_linear_backward_workspace_bytes.restype = c_size_t
    lib.lt_linear_backward_workspace_bytes.argtypes = [POINTER(LtLinear), c_int64, c_int32]
    lib.lt_linear_forward.argtypes = [POINTER(LtLinear), c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.lt_linear_check_out_group.argtypes = [POINTER(LtLinear), c_void_p, c_void_p]
    lib.lt_linear_check_in_group.argtypes = [POINTER(LtLinear), c_void_p, c_void_p]
    lib.lt_linear_backward.argtypes = [POINTER(LtLinear), c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p,
                                       POINTER(LtLinearGrads), c_void_p, c_size_t, c_void_p]
    lib.lt_blocksparse_forward.argtypes = [POINTER(LtLinear), c_int64, c_int32, c_void_p, c_void_p, c_void_p]
    lib.lt_blocksparse_backward.argtypes = [POINTER(LtLinear), c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_void_p]
    lib.lt_layernorm_forward.argtypes = [c_int64, c_int32, c_float, c_int32, c_void_p, c_void_p, c_void_p, c_int32,
                                         c_void_p, c_void_p, c_void_p]
    lib.lt_layernorm_backward_workspace_bytes.restype = c_size_t
    lib.lt_layernorm_backward_workspace_bytes.argtypes = [c_int64, c_int32]
    lib.lt_layernorm_backward.argtypes = [c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_void_p,
                                          c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]
    lib.lt_layernorm_backward_static_scratch_bytes.restype = c_size_t
    lib.lt_layernorm_backward_static_scratch_bytes.argtypes = []
    lib.lt_layernorm_backward_static.argtypes = [c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_void_p,
                                                 c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.lt_activation_forward.argtypes = [c_int64, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p]
    lib.lt_activation_backward.argtypes = [c_int64, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p,
                                           c_void_p]
    lib.lt_dropout_mask.argtypes = [c_int64, c_int32, c_float, c_uint64, c_uint64, c_void_p, c_void_p]
    lib.lt_gemm.argtypes = [c_int32, c_int64, c_int64, c_int64, c_void_p, c_int32, c_void_p, c_int32, c_int32, c_void_p,
                            c_int32, c_void_p]
    lib.lt_profile_enable.argtypes = [c_int32]
    lib.lt_profile_reset.argtypes = []
    lib.lt_profile_read.argtypes = [POINTER(LtProfileEntry), c_int32]
    for name in EXPORTED_SYMBOLS:
        fn = getattr(lib, name)
        if fn.restype is ctypes.c_int:  # default restype: these return lt_status
            fn.restype = c_int32


def available() -> bool:
    """whether the built library is there (the only caller: the stock-op path's choice of dropout mask; every kernel path
    calls lib() and fails loudly without it)"""
    return bool(_libs) or os.path.exists(LIB_PATH)


def lib(*dtypes: Optional[torch.dtype]):
    """The loaded library that computes in the given dtypes: libleanffn_f16.so when one of them is float16, libleanffn.so
    otherwise (float32 work runs on the same kernels in either).  Raises if the library was never built, and when float16
    and bfloat16 meet in one call (no kernel mixes them)."""
    f16 = torch.float16 in dtypes
    if f16 and torch.bfloat16 in dtypes:
        raise TypeError("float16 and bfloat16 tensors in one call: the kernels compute in one 16-bit type at a time")
    path = F16_LIB_PATH if f16 else LIB_PATH
    loaded = _libs.get(path)
    if loaded is None:
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} is missing: the HIP kernels of lean_transformer_amd are not built. "
                "Run `python -m lean_transformer_amd._build` (needs hipcc; cross-compiles for gfx950 without a GPU).")
        loaded = ctypes.CDLL(path)
        _declare(loaded)
        _libs[path] = loaded
    return loaded


def check(status: int, what: str, library=None):
    """raise with the message of the library that returned ``status`` (the bfloat16 one unless ``library`` is given)"""
    if status != 0:
        message = (library or lib()).lt_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (lt_status {status}): {message}")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TypeError(f"the HIP kernels take float32, bfloat16 and float16 tensors, not {dtype}") from None


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    """device address of a tensor (None -> NULL)"""
    return None if t is None else t.data_ptr()


def require_gpu(*tensors: Optional[torch.Tensor]):
    """All tensors must live on one GPU; there is no CPU implementation behind this package."""
    device = None
    for t in tensors:
        if t is None:
            continue
        if t.device.type != "cuda":
            raise RuntimeError(
                f"lean_transformer_amd runs on AMD GPUs only (got a tensor on {t.device}); its HIP kernels have no CPU "
                "counterpart. Move the module and its inputs to the GPU.")
        if device is None:
            device = t.device
        elif t.device != device:
            raise RuntimeError(f"tensors on different devices: {device} and {t.device}")
    return device


def current_stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    """scratch memory from PyTorch's caching allocator (256-byte aligned like every fresh block of it)"""
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def profile_read(library=None):
    """[(kernel tag, launches, total ms, algorithmic flops, algorithmic bytes)] recorded by ``library`` (the bfloat16 one
    unless given) since the last lt_profile_reset"""
    library = library or lib()
    entries = (LtProfileEntry * 64)()
    n = library.lt_profile_read(entries, 64)
    if n < 0:
        check(-n, "lt_profile_read", library)
    return [(e.name.decode(), e.launches, e.ms, e.flops, e.bytes) for e in entries[:min(n, 64)]]
