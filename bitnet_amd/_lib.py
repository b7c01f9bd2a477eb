"""ctypes binding of libbitlinear_hip.so (the C ABI in include/bitlinear_hip.h).

The library is the only compute path: if it has not been built, loading
raises -- there is no fallback.
"""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "lib", "libbitlinear_hip.so")

_c_int = ctypes.c_int
_c_ptr = ctypes.c_void_p

# name -> (restype, argtypes); mirrors include/bitlinear_hip.h one to one
SIGNATURES = {
    "bitlinear_int8xint2": (None, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr]),
    "bitlinear_last_status": (_c_int, []),
    "bitlinear_status_string": (ctypes.c_char_p, [_c_int]),
    "bitlinear_ws_num": (_c_int, [_c_int, _c_int]),
    "bitlinear_last_kernel": (ctypes.c_char_p, []),
    "bitlinear_forward_bf16_acc_i32": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "bitlinear_int8xint2_acc_i32": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "bitlinear_int8xint2_seg": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, ctypes.POINTER(_c_int), _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "bitlinear_quant_absmax": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr]),
    "bitlinear_quant_absmax_rowsum": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr]),
    "bitlinear_repacked_size": (ctypes.c_size_t, [_c_int, _c_int]),
    "bitlinear_repack": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr]),
    "bitlinear_forward_bf16": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "bitlinear_forward_bf16_static": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "bitlinear_norm_forward_bf16": (
        _c_int,
        [_c_ptr, _c_ptr, ctypes.c_float, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
         _c_int, _c_ptr],
    ),
    "bitlinear_forward_bf16_seg": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, ctypes.POINTER(_c_int), _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
         _c_ptr],
    ),
    "bitlinear_norm_forward_bf16_seg": (
        _c_int,
        [_c_ptr, _c_ptr, ctypes.c_float, _c_int, _c_ptr, _c_ptr, ctypes.POINTER(_c_int), _c_int, _c_ptr, _c_ptr, _c_ptr,
         _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "bitnet_attn_decode": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_ptr],
    ),
    "bitnet_attn_decode_rows": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_int, _c_ptr],
    ),
    "bitnet_decode_step_begin": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "bitnet_attn_decode_workspace_floats": (_c_int, [_c_int, _c_int, _c_int, _c_int]),
    "bitnet_attn_decode_error_index": (_c_int, [_c_int, _c_int, _c_int, _c_int]),
    "bitnet_attn_decode_set_spin_limit": (_c_int, [_c_int]),
    "bitnet_attn_prefill": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "bitnet_rope_cache_tokens": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "bitnet_attn_decode_set_threads": (_c_int, [_c_int]),
    "bitnet_lm_head_greedy": (
        _c_int,
        [_c_ptr, _c_ptr, ctypes.c_float, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "bitnet_lm_head_greedy_step": (
        _c_int,
        [_c_ptr, _c_ptr, ctypes.c_float, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
         _c_int, _c_int, _c_int, _c_ptr],
    ),
    "bitnet_lm_head_workgroups": (_c_int, [_c_int]),
    "bitnet_lm_head_set_kernel": (_c_int, [_c_int]),
    "bitlinear_set_tuning": (_c_int, [_c_int, _c_int, _c_int, _c_int]),
    "bitlinear_plan_name": (_c_int, [_c_int, _c_int, _c_int, _c_int, ctypes.c_char_p, _c_int]),
    "bitlinear_int8xint2_grouped": (_c_int, [_c_ptr, _c_int, _c_ptr]),
    # include/bitlinear_probes.h
    "bitlinear_probe_empty": (_c_int, [_c_int, _c_int, _c_ptr]),
    "bitlinear_probe_weight_stream": (_c_int, [_c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr]),
    "bitlinear_probe_mfma_i8": (_c_int, [_c_int, _c_int, _c_ptr, _c_ptr, _c_ptr]),
    "bitlinear_probe_flag_roundtrip": (_c_int, [_c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr]),
}


class Problem(ctypes.Structure):
    """struct bitlinear_problem of include/bitlinear_hip.h."""

    _fields_ = [
        ("input0", _c_ptr),
        ("input1", _c_ptr),
        ("output0", _c_ptr),
        ("s", _c_ptr),
        ("ws", _c_ptr),
        ("M", _c_int),
        ("N", _c_int),
        ("K", _c_int),
    ]

_lib = None


class BitLinearLibraryError(RuntimeError):
    pass


def load_library(path: str = None) -> ctypes.CDLL:
    """Open the shared library and type its entry points.  Raises
    BitLinearLibraryError when the .so is missing or lacks a symbol."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or os.environ.get("BITLINEAR_HIP_LIB", LIB_PATH)
    if not os.path.exists(p):
        raise BitLinearLibraryError(
            f"{p} not found: build it with `python -m bitnet_amd.build` (hipcc, gfx950); there is no fallback path"
        )
    try:
        lib = ctypes.CDLL(p)
    except OSError as e:  # missing ROCm runtime, wrong arch, ...
        raise BitLinearLibraryError(f"cannot load {p}: {e}") from e
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise BitLinearLibraryError(f"{p} does not export {name}") from e
        fn.restype = restype
        fn.argtypes = argtypes
    if path is None:
        _lib = lib
    return lib


def plan_name(entry: int, M: int, N: int, K: int) -> str:
    """bitlinear_plan_name: the kernels (template arguments, grid, block, LDS) a call would launch; needs no GPU."""
    buf = ctypes.create_string_buffer(1024)
    st = load_library().bitlinear_plan_name(entry, M, N, K, buf, len(buf))
    if st != 0:
        raise BitLinearLibraryError(f"bitlinear_plan_name(entry={entry}, M={M}, N={N}, K={K}): status {st}")
    return buf.value.decode()


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load_library().bitlinear_status_string(status).decode()
        raise BitLinearLibraryError(f"{what}: status {status} ({msg})")
