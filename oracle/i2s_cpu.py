"""ctypes access to the C restatement of the reference's CPU I2_S kernels
(oracle/i2s_cpu.c).  TEST INFRASTRUCTURE ONLY -- checker and CPU baseline."""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "_build", "libi2s_oracle.so")
_lib = None


def build(verbose: bool = False) -> str:
    res = subprocess.run(["make", "-C", _DIR, "-B"], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + res.stdout + res.stderr)
    if verbose:
        print(res.stdout)
    return LIB_PATH


_path = LIB_PATH
_build_note = "-O3 -mavx2 -fopenmp (built beforehand)"


def use_native_build() -> str:
    """For timing runs: rebuild the library on THIS host with -O3 -march=native (what the reference's own
    harness uses, utils/test_gemm_kernel.sh:392-397) next to the portable build and load that one from now on.
    Falls back to the portable build when no compiler is at hand.  Returns a note saying which build is loaded."""
    global _lib, _path, _build_note
    native = os.path.join(_DIR, "_build", "libi2s_oracle_native.so")
    try:
        res = subprocess.run(
            ["make", "-C", _DIR, "-B", "OUT=_build/libi2s_oracle_native.so",
             "CFLAGS=-O3 -march=native -fopenmp -fPIC -shared -Wall -Wextra"],
            capture_output=True, text=True, timeout=120,
        )
        ok = res.returncode == 0 and os.path.exists(native)
    except (OSError, subprocess.SubprocessError):
        ok = False
    if ok:
        try:
            ctypes.CDLL(native)
        except OSError:
            ok = False
    if ok:
        _lib, _path, _build_note = None, native, "-O3 -march=native -fopenmp (built on this host)"
    return _build_note


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_path):
            build()
        lib = ctypes.CDLL(_path)
        vp, i64, ci, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t
        lib.i2s_pack_row.argtypes = [vp, vp, i64]
        lib.i2s_pack_row.restype = None
        lib.i2s_quantize.argtypes = [vp, vp, i64, i64]
        lib.i2s_quantize.restype = ctypes.c_float
        for name in ("i2s_vec_dot", "i2s_vec_dot_1x1", "i2s_vec_dot_Nx1"):
            fn = getattr(lib, name)
            fn.argtypes = [ci, vp, sz, vp, sz, vp, sz, ci]
            fn.restype = None
        lib.i2s_gemm.argtypes = [ci, vp, sz, vp, vp, ci, ci]
        lib.i2s_gemm.restype = None
        lib.i2s_bitlinear_acc.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci]
        lib.i2s_bitlinear_acc.restype = None
        lib.i2s_has_avx2.restype = ci
        _lib = lib
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def pack(w: np.ndarray) -> np.ndarray:
    """Ternary int8 [N, K] -> uint8 [N, K/4], x86 I2_S layout."""
    w = np.ascontiguousarray(w, dtype=np.int8)
    n, k = w.shape
    out = np.empty((n, k // 4), dtype=np.uint8)
    load().i2s_pack_row(_p(w), _p(out), n * k)
    return out


def quantize(src: np.ndarray):
    src = np.ascontiguousarray(src, dtype=np.float32)
    n, k = src.shape
    out = np.empty((n, k // 4), dtype=np.uint8)
    scale = load().i2s_quantize(_p(src), _p(out), n, k)
    return out, float(scale)


def vec_dot(packed: np.ndarray, y: np.ndarray, which: str = "i2s_vec_dot") -> np.ndarray:
    """Raw dispatcher call as the M=1 decode path issues it: one call per
    weight row (nrc = 1), returning the float sums of codes q = w + 1."""
    n_rows, kb = packed.shape
    k = kb * 4
    y = np.ascontiguousarray(y, dtype=np.int8).reshape(-1)
    out = np.empty(n_rows, dtype=np.float32)
    fn = getattr(load(), which)
    for r in range(n_rows):
        fn(k, ctypes.c_void_p(out.ctypes.data + 4 * r), 1, ctypes.c_void_p(packed.ctypes.data + r * kb), k, _p(y), k, 1)
    return out


def gemm(packed: np.ndarray, y: np.ndarray) -> np.ndarray:
    """Tiled driver: float [M, N] of sum_k q[n, k] * y[m, k]."""
    n_rows, kb = packed.shape
    k = kb * 4
    y = np.ascontiguousarray(y, dtype=np.int8)
    m = y.shape[0]
    out = np.zeros((m, n_rows), dtype=np.float32)
    load().i2s_gemm(k, _p(out), n_rows, _p(packed), _p(y), m, n_rows)
    return out


def bitlinear_acc(packed: np.ndarray, y: np.ndarray, nthreads: int = 1, tmp=None, acc=None) -> np.ndarray:
    """int32 [M, N] accumulators sum_k w[n, k] * y[m, k] (dot kernels plus the
    explicit -sum(y) correction), weight rows split over nthreads."""
    n_rows, kb = packed.shape
    k = kb * 4
    y = np.ascontiguousarray(y, dtype=np.int8)
    m = y.shape[0]
    if acc is None:
        acc = np.empty((m, n_rows), dtype=np.int32)
    if tmp is None:
        tmp = np.empty((m, n_rows), dtype=np.float32)
    load().i2s_bitlinear_acc(_p(packed), _p(y), _p(acc), _p(tmp), m, n_rows, k, nthreads)
    return acc
