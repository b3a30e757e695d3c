"""ctypes front end of oracle/libcpu_ref.so (TEST INFRASTRUCTURE ONLY: same-precision parity checker and
timed CPU baseline; see cpu_ref_impl.h for the reference lines it restates)."""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force: bool = False) -> str:
    path = os.path.join(_DIR, "libcpu_ref.so")
    if force or not os.path.exists(path):
        subprocess.run(["make", "-B", "-C", _DIR, "libcpu_ref.so"], check=True, stdout=subprocess.DEVNULL)
    return path


def lib():
    global _LIB
    if _LIB is None:
        _LIB = ctypes.CDLL(build())
        _LIB.cpu_ref_max_threads.restype = ctypes.c_int
    return _LIB


def max_threads() -> int:
    return int(lib().cpu_ref_max_threads())


def _sfx(dtype):
    return {np.dtype(np.float32): "_f32", np.dtype(np.float64): "_f64"}[np.dtype(dtype)]


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _boxes(lower, upper, dtype):
    if lower is None:
        return None
    return np.ascontiguousarray(np.concatenate([lower, upper], axis=-1), dtype=dtype)


def forward(mixture: np.ndarray, xes: np.ndarray, lower=None, upper=None, n_threads: int = 128) -> np.ndarray:
    """Reference CPU forward in the precision of `mixture`; n_threads=128 is the reference's own choice
    (parallel_start.h:94-99)."""
    mixture = np.ascontiguousarray(mixture)
    xes = np.ascontiguousarray(xes, dtype=mixture.dtype)
    B, L, M, G = mixture.shape
    D = 2 if G == 7 else 3
    Bx, Lx, N, _ = xes.shape
    out = np.empty((B, L, N), dtype=mixture.dtype)
    boxes = _boxes(lower, upper, mixture.dtype)
    getattr(lib(), "cpu_ref_forward" + _sfx(mixture.dtype))(
        _ptr(mixture), _ptr(xes), _ptr(out), _ptr(boxes), B, L, M, N, D, Bx, Lx, n_threads)
    return out


def backward(grad_out, mixture, xes, lower=None, upper=None, need_mixture=True, need_xes=True,
             n_threads: int = 128):
    mixture = np.ascontiguousarray(mixture)
    xes = np.ascontiguousarray(xes, dtype=mixture.dtype)
    grad_out = np.ascontiguousarray(grad_out, dtype=mixture.dtype)
    B, L, M, G = mixture.shape
    D = 2 if G == 7 else 3
    Bx, Lx, N, _ = xes.shape
    gm = np.empty_like(mixture)
    gx = np.empty_like(xes)
    boxes = _boxes(lower, upper, mixture.dtype)
    getattr(lib(), "cpu_ref_backward" + _sfx(mixture.dtype))(
        _ptr(grad_out), _ptr(mixture), _ptr(xes), _ptr(gm), _ptr(gx), _ptr(boxes),
        B, L, M, N, D, Bx, Lx, int(need_mixture), int(need_xes), n_threads)
    return gm, gx
