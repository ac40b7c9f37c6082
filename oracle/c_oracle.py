"""ctypes front end of oracle/optim_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Builds oracle/_build/liboptim_oracle.so with the Makefile next to this file if it is missing.
Only tests, the smoke check and the benchmark's cpu_baseline leg may import this module.
"""
from __future__ import annotations

import ctypes
import subprocess
from ctypes import POINTER, Structure, c_double, c_float, c_int, c_int32, c_int64, c_void_p
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB = HERE / "_build" / "liboptim_oracle.so"


class OracleHParams(Structure):
    _fields_ = [
        ("learning_rate", c_float), ("beta1", c_float), ("beta2", c_float), ("eps", c_float),
        ("weight_decay", c_float),
        ("bias_correction", c_int32), ("grad_averaging", c_int32), ("mode", c_int32),
        ("normalize_grad", c_int32),
        ("grad_unscale", c_float),
    ]


def build(force: bool = False) -> Path:
    if force or not LIB.exists() or LIB.stat().st_mtime < (HERE / "optim_oracle.c").stat().st_mtime:
        subprocess.run(["make", "-C", str(HERE), "-B" if force else "-s"], check=True)
    return LIB


_lib = None


def lib():
    global _lib
    if _lib is None:
        l = ctypes.CDLL(str(build()))
        l.oracle_sgd_f32.restype = None
        l.oracle_sgd_f32.argtypes = [c_void_p] * 5 + [c_int64, c_double, c_double, c_int]
        l.oracle_lans_step.restype = None
        l.oracle_lans_step.argtypes = [c_int32, POINTER(c_int64), POINTER(c_void_p), c_int,
                                       POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                       c_float, POINTER(OracleHParams), POINTER(c_double), c_int,
                                       POINTER(c_void_p), c_int]
        for fn in (l.oracle_f32_to_f16_bits, l.oracle_f32_to_bf16_bits):
            fn.restype = None
            fn.argtypes = [c_void_p, c_void_p, c_int64]
        l.oracle_max_threads.restype = c_int
        _lib = l
    return _lib


def max_threads() -> int:
    return lib().oracle_max_threads()


def sgd_step(x0, dx, v0, learning_rate, mu, threads: int = 1):
    x0 = np.ascontiguousarray(x0, dtype=np.float32)
    dx = np.ascontiguousarray(dx, dtype=np.float32)
    v0 = np.ascontiguousarray(v0, dtype=np.float32)
    v1 = np.empty_like(dx)
    x1 = np.empty_like(dx)
    lib().oracle_sgd_f32(x0.ctypes.data, dx.ctypes.data, v0.ctypes.data, v1.ctypes.data,
                         x1.ctypes.data, x0.size, float(learning_rate), float(mu), int(threads))
    return v1, x1


def hparams_from(hp) -> OracleHParams:
    """From oracle.lans_f64.LansHParams (or anything with the same attributes)."""
    return OracleHParams(hp.learning_rate, hp.beta1, hp.beta2, hp.eps, hp.weight_decay,
                         int(hp.bias_correction), int(hp.grad_averaging), int(hp.mode),
                         int(bool(hp.normalize_grad)), hp.grad_unscale)


_DTYPE_CODE = {np.dtype(np.float32): 0, np.dtype(np.float16): 1, np.dtype(np.uint16): 2}


def narrow_bits(x, dtype: str):
    """fp32 -> float16 / bfloat16 bit patterns (uint16) with the C oracle's own conversions."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    fn = lib().oracle_f32_to_bf16_bits if dtype == "bfloat16" else lib().oracle_f32_to_f16_bits
    fn(x.ctypes.data, out.ctypes.data, x.size)
    return out


def lans_step_inplace(g_list, w_list, m_list, v_list, step, hp, threads: int = 0, p_list=None,
                      model_dtype: str = "float16"):
    """In place on the fp32 arrays of w/m/v; g may be fp32, fp16 or uint16 (bfloat16 bit patterns)
    arrays.  ``p_list``: optional uint16/float16 arrays that receive the new weights narrowed to
    ``model_dtype``.  Returns [n,4] norms."""
    n = len(w_list)
    gdt = g_list[0].dtype if n > 0 else np.dtype(np.float32)
    g_dtype = _DTYPE_CODE[np.dtype(gdt)]
    for arrs, dt in ((g_list, gdt), (w_list, np.float32), (m_list, np.float32), (v_list, np.float32)):
        for a in arrs:
            assert a.dtype == dt and a.flags.c_contiguous, (a.dtype, dt)
    if p_list is not None:
        for a, w in zip(p_list, w_list):
            assert a.dtype.itemsize == 2 and a.flags.c_contiguous and a.size == w.size
    numel = (c_int64 * max(n, 1))(*[int(a.size) for a in w_list])

    def ptrs(arrs):
        return (c_void_p * max(n, 1))(*[a.ctypes.data for a in arrs])

    norms = np.zeros((n, 4), dtype=np.float64)
    ohp = hparams_from(hp)
    lib().oracle_lans_step(n, numel, ptrs(g_list), g_dtype, ptrs(w_list), ptrs(m_list),
                           ptrs(v_list), float(np.float32(step)), ctypes.byref(ohp),
                           norms.ctypes.data_as(POINTER(c_double)), int(threads),
                           ptrs(p_list) if p_list is not None else None,
                           2 if model_dtype == "bfloat16" else 1)
    return norms
