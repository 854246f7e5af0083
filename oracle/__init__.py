"""ctypes binding of the CPU oracle (``liboracle.so`` built from ``gpt2_cpu.c``).

TEST INFRASTRUCTURE ONLY: tests, the smoke check and the benchmark's
``cpu_baseline`` leg load this; the product package never does.

All functions take and return C-contiguous numpy arrays (float32 / int32).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# ORACLE_LIB: another build of the same source to check against (the sanitizer build of the Makefile)
_LIB_PATH = os.environ.get("ORACLE_LIB") or os.path.join(_HERE, "liboracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int)


def build() -> str:
    """Compile liboracle.so with the Makefile next to this file."""
    subprocess.run(["make", "-B", "-C", _HERE, "liboracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        c_int, c_size = ctypes.c_int, ctypes.c_size_t
        L.oracle_num_threads.restype = c_int
        L.oracle_encoder_forward.argtypes = [_f32p, _i32p, _f32p, _f32p, c_int, c_int, c_int]
        L.oracle_layernorm_forward.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, c_int,
                                               c_int, c_int]
        L.oracle_fused_residual_layernorm_forward.argtypes = [_f32p] * 8 + [c_int] * 3
        L.oracle_residual_forward.argtypes = [_f32p, _f32p, _f32p, c_size]
        L.oracle_gelu_forward.argtypes = [_f32p, _f32p, c_size]
        for fn in (L.oracle_matmul_forward, L.oracle_matmul_forward_naive):
            fn.argtypes = [_f32p, _f32p, _f32p, _f32p, c_int, c_int, c_int, c_int]
        L.oracle_attention_forward.argtypes = [_f32p, _f32p, c_int, c_int, c_int, c_int]
        L.oracle_argmax_forward.argtypes = [_i32p, _f32p, c_int, c_int]
        L.oracle_num_parameters.argtypes = [c_int] * 4
        L.oracle_num_parameters.restype = c_size
        L.oracle_param_sizes.argtypes = [ctypes.POINTER(c_size), c_int, c_int, c_int, c_int]
        L.oracle_gpt2_forward.argtypes = [_f32p, _i32p, _f32p, _f32p, _i32p] + [c_int] * 7
        L.oracle_gpt2_forward.restype = c_int
        _lib = L
    return _lib


def _f(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(_f32p)


def _i(a: np.ndarray):
    assert a.dtype == np.int32 and a.flags.c_contiguous
    return a.ctypes.data_as(_i32p)


def _c(a, dtype=np.float32):
    return np.ascontiguousarray(a, dtype=dtype)


def num_threads() -> int:
    return lib().oracle_num_threads()


def encoder_forward(inp, wte, wpe):
    inp, wte, wpe = _c(inp, np.int32), _c(wte), _c(wpe)
    B, T = inp.shape
    C = wte.shape[1]
    out = np.empty((B, T, C), np.float32)
    lib().oracle_encoder_forward(_f(out), _i(inp), _f(wte), _f(wpe), B, T, C)
    return out


def layernorm_forward(inp, weight, bias):
    """inp (N, C) -> out (N, C), mean (N,), rstd (N,)."""
    inp, weight, bias = _c(inp), _c(weight), _c(bias)
    N, C = inp.shape
    out = np.empty_like(inp)
    mean = np.empty(N, np.float32)
    rstd = np.empty(N, np.float32)
    lib().oracle_layernorm_forward(_f(out), _f(mean), _f(rstd), _f(inp), _f(weight), _f(bias), 1,
                                   N, C)
    return out, mean, rstd


def fused_residual_layernorm_forward(inp1, inp2, weight, bias):
    """-> res (N, C), ln (N, C), mean (N,), rstd (N,)."""
    inp1, inp2, weight, bias = _c(inp1), _c(inp2), _c(weight), _c(bias)
    N, C = inp1.shape
    res = np.empty_like(inp1)
    ln = np.empty_like(inp1)
    mean = np.empty(N, np.float32)
    rstd = np.empty(N, np.float32)
    lib().oracle_fused_residual_layernorm_forward(_f(res), _f(ln), _f(mean), _f(rstd), _f(inp1),
                                                  _f(inp2), _f(weight), _f(bias), 1, N, C)
    return res, ln, mean, rstd


def residual_forward(inp1, inp2):
    inp1, inp2 = _c(inp1), _c(inp2)
    out = np.empty_like(inp1)
    lib().oracle_residual_forward(_f(out), _f(inp1), _f(inp2), inp1.size)
    return out


def gelu_forward(inp):
    inp = _c(inp)
    out = np.empty_like(inp)
    lib().oracle_gelu_forward(_f(out), _f(inp), inp.size)
    return out


def matmul_forward(inp, weight, bias=None, naive=False):
    """inp (N, C), weight (OC, C), bias (OC,) or None -> (N, OC)."""
    inp, weight = _c(inp), _c(weight)
    N, C = inp.shape
    OC = weight.shape[0]
    assert weight.shape[1] == C
    out = np.empty((N, OC), np.float32)
    b = None
    if bias is not None:
        bias = _c(bias)
        b = _f(bias)
    fn = lib().oracle_matmul_forward_naive if naive else lib().oracle_matmul_forward
    fn(_f(out), _f(inp), _f(weight), b, 1, N, C, OC)
    return out


def attention_forward(qkv, NH):
    """qkv (B, T, 3C) packed -> (B, T, C)."""
    qkv = _c(qkv)
    B, T, C3 = qkv.shape
    C = C3 // 3
    out = np.empty((B, T, C), np.float32)
    lib().oracle_attention_forward(_f(out), _f(qkv), B, T, C, NH)
    return out


def argmax_forward(logits):
    logits = _c(logits)
    V = logits.shape[-1]
    N = logits.size // V
    ids = np.empty(N, np.int32)
    lib().oracle_argmax_forward(_i(ids), _f(logits), N, V)
    return ids.reshape(logits.shape[:-1])


PARAM_NAMES = ("wte", "wpe", "ln1w", "ln1b", "qkvw", "qkvb", "attprojw", "attprojb", "ln2w",
               "ln2b", "fcw", "fcb", "fcprojw", "fcprojb", "lnfw", "lnfb")


def param_sizes(maxT, V, L, C):
    s = (ctypes.c_size_t * len(PARAM_NAMES))()
    lib().oracle_param_sizes(s, maxT, V, L, C)
    return dict(zip(PARAM_NAMES, (int(x) for x in s)))


def num_parameters(maxT, V, L, C) -> int:
    return int(lib().oracle_num_parameters(maxT, V, L, C))


def gpt2_forward(params, inputs, *, maxT, V, L, NH, C, want_lnf=False):
    """params: flat float32 buffer in checkpoint order; inputs (B, T) int32.

    Returns (logits (B,T,V), ids (B,T)[, lnf (B,T,C)]).
    """
    params, inputs = _c(params), _c(inputs, np.int32)
    B, T = inputs.shape
    assert params.size == num_parameters(maxT, V, L, C)
    logits = np.empty((B, T, V), np.float32)
    ids = np.empty((B, T), np.int32)
    lnf = np.empty((B, T, C), np.float32) if want_lnf else None
    rc = lib().oracle_gpt2_forward(_f(logits), _i(ids), _f(lnf) if want_lnf else None, _f(params),
                                   _i(inputs), B, T, maxT, V, L, NH, C)
    if rc != 0:
        raise RuntimeError(f"oracle_gpt2_forward failed ({rc})")
    return (logits, ids, lnf) if want_lnf else (logits, ids)
