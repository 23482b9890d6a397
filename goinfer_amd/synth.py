"""Deterministic synthetic weights (libgoinfer_synth.so): N(0, sigma) values quantized to the repo's weight formats."""
import ctypes as C
import os

import numpy as np

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libgoinfer_synth.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_PATH):
            raise RuntimeError("%s is missing: run `python -m goinfer_amd.build`" % _PATH)
        _lib = C.CDLL(_PATH)
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def normal(seed, n, sigma=1.0, mean=0.0, offset=0):
    out = np.empty(int(n), np.float32)
    lib().synth_normal(C.c_uint64(seed), C.c_uint64(offset), C.c_size_t(int(n)), C.c_float(mean), C.c_float(sigma), _p(out))
    return out


def q4k_normal(seed, N, K, sigma=0.02):
    """N x K weights ~ N(0, sigma) as raw Q4_K super-blocks: uint8 [N * K/256 * 144]."""
    out = np.empty(N * (K // 256) * 144, np.uint8)
    lib().synth_q4k_normal(C.c_uint64(seed), N, K, C.c_float(sigma), _p(out))
    return out


def kquant_normal(fmt, seed, N, K, sigma=0.02):
    """N x K weights ~ N(0, sigma) as raw Q5_K ('q5k', 176 B) or Q6_K ('q6k', 210 B) super-blocks."""
    bb, code = {"q5k": (176, 5), "q6k": (210, 6)}[fmt]
    out = np.empty(N * (K // 256) * bb, np.uint8)
    lib().synth_kquant_normal(code, C.c_uint64(seed), N, K, C.c_float(sigma), _p(out))
    return out


def quantize_q4k(w):
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, K = w.shape
    out = np.empty(N * (K // 256) * 144, np.uint8)
    lib().synth_quantize_q4k(_p(w), N, K, _p(out))
    return out


def w8a8_normal(seed, N, K, sigma=0.02):
    q = np.empty((N, K), np.int8)
    s = np.empty(N, np.float32)
    lib().synth_w8a8_normal(C.c_uint64(seed), N, K, C.c_float(sigma), _p(q), _p(s))
    return q, s


def w4a8_normal(seed, N, K, sigma=0.02):
    nib = np.empty((N, K // 2), np.uint8)
    s16 = np.empty((N, K // 32), np.uint16)
    lib().synth_w4a8_normal(C.c_uint64(seed), N, K, C.c_float(sigma), _p(nib), _p(s16))
    return nib, s16
