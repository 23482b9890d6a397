"""CPU-side checks of the C ABI: the library loads, exports every entry point include/rocmdecode.h declares, and declines
cleanly (no crash, no fallback) when no GPU is present."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from goinfer_amd import capi, synth
from oracle import binding as ob

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "rocmdecode.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rd_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    names = declared_functions()
    assert len(names) >= 30
    assert sorted(capi.EXPORTS) == names


def test_library_exports_every_declared_symbol():
    lib = capi.lib()
    for n in declared_functions():
        assert hasattr(lib, n), n


def test_code_object_is_built_for_gfx950():
    blob = open(capi.HSACO_PATH, "rb").read()
    assert (blob[:4] == b"\x7fELF" or blob.startswith(b"__CLANG_OFFLOAD_BUNDLE__")) and b"gfx950" in blob
    for k in (b"rd_k_gemm8_q4k_kw4", b"rd_k_attn_partial", b"rd_k_dequant_q4k", b"rd_k_moe_route", b"rd_k_gemm8_q4k_gateup"):
        assert k in blob


def test_backend_name():
    assert capi.lib().rd_backend_name() == b"rocm"


def test_device_open_without_gpu_declines_or_opens():
    """No GPU here: rd_device_open must return RD_DECLINED with a reason (the caller stays on its own CPU path); with a GPU
    it opens. Either way nothing computes on the CPU inside this library."""
    h = C.c_void_p()
    rc = capi.lib().rd_device_open(0, C.byref(h))
    if rc == capi.RD_OK:
        capi.lib().rd_device_close(h)
    else:
        assert rc == capi.RD_DECLINED
        assert len(capi.lib().rd_last_error()) > 0
        with pytest.raises(capi.RocmError):
            capi.Device(0)


def test_null_arguments_are_rejected():
    L = capi.lib()
    assert L.rd_dequant_q4k(None, None, 1, 256, None) < 0
    assert L.rd_step_batch(None, 1, None, None, None, 1, None, None) < 0
    assert L.rd_model_create(None, None, None) < 0


def test_synthetic_q4k_is_a_valid_quantization():
    """The benchmark's 'N(0,0.02) quantized to Q4_K' inputs: dequantizing the blocks (oracle, pinned bit-exact by the
    reference fingerprint) recovers the source values to Q4_K's resolution."""
    N, K = 16, 1024
    w = synth.normal(9, N * K, 0.02).reshape(N, K)
    blocks = synth.quantize_q4k(w)
    assert blocks.size == N * (K // 256) * 144
    back = ob.dequant_q4k(blocks).reshape(N, K)
    err = np.abs(back - w)
    assert err.max() < 0.02 * 0.5 and np.sqrt((err ** 2).mean()) < 0.02 * 0.12
    assert np.array_equal(blocks, synth.q4k_normal(9, N, K, 0.02))  # the fused generator quantizes the same values


def test_synthetic_int_weights_follow_the_reference_quantizers():
    N, K = 8, 256
    w = synth.normal(5, N * K, 0.02).reshape(N, K)
    q, s = synth.w8a8_normal(5, N, K)
    q2, s2 = ob.quantize_rows_int8(w)
    assert np.array_equal(q, q2) and np.array_equal(s, s2)
    w = synth.normal(8, N * K, 0.02).reshape(N, K)
    nib, s16 = synth.w4a8_normal(8, N, K)
    n2, t2 = ob.quantize_int4(w)
    assert np.array_equal(nib, n2) and np.array_equal(s16, t2)
