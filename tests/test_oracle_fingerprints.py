"""The oracle's restatements reproduce goinfer's committed kernel fingerprints bit for bit.

tests/golden/kernel_fingerprints.json is the reference's testdata/kernel_fingerprints.json (data). oracle/kprint.c
regenerates the reference's splitmix64 input suite and hashes the oracle's outputs the way
internal/diag/kernelprint does; a digest match pins the exact f32 expression order of each function.
"""
import json
import os

import pytest

from oracle import binding as ob

ALL = "amd64[avx2,avx512vnni,avx512vnni+vl,f16c,popcnt]", "amd64[avx2,f16c,popcnt]", "arm64[dotprod]"
# digest name -> the reference configurations it must equal
PINS = {
    "linalg.F32ToF16": ALL,
    "linalg.F16ToF32": ALL,
    "embed.GGUFFile(Q4_K).Tensor": ALL,
    "embed.GGUFFile(Q5_K).Tensor": ALL,
    "embed.GGUFFile(Q6_K).Tensor": ALL,
    "linalg.QuantizeRowInt8": ALL,
    "linalg.DequantizeRowsInt8Into": ALL,  # with QuantizeRowInt8: the int8 KV cache's store and read
    "linalg.QuantizeActQ": ALL,
    "linalg.QuantizeGroupInt4Row": ALL,
    "linalg.QuantizeInt4": ALL,
    "linalg.MatmulQKAcc64": ALL,
    "linalg.MatmulAVAcc64": ALL,
    "linalg.MatmulBTW8A8": ALL,  # per-row int8 activations: ((f32)idot*aS)*wS
    # per-32 activations: the reference's own result differs between amd64 and arm64; the oracle's ascending-group
    # fused fold is the arm64 one
    "linalg.MatmulBTW8A8Into": ("arm64[dotprod]",),
}


@pytest.fixture(scope="module")
def table(golden_dir):
    return json.load(open(os.path.join(golden_dir, "kernel_fingerprints.json")))


@pytest.fixture(scope="module")
def got():
    return ob.fingerprints()


@pytest.mark.parametrize("name", sorted(PINS))
def test_fingerprint(name, table, got):
    assert name in got, "oracle/kprint.c does not compute " + name
    for cfg in PINS[name]:
        assert got[name] == table[cfg][name], (name, cfg)
