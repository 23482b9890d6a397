"""The oracle's decodeMultiStep reproduces the reference's committed Hugging Face goldens on its tiny f32 checkpoints.

Bars are the reference's own: cosine >= 0.9999 and max-abs <= 5e-2 on the last-position logits, argmax equal, greedy
continuation equal (decoder/llama_tiny_test.go:21-90); top-k / sampled logits to 1e-3 for the MoE goldens.
"""
import json
import os

import numpy as np
import pytest

from oracle import binding as ob
from tests.util import GOLDEN, tiny_model


def run_prompt(m, emb, ids, cap=64):
    c = m.new_cache(cap)
    try:
        for t in ids:
            logits = m.step(emb[t][None, :], [c])
        return logits[0], c
    except Exception:
        m.free_cache(c)
        raise


def test_llama_tiny_text_parity():
    g = json.load(open(os.path.join(GOLDEN, "llama_tiny_text_golden.json")))
    m, emb, _ = tiny_model("llama-tiny")
    logits, c = run_prompt(m, emb, g["prompt_ids"])
    want = np.array(g["last_logits"], np.float64)
    got = logits.astype(np.float64)
    cos = got @ want / np.linalg.norm(got) / np.linalg.norm(want)
    assert cos >= 0.9999
    assert np.abs(got - want).max() <= 5e-2
    assert np.abs(got - want).max() <= 2e-5  # what this restatement actually reaches
    assert ob.argmax(logits) == g["argmax"]
    cont = []
    tok = ob.argmax(logits)
    for _ in range(g["n_new"]):
        cont.append(tok)
        tok = ob.argmax(m.step(emb[tok][None, :], [c])[0])
    m.free_cache(c)
    assert cont == g["continuation_ids"]


@pytest.mark.parametrize("name,golden", [("qwen3moe-tiny", "qwen3moe_forward_golden.json"),
                                         ("mixtral-tiny", "mixtral_forward_golden.json")])
def test_moe_tiny_forward(name, golden):
    g = json.load(open(os.path.join(GOLDEN, golden)))
    m, emb, _ = tiny_model(name)
    logits, c = run_prompt(m, emb, g["ids"])
    m.free_cache(c)
    assert ob.argmax(logits) == g["argmax"]
    for i, v in g["top_k"] + g["sample"]:
        assert abs(float(logits[i]) - v) <= 1e-4, (i, logits[i], v)
    st = g["stats"]
    l64 = logits.astype(np.float64)
    assert abs(l64.sum() - st["sum"]) <= 1e-3 and abs((l64 * l64).sum() - st["sum_sq"]) <= 1e-3
    assert abs(l64.min() - st["min"]) <= 1e-4 and abs(l64.max() - st["max"]) <= 1e-4


def test_batched_rows_equal_single_rows():
    """decoder/cpu_batch_test.go:14-53: each row of a batched step is bit-identical to that sequence alone."""
    m, emb, _ = tiny_model("llama-tiny")
    prompts = [[2, 7, 42], [100, 5, 200, 13, 88, 1, 9], [3], [250, 249, 248, 247, 246]]
    solo = []
    for p in prompts:
        c = m.new_cache(32)
        for t in p:
            m.step(emb[t][None, :], [c])
        solo.append(c)
    nxt = [11, 22, 33, 44]
    want = []
    for b, c in enumerate(solo):
        c2 = m.new_cache(32)
        for t in prompts[b]:
            m.step(emb[t][None, :], [c2])
        want.append(m.step(emb[nxt[b]][None, :], [c2])[0])
        m.free_cache(c2)
    got = m.step(emb[nxt], solo)
    for b in range(4):
        assert np.array_equal(got[b].view(np.uint32), want[b].view(np.uint32))
    for c in solo:
        m.free_cache(c)
