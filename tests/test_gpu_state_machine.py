"""A random walk over the resident's entry points (batched steps, ragged steps with several rows per slot, prompt passes,
truncation, reset, uploaded prefixes) on a few KV slots, checked by replay: whatever order the calls came in, the logits a slot
last returned are, bit for bit, those of its token history stepped one token at a time on a fresh slot.

This is goinfer's resident contract read as a whole (resident/forward.go:5-38: ForwardN == K x Forward, TruncateTo and Reset
leave a prefix that behaves as if nothing else had been there; resident/subsystems.go:102-117: a row in a batch == the row
alone), exercised for what single-feature tests miss: stale state between calls."""
import numpy as np
import pytest

from goinfer_amd import capi
from tests.models import Pair, dense_cfg, moe_cfg

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = capi.Device(0)
    yield d
    d.close()


def bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)


def walk(pair, emb, vocab, slots, cap, seed, n_ops, max_batch, chains=False, max_prefill=50, max_ragged=7, moves=None):
    """emb: the embedding rows by token id. Returns (history per slot, last logits per slot). Slot `slots` (one past the last) is
    left for the replay. chains: the device-side greedy chain is one of the moves (emb must then be the resident table's rows)."""
    rng = np.random.default_rng(seed)
    hist = [[] for _ in range(slots)]  # what each slot holds: a list of ("tok", id) or ("kv", layer arrays)
    last = [None] * slots
    g = pair.gpu
    for _ in range(n_ops):
        op = rng.choice(moves or (["batch", "batch", "ragged", "prefill", "truncate", "reset", "nologits"] + (["chain"] if chains else [])))
        if op == "batch":
            k = int(rng.integers(1, min(slots, max_batch) + 1))
            chosen = [int(s) for s in rng.permutation(slots)[:k] if len(hist[s]) < cap - 1]
            if not chosen:
                continue
            toks = rng.integers(0, vocab, len(chosen))
            out, ids = g.step_batch(chosen, [len(hist[s]) for s in chosen], emb[toks], capi.WANT_LOGITS | capi.WANT_ARGMAX)
            for i, s in enumerate(chosen):
                hist[s].append(int(toks[i]))
                last[s] = out[i].copy()
                assert ids[i] == int(np.argmax(out[i]))
        elif op == "ragged":
            k = int(rng.integers(1, min(3, slots) + 1))
            chosen = [int(s) for s in rng.permutation(slots)[:k]]
            rows = [int(rng.integers(1, max_ragged)) for _ in chosen]
            keep = [(s, r) for s, r in zip(chosen, rows) if len(hist[s]) + r < cap]
            if not keep or sum(r for _, r in keep) > max_batch:
                continue
            toks = [rng.integers(0, vocab, r) for _, r in keep]
            out, _ = g.step_ragged([s for s, _ in keep], [len(hist[s]) for s, _ in keep], [emb[t] for t in toks])
            off = 0
            for (s, r), t in zip(keep, toks):
                hist[s].extend(int(x) for x in t)
                last[s] = out[off + r - 1].copy()
                off += r
        elif op == "prefill":
            s = int(rng.integers(0, slots))
            n = int(rng.integers(1, max_prefill))
            if len(hist[s]) + n >= cap:
                continue
            toks = rng.integers(0, vocab, n)
            last[s] = g.prefill_last(s, len(hist[s]), emb[toks]).copy()
            hist[s].extend(int(x) for x in toks)
        elif op == "nologits":
            s = int(rng.integers(0, slots))
            if len(hist[s]) >= cap - 1:
                continue
            t = int(rng.integers(0, vocab))
            g.forward_no_logits(s, len(hist[s]), emb[t])
            hist[s].append(t)
            last[s] = None  # this call returns nothing to compare; the tokens after it will
        elif op == "chain":
            s = int(rng.integers(0, slots))
            n = int(rng.integers(1, 9))
            if len(hist[s]) + n >= cap - 1:
                continue
            t = int(rng.integers(0, vocab))
            g.greedy_chain_start(s, t, len(hist[s]))
            ids = [g.greedy_chain_next() for _ in range(n)]
            g.chain_stop()
            hist[s].extend([t] + ids[:-1])  # the chain fed its first token and every pick but the last
            last[s] = None
        elif op == "truncate":
            s = int(rng.integers(0, slots))
            if len(hist[s]) < 2:
                continue
            n = int(rng.integers(1, len(hist[s])))
            g.kv_truncate(s, n)
            del hist[s][n:]
            last[s] = None
        else:
            s = int(rng.integers(0, slots))
            g.kv_reset(s)
            hist[s] = []
            last[s] = None
    return hist, last


@pytest.mark.parametrize("seed", [82, 83, 84, "long"])
@pytest.mark.parametrize("kind,kv", [("dense", "f16"), ("dense", "i8"), ("moe", "f16"), ("dense-chains", "f16")])
def test_random_walk_replays_bit_identically(dev, kind, kv, seed):
    cfg = moe_cfg(n_layers=2) if kind == "moe" else dense_cfg(n_layers=2)
    slots, cap = 5, 160
    grow = {}
    if seed == "long":  # moves that mostly add rows, many at a time: the slots pass 1024 positions, where a sequence's attention is cut in pieces of several blocks
        slots, cap, seed = 4, 2600, 86
        grow = dict(max_prefill=500, max_ragged=41, moves=["batch"] * 8 + ["ragged"] * 6 + ["prefill"] * 6 + ["nologits", "truncate"] + (["chain"] if kind == "dense-chains" else []))
    pair = Pair(cfg, seed=81, dev=dev, slots=slots + 1, ctx_cap=cap, kv=kv)
    try:
        emb = pair.emb
        if kind == "dense-chains":  # the chain looks its tokens up in the resident int8 table: every move uses that table's rows
            from goinfer_amd import synth
            q, sc = synth.w8a8_normal(85, cfg["vocab"], cfg["hidden"], 0.02)
            pair.gpu.upload_embedding(q, sc)
            emb = q.astype(np.float32) * sc[:, None]
        hist, last = walk(pair, emb, cfg["vocab"], slots, cap, seed=seed, n_ops=120 if grow else 300, max_batch=32 if kind == "moe" else 128,
                          chains=kind == "dense-chains", **grow)
        if grow:
            assert max(len(h) for h in hist) > 1024
        checked = 0
        for s in range(slots):
            if not hist[s]:
                continue
            # the slot's state, not only its last answer: one more token on the slot and on the replay must agree too
            pair.gpu.kv_reset(slots)
            replay = None
            for p, t in enumerate(hist[s]):
                replay = pair.gpu.forward(slots, p, emb[t])
            if last[s] is not None:
                assert np.array_equal(bits(last[s]), bits(replay)), ("last logits", s, len(hist[s]))
                checked += 1
            nxt = 7
            a = pair.gpu.forward(s, len(hist[s]), emb[nxt])
            b = pair.gpu.forward(slots, len(hist[s]), emb[nxt])
            assert np.array_equal(bits(a), bits(b)), ("next token", s, len(hist[s]))
        assert checked >= 1
    finally:
        pair.close()
