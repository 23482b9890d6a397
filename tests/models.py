"""Synthetic decoder models built twice from the same bytes: once for the CPU oracle, once resident on the GPU."""
import numpy as np

from goinfer_amd import capi, synth
from oracle import binding as ob
from tests.util import inv_freq


def dense_cfg(n_layers=2, hidden=256, n_heads=4, n_kv=2, head_dim=64, inter=512, vocab=512, theta=5e5, eps=1e-5, softcap=0.0):
    return dict(n_layers=n_layers, hidden=hidden, n_heads=n_heads, n_kv=n_kv, head_dim=head_dim, inter=inter, vocab=vocab,
                eps=eps, attn_scale=float(1.0 / np.sqrt(head_dim)), softcap=softcap, theta=theta, kv_f16=1)


def moe_cfg(n_layers=2, hidden=256, n_heads=4, n_kv=2, head_dim=64, n_experts=8, top_k=2, exp_inter=128, vocab=512, exp_act_group=32):
    """exp_act_group: the experts' ActQuantGroup, 32 (activations quantized per group of 32) or 0 (one scale per token row)."""
    c = dense_cfg(n_layers, hidden, n_heads, n_kv, head_dim, 0, vocab, theta=1e6, eps=1e-6)
    c.update(n_experts=n_experts, top_k=top_k, norm_topk=1, exp_inter=exp_inter, qk_norm=1, exp_act_group=exp_act_group)
    return c


class LazyEmbedding:
    """Embedding rows generated on demand (row t from its own seed): a 128k x 4096 f32 table is 2 GB nobody needs whole."""

    def __init__(self, seed, vocab, hidden, sigma):
        self.seed, self.shape, self.sigma = seed, (vocab, hidden), sigma

    def row(self, t):
        return synth.normal(self.seed * 1000003 + int(t), self.shape[1], self.sigma)

    def __getitem__(self, idx):
        if np.ndim(idx) == 0:
            return self.row(idx)
        return np.stack([self.row(t) for t in idx])


class Pair:
    """The same synthetic model as an oracle model and (when dev is given) a resident GPU model."""

    def __init__(self, cfg, seed, dev=None, slots=8, ctx_cap=512, sigma=0.02, kinds=None, kv="f16"):
        """kinds: optional {projection: 'q5k' | 'q6k' | 'w8a8' | 'w4a8'} for dense projections stored as those super-blocks, int8 rows
        or int4-g32 rows. cfg["act_group"] / cfg["exp_act_group"] (default 32): goinfer's ActQuantGroup of the dense int8 / int4
        tensors and of the experts, 0 = one activation scale per row."""
        if kv == "i8":  # the int8 KV cache on both sides
            cfg = dict(cfg, kv_f16=2)
        self.cfg = cfg
        kinds = kinds or {}
        H, nH, nKV, hd = cfg["hidden"], cfg["n_heads"], cfg["n_kv"], cfg["head_dim"]
        qd, kvd, I, V = nH * hd, nKV * hd, cfg["inter"], cfg["vocab"]
        nE = cfg.get("n_experts", 0)
        inv = inv_freq(hd, cfg["theta"])
        self.gpu = capi.Model(dev, cfg, inv) if dev is not None else None
        if V * H > (1 << 26):
            self.emb = LazyEmbedding(seed * 1000 + 999, V, H, sigma)
        else:
            self.emb = synth.normal(seed * 1000 + 999, V * H, sigma).reshape(V, H)
        s = [seed * 1000]

        def nxt():
            s[0] += 1
            return s[0]

        def mat(layer, proj, N, K, expert=-1):
            """Q4_K when K is a multiple of 256, else int8 W8A8 (goinfer's q4k-mode policy, weightmat.go:33-38)."""
            ag, eag = cfg.get("act_group", 32), cfg.get("exp_act_group", 32)
            if expert >= 0:
                nib, s16 = synth.w4a8_normal(nxt(), N, K, sigma)
                if self.gpu:
                    self.gpu.set_act_group(eag)
                    self.gpu.upload_w4a8(layer, proj, expert, nib, s16, K)
                return ob.WMat(ob.OR_W4A8, N, K, nib, s16, act_group=eag)
            if self.gpu:
                self.gpu.set_act_group(ag)
            if kinds.get(proj) == "w4a8":
                nib, s16 = synth.w4a8_normal(nxt(), N, K, sigma)
                if self.gpu:
                    self.gpu.upload_w4a8(layer, proj, -1, nib, s16, K)
                return ob.WMat(ob.OR_W4A8, N, K, nib, s16, act_group=ag)
            if kinds.get(proj) == "w8a8":
                q, sc = synth.w8a8_normal(nxt(), N, K, sigma)
                if self.gpu:
                    self.gpu.upload_w8a8(layer, proj, q, sc)
                return ob.WMat(ob.OR_W8A8, N, K, q, sc, act_group=ag)
            if proj in kinds:
                fmt = kinds[proj]
                blocks = synth.kquant_normal(fmt, nxt(), N, K, sigma)
                if self.gpu:
                    self.gpu.upload_kquant(fmt, layer, proj, blocks, N, K)
                return ob.WMat(ob.OR_Q5K if fmt == "q5k" else ob.OR_Q6K, N, K, blocks, act_group=32)
            if K % 256 == 0 and proj != "head":
                blocks = synth.q4k_normal(nxt(), N, K, sigma)
                if self.gpu:
                    self.gpu.upload_q4k(layer, proj, blocks, N, K)
                return ob.WMat(ob.OR_Q4K, N, K, blocks, act_group=32)
            q, sc = synth.w8a8_normal(nxt(), N, K, sigma)
            if self.gpu:
                self.gpu.upload_w8a8(layer, proj, q, sc)
            return ob.WMat(ob.OR_W8A8, N, K, q, sc, act_group=ag)

        def vec(layer, which, n):
            # norm weights around one; stored as the deviation from one where the model scales by (1 + w)
            v = synth.normal(nxt(), n, 0.02, 0.0 if cfg.get("norm_add_one") else 1.0)
            if self.gpu:
                self.gpu.upload_f32(layer, which, v)
            return v

        layers = []
        for l in range(cfg["n_layers"]):
            lw = dict(q=mat(l, "q", qd, H), k=mat(l, "k", kvd, H), v=mat(l, "v", kvd, H), o=mat(l, "o", H, qd))
            lw["attn_norm"], lw["ffn_norm"] = vec(l, "attn_norm", H), vec(l, "ffn_norm", H)
            if cfg.get("post_norms"):  # Gemma 2: each branch's output is normed before it joins the residual
                lw["post_attn_norm"], lw["post_ffn_norm"] = vec(l, "post_attn_norm", H), vec(l, "post_ffn_norm", H)
            if cfg.get("qk_norm"):
                lw["q_norm"], lw["k_norm"] = vec(l, "q_norm", hd), vec(l, "k_norm", hd)
            if cfg.get("attn_sinks"):  # one learned logit per query head joining the softmax (decoder/attention.go:305-322)
                lw["sinks"] = synth.normal(nxt(), nH, 2.0)
                if self.gpu:
                    self.gpu.upload_f32(l, "attn_sinks", lw["sinks"])
            if cfg.get("window") and l % 2 == 0:  # sliding-window layers alternate with whole-context ones, as in Gemma-2
                lw["window"] = int(cfg["window"])
                if self.gpu:
                    self.gpu.set_window(l, lw["window"])
            if cfg.get("qkv_bias"):  # Qwen2: biases on the q, k and v projections, sent to the GPU as one vector
                b = synth.normal(nxt(), qd + 2 * kvd, 0.5)
                lw["q_bias"], lw["k_bias"], lw["v_bias"] = b[:qd].copy(), b[qd:qd + kvd].copy(), b[qd + kvd:].copy()
                if self.gpu:
                    self.gpu.upload_f32(l, "qkv_bias", b)
            if nE == 0:
                lw["gate"], lw["up"], lw["down"] = mat(l, "gate", I, H), mat(l, "up", I, H), mat(l, "down", H, I)
            else:
                EI = cfg["exp_inter"]
                r = synth.normal(nxt(), nE * H, sigma).reshape(nE, H)
                if self.gpu:
                    self.gpu.upload_f32(l, "router", r)
                lw["router"] = ob.WMat.from_f32(r)
                if cfg.get("router_bias"):  # e_score_correction_bias: shifts the selection, not the weights
                    lw["router_bias"] = synth.normal(nxt(), nE, 0.2)
                    if self.gpu:
                        self.gpu.upload_f32(l, "router_bias", lw["router_bias"])
                lw["exp_gate"] = [mat(l, "gate", EI, H, e) for e in range(nE)]
                lw["exp_up"] = [mat(l, "up", EI, H, e) for e in range(nE)]
                lw["exp_down"] = [mat(l, "down", H, EI, e) for e in range(nE)]
            layers.append(lw)
        fn = synth.normal(nxt(), H, 0.02, 0.0 if cfg.get("norm_add_one") else 1.0)
        if self.gpu:
            self.gpu.upload_f32(-1, "final_norm", fn)
        head = mat(-1, "head", V, H)
        self.oracle = ob.OracleModel(cfg, layers, fn, head, inv)
        if self.gpu:
            self.gpu.finalize()
            self.gpu.kv_configure(slots, ctx_cap, kv)
        self.ctx_cap = ctx_cap

    def close(self):
        if self.gpu:
            self.gpu.close()


def logits_close(got, want, floor=0.0, abs_tol=2e-2, rel_tol=1e-2):
    """The north-star logit bar: max-abs 2e-2 and relative 1e-2 (of the row's largest |logit|) — widened to twice the
    oracle's own noise floor where that is larger. The floor is how far the oracle's logits move when its input embedding
    is perturbed by 1e-6 relative: per-32 int8 activation quantization makes a random-weight decoder chaotic (one flipped
    code flips ~3 % of the next layer's codes), so no implementation that is not bit-identical can sit below it
    (tests/test_oracle_sensitivity.py pins this behaviour of the reference arithmetic)."""
    d = np.abs(got.astype(np.float64) - want.astype(np.float64)).max()
    tol = max(min(abs_tol, rel_tol * float(np.abs(want).max())), 2.0 * floor)
    return d <= tol, d


def perturbed(emb, eps, key):
    """emb * (1 + eps * n), n ~ N(0,1): the probe of the oracle's sensitivity."""
    n = np.random.default_rng(key).standard_normal(emb.shape).astype(np.float32)
    return (emb * (1 + eps * n)).astype(np.float32)


def near_tie_ok(ref, cand_arg, pct=0.03):
    """goinfer's near-tie rule (decoder/fidelity_testhook.go:126-152): a differing argmax passes only if the reference's
    gap between its own argmax and the candidate's is at most 3 % of the reference logit range."""
    ra = int(ob.argmax(ref))
    if ra == cand_arg:
        return True
    gap = (ref[ra] - ref[cand_arg]) / (ref.max() - ref.min())
    return gap <= pct
