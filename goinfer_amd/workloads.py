"""The benchmark workloads: synthetic models of the shapes BASELINE.json names, resident on the GPU.

Weights are N(0, 0.02) drawn from a counter-based generator and quantized to the repo's formats (synth.py); norm weights
are 1 + N(0, 0.02) in f32; the LM head and the embedding table are int8 per goinfer's q4k-mode policy
(decoder/weightmat.go:79-84). KV caches are pre-filled with N(0,1) values narrowed to binary16 by the backend.
"""
import numpy as np

from . import capi, synth

SIGMA = 0.02


def llama3_8b_cfg(n_layers=32):
    """Llama-3-8B shape: 32 layers, hidden 4096, 32 Q / 8 KV heads, head_dim 128, SwiGLU FFN 14336, vocab 128256, theta 5e5."""
    return dict(name="llama3-8b-shape", n_layers=n_layers, hidden=4096, n_heads=32, n_kv=8, head_dim=128, inter=14336, vocab=128256,
                eps=1e-5, attn_scale=float(1.0 / np.sqrt(128)), softcap=0.0, theta=5e5)


def qwen3_moe_cfg(n_layers=48, exp_act_group=0):
    """Qwen3-MoE-30B-A3B shape: 48 layers, hidden 2048, 32 Q / 4 KV heads, head_dim 128, 128 experts top-8, expert FFN 768.
    The experts are int4-g32 with int8 activations quantized per token row (exp_act_group 0, goinfer's int4 mode); 32 gives the
    variant whose expert activations are quantized per group of 32."""
    return dict(name="qwen3-moe-30b-a3b-shape", n_layers=n_layers, hidden=2048, n_heads=32, n_kv=4, head_dim=128, inter=0, vocab=151936,
                eps=1e-6, attn_scale=float(1.0 / np.sqrt(128)), softcap=0.0, theta=1e6, n_experts=128, top_k=8, norm_topk=1,
                exp_inter=768, qk_norm=1, exp_act_group=exp_act_group)


def inv_freq(head_dim, theta):
    d = np.arange(0, head_dim, 2, dtype=np.float64)
    return 1.0 / (float(theta) ** (d / head_dim))


def weight_bytes(cfg):
    """Algorithmic weight bytes one decode step streams (each byte once, shared by the batch), excluding MoE experts."""
    H, qd, kvd = cfg["hidden"], cfg["n_heads"] * cfg["head_dim"], cfg["n_kv"] * cfg["head_dim"]
    per_layer = (qd * H + 2 * kvd * H + H * qd) * 0.5625
    if not cfg.get("n_experts"):
        per_layer += 3 * cfg["inter"] * H * 0.5625
    else:
        per_layer += cfg["n_experts"] * H * 4  # f32 router
    head = cfg["vocab"] * H + cfg["vocab"] * 4  # int8 codes + f32 row scales
    norms = (2 * cfg["n_layers"] + 1) * H * 4
    return cfg["n_layers"] * per_layer + head + norms


def expert_bytes(cfg):
    """Bytes of one expert's three int4-g32 matrices (codes + f16 group scales)."""
    return 3 * cfg["exp_inter"] * cfg["hidden"] * 0.5625


def kv_bytes_per_position(cfg, kv="f16"):
    """K and V of one position over all layers: binary16, or int8 codes plus one f32 scale per kv head."""
    per_head = cfg["head_dim"] * 2 if kv == "f16" else cfg["head_dim"] + 4
    return cfg["n_layers"] * 2 * cfg["n_kv"] * per_head


class Resident:
    """A synthetic model resident on the device, with its KV slots pre-filled."""

    def __init__(self, dev, cfg, seed=1234, slots=32, ctx_cap=4352, keep_layers=0, progress=None, kv="f16"):
        self.dev, self.cfg = dev, cfg
        H, hd = cfg["hidden"], cfg["head_dim"]
        qd, kvd, V = cfg["n_heads"] * hd, cfg["n_kv"] * hd, cfg["vocab"]
        nE = cfg.get("n_experts", 0)
        self.model = capi.Model(dev, cfg, inv_freq(hd, cfg["theta"]))
        self.kept = []  # host copies of the first keep_layers layers (for the CPU baseline)
        s = [seed * 100003]

        def nxt():
            s[0] += 1
            return s[0]

        m = self.model
        for l in range(cfg["n_layers"]):
            keep = {} if l < keep_layers else None
            for proj, N, K in (("q", qd, H), ("k", kvd, H), ("v", kvd, H), ("o", H, qd)):
                b = synth.q4k_normal(nxt(), N, K, SIGMA)
                m.upload_q4k(l, proj, b, N, K)
                if keep is not None:
                    keep[proj] = (b, N, K)
            for which in ("attn_norm", "ffn_norm"):
                v = synth.normal(nxt(), H, 0.02, 1.0)
                m.upload_f32(l, which, v)
                if keep is not None:
                    keep[which] = v
            if cfg.get("qk_norm"):
                for which in ("q_norm", "k_norm"):
                    v = synth.normal(nxt(), hd, 0.02, 1.0)
                    m.upload_f32(l, which, v)
                    if keep is not None:
                        keep[which] = v
            if not nE:
                I = cfg["inter"]
                for proj, N, K in (("gate", I, H), ("up", I, H), ("down", H, I)):
                    b = synth.q4k_normal(nxt(), N, K, SIGMA)
                    m.upload_q4k(l, proj, b, N, K)
                    if keep is not None:
                        keep[proj] = (b, N, K)
            else:
                EI = cfg["exp_inter"]
                r = synth.normal(nxt(), nE * H, SIGMA).reshape(nE, H)
                m.upload_f32(l, "router", r)
                if keep is not None:
                    keep["router"] = r
                    keep["experts"] = []
                m.set_act_group(cfg.get("exp_act_group", 32))
                for e in range(nE):
                    ex = {}
                    for proj, N, K in (("gate", EI, H), ("up", EI, H), ("down", H, EI)):
                        nib, s16 = synth.w4a8_normal(nxt(), N, K, SIGMA)
                        m.upload_w4a8(l, proj, e, nib, s16, K)
                        ex[proj] = (nib, s16, N, K)
                    if keep is not None:
                        keep["experts"].append(ex)
            if keep is not None:
                self.kept.append(keep)
            if progress and ((l + 1) % 8 == 0 or l + 1 == cfg["n_layers"]):
                progress("layer %d/%d uploaded" % (l + 1, cfg["n_layers"]))
        self.final_norm = synth.normal(nxt(), H, 0.02, 1.0)
        m.upload_f32(-1, "final_norm", self.final_norm)
        m.set_act_group(cfg.get("act_group", 32))
        self.head = synth.w8a8_normal(nxt(), V, H, SIGMA)
        m.upload_w8a8(-1, "head", *self.head)
        self.embed = synth.w8a8_normal(nxt(), V, H, SIGMA)
        m.upload_embedding(*self.embed)
        m.finalize()
        m.kv_configure(slots, ctx_cap, kv)
        if progress:
            progress("model resident")

    def embed_rows(self, ids):
        """Host embedding lookup, as goinfer's embedResidentInto does it (decoder/residency.go:1077-1123)."""
        q, sc = self.embed
        return q[ids].astype(np.float32) * sc[ids][:, None]

    def prefill_kv(self, lens, seed=77, progress=None):
        """Positions [0, lens[i]) of slot i, every layer: K,V ~ N(0,1). One [max len][kv dim] pair of arrays per layer,
        each slot takes its prefix. Returns the per-layer arrays of the first len(self.kept) layers."""
        cfg = self.cfg
        kvd = cfg["n_kv"] * cfg["head_dim"]
        mx = int(max(lens))
        kept = []
        for l in range(cfg["n_layers"]):
            k = synth.normal(seed * 1000 + 2 * l, mx * kvd).reshape(mx, kvd)
            v = synth.normal(seed * 1000 + 2 * l + 1, mx * kvd).reshape(mx, kvd)
            for i, n in enumerate(lens):
                self.model.kv_upload(i, l, 0, k[:n], v[:n])
            if l < len(self.kept):
                kept.append((k, v))
            if progress and (l + 1) % 8 == 0:
                progress("KV layer %d/%d filled" % (l + 1, cfg["n_layers"]))
        return kept

    def close(self):
        self.model.close()
