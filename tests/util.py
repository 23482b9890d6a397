"""Shared helpers for the tests: safetensors reading (numpy only) and oracle models of the tiny fixtures."""
import json
import os
import struct

import numpy as np

from oracle import binding as ob

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_safetensors(path):
    with open(path, "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        hdr = json.loads(f.read(n))
        base = 8 + n
        out = {}
        for k, v in hdr.items():
            if k == "__metadata__":
                continue
            assert v["dtype"] == "F32", v["dtype"]
            lo, hi = v["data_offsets"]
            f.seek(base + lo)
            out[k] = np.frombuffer(f.read(hi - lo), dtype="<f4").reshape(v["shape"]).copy()
    return out


def inv_freq(head_dim, theta):
    """decoder/rope.go: invFreq[d] = theta^(-2d/headDim) as float64."""
    d = np.arange(0, head_dim, 2, dtype=np.float64)
    return 1.0 / (float(theta) ** (d / head_dim))


def tiny_model(name, wrap=ob.WMat.from_f32):
    """An oracle model over one of the committed tiny HF checkpoints; every matmul weight goes through wrap."""
    d = os.path.join(GOLDEN, name)
    cfg = json.load(open(os.path.join(d, "config.json")))
    t = load_safetensors(os.path.join(d, "model.safetensors"))
    H, nH, nKV = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim") or H // nH
    theta = cfg.get("rope_parameters", {}).get("rope_theta", cfg.get("rope_theta", 10000.0))
    nE = cfg.get("num_experts", cfg.get("num_local_experts", 0))
    gemma2 = cfg["model_type"] == "gemma2"
    layers = []
    for l in range(cfg["num_hidden_layers"]):
        p = "model.layers.%d." % l
        lw = {n: wrap(t[p + "self_attn.%s_proj.weight" % n]) for n in ("q", "k", "v", "o")}
        lw["attn_norm"] = t[p + "input_layernorm.weight"]
        if gemma2:  # four norm slots: before and after each branch
            lw["post_attn_norm"] = t[p + "post_attention_layernorm.weight"]
            lw["ffn_norm"] = t[p + "pre_feedforward_layernorm.weight"]
            lw["post_ffn_norm"] = t[p + "post_feedforward_layernorm.weight"]
            if cfg["layer_types"][l] == "sliding_attention":
                lw["window"] = cfg["sliding_window"]
        else:
            lw["ffn_norm"] = t[p + "post_attention_layernorm.weight"]
            if cfg["model_type"] == "mistral" and cfg.get("sliding_window"):  # every layer slides
                lw["window"] = cfg["sliding_window"]
        if p + "self_attn.q_norm.weight" in t:
            lw["q_norm"] = t[p + "self_attn.q_norm.weight"]
            lw["k_norm"] = t[p + "self_attn.k_norm.weight"]
        if nE == 0:
            for n in ("gate", "up", "down"):
                lw[n] = wrap(t[p + "mlp.%s_proj.weight" % n])
        elif cfg["model_type"] == "mixtral":
            q = p + "block_sparse_moe."
            lw["router"] = ob.WMat.from_f32(t[q + "gate.weight"])
            lw["exp_gate"] = [wrap(t[q + "experts.%d.w1.weight" % e]) for e in range(nE)]
            lw["exp_down"] = [wrap(t[q + "experts.%d.w2.weight" % e]) for e in range(nE)]
            lw["exp_up"] = [wrap(t[q + "experts.%d.w3.weight" % e]) for e in range(nE)]
        else:
            q = p + "mlp."
            lw["router"] = ob.WMat.from_f32(t[q + "gate.weight"])
            for n in ("gate", "up", "down"):
                lw["exp_" + n] = [wrap(t[q + "experts.%d.%s_proj.weight" % (e, n)]) for e in range(nE)]
        layers.append(lw)
    c = dict(hidden=H, n_heads=nH, n_kv=nKV, head_dim=hd, inter=cfg.get("intermediate_size", 0),
             vocab=cfg["vocab_size"], eps=cfg["rms_norm_eps"], attn_scale=1.0 / np.sqrt(hd),
             n_experts=nE, top_k=cfg.get("num_experts_per_tok", 0),
             norm_topk=1 if (cfg["model_type"] == "mixtral" or cfg.get("norm_topk_prob")) else 0,
             exp_inter=cfg.get("moe_intermediate_size", cfg.get("intermediate_size", 0)) if nE else 0)
    emb = t["model.embed_tokens.weight"]
    if gemma2:
        # decoder/model_forward.go:41-53: embedding rows scaled by float32(sqrt(hidden)); tied head; (1+w) norms; GeGLU;
        # attention scale query_pre_attn_scalar^-0.5; attention and final-logit softcaps
        c.update(attn_scale=float(cfg["query_pre_attn_scalar"]) ** -0.5, softcap=cfg["attn_logit_softcapping"],
                 final_softcap=cfg["final_logit_softcapping"], norm_add_one=1, act_gelu_tanh=1)
        head = wrap(emb)
        emb = emb * np.float32(np.sqrt(np.float64(H)))
    else:
        head = wrap(t["lm_head.weight"])
    if cfg["model_type"] == "granite":  # decoder/arch_granite.go:50-62: the three multipliers of a llama block (residual_multiplier is 1)
        assert cfg["residual_multiplier"] == 1.0
        c.update(attn_scale=float(cfg["attention_multiplier"]), logit_scale=float(cfg["logits_scaling"]))
        emb = emb * np.float32(cfg["embedding_multiplier"])
    m = ob.OracleModel(c, layers, t["model.norm.weight"], head, inv_freq(hd, theta))
    return m, emb, cfg
