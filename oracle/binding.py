"""ctypes binding of oracle/liboracle.so (the C restatement in oracle.c). Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

OR_F32, OR_Q4K, OR_W4A8, OR_W8A8, OR_Q5K, OR_Q6K = 0, 1, 2, 3, 4, 5


class Mat(C.Structure):
    _fields_ = [("kind", C.c_int), ("N", C.c_int), ("K", C.c_int), ("data", C.c_void_p),
                ("scales", C.c_void_p), ("act_group", C.c_int)]


class Layer(C.Structure):
    _fields_ = [(n, Mat) for n in ("q", "k", "v", "o", "gate", "up", "down")] + [
        ("attn_norm", C.c_void_p), ("ffn_norm", C.c_void_p), ("q_norm", C.c_void_p), ("k_norm", C.c_void_p),
        ("q_bias", C.c_void_p), ("k_bias", C.c_void_p), ("v_bias", C.c_void_p),
        ("router", Mat), ("exp_gate", C.POINTER(Mat)), ("exp_up", C.POINTER(Mat)), ("exp_down", C.POINTER(Mat)),
        ("router_bias", C.c_void_p), ("window", C.c_int), ("sinks", C.c_void_p),
        ("post_attn_norm", C.c_void_p), ("post_ffn_norm", C.c_void_p)]


class Model(C.Structure):
    _fields_ = [("n_layers", C.c_int), ("hidden", C.c_int), ("n_heads", C.c_int), ("n_kv", C.c_int),
                ("head_dim", C.c_int), ("inter", C.c_int), ("vocab", C.c_int),
                ("eps", C.c_double), ("attn_scale", C.c_double), ("softcap", C.c_double),
                ("inv_freq", C.c_void_p),
                ("n_experts", C.c_int), ("top_k", C.c_int), ("norm_topk", C.c_int), ("exp_inter", C.c_int),
                ("kv_f16", C.c_int), ("layers", C.POINTER(Layer)), ("final_norm", C.c_void_p), ("head", Mat),
                ("router_sigmoid", C.c_int), ("router_scale", C.c_double), ("n_group", C.c_int), ("topk_group", C.c_int),
                ("norm_add_one", C.c_int), ("act_gelu_tanh", C.c_int), ("final_softcap", C.c_double),
                ("logit_scale", C.c_double)]


def f16_round_trip(x):
    """What an f16 cache holds of x (round-half-up narrowing, widened back)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().or_f16_round_trip(x.ctypes.data, out.ctypes.data, x.size)
    return out


def build():
    """Compile liboracle.so from the C sources beside this file."""
    subprocess.check_call(["make", "-s", "-C", _HERE])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        L = C.CDLL(path)
        L.or_f32_to_f16.restype = C.c_uint16
        L.or_f32_to_f16.argtypes = [C.c_float]
        L.or_f16_to_f32.restype = C.c_float
        L.or_f16_to_f32.argtypes = [C.c_uint16]
        L.or_silu.restype = C.c_float
        L.or_silu.argtypes = [C.c_float]
        L.or_gelu_tanh.restype = C.c_float
        L.or_gelu_tanh.argtypes = [C.c_float]
        L.or_softcap_logits.argtypes = [C.c_void_p, C.c_size_t, C.c_float]
        L.or_quantize_row_int8.restype = C.c_float
        L.or_kprint_name.restype = C.c_char_p
        L.or_softmax_z.restype = C.c_double
        L.or_cache_new.restype = C.c_void_p
        L.or_cache_new.argtypes = [C.POINTER(Model), C.c_int]
        L.or_cache_free.argtypes = [C.POINTER(Model), C.c_void_p]
        L.or_cache_upload.restype = C.c_int
        L.or_cache_upload.argtypes = [C.POINTER(Model), C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.or_f16_round_trip.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        _LIB = L
    return _LIB


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def fingerprints():
    L = lib()
    out = {}
    buf = C.create_string_buffer(80)
    for i in range(L.or_kprint_count()):
        L.or_kprint_run(i, buf)
        out[L.or_kprint_name(i).decode()] = buf.value.decode()
    return out


def set_threads(n):
    lib().or_set_threads(int(n))


FAULTS = dict(none=0, rope_pos=1, gqa_head=2, q4k_scale_index=3, no_softcap=4, q4k_no_min=5, causal_range=6, w4a8_scale_index=7)


def set_fault(name):
    """Turns the oracle into a deliberately wrong one (see oracle.h OR_FAULT_*): only for measuring what a parity test can see."""
    lib().or_set_fault(FAULTS[name])


def dequant_q4k(blocks):
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    nb = blocks.size // 144
    out = np.empty(nb * 256, np.float32)
    lib().or_dequant_q4k(_p(blocks), C.c_size_t(nb), _p(out))
    return out


def dequant_q5k(blocks):
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    nb = blocks.size // 176
    out = np.empty(nb * 256, np.float32)
    lib().or_dequant_q5k(_p(blocks), C.c_size_t(nb), _p(out))
    return out


def dequant_q6k(blocks):
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    nb = blocks.size // 210
    out = np.empty(nb * 256, np.float32)
    lib().or_dequant_q6k(_p(blocks), C.c_size_t(nb), _p(out))
    return out


def quantize_act(a, group):
    a = f32(a)
    M, K = a.shape
    nG = (K + group - 1) // group if group > 0 else 1
    q = np.empty((M, K), np.int8)
    S = np.empty((M, nG), np.float32)
    lib().or_quantize_act(_p(a), M, K, group, _p(q), _p(S))
    return q, S


def quantize_rows_int8(w):
    w = f32(w)
    N, K = w.shape
    q = np.empty((N, K), np.int8)
    S = np.empty(N, np.float32)
    lib().or_quantize_act(_p(w), N, K, 0, _p(q), _p(S))
    return q, S


def quantize_int4(w, group=32):
    w = f32(w)
    N, K = w.shape
    q4 = np.empty((N, (K + 1) // 2), np.uint8)
    s16 = np.empty((N, (K + group - 1) // group), np.uint16)
    lib().or_quantize_int4_mat(_p(w), N, K, group, _p(q4), _p(s16))
    return q4, s16


class WMat:
    """A weight matrix handed to the oracle; keeps its numpy buffers alive."""

    def __init__(self, kind, N, K, data, scales=None, act_group=0):
        self.kind, self.N, self.K, self.act_group = kind, N, K, act_group
        self.data = np.ascontiguousarray(data)
        self.scales = None if scales is None else np.ascontiguousarray(scales)

    @staticmethod
    def from_f32(w):
        w = f32(w)
        return WMat(OR_F32, w.shape[0], w.shape[1], w)

    def c(self):
        return Mat(self.kind, self.N, self.K, _p(self.data), _p(self.scales) if self.scales is not None else None,
                   self.act_group)


def matmul(w, a):
    a = f32(a)
    M = a.shape[0]
    dst = np.empty((M, w.N), np.float32)
    m = w.c()
    lib().or_matmul(C.byref(m), _p(a), M, _p(dst))
    return dst


def matmul_f64ref(w, a):
    a = f32(a)
    M = a.shape[0]
    dst = np.empty((M, w.N), np.float64)
    m = w.c()
    lib().or_matmul_f64ref(C.byref(m), _p(a), M, _p(dst))
    return dst


def rmsnorm(x, w, eps, add_one=False):
    x = f32(x)
    w = f32(w)
    out = np.empty_like(x)
    rows, dim = x.shape
    lib().or_rmsnorm(_p(out), _p(x), _p(w), rows, dim, C.c_double(eps), int(add_one))
    return out


def rope(vec, heads, head_dim, pos, inv_freq, scale=1.0):
    v = f32(vec).copy()
    inv = np.ascontiguousarray(inv_freq, dtype=np.float64)
    lib().or_rope(_p(v), heads, head_dim, int(pos), _p(inv), len(inv), C.c_double(scale))
    return v


def swiglu(gate, up):
    g = f32(gate).copy()
    u = f32(up)
    lib().or_swiglu(_p(g), _p(u), g.size)
    return g


def geglu(gate, up):
    """geluTanh(gate) * up, element by element."""
    g = f32(gate).copy()
    u = f32(up)
    lib().or_geglu(_p(g), _p(u), g.size)
    return g


def softcap_logits(x, cap):
    """cap * tanh(x / cap) as the final-logit softcap computes it."""
    x = f32(x).copy()
    lib().or_softcap_logits(_p(x), C.c_size_t(x.size), C.c_float(cap))
    return x


def route_experts(logits, k, norm, scale=0.0, bias=None, sigmoid=False, n_group=0, topk_group=0):
    lg = f32(logits)
    idx = np.empty(k, np.int32)
    wts = np.empty(k, np.float32)
    bs = f32(bias) if bias is not None else None
    n = lib().or_route_experts_ex(_p(lg), _p(bs), lg.size, k, int(sigmoid), int(norm), C.c_double(scale), int(n_group), int(topk_group),
                                  _p(idx), _p(wts))
    return idx[:n], wts[:n]


def group_limit(sel, n_group, topk_group):
    sel = f32(sel)
    out = np.empty_like(sel)
    lib().or_group_limit(_p(sel), sel.size, int(n_group), int(topk_group), _p(out))
    return out


def topk_by_logit(x, k):
    x = f32(x)
    ids = np.empty(min(k, x.size), np.int32)
    vals = np.empty(min(k, x.size), np.float32)
    n = lib().or_topk_by_logit(_p(x), x.size, k, _p(ids), _p(vals))
    return ids[:n], vals[:n]


def softmax_z(x, temperature):
    x = f32(x)
    return lib().or_softmax_z(_p(x), x.size, C.c_double(temperature))


def argmax(x):
    x = f32(x)
    return lib().or_argmax(_p(x), x.size)


def attend(q, keys, vals, n_keys, nH, nKV, hd, scale, softcap=0.0, start=0, sinks=None):
    q = f32(q)
    keys = f32(keys)
    vals = f32(vals)
    ctx = np.empty(nH * hd, np.float32)
    sk = f32(sinks) if sinks is not None else None
    lib().or_attend_sinks(_p(q), _p(ctx), _p(keys), _p(vals), int(n_keys), int(start), nH, nKV, hd,
                          C.c_double(scale), C.c_double(softcap), _p(sk))
    return ctx


class OracleModel:
    """decodeMultiStep over numpy weights. layers: list of dicts with WMat entries q,k,v,o,(gate,up,down | router,
    exp_gate[],exp_up[],exp_down[]) and f32 arrays attn_norm, ffn_norm, optional q_norm,k_norm, q_bias,k_bias,v_bias,
    router_bias, sinks, post_attn_norm, post_ffn_norm and an int window."""

    def __init__(self, cfg, layers, final_norm, head, inv_freq):
        self.cfg = cfg
        self._keep = []
        nL = len(layers)
        self._layers = (Layer * nL)()
        nE = cfg.get("n_experts", 0)
        for i, lw in enumerate(layers):
            L = self._layers[i]
            for n in ("q", "k", "v", "o"):
                setattr(L, n, lw[n].c())
            self._keep.append(lw)
            L.window = int(lw.get("window", 0))
            for n in ("attn_norm", "ffn_norm", "q_norm", "k_norm", "q_bias", "k_bias", "v_bias", "router_bias", "sinks",
                      "post_attn_norm", "post_ffn_norm"):
                if lw.get(n) is not None:
                    arr = f32(lw[n])
                    self._keep.append(arr)
                    setattr(L, n, _p(arr))
            if nE == 0:
                for n in ("gate", "up", "down"):
                    setattr(L, n, lw[n].c())
            else:
                L.router = lw["router"].c()
                for n in ("exp_gate", "exp_up", "exp_down"):
                    arr = (Mat * nE)(*[m.c() for m in lw[n]])
                    self._keep.append(arr)
                    setattr(L, n, arr)
        self._fn = f32(final_norm)
        self._inv = np.ascontiguousarray(inv_freq, dtype=np.float64)
        self._head = head
        self.m = Model(nL, cfg["hidden"], cfg["n_heads"], cfg["n_kv"], cfg["head_dim"], cfg.get("inter", 0),
                       cfg["vocab"], cfg["eps"], cfg["attn_scale"], cfg.get("softcap", 0.0), _p(self._inv),
                       nE, cfg.get("top_k", 0), int(cfg.get("norm_topk", 0)), cfg.get("exp_inter", 0),
                       int(cfg.get("kv_f16", 0)), self._layers, _p(self._fn), head.c(),
                       int(cfg.get("router_sigmoid", 0)), float(cfg.get("router_scale", 0.0)), int(cfg.get("n_group", 0)), int(cfg.get("topk_group", 0)),
                       int(cfg.get("norm_add_one", 0)), int(cfg.get("act_gelu_tanh", 0)), float(cfg.get("final_softcap", 0.0)),
                       float(cfg.get("logit_scale", 0.0)))

    def new_cache(self, cap):
        return lib().or_cache_new(C.byref(self.m), cap)

    def cache_upload(self, c, layer, base, keys, vals):
        """UploadKV: rows [n][kv dim] of one layer at positions base.., narrowed as the cache stores them."""
        keys = np.ascontiguousarray(keys, dtype=np.float32)
        vals = np.ascontiguousarray(vals, dtype=np.float32)
        if lib().or_cache_upload(C.byref(self.m), C.c_void_p(c), layer, base, keys.shape[0], keys.ctypes.data, vals.ctypes.data):
            raise RuntimeError("oracle: cache upload out of range")

    def free_cache(self, c):
        lib().or_cache_free(C.byref(self.m), C.c_void_p(c))

    def step(self, emb, caches, want_moe=False, want_weights=False, replay=None):
        """One decodeMultiStep. want_moe: also the expert indices [B][layers][k]; want_weights: and the routing weights.
        replay=(idx, wts): use this routing instead of the step's own."""
        emb = f32(emb)
        B = emb.shape[0]
        logits = np.empty((B, self.cfg["vocab"]), np.float32)
        arr = (C.c_void_p * B)(*caches)
        trace = wts = None
        if replay is not None:
            trace = np.ascontiguousarray(replay[0], dtype=np.int32).copy()
            wts = np.ascontiguousarray(replay[1], dtype=np.float32).copy()
        elif want_moe or want_weights:
            trace = np.full((B, self.cfg_layers(), self.cfg["top_k"]), -1, np.int32)
            wts = np.zeros((B, self.cfg_layers(), self.cfg["top_k"]), np.float32)
        rc = lib().or_decode_multi_step_traced(C.byref(self.m), B, _p(emb), arr, _p(logits), _p(trace) if trace is not None else None,
                                               _p(wts) if wts is not None else None, 1 if replay is not None else 0)
        if rc != 0:
            raise RuntimeError("oracle: cache full")
        if want_weights:
            return logits, trace, wts
        return (logits, trace) if want_moe else logits

    def cfg_layers(self):
        return self.m.n_layers


def philox4x32(ctr, key):
    c = (C.c_uint32 * 4)(*ctr)
    k = (C.c_uint32 * 2)(*key)
    out = (C.c_uint32 * 4)()
    lib().or_philox4x32(c, k, out)
    return tuple(out)


def gumbel_noise(h):
    f = lib().or_gumbel_noise
    f.restype = C.c_float
    return float(f(C.c_uint32(int(h))))


def gumbel_draw(logits, temperature, seed, draw, guarded=False):
    """GumbelDraw(logits, temperature, seed, draw); guarded=True adds Sampler.gumbelDraw's temperature guards."""
    x = f32(logits)
    f = lib().or_sampler_gumbel_draw if guarded else lib().or_gumbel_draw
    return int(f(_p(x), x.size, C.c_double(temperature), C.c_uint64(seed), C.c_uint64(draw)))


def gumbel_draw_many(logits, temperature, seed, draw0, count):
    x = f32(logits)
    out = np.empty(count, np.int32)
    lib().or_gumbel_draw_many(_p(x), x.size, C.c_double(temperature), C.c_uint64(seed), C.c_uint64(draw0), count, _p(out))
    return out


def gumbel_noise_many(h):
    h = np.ascontiguousarray(h, dtype=np.uint32)
    out = np.empty(h.size, np.float32)
    lib().or_gumbel_noise_many(_p(h), C.c_size_t(h.size), _p(out))
    return out


def dequantize_rows_int8(q, scales):
    q = np.ascontiguousarray(q, dtype=np.int8)
    scales = f32(scales)
    rows, cols = q.shape
    out = np.empty((rows, cols), np.float32)
    lib().or_dequantize_rows_int8(_p(out), _p(q), _p(scales), rows, cols)
    return out
