"""ctypes binding of librocmdecode.so (include/rocmdecode.h). numpy in, numpy out; no torch."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "librocmdecode.so")
HSACO_PATH = os.path.join(HERE, "lib", "rocmdecode_gfx950.hsaco")

RD_OK, RD_DECLINED = 0, 1
PROJ = dict(q=0, k=1, v=2, o=3, gate=4, up=5, down=6, head=7)
VEC = dict(attn_norm=0, ffn_norm=1, q_norm=2, k_norm=3, final_norm=4, router=5, qkv_bias=6, router_bias=7, attn_sinks=8, post_attn_norm=9, post_ffn_norm=10)
WANT_LOGITS, WANT_ARGMAX = 1, 2

EXPORTS = [
    "rd_device_open", "rd_device_open_image", "rd_device_close", "rd_last_error", "rd_backend_name", "rd_device_sync",
    "rd_device_mem_info", "rd_matmul_bt", "rd_dequant_q4k", "rd_gemm_q4k", "rd_gemm_w8a8", "rd_gemm_w4a8",
    "rd_attn_ragged", "rd_moe_route", "rd_rmsnorm", "rd_rope", "rd_model_create", "rd_model_destroy",
    "rd_model_upload_q4k", "rd_model_upload_w8a8", "rd_model_upload_w4a8", "rd_model_upload_f32", "rd_model_finalize",
    "rd_kv_configure", "rd_kv_upload", "rd_kv_truncate", "rd_kv_reset", "rd_step_batch", "rd_model_max_rows", "rd_forward",
    "rd_last_moe_indices", "rd_model_upload_embedding", "rd_bench_steps", "rd_bench_profile", "rd_bench_attn_chain", "rd_bench_enqueue", "rd_bench_attn_kernel_name", "rd_bench_attn_in_step", "rd_moe_route_ex", "rd_attn_ragged_ex", "rd_model_set_router", "rd_model_set_window", "rd_model_set_block", "rd_model_set_graph", "rd_model_graph_stats", "rd_bench_prefill", "rd_bench_class_count",
    "rd_bench_class_name", "rd_bench_kernel", "rd_gateup_q4k_quant", "rd_moe_replay", "rd_bench_attn", "rd_step_ragged", "rd_prefill_last",
    "rd_kv_configure_typed", "rd_attn_ragged_i8", "rd_attn_ragged_rows", "rd_plan_attention", "rd_plan_gemm", "rd_step_batch_topk", "rd_last_logits", "rd_topk_rows", "rd_bench_attn_i8", "rd_step_ragged_draw", "rd_forward_no_logits",
    "rd_step_batch_draw", "rd_sample_rows", "rd_greedy_chain_start", "rd_greedy_chain_next", "rd_sample_chain_start",
    "rd_sample_chain_next", "rd_greedy_chain_stop",
    "rd_dequant_q5k", "rd_dequant_q6k", "rd_gemm_q5k", "rd_gemm_q6k", "rd_model_upload_q5k", "rd_model_upload_q6k",
    "rd_kv_download", "rd_qkv_rope_store", "rd_topk_rows_static", "rd_quant_act", "rd_model_set_act_group",
]


class RocmError(RuntimeError):
    pass


def plan_attention(lens, slots, heads_per_kv, n_kv, max_items=1 << 16):
    """The step's attention work list (host planning, no device): (items [n][4], ranges [rows][n_kv][3], grouped)."""
    lens = np.ascontiguousarray(lens, dtype=np.int32)
    sl = None if slots is None else np.ascontiguousarray(slots, dtype=np.int32)
    items = np.zeros((max_items, 4), np.int32)
    ranges = np.zeros((len(lens), n_kv, 3), np.int32)
    n, g = C.c_int(0), C.c_int(0)
    check(lib().rd_plan_attention(len(lens), _p(lens), None if sl is None else _p(sl), heads_per_kv, n_kv, _p(items), max_items, _p(ranges),
                                  C.byref(n), C.byref(g)), "rd_plan_attention")
    return items[:n.value].copy(), ranges, bool(g.value)


def plan_gemm(N, n_kblocks):
    s, k = C.c_int(0), C.c_int(0)
    check(lib().rd_plan_gemm(N, n_kblocks, C.byref(s), C.byref(k)), "rd_plan_gemm")
    return s.value, k.value


class Draw(C.Structure):
    _fields_ = [("temperature", C.c_double), ("seed", C.c_uint64), ("draw", C.c_uint64), ("mode", C.c_int32), ("reserved", C.c_int32)]


DRAW_NONE, DRAW_GREEDY, DRAW_GUMBEL = 0, 1, 2


def make_draws(draws):
    """per row None, "greedy" or (temperature, seed, draw) -> a ctypes array of rd_draw"""
    arr = (Draw * len(draws))()
    for i, dw in enumerate(draws):
        if dw is None:
            arr[i].mode = DRAW_NONE
        elif isinstance(dw, str):
            arr[i].mode = DRAW_GREEDY
        else:
            arr[i].mode, arr[i].temperature, arr[i].seed, arr[i].draw = DRAW_GUMBEL, dw[0], dw[1], dw[2]
    return arr


class ModelDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "hidden", "n_heads", "n_kv_heads", "head_dim", "inter", "vocab")] + [
        ("rms_eps", C.c_float), ("attn_scale", C.c_float), ("attn_softcap", C.c_float),
        ("n_experts", C.c_int32), ("top_k", C.c_int32), ("norm_topk_prob", C.c_int32), ("expert_inter", C.c_int32),
        ("qk_norm", C.c_int32), ("rope_inv_freq", C.c_void_p)]


_lib = None


def lib():
    """The loaded C-ABI library. Raises when it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RocmError("%s is missing: run `python -m goinfer_amd.build`" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        L.rd_last_error.restype = C.c_char_p
        L.rd_backend_name.restype = C.c_char_p
        for name in ("rd_device_close", "rd_model_destroy", "rd_greedy_chain_stop"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def check(rc, what):
    if rc != RD_OK:
        kind = "declined" if rc == RD_DECLINED else "failed (%d)" % rc
        raise RocmError("%s %s: %s" % (what, kind, lib().rd_last_error().decode()))


class Device:
    """rd_device: one MI355X, its code object and stream."""

    def __init__(self, ordinal=0):
        self.h = C.c_void_p()
        check(lib().rd_device_open(ordinal, C.byref(self.h)), "rd_device_open")

    def close(self):
        if self.h:
            lib().rd_device_close(self.h)
            self.h = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def sync(self):
        check(lib().rd_device_sync(self.h), "rd_device_sync")

    def mem_info(self):
        f, t = C.c_size_t(), C.c_size_t()
        check(lib().rd_device_mem_info(self.h, C.byref(f), C.byref(t)), "rd_device_mem_info")
        return f.value, t.value

    def matmul_bt(self, a, b):
        a, b = _f32(a), _f32(b)
        M, K = a.shape
        N = b.shape[0]
        dst = np.empty((M, N), np.float32)
        check(lib().rd_matmul_bt(self.h, _p(a), _p(b), _p(dst), M, K, N), "rd_matmul_bt")
        return dst

    def dequant_q4k(self, blocks, N, K):
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        out = np.empty((N, K), np.float32)
        check(lib().rd_dequant_q4k(self.h, _p(blocks), N, K, _p(out)), "rd_dequant_q4k")
        return out

    def dequant_kquant(self, fmt, blocks, N, K):
        """fmt 'q5k' or 'q6k': raw super-blocks -> f32 [N][K]."""
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        out = np.empty((N, K), np.float32)
        name = "rd_dequant_" + fmt
        check(getattr(lib(), name)(self.h, _p(blocks), N, K, _p(out)), name)
        return out

    def gemm_kquant(self, fmt, blocks, N, K, a):
        a = _f32(a)
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        dst = np.empty((a.shape[0], N), np.float32)
        name = "rd_gemm_" + fmt
        check(getattr(lib(), name)(self.h, _p(blocks), N, K, _p(a), a.shape[0], _p(dst)), name)
        return dst

    def sample_rows(self, logits, draws):
        """draws: per row "greedy" or (temperature, seed, draw). Returns int32 ids."""
        logits = _f32(logits)
        rows, V = logits.shape
        arr = make_draws(draws)
        ids = np.empty(rows, np.int32)
        check(lib().rd_sample_rows(self.h, _p(logits), rows, V, arr, _p(ids)), "rd_sample_rows")
        return ids

    def gemm_q4k(self, blocks, N, K, a, blocks2=None):
        a = _f32(a)
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        b2 = None if blocks2 is None else np.ascontiguousarray(blocks2, dtype=np.uint8)
        dst = np.empty((a.shape[0], N), np.float32)
        check(lib().rd_gemm_q4k(self.h, _p(blocks), N, K, _p(a), a.shape[0], _p(dst), _p(b2)), "rd_gemm_q4k")
        return dst

    def gateup_q4k_quant(self, gate, up, I, K, a):
        a = _f32(a)
        gate = np.ascontiguousarray(gate, dtype=np.uint8)
        up = np.ascontiguousarray(up, dtype=np.uint8)
        dst = np.empty((a.shape[0], I), np.float32)
        check(lib().rd_gateup_q4k_quant(self.h, _p(gate), _p(up), I, K, _p(a), a.shape[0], _p(dst)), "rd_gateup_q4k_quant")
        return dst

    def gemm_w8a8(self, q, scales, a, act_group=32):
        """act_group 32: activations quantized per group of 32; 0: one scale per row (goinfer's ActQuantGroup)."""
        a = _f32(a)
        q = np.ascontiguousarray(q, dtype=np.int8)
        scales = _f32(scales)
        N, K = q.shape
        dst = np.empty((a.shape[0], N), np.float32)
        check(lib().rd_gemm_w8a8(self.h, _p(q), _p(scales), N, K, _p(a), a.shape[0], int(act_group), _p(dst)), "rd_gemm_w8a8")
        return dst

    def gemm_w4a8(self, nib, s16, K, a, act_group=32):
        a = _f32(a)
        nib = np.ascontiguousarray(nib, dtype=np.uint8)
        s16 = np.ascontiguousarray(s16, dtype=np.uint16)
        N = nib.shape[0]
        dst = np.empty((a.shape[0], N), np.float32)
        check(lib().rd_gemm_w4a8(self.h, _p(nib), _p(s16), N, K, _p(a), a.shape[0], int(act_group), _p(dst)), "rd_gemm_w4a8")
        return dst

    def topk_rows(self, logits, k, temperature=1.0, want_z=True):
        """Each row's k best entries in (logit descending, id ascending) order: (ids [rows][k'], vals [rows][k'], z [rows] or None)."""
        logits = _f32(logits)
        rows, V = logits.shape
        kk = min(k, V)
        ids = np.empty((rows, kk), np.int32)
        vals = np.empty((rows, kk), np.float32)
        z = np.empty(rows, np.float64) if want_z else None
        check(lib().rd_topk_rows(self.h, _p(logits), rows, V, k, C.c_double(temperature), int(want_z), _p(ids), _p(vals), _p(z)), "rd_topk_rows")
        return ids, vals, z

    def attn_ragged(self, lens, k, v, q, n_h, n_kv, hd, scale, softcap=0.0, kv="f16"):
        """kv: "f16" (the binary16 cache) or "i8" (the int8 cache with one scale per position and kv head)."""
        lens = np.ascontiguousarray(lens, dtype=np.int32)
        off = np.zeros(len(lens), np.int64)
        off[1:] = np.cumsum(lens[:-1])
        k, v, q = _f32(k), _f32(v), _f32(q)
        out = np.empty((len(lens), n_h * hd), np.float32)
        name = "rd_attn_ragged" if kv == "f16" else "rd_attn_ragged_i8"
        check(getattr(lib(), name)(self.h, len(lens), _p(lens), _p(off), _p(k), _p(v), _p(q), n_h, n_kv, hd,
                                   C.c_float(scale), C.c_float(softcap), _p(out)), name)
        return out

    def attn_ragged_rows(self, lens, nq, k, v, q, n_h, n_kv, hd, scale, softcap=0.0, kv="f16"):
        """Sequence i brings nq[i] query rows (its last nq[i] positions); q, out: [sum nq][n_h*hd]."""
        lens = np.ascontiguousarray(lens, dtype=np.int32)
        nq = np.ascontiguousarray(nq, dtype=np.int32)
        off = np.zeros(len(lens), np.int64)
        off[1:] = np.cumsum(lens[:-1])
        k, v, q = _f32(k), _f32(v), _f32(q)
        out = np.empty((int(nq.sum()), n_h * hd), np.float32)
        check(lib().rd_attn_ragged_rows(self.h, 0 if kv == "f16" else 1, len(lens), _p(lens), _p(nq), _p(off), _p(k), _p(v), _p(q), n_h, n_kv,
                                        hd, C.c_float(scale), C.c_float(softcap), _p(out)), "rd_attn_ragged_rows")
        return out

    def attn_ragged_ex(self, lens, k, v, q, n_h, n_kv, hd, scale, softcap=0.0, kv="f16", nq=None, window=0, sinks=None):
        """rd_attn_ragged_rows (nq=None: one query row per sequence) with a sliding window and attention sinks."""
        lens = np.ascontiguousarray(lens, dtype=np.int32)
        off = np.zeros(len(lens), np.int64)
        off[1:] = np.cumsum(lens[:-1])
        k, v, q = _f32(k), _f32(v), _f32(q)
        rows = len(lens) if nq is None else int(np.sum(nq))
        nq_a = None if nq is None else np.ascontiguousarray(nq, dtype=np.int32)
        sk = None if sinks is None else _f32(sinks)
        out = np.empty((rows, n_h * hd), np.float32)
        check(lib().rd_attn_ragged_ex(self.h, 0 if kv == "f16" else 1, len(lens), _p(lens), _p(nq_a), _p(off), _p(k), _p(v), _p(q), n_h, n_kv, hd,
                                      C.c_float(scale), C.c_float(softcap), int(window), _p(sk), _p(out)), "rd_attn_ragged_ex")
        return out

    def qkv_rope_store(self, x, pos, n_h, n_kv, hd, inv_freq, q_norm=None, k_norm=None, eps=1e-6, bias=None, kv="f16"):
        """The step's q|k|v epilogue on rows x [rows][(n_h+2n_kv)*hd]: (q, k as stored, v as stored)."""
        x = _f32(x)
        rows = x.shape[0]
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        inv = np.ascontiguousarray(inv_freq, dtype=np.float64)
        qn = None if q_norm is None else _f32(q_norm)
        kn = None if k_norm is None else _f32(k_norm)
        bi = None if bias is None else _f32(bias)
        q = np.empty((rows, n_h * hd), np.float32)
        k = np.empty((rows, n_kv * hd), np.float32)
        v = np.empty((rows, n_kv * hd), np.float32)
        check(lib().rd_qkv_rope_store(self.h, 0 if kv == "f16" else 1, rows, _p(x), _p(pos), n_h, n_kv, hd, _p(inv), _p(qn), _p(kn), C.c_float(eps),
                                      _p(bi), _p(q), _p(k), _p(v)), "rd_qkv_rope_store")
        return q, k, v

    def quant_act(self, a, act_group=32):
        """int8 quantization of rows a [M][K]. act_group 32: (codes int8 [M][K], scales f32 [M][K/32], sums f32 [M][K/32]);
        act_group 0, one scale per row: (codes, scales f32 [M], None)."""
        a = _f32(a)
        M, K = a.shape
        codes = np.empty((M, K), np.int8)
        scales = np.empty((M, K // 32) if act_group else (M,), np.float32)
        sums = np.empty((M, K // 32), np.float32) if act_group else None
        check(lib().rd_quant_act(self.h, _p(a), M, K, int(act_group), _p(codes), _p(scales), _p(sums)), "rd_quant_act")
        return codes, scales, sums

    def moe_route(self, logits, k, norm, bias=None, sigmoid=False, scale=0.0, n_group=0, topk_group=0):
        logits = _f32(logits)
        T, nE = logits.shape
        idx = np.full((T, k), -1, np.int32)
        wgt = np.zeros((T, k), np.float32)
        bs = None if bias is None else _f32(bias)
        check(lib().rd_moe_route_ex(self.h, _p(logits), _p(bs), T, nE, k, int(sigmoid), int(norm), C.c_double(scale), int(n_group), int(topk_group),
                                    _p(idx), _p(wgt)), "rd_moe_route_ex")
        return idx, wgt

    def rmsnorm(self, x, w, eps):
        x, w = _f32(x), _f32(w)
        out = np.empty_like(x)
        check(lib().rd_rmsnorm(self.h, _p(x), _p(w), x.shape[0], x.shape[1], C.c_float(eps), _p(out)), "rd_rmsnorm")
        return out

    def rope(self, vec, heads, head_dim, pos, inv_freq):
        v = _f32(vec).copy()
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        inv = np.ascontiguousarray(inv_freq, dtype=np.float64)
        check(lib().rd_rope(self.h, _p(v), v.shape[0], heads, head_dim, _p(pos), _p(inv)), "rd_rope")
        return v

    def bench_attn(self, lens, n_h, n_kv, hd, scale, softcap, warmup, iters, kv="f16"):
        lens = np.ascontiguousarray(lens, dtype=np.int32)
        tot, part = np.empty(iters, np.float32), np.empty(iters, np.float32)
        name = "rd_bench_attn" if kv == "f16" else "rd_bench_attn_i8"
        check(getattr(lib(), name)(self.h, len(lens), _p(lens), n_h, n_kv, hd, C.c_float(scale), C.c_float(softcap), warmup, iters,
                                   _p(tot), _p(part)), name)
        return tot, part

    def bench_kernel(self, name, args, warmup, iters):
        a = np.ascontiguousarray(args, dtype=np.int64)
        ms = np.empty(iters, np.float32)
        check(lib().rd_bench_kernel(self.h, name.encode(), _p(a), len(a), warmup, iters, _p(ms)), "rd_bench_kernel")
        return ms


class Model:
    """rd_model: the resident decoder (goinfer's resident.Forward + DecodeSubsystem for this backend)."""

    def __init__(self, dev, cfg, inv_freq):
        self.dev, self.cfg = dev, dict(cfg)
        self._inv = np.ascontiguousarray(inv_freq, dtype=np.float64)
        d = ModelDesc(cfg["n_layers"], cfg["hidden"], cfg["n_heads"], cfg["n_kv"], cfg["head_dim"], cfg.get("inter", 0),
                      cfg["vocab"], cfg["eps"], cfg["attn_scale"], cfg.get("softcap", 0.0), cfg.get("n_experts", 0),
                      cfg.get("top_k", 0), int(cfg.get("norm_topk", 0)), cfg.get("exp_inter", 0), int(cfg.get("qk_norm", 0)),
                      _p(self._inv))
        self.h = C.c_void_p()
        check(lib().rd_model_create(dev.h, C.byref(d), C.byref(self.h)), "rd_model_create")
        if cfg.get("router_sigmoid") or cfg.get("router_scale") or cfg.get("n_group"):  # the router's variant (mlp.go:130-228)
            check(lib().rd_model_set_router(self.h, int(cfg.get("router_sigmoid", 0)), C.c_double(cfg.get("router_scale", 0.0)),
                                            int(cfg.get("n_group", 0)), int(cfg.get("topk_group", 0))), "rd_model_set_router")

        if cfg.get("norm_add_one") or cfg.get("act_gelu_tanh") or cfg.get("final_softcap") or cfg.get("logit_scale"):
            # Gemma's block (rmsnorm.go:10-13,229-234), Granite's logits_scaling (model_forward.go:304-320)
            check(lib().rd_model_set_block(self.h, int(cfg.get("norm_add_one", 0)), int(cfg.get("act_gelu_tanh", 0)),
                                           C.c_float(cfg.get("final_softcap", 0.0)), C.c_double(cfg.get("logit_scale", 0.0))), "rd_model_set_block")

    def bench_attn_in_step(self, slots, pos, ids0, reps=8):
        """(ms per attention launch inside the step, ms per whole step): whole steps against steps without their attention launches."""
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        ids0 = np.ascontiguousarray(ids0, dtype=np.int32)
        a, b = C.c_float(0), C.c_float(0)
        check(lib().rd_bench_attn_in_step(self.h, len(slots), _p(slots), _p(pos), _p(ids0), int(reps), C.byref(a), C.byref(b)), "rd_bench_attn_in_step")
        return a.value, b.value

    def attn_kernel_name(self):
        """The attention kernel the last step launched for its whole-context work list."""
        f = lib().rd_bench_attn_kernel_name
        f.restype = C.c_char_p
        return f(self.h).decode()

    def bench_enqueue(self, slots, pos0, ids0, steps):
        """Host microseconds per step to enqueue `steps` chained greedy steps (nothing waits for the GPU inside the loop)."""
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        pos0 = np.ascontiguousarray(pos0, dtype=np.int32)
        ids0 = np.ascontiguousarray(ids0, dtype=np.int32)
        us = C.c_double(0)
        check(lib().rd_bench_enqueue(self.h, len(slots), _p(slots), _p(pos0), _p(ids0), int(steps), C.byref(us)), "rd_bench_enqueue")
        return us.value

    def set_graph(self, on):
        """Returns False when the library keeps graph replay off (a profiler tool library is attached)."""
        rc = lib().rd_model_set_graph(self.h, 1 if on else 0)
        if rc == 1:  # RD_DECLINED
            return False
        check(rc, "rd_model_set_graph")
        return True

    def graph_stats(self):
        """(graphs captured, steps replayed from a graph)"""
        a, b = C.c_longlong(0), C.c_longlong(0)
        check(lib().rd_model_graph_stats(self.h, C.byref(a), C.byref(b)), "rd_model_graph_stats")
        return a.value, b.value

    def set_window(self, layer, window):
        check(lib().rd_model_set_window(self.h, layer, int(window)), "rd_model_set_window")

    def close(self):
        if self.h:
            lib().rd_model_destroy(self.h)
            self.h = C.c_void_p()

    def upload_q4k(self, layer, proj, blocks, N, K):
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        check(lib().rd_model_upload_q4k(self.h, layer, PROJ[proj], _p(blocks), N, K), "rd_model_upload_q4k")

    def upload_kquant(self, fmt, layer, proj, blocks, N, K):
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        name = "rd_model_upload_" + fmt
        check(getattr(lib(), name)(self.h, layer, PROJ[proj], _p(blocks), N, K), name)

    def upload_w8a8(self, layer, proj, q, scales):
        q = np.ascontiguousarray(q, dtype=np.int8)
        scales = _f32(scales)
        check(lib().rd_model_upload_w8a8(self.h, layer, PROJ[proj], _p(q), _p(scales), q.shape[0], q.shape[1]),
              "rd_model_upload_w8a8")

    def upload_w4a8(self, layer, proj, expert, nib, s16, K):
        nib = np.ascontiguousarray(nib, dtype=np.uint8)
        s16 = np.ascontiguousarray(s16, dtype=np.uint16)
        check(lib().rd_model_upload_w4a8(self.h, layer, PROJ[proj], expert, _p(nib), _p(s16), nib.shape[0], K),
              "rd_model_upload_w4a8")

    def set_act_group(self, act_group):
        """goinfer's ActQuantGroup of the int8 / int4 tensors uploaded from here on: 32, or 0 = one activation scale per row."""
        check(lib().rd_model_set_act_group(self.h, int(act_group)), "rd_model_set_act_group")

    def upload_f32(self, layer, which, v):
        v = _f32(v)
        check(lib().rd_model_upload_f32(self.h, layer, VEC[which], _p(v), C.c_size_t(v.size)), "rd_model_upload_f32")

    def finalize(self):
        check(lib().rd_model_finalize(self.h), "rd_model_finalize")

    def kv_configure(self, slots, ctx_cap, kv="f16"):
        if kv == "f16":
            check(lib().rd_kv_configure(self.h, slots, ctx_cap), "rd_kv_configure")
        else:
            check(lib().rd_kv_configure_typed(self.h, slots, ctx_cap, {"i8": 1}[kv]), "rd_kv_configure_typed")

    def kv_upload(self, slot, layer, base, keys, vals):
        keys, vals = _f32(keys), _f32(vals)
        check(lib().rd_kv_upload(self.h, slot, layer, base, keys.shape[0], _p(keys), _p(vals)), "rd_kv_upload")

    def kv_download(self, slot, layer, base, n):
        """Rows base..base+n-1 of a slot as the cache holds them, widened to f32: (keys, vals), each [n][n_kv*hd]."""
        kvd = self.cfg["n_kv"] * self.cfg["head_dim"]
        keys, vals = np.empty((n, kvd), np.float32), np.empty((n, kvd), np.float32)
        check(lib().rd_kv_download(self.h, slot, layer, base, n, _p(keys), _p(vals)), "rd_kv_download")
        return keys, vals

    def kv_reset(self, slot):
        check(lib().rd_kv_reset(self.h, slot), "rd_kv_reset")

    def kv_truncate(self, slot, pos):
        check(lib().rd_kv_truncate(self.h, slot, pos), "rd_kv_truncate")

    def max_rows(self):
        """The widest step (BatchStepRange's hi) and the rows of a prompt pass."""
        return int(lib().rd_model_max_rows(self.h))

    def step_batch(self, slots, pos, emb, want=WANT_LOGITS):
        emb = _f32(emb)
        B = emb.shape[0]
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        logits = np.empty((B, self.cfg["vocab"]), np.float32) if want & WANT_LOGITS else None
        ids = np.empty(B, np.int32) if want & WANT_ARGMAX else None
        check(lib().rd_step_batch(self.h, B, _p(slots), _p(pos), _p(emb), want, _p(logits), _p(ids)), "rd_step_batch")
        return logits, ids

    def step_batch_draw(self, slots, pos, emb, draws, want=0):
        """draws: per row None, "greedy" or (temperature, seed, draw). Returns (logits or None, ids with -1 for rows without a draw)."""
        emb = _f32(emb)
        B = emb.shape[0]
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        arr = make_draws(draws)
        logits = np.empty((B, self.cfg["vocab"]), np.float32) if want & WANT_LOGITS else None
        ids = np.empty(B, np.int32)
        check(lib().rd_step_batch_draw(self.h, B, _p(slots), _p(pos), _p(emb), arr, want, _p(logits), _p(ids)), "rd_step_batch_draw")
        return logits, ids

    def greedy_chain_start(self, slot, tok, pos):
        check(lib().rd_greedy_chain_start(self.h, slot, int(tok), pos), "rd_greedy_chain_start")

    def greedy_chain_next(self):
        out = C.c_int(-1)
        check(lib().rd_greedy_chain_next(self.h, C.byref(out)), "rd_greedy_chain_next")
        return out.value

    def sample_chain_start(self, slot, tok, pos, temperature, seed, draw):
        check(lib().rd_sample_chain_start(self.h, slot, int(tok), pos, C.c_double(temperature), C.c_uint64(seed), C.c_uint64(draw)),
              "rd_sample_chain_start")

    def sample_chain_next(self, seed, draw):
        out = C.c_int(-1)
        check(lib().rd_sample_chain_next(self.h, C.c_uint64(seed), C.c_uint64(draw), C.byref(out)), "rd_sample_chain_next")
        return out.value

    def chain_stop(self):
        lib().rd_greedy_chain_stop(self.h)

    def step_ragged(self, slots, pos, embs, want=WANT_LOGITS):
        """embs: one [rows_i][hidden] array per sequence. Returns (logits [sum rows][vocab] or None, ids [sum rows] or None)."""
        n_rows = np.ascontiguousarray([len(e) for e in embs], dtype=np.int32)
        emb = _f32(np.concatenate([np.asarray(e, dtype=np.float32).reshape(len(e), -1) for e in embs], axis=0))
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        R = int(n_rows.sum())
        logits = np.empty((R, self.cfg["vocab"]), np.float32) if want & WANT_LOGITS else None
        ids = np.empty(R, np.int32) if want & WANT_ARGMAX else None
        check(lib().rd_step_ragged(self.h, len(slots), _p(slots), _p(pos), _p(n_rows), _p(emb), want, _p(logits), _p(ids)), "rd_step_ragged")
        return logits, ids

    def step_ragged_draw(self, slots, pos, embs, draws, want=0):
        """draws: per sequence None, "greedy" or (temperature, seed, draw), for its last row. Returns (logits or None, ids per row)."""
        n_rows = np.ascontiguousarray([len(e) for e in embs], dtype=np.int32)
        emb = _f32(np.concatenate([np.asarray(e, dtype=np.float32).reshape(len(e), -1) for e in embs], axis=0))
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        R = int(n_rows.sum())
        logits = np.empty((R, self.cfg["vocab"]), np.float32) if want & WANT_LOGITS else None
        ids = np.empty(R, np.int32)
        check(lib().rd_step_ragged_draw(self.h, len(slots), _p(slots), _p(pos), _p(n_rows), _p(emb), make_draws(draws), want, _p(logits), _p(ids)),
              "rd_step_ragged_draw")
        return logits, ids

    def step_batch_topk(self, slots, pos, emb, k, temperature=None):
        """The step with each row's logits reduced to its k best entries: (ids [B][k'], vals [B][k'], z [B] or None)."""
        emb = _f32(emb)
        B = emb.shape[0]
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        kk = min(k, self.cfg["vocab"])
        ids = np.empty((B, kk), np.int32)
        vals = np.empty((B, kk), np.float32)
        t = None if temperature is None else np.ascontiguousarray(np.broadcast_to(temperature, (B,)), dtype=np.float64)
        z = None if t is None else np.empty(B, np.float64)
        check(lib().rd_step_batch_topk(self.h, B, _p(slots), _p(pos), _p(emb), k, _p(t), int(t is not None), _p(ids), _p(vals), _p(z)),
              "rd_step_batch_topk")
        return ids, vals, z

    def last_logits(self, row):
        out = np.empty(self.cfg["vocab"], np.float32)
        check(lib().rd_last_logits(self.h, row, _p(out)), "rd_last_logits")
        return out

    def forward_no_logits(self, slot, pos, emb):
        emb = _f32(emb)
        check(lib().rd_forward_no_logits(self.h, slot, pos, _p(emb)), "rd_forward_no_logits")

    def prefill_last(self, slot, start_pos, emb):
        emb = _f32(emb)
        logits = np.empty(self.cfg["vocab"], np.float32)
        check(lib().rd_prefill_last(self.h, slot, start_pos, emb.shape[0], _p(emb), _p(logits)), "rd_prefill_last")
        return logits

    def moe_replay(self, idx, wgt):
        """The next step replays this routing ([B][layers][k] indices and weights) instead of its own."""
        idx = np.ascontiguousarray(idx, dtype=np.int32)
        wgt = _f32(wgt)
        check(lib().rd_moe_replay(self.h, idx.shape[0], _p(idx), _p(wgt)), "rd_moe_replay")

    def forward(self, slot, pos, emb):
        emb = _f32(emb)
        logits = np.empty(self.cfg["vocab"], np.float32)
        check(lib().rd_forward(self.h, slot, pos, _p(emb), _p(logits)), "rd_forward")
        return logits

    def last_moe_indices(self, B):
        idx = np.empty((B, self.cfg["n_layers"], self.cfg["top_k"]), np.int32)
        check(lib().rd_last_moe_indices(self.h, _p(idx)), "rd_last_moe_indices")
        return idx

    def upload_embedding(self, q, scales):
        q = np.ascontiguousarray(q, dtype=np.int8)
        scales = _f32(scales)
        assert q.shape == (self.cfg["vocab"], self.cfg["hidden"])
        check(lib().rd_model_upload_embedding(self.h, _p(q), _p(scales)), "rd_model_upload_embedding")

    def bench_steps(self, slots, pos0, ids0, warmup, steps, want_ids=False):
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        pos0 = np.ascontiguousarray(pos0, dtype=np.int32)
        ids0 = np.ascontiguousarray(ids0, dtype=np.int32)
        ms = np.empty(steps, np.float32)
        ids = np.empty((steps, len(slots)), np.int32) if want_ids else None
        check(lib().rd_bench_steps(self.h, len(slots), _p(slots), _p(pos0), _p(ids0), warmup, steps, _p(ms), _p(ids)), "rd_bench_steps")
        return (ms, ids) if want_ids else ms

    def bench_prefill(self, slot, ids, profile=False):
        """A prompt of len(ids) tokens into `slot` (reset first), inputs on the device: milliseconds, and with profile the per-class
        (milliseconds, launches) as bench_profile gives them."""
        L = lib()
        L.rd_bench_class_name.restype = C.c_char_p
        n = L.rd_bench_class_count()
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        total = C.c_float(0)
        ms = np.zeros(n, np.float32)
        cnt = np.zeros(n, np.int32)
        check(L.rd_bench_prefill(self.h, int(slot), len(ids), _p(ids), 1 if profile else 0, C.byref(total), _p(ms), _p(cnt)), "rd_bench_prefill")
        classes = {L.rd_bench_class_name(i).decode(): (float(ms[i]), int(cnt[i])) for i in range(n) if cnt[i]}
        return (float(total.value), classes) if profile else float(total.value)

    def bench_attn_chain(self, slots, pos, ids0, reps=1):
        """(ms per launch, launches) of the attention kernel launched back to back for every layer between one pair of events."""
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        ids0 = np.ascontiguousarray(ids0, dtype=np.int32)
        ms, n = C.c_float(0), C.c_int(0)
        check(lib().rd_bench_attn_chain(self.h, len(slots), _p(slots), _p(pos), _p(ids0), reps, C.byref(ms), C.byref(n)), "rd_bench_attn_chain")
        return float(ms.value), int(n.value)

    def bench_profile(self, slots, pos, ids0):
        L = lib()
        L.rd_bench_class_name.restype = C.c_char_p
        n = L.rd_bench_class_count()
        slots = np.ascontiguousarray(slots, dtype=np.int32)
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        ids0 = np.ascontiguousarray(ids0, dtype=np.int32)
        ms = np.zeros(n, np.float32)
        cnt = np.zeros(n, np.int32)
        check(L.rd_bench_profile(self.h, len(slots), _p(slots), _p(pos), _p(ids0), _p(ms), _p(cnt)), "rd_bench_profile")
        return {L.rd_bench_class_name(i).decode(): (float(ms[i]), int(cnt[i])) for i in range(n) if cnt[i]}
