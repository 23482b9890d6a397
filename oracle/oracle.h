/*
 * oracle.h — CPU restatement of goinfer's ragged batched decode step.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing the product ships (the HIP kernels, the C-ABI host library, the
 * benchmark's GPU leg) may call into this file; it exists so the GPU path has something to be checked
 * against, and so the benchmark can time a CPU baseline beside the GPU number.
 *
 * Every function cites the reference file:line (relative to the goinfer tree) it restates. The
 * arithmetic owned by the un-vendored module github.com/townsendmerino/aikit v1.78.0 (go.mod:8) is
 * restated from its in-tree call sites and twins, and pinned by the SHA-256 fingerprints in
 * testdata/kernel_fingerprints.json (see kprint.c).
 *
 * Pin status (checked by tests/test_oracle_fingerprints.py and tests/test_oracle_golden.py):
 *   or_f32_to_f16 / or_f16_to_f32        pinned: linalg.F32ToF16, linalg.F16ToF32 fingerprints
 *   or_dequant_q4k                       pinned: embed.GGUFFile(Q4_K).Tensor fingerprint
 *   or_dequant_q5k / or_dequant_q6k      pinned: embed.GGUFFile(Q5_K).Tensor, embed.GGUFFile(Q6_K).Tensor fingerprints
 *   or_quantize_row_int8                 pinned: linalg.QuantizeRowInt8 fingerprint
 *   or_quantize_act                      pinned: linalg.QuantizeActQ fingerprint (per-row and per-32)
 *   or_dequantize_rows_int8              pinned: linalg.DequantizeRowsInt8Into fingerprint (with or_quantize_row_int8 the
 *                                        whole of the int8 KV cache's store and read)
 *   or_quantize_int4_row / _mat          pinned: linalg.QuantizeGroupInt4Row, linalg.QuantizeInt4
 *   or_qk_acc64 / or_av_acc64            pinned: linalg.MatmulQKAcc64, linalg.MatmulAVAcc64
 *   or_rmsnorm, or_rope, or_swiglu, or_softmax_f32, or_topk, or_route_experts, or_argmax
 *                                        plain Go in the reference, restated statement by statement;
 *                                        pinned by closed forms + the HF goldens (llama-tiny, internlm3-tiny, qwen3moe-tiny, mixtral-tiny)
 *   or_route_experts_ex, or_group_limit  pinned: the known answers of the reference's decoder/moe_route_test.go (sigmoid scoring, the
 *                                        selection bias, group-limited selection, the scaling factor), tests/test_oracle_routing.py;
 *                                        top-3 routing also by the qwen3moe-tiny-k3 golden
 *   the attention window (or_layer.window, `start` of or_attend)
 *                                        pinned: the mistral-tiny-window golden (window 16 on every layer, the reference's bars
 *                                        of decoder/mistral_tiny_window_test.go) and the gemma2-tiny golden (window 4 on alternate
 *                                        layers); both fail with the window off
 *   attention softcap, or_gelu_tanh / or_geglu, or_softcap_logits, (1 + w) norms, post-branch norms
 *                                        pinned: the gemma2-tiny golden to 1e-5 (tests/test_oracle_golden.py shows each knob moves
 *                                        the logits by > 1e-3 when switched off)
 *   or_model.logit_scale                 pinned: the granite-dense-tiny golden (embedding x 12, attention scale 0.5, logits / 6)
 *   or_attend_sinks                      pinned by the closed form only (a softmax with one more logit per head, numpy f64):
 *                                        the reference's fixture with sinks is a GGUF file with MXFP4 experts, outside this path
 *   or_topk_by_logit, or_softmax_z       pinned by what the definition fixes: the first K of the row sorted by (logit desc, id asc) is
 *                                        unique, so the heap restatement is checked against an independent full sort (numpy
 *                                        lexsort) on normal, heavily tied and signed-zero rows, K from 1 to the row (the shapes of
 *                                        the reference's own topk_test.go); Z against numpy's f64 sum
 *   or_philox4x32                        pinned: the Random123 known-answer vectors the reference's philox_test.go holds
 *   or_gumbel_noise / _key / _draw       pinned by the closed form the reference's tests state (f64 -log(-log1p(-w)), range,
 *                                        monotone), by chi-square fit of the draw to softmax(l/T) under the reference's own
 *                                        pre-registered rule, and by its edge rows (-Inf never drawn, masked row -> argmax).
 *                                        The reference holds no golden token stream, so the counter layout (i>>2, draw,
 *                                        draw>>32, 0; lane i&3) is "parity unpinned" beyond its statement in the source.
 *   or_matmul (f32 kind)                 parity unpinned at bit level (aikit's summation order is arch dependent);
 *                                        pinned to tolerance by the HF goldens
 *   or_matmul (w8a8 kind)                pinned: linalg.MatmulBTW8A8 fingerprint (per-row activations, every reference
 *                                        configuration); per-32 activations: linalg.MatmulBTW8A8Into, bit-exact to the
 *                                        arm64[dotprod] entry (the reference's own amd64 and arm64 digests differ)
 *   or_matmul (q4k / w4a8 kinds)         parity unpinned at bit level: the reference's own result differs between
 *                                        amd64 and arm64 (kernel_fingerprints.json). Restated in the mathematically
 *                                        specified form (exact int32 dot per 32-group, f32 fold in ascending group
 *                                        order, backend/cuda/actgroup.cu:298-355) and checked against an f64 sum.
 *   or_matmul (q5k / q6k kinds)          parity unpinned at bit level: the reference holds no digest or golden for its
 *                                        native Q5_K / Q6_K lanes (they exist only as CUDA / Metal kernels). Restated in
 *                                        the specified form (backend/cuda/actgroup.cu:77-205) and held to 1e-5 of the f64
 *                                        sum over the fingerprint-pinned dequantizer and activation quantizer
 *                                        (tests/test_oracle_matmul.py).
 */
#ifndef GOINFER_ORACLE_H
#define GOINFER_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- 16-bit conversions: internal/runtime/f16/f16.go:14-63 ---- */
uint16_t or_f32_to_f16(float f);      /* round-half-up on the dropped bits */
float or_f16_to_f32(uint16_t h);

/* ---- Q4_K: decoder/gguf.go:1508-1537, backend/metal/kernels/gemm_kq_test.go:27-70 ---- */
void or_q4k_scale_min(int j, const uint8_t *q12, int *sc, int *m);
void or_dequant_q4k(const uint8_t *blocks, size_t n_blocks, float *out); /* 144 B -> 256 f32 each */
/* GGUF Q5_K (176-byte super-blocks: d, dmin f16; 12 bytes of 6-bit scales and mins as Q4_K; qh[32] fifth bits; qs[128] nibbles):
 * w = d*sc_j*q - dmin*m_j with q = nibble | fifth bit << 4. Pinned bit-exact by fingerprint embed.GGUFFile(Q5_K).Tensor. */
void or_dequant_q5k(const uint8_t *blocks, size_t n_blocks, float *out);
/* GGUF Q6_K (210-byte super-blocks: ql[128] low nibbles, qh[64] two high bits each, 16 int8 sub-block scales, d f16):
 * w = d*sc_s*(q-32), 16 sub-blocks of 16. Pinned bit-exact by fingerprint embed.GGUFFile(Q6_K).Tensor. */
void or_dequant_q6k(const uint8_t *blocks, size_t n_blocks, float *out);

/* ---- int8 rows back to f32: decoder/kvcache.go:54-59, backend/cuda/kvtype.cuh:48-52 ---- */
void or_dequantize_rows_int8(float *dst, const int8_t *q, const float *scales, int rows, int cols);

/* ---- activation quantizers: backend/cuda/kv8_store.cu:3-35, actgroup.cu:26-54 ---- */
float or_quantize_row_int8(const float *row, int n, int8_t *q);
/* group==0: one scale per row (S[m]); group>0: S[m*nG+g], nG=ceil(K/group) */
void or_quantize_act(const float *a, int M, int K, int group, int8_t *q, float *S);

/* ---- int4 g32: decoder/fakequant.go:99-131, backend/cuda/internal/wpack/wpack.go:165-207 ---- */
void or_quantize_int4_row(const float *row, int cols, int group, uint8_t *packed, float *scales);
void or_quantize_int4_mat(const float *w, int rows, int cols, int group, uint8_t *q4, uint16_t *s16);

/* ---- attention primitives: decoder/forwardn.go:379-383,488-490 (call sites of aikit MatmulQKAcc64/AVAcc64) ---- */
void or_qk_acc64(const float *a, const float *keys, float *dst, int M, int hd, int nKeys, int off, int kvDim);
void or_av_acc64(const float *scores, const float *vals, float *dst, int M, int nKeys, int hd, int off, int kvDim);

/* ---- glue: decoder/rmsnorm.go:29-92,204-207; rope.go:28-64; mlp.go:269-290,370-440,130-184 ---- */
void or_rmsnorm(float *dst, const float *src, const float *w, int rows, int dim, double eps, int add_one);
void or_rope(float *vec, int heads, int head_dim, int pos, const double *inv_freq, int half, double scale);
float or_silu(float x);
void or_swiglu(float *gate, const float *up, int n);
void or_softmax_f32(const float *x, int n, float *out);
int or_topk(const float *x, int n, int k, int *idx, float *val);
int or_route_experts(const float *logits, int nE, int k, int norm, double scale, int *idx, float *wts);
/* the whole of routeExperts: sigmoid scoring, selection bias, group-limited selection (decoder/mlp.go:130-228) */
int or_route_experts_ex(const float *logits, const float *bias, int nE, int k, int sigmoid, int norm, double scale, int nGroup,
                        int topkGroup, int *idx, float *wts);
void or_group_limit(const float *sel, int nE, int nGroup, int topkGroup, float *out);
int or_argmax(const float *x, int n); /* internal/runtime/sampling/sampler.go:485-520: first maximum wins */
int or_topk_by_logit(const float *x, int n, int k, int *ids, float *vals); /* sampler.go:726-782 + the (logit desc, id asc) order of TopKRow */
double or_softmax_z(const float *x, int n, double temperature);            /* the top-p denominator, f64 */

/* ---- temperature-only sampling by Gumbel-max: internal/runtime/sampling/philox.go, sampler_gumbel.go ---- */
void or_philox4x32(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);
float or_gumbel_noise(uint32_t h);
float or_gumbel_key(float logit, float invT, uint32_t h);
int or_gumbel_draw(const float *logits, int n, double temperature, uint64_t seed, uint64_t draw);         /* GumbelDraw */
int or_sampler_gumbel_draw(const float *logits, int n, double temperature, uint64_t seed, uint64_t draw); /* Sampler.gumbelDraw's guards */
void or_gumbel_draw_many(const float *logits, int n, double temperature, uint64_t seed, uint64_t draw0, int count, int *out);
void or_gumbel_noise_many(const uint32_t *h, size_t n, float *out);

/* ---- weight matrices and the matmul dispatch: decoder/weightmat.go:845-985 ---- */
enum { OR_F32 = 0, OR_Q4K = 1, OR_W4A8 = 2, OR_W8A8 = 3, OR_Q5K = 4, OR_Q6K = 5 };
typedef struct {
    int kind;           /* OR_* */
    int N, K;           /* rows (outputs), cols (inputs) */
    const void *data;   /* f32[N*K] | q4k blocks N*K/256*144 | nibbles N*((K+1)/2) | int8[N*K] */
    const void *scales; /* w4a8: uint16 f16[N*ceil(K/32)] | w8a8: f32[N] */
    int act_group;      /* activation quant group for int kinds: 32 (q4k mode) or 0 (per row) */
} or_mat;
void or_matmul(const or_mat *w, const float *a, int M, float *dst);
/* the same product with f64 accumulation over dequantized weights and dequantized activations */
void or_matmul_f64ref(const or_mat *w, const float *a, int M, double *dst);
void or_set_threads(int n);
/* Mutations of the oracle, used only to measure what size of mistake a parity test catches (never by a parity check itself). */
enum { OR_FAULT_NONE = 0, OR_FAULT_ROPE_POS = 1, OR_FAULT_GQA_HEAD = 2, OR_FAULT_Q4K_SCALE_INDEX = 3, OR_FAULT_NO_SOFTCAP = 4, OR_FAULT_Q4K_NO_MIN = 5,
       OR_FAULT_CAUSAL_RANGE = 6, OR_FAULT_W4A8_SCALE_INDEX = 7 };
void or_set_fault(int fault);

/* ---- one sequence's decode attention over its own cache:
 * decoder/program_cpu_n.go:497-515 + forwardn.go:295-500 (useAcc64, K=1) + kvcache.go:21-40 (f16 narrowing) ---- */
void or_attend(const float *q, float *ctx, const float *keys, const float *vals, int n_keys, int start,
               int nH, int nKV, int hd, double scale, double softcap);
/* the same with attention sinks (decoder/attention.go:305-322): sinks[nH] or NULL */
void or_attend_sinks(const float *q, float *ctx, const float *keys, const float *vals, int n_keys, int start,
                     int nH, int nKV, int hd, double scale, double softcap, const float *sinks);

/* decoder/rmsnorm.go:229-234 (geluTanh) and the GeGLU gate; decoder/model_forward.go:259-266 (softcapParallel) */
float or_gelu_tanh(float x);
void or_geglu(float *gate, const float *up, int n);
void or_softcap_logits(float *logits, size_t n, float cap);

/* ---- the model and decodeMultiStep: decoder/cpu_batch.go:166-197, program_cpu_n.go:406-563, mlp.go:36-120 ---- */
typedef struct {
    or_mat q, k, v, o, gate, up, down; /* dense FFN when n_experts==0 */
    const float *attn_norm, *ffn_norm; /* [hidden] */
    const float *q_norm, *k_norm;      /* [hd] or NULL (Qwen3 QK-norm) */
    const float *q_bias, *k_bias, *v_bias; /* [nH*hd], [nKV*hd], [nKV*hd] or NULL (Qwen2 projection biases) */
    or_mat router;                     /* [nE, hidden] */
    or_mat *exp_gate, *exp_up, *exp_down; /* [nE] each */
    const float *router_bias;          /* [nE] or NULL: e_score_correction_bias, shifts the selection only */
    int window;                        /* > 0: this layer attends to the last `window` positions only (keys from pos-window+1) */
    const float *sinks;                /* [nH] or NULL: a learned logit per query head that joins the softmax's max and denominator */
    const float *post_attn_norm;       /* [hidden] or NULL: Gemma 2's norm of the attention output before it joins the residual */
    const float *post_ffn_norm;        /* [hidden] or NULL: the same for the FFN output */
} or_layer;

typedef struct {
    int n_layers, hidden, n_heads, n_kv, head_dim, inter, vocab;
    double eps, attn_scale, softcap;
    const double *inv_freq; /* [head_dim/2] */
    int n_experts, top_k, norm_topk, exp_inter;
    int kv_f16;     /* KV cache element: 0 f32, 1 binary16 (round-half-up on append), 2 int8 per (position, kv head) with an f32 scale */
    or_layer *layers;
    const float *final_norm;
    or_mat head;
    int router_sigmoid;  /* 1: per-expert sigmoid scores instead of a softmax (DeepSeek / GLM) */
    double router_scale; /* routed_scaling_factor; 0 or 1 = none */
    int n_group, topk_group; /* > 1: group-limited selection */
    int norm_add_one;     /* 1: every RMSNorm scales by (1 + w) (Gemma stores weights as deviations from one) */
    int act_gelu_tanh;    /* 1: the gated FFN is GeGLU with the tanh-approximate GELU instead of SwiGLU */
    double final_softcap; /* > 0: logits become cap * tanh(logit / cap) */
    double logit_scale;   /* not 0 or 1: logits are multiplied by f32(1 / logit_scale) after the softcap (Granite logits_scaling) */
} or_model;

typedef struct {
    int pos;       /* rows stored so far */
    int cap;       /* allocated rows */
    float **k, **v; /* per layer [cap][n_kv*head_dim] (values already narrowed when kv_f16) */
} or_cache;

or_cache *or_cache_new(const or_model *m, int cap);
void or_cache_free(const or_model *m, or_cache *c);
/* The prefill bridge, resident.Forward.UploadKV (decoder/resident/forward.go:17-22): writes post-RoPE K and raw V rows
 * [n][n_kv*head_dim] of one layer at positions base..base+n-1, narrowed as the cache stores them; pos becomes
 * max(pos, base+n) once the caller has uploaded every layer. Returns -1 when the rows do not fit. */
int or_cache_upload(const or_model *m, or_cache *c, int layer, int base, int n, const float *keys, const float *vals);
/* dst[i] = f16_to_f32(f32_to_f16(src[i])): what an f16 cache holds of src. */
void or_f16_round_trip(const float *src, float *dst, size_t n);
/* emb: [B][hidden] (embedding rows, already scaled); logits: [B][vocab]. Appends one position to every cache. */
int or_decode_multi_step(const or_model *m, int B, const float *emb, or_cache **caches, float *logits,
                         int *moe_idx_trace /* [B][layers][top_k] or NULL */);
/* The same, also recording the routing weights (decoder/mlp.go:17-27 moeSelTrace / moeWtsTrace) or, with replay != 0,
 * reading both arrays as the routing to replay (moeSelOverride / moeWtsOverride, mlp.go:53-56). */
int or_decode_multi_step_traced(const or_model *m, int B, const float *emb, or_cache **caches, float *logits, int *moe_idx_trace,
                                float *moe_wts_trace /* [B][layers][top_k] or NULL */, int replay);

#ifdef __cplusplus
}
#endif
#endif
