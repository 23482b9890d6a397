/*
 * rocmdecode.h — C ABI of librocmdecode.so: the MI355X (gfx950) decode backend that sits behind goinfer's
 * backend seam. A Go `backend/rocm` module binds these entry points with purego (cgo-free, the way
 * backend/cuda/internal/gpudev binds libcuda); the library itself loads libamdhip64 at run time with
 * dlopen and its gfx950 code object with hipModuleLoadData.
 *
 * Conventions: every call returns RD_OK (0), RD_DECLINED (1: this backend does not take the request —
 * goinfer's DeclineResident, decoder/residency.go:240-255) or a negative failure; rd_last_error() holds the
 * reason. All calls on one model come from one thread (goinfer's resident executor, backend/cuda/resident.go:2135).
 * Host pointers are caller-owned and only read/written during the call.
 *
 * Reference interfaces replaced (paths relative to the goinfer tree):
 *   decoder/backend.go:23-32        Backend{Name, MatmulBT, Close}
 *   decoder/residency.go:208-210    ResidencyBackend.BuildResident
 *   decoder/resident/forward.go:5-38   Forward{Forward, ForwardN, UploadKV, TruncateTo, Reset, Close}
 *   decoder/resident/subsystems.go:102-117  DecodeSubsystem{StepBatch, ForwardArgmax}
 *   decoder/resident/subsystems.go:236-251  KVSubsystem{KVSlots, UseKVSlot}
 */
#ifndef ROCMDECODE_H
#define ROCMDECODE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RD_OK 0
#define RD_DECLINED 1
#define RD_ERR_ARG (-1)
#define RD_ERR_HIP (-2)
#define RD_ERR_STATE (-3)
#define RD_ERR_KV_FULL (-4) /* goinfer's ErrKVPoolFull (decoder/mc3_batch.go:492-499): the step wrote nothing */

typedef struct rd_device rd_device;
typedef struct rd_model rd_model;

/* projection ids for the upload calls */
enum { RD_PROJ_Q = 0, RD_PROJ_K, RD_PROJ_V, RD_PROJ_O, RD_PROJ_GATE, RD_PROJ_UP, RD_PROJ_DOWN, RD_PROJ_HEAD, RD_PROJ_COUNT };
/* f32 vectors. RD_VEC_QKV_BIAS (optional): the q, k and v projection biases end to end, (n_heads + 2 n_kv_heads) * head_dim values,
 * added right after the projections (Qwen2; decoder/attention.go:12-34 addBias, program_cpu_n.go:470-476). */
enum { RD_VEC_ATTN_NORM = 0, RD_VEC_FFN_NORM, RD_VEC_Q_NORM, RD_VEC_K_NORM, RD_VEC_FINAL_NORM, RD_VEC_ROUTER, RD_VEC_QKV_BIAS, RD_VEC_ROUTER_BIAS, RD_VEC_ATTN_SINKS,
       RD_VEC_POST_ATTN_NORM, RD_VEC_POST_FFN_NORM };
/* rd_step_batch `want` */
enum { RD_WANT_LOGITS = 1, RD_WANT_ARGMAX = 2 };

/* What BuildResident reads through Model.BackendView() (decoder/backend_view.go:17-108). */
typedef struct {
    int32_t n_layers, hidden, n_heads, n_kv_heads, head_dim, inter, vocab;
    float rms_eps;
    float attn_scale;        /* AttnScale(): 1/sqrt(head_dim) or query_pre_attn_scalar^-0.5 */
    float attn_softcap;      /* AttnLogitSoftcap(): 0 = off */
    int32_t n_experts;       /* 0 = dense FFN */
    int32_t top_k, norm_topk_prob, expert_inter;
    int32_t qk_norm;         /* per-head RMSNorm of q and k (Qwen3) */
    const double *rope_inv_freq; /* Layer(i).RopeInvFreq: head_dim/2 float64 entries */
} rd_model_desc;

/* ---- device: replaces backend/cuda/internal/gpudev/cuda.go:65-83 (Device open/close) ---- */
int rd_device_open(int ordinal, rd_device **out);
/* the same, from a code-object image the caller embeds (Go's go:embed of the .hsaco) */
int rd_device_open_image(int ordinal, const void *hsaco, size_t len, rd_device **out);
void rd_device_close(rd_device *d);
const char *rd_last_error(void);
/* "rocm": Backend.Name(), decoder/backend.go:24 */
const char *rd_backend_name(void);
int rd_device_sync(rd_device *d);
/* free and total device memory in bytes: decoder.RegisterMemoryProbe, backend/cuda/backend.go:20-25 */
int rd_device_mem_info(rd_device *d, size_t *free_b, size_t *total_b);

/* ---- Backend.MatmulBT (decoder/backend.go:26-30): dst[M,N] = a[M,K] . b[N,K]^T, f32, host pointers ---- */
int rd_matmul_bt(rd_device *d, const float *a, const float *b, float *dst, int M, int K, int N);

/* ---- kernel-level entry points (the reference's kernel tests bind these: backend/cuda/kernels tests) ---- */
/* Q4_K super-blocks (144 B per 256 weights, decoder/gguf.go:1508-1537) -> f32, bit-exact d*sc*q - dmin*m.
 * blocks: host, N*K/256*144 bytes; out: host f32[N*K]. */
int rd_dequant_q4k(rd_device *d, const void *blocks, int N, int K, float *out);
/* dst[M,N] = a[M,K] . W^T with W raw Q4_K blocks and per-32 int8 activation quantization
 * (decoder/weightmat.go:961-971; backend/cuda/actgroup.cu:298-355 gemv_q4k_g32). If W2 != NULL the call is the
 * fused gate/up SwiGLU: dst = silu(a.W^T) * (a.W2^T) (decoder/cpu_gateup_fused.go:83-148). Host pointers. */
int rd_gemm_q4k(rd_device *d, const void *W, int N, int K, const float *a, int M, float *dst, const void *W2);
/* The decode step's own fused kernel on its own: gate|up projection + SwiGLU + per-32 quantization in one launch
 * (decoder/cpu_gateup_fused.go:83-148 followed by linalg.QuantizeActQ at the down projection's input). dst[M][I] receives
 * the quantized activations, code * scale, exactly as the down projection reads them. I and K multiples of 256. */
int rd_gateup_q4k_quant(rd_device *d, const void *Wg, const void *Wu, int I, int K, const float *a, int M, float *dst);
/* Q5_K (176 B) and Q6_K (210 B) super-blocks, the file's own bytes as decoder.KQuantReader.RowSource hands them out
 * (decoder/kquant_native.go:240-265): -> f32 bit-exactly as (d*sc)*q - dmin*m and (d*sc)*(q-32), and
 * dst[M,N] = a[M,K] . W^T against per-32 int8 activations (backend/cuda/actgroup.cu:457-530 gemv_q5k_g32 / gemv_q6k_g32,
 * arithmetic at :77-205). Host pointers; K a multiple of 256, N of 32. */
int rd_dequant_q5k(rd_device *d, const void *blocks, int N, int K, float *out);
int rd_dequant_q6k(rd_device *d, const void *blocks, int N, int K, float *out);
int rd_gemm_q5k(rd_device *d, const void *W, int N, int K, const float *a, int M, float *dst);
int rd_gemm_q6k(rd_device *d, const void *W, int N, int K, const float *a, int M, float *dst);
/* The activation quantizer every int projection's input goes through (aikit QuantizeActQ, call sites decoder/weightmat.go:845-862,
 * cpu_gateup_fused.go:110-117; device twins backend/cuda/actgroup.cu:32-54 quantG32 and kv8_store.cu:27-35 — with the CPU path's
 * round-half-away, not the twins' round-to-even): a host f32 [M][K] -> codes int8 [M][K] and
 *   act_group 32: scales f32 [M][K/32] (maxabs/127, 1 for an all-zero group) and sums f32 [M][K/32] (scale * sum of the group's codes);
 *   act_group 0 (linalg.QuantizeRowInt8, one scale per row): scales f32 [M]; sums is not written and may be NULL.
 * K a multiple of 32. */
int rd_quant_act(rd_device *d, const float *a, int M, int K, int act_group, int8_t *codes, float *scales, float *sums);
/* act_group below is goinfer's WeightMat.ActQuantGroup(): 32 = activations quantized per group of 32 (the lanes its q4k mode runs
 * on the CPU, decoder/weightmat.go:961-971), 0 = one scale per row, the only case in which goinfer consults a backend's staged
 * QuantBackend.MatmulW8A8 / QuantBackend4.MatmulW4A8 hooks (decoder/backend.go:38-75, weightmat.go:909-912,936-938). */
/* int8 per-row weights x int8 activations. act_group 32: backend/cuda/actgroup.cu:421-437 gemv_w8a8_g32. act_group 0:
 * dst = (f32(int32 dot over K) * aScale[m]) * wScale[n], linalg.MatmulBTW8A8 bit for bit (internal/gpudev/gemv_quant.cu:99-112). */
int rd_gemm_w8a8(rd_device *d, const int8_t *q, const float *row_scale, int N, int K, const float *a, int M, int act_group, float *dst);
/* int4 group-32 weights with f16 scales x int8 activations. act_group 32: backend/cuda/actgroup.cu:243-275. act_group 0: per weight
 * group facc = fma(f32(idot_g), ws_g, facc), dst = facc * aScale[m] (internal/gpudev/gemv_quant.cu:40-95, backend/cuda/moe_rows.cu:24-106). */
int rd_gemm_w4a8(rd_device *d, const uint8_t *nib, const uint16_t *s16, int N, int K, const float *a, int M, int act_group, float *dst);
/* The step's q|k|v epilogue on its own (backend/cuda/gemv_fwd.cu:51-101 rope_kv, prefill_batched.cu rope_kv_ragged; CPU:
 * decoder/attention.go:12-34 addBias, program_cpu.go:351-375 applyQKNorm / applyRope, kvcache.go:21-40,43-52 Append's narrowing):
 * x: host f32 [rows][(n_h+2*n_kv)*hd], the projections of `rows` (<= 32) sequences, row r at position pos[r] of its own cache.
 * Adds bias, applies the per-head RMSNorm of q and k (either may be NULL) and NeoX RoPE with f64 angles, and stores k and v into
 * a cache of kv_type. q_out: f32 [rows][n_h*hd]; k_out, v_out: f32 [rows][n_kv*hd], the stored row read back from the cache
 * (binary16 narrowed half-up and widened, or code * scale of the int8 cache). */
int rd_qkv_rope_store(rd_device *d, int kv_type, int rows, const float *x, const int *pos, int n_h, int n_kv, int hd, const double *inv_freq,
                      const float *q_norm, const float *k_norm, float eps, const float *bias, float *q_out, float *k_out, float *v_out);
/* Ragged flash-decode attention (backend/cuda/decode_fa.cu fa_partial_ragged/fa_combine_ragged;
 * decoder/forwardn.go:295-500): n_seq sequences, sequence i has len[i] keys; k,v: host f32 [sum len][n_kv*hd]
 * (rows of sequence i start at row off[i]); they are narrowed to binary16 (round-half-up) into a paged pool
 * as the cache does. q: host f32 [n_seq][n_h*hd]; out: host f32 [n_seq][n_h*hd]. softcap 0 = off. */
int rd_attn_ragged(rd_device *d, int n_seq, const int *len, const int64_t *off, const float *k, const float *v,
                   const float *q, int n_h, int n_kv, int hd, float scale, float softcap, float *out);
/* The same through the int8 cache (RD_KV_I8 below): k and v are quantized per (position, kv head) as the cache stores them. */
int rd_attn_ragged_i8(rd_device *d, int n_seq, const int *len, const int64_t *off, const float *k, const float *v,
                      const float *q, int n_h, int n_kv, int hd, float scale, float softcap, float *out);
/* Several query rows per sequence, as a prompt pass or a verification step brings them (decoder/forwardn.go:295-500: row j of
 * a sequence's n rows attends to the keys up to its own position): sequence i has nq[i] <= len[i] query rows, its last
 * nq[i] positions, and row j sees keys 0..len[i]-nq[i]+j. q, out: host f32 [sum nq][n_h*hd] in sequence order. kv_type
 * RD_KV_F16 or RD_KV_I8. Consecutive rows of a sequence share one pass over its keys and values; each row's result is
 * bit-identical to the row computed alone. */
int rd_attn_ragged_rows(rd_device *d, int kv_type, int n_seq, const int *len, const int *nq, const int64_t *off, const float *k,
                        const float *v, const float *q, int n_h, int n_kv, int hd, float scale, float softcap, float *out);
/* rd_attn_ragged_rows (nq may be NULL: one query row per sequence) with the two knobs of decoder/attention.go:57-143 /
 * forwardn.go:379-500 that are not on every model: window > 0, each row reads only the last `window` positions up to its own
 * (kvmgr.WindowNeedStart: start = max(pos - window + 1, 0)); sinks (host f32 [n_h] or NULL), one learned logit per query head
 * that joins the softmax's maximum and denominator and nothing else (attention.go:305-322). */
int rd_attn_ragged_ex(rd_device *d, int kv_type, int n_seq, const int *len, const int *nq, const int64_t *off, const float *k, const float *v,
                      const float *q, int n_h, int n_kv, int hd, float scale, float softcap, int window, const float *sinks, float *out);
/* MoE routing (decoder/mlp.go:130-184 routeExperts, softmax scoring; backend/cuda/moe.cu:49-104 moe_route):
 * logits host f32 [T][nE]; idx int32 [T][k], wgt f32 [T][k], rank order. */
int rd_moe_route(rd_device *d, const float *logits, int T, int nE, int k, int norm, int *idx, float *wgt);
/* The whole of routeExperts (decoder/mlp.go:130-228): sigmoid != 0 scores every expert by its own sigmoid instead of a softmax
 * (DeepSeek / GLM); bias (host f32 [nE] or NULL, e_score_correction_bias) shifts the selection only, the weights stay the unbiased
 * scores; n_group > 1 keeps only the experts of the topk_group best of n_group contiguous groups eligible (groupLimit; at most 32
 * groups); scale (routed_scaling_factor) multiplies the weights when it is neither 0 nor 1. */
int rd_moe_route_ex(rd_device *d, const float *logits, const float *bias, int T, int nE, int k, int sigmoid, int norm, double scale,
                    int n_group, int topk_group, int *idx, float *wgt);
/* RMSNorm rows (decoder/rmsnorm.go:29-92) and NeoX RoPE (decoder/rope.go:28-64), host pointers. */
int rd_rmsnorm(rd_device *d, const float *x, const float *w, int rows, int dim, float eps, float *out);
int rd_rope(rd_device *d, float *vec, int rows, int heads, int head_dim, const int *pos, const double *inv_freq);

/* ---- resident model: replaces backend/cuda/backend.go:138-259 (BuildResident) ---- */
int rd_model_create(rd_device *d, const rd_model_desc *desc, rd_model **out);
void rd_model_destroy(rd_model *m);
/* raw 144-byte super-blocks, N rows of K/256 blocks (Model.OpenKQuant, decoder/kquant_native.go:198-273) */
int rd_model_upload_q4k(rd_model *m, int layer, int proj, const void *blocks, int N, int K);
/* raw Q5_K / Q6_K super-blocks of a tensor the file stores that way (decoder/kquant_native.go:49-80 noteKQuant records the
 * source, :240-265 serves the rows; backend/cuda/resident_build.go:1030 binds the native lanes). Projections that feed one
 * consumer (q|k|v, gate|up) may differ in kind, as a Q4_K_M file's attn_v does: each run of one kind is multiplied by its
 * own kernel into the shared partial sums. */
int rd_model_upload_q5k(rd_model *m, int layer, int proj, const void *blocks, int N, int K);
int rd_model_upload_q6k(rd_model *m, int layer, int proj, const void *blocks, int N, int K);
/* int8 rows + per-row f32 scale (WeightMat.Int8, decoder/weightmat.go:931) */
int rd_model_upload_w8a8(rd_model *m, int layer, int proj, const int8_t *q, const float *row_scale, int N, int K);
/* canonical int4 nibbles + binary16 group-32 scales (WeightMat.Int4F16, decoder/weightmat.go:904); expert < 0 = dense */
int rd_model_upload_w4a8(rd_model *m, int layer, int proj, int expert, const uint8_t *nib, const uint16_t *s16, int N, int K);
/* WeightMat.ActQuantGroup() of the int8 / int4 tensors (dense and expert) uploaded from here on: 32 (the default; goinfer's q4k
 * mode) or 0 (one activation scale per row: its int8 / int4 modes, decoder/weightmat.go:837,909,936; the experts' kernels
 * backend/cuda/moe_rows.cu:24-106, moe.cu:111-216). Projections that share a quantized input (q|k|v, gate|up) and all experts of a
 * model must agree, RD_DECLINED otherwise; Q4_K / Q5_K / Q6_K tensors are per-32 by kind. Before rd_model_finalize. */
int rd_model_set_act_group(rd_model *m, int act_group);
/* norms, router; RD_VEC_ROUTER_BIAS: a layer's e_score_correction_bias [n_experts]; RD_VEC_ATTN_SINKS: its attention sinks [n_heads];
 * RD_VEC_POST_ATTN_NORM / RD_VEC_POST_FFN_NORM [hidden]: Gemma 2's norm of the attention / feed-forward output before it joins the
 * residual (decoder/program_cpu.go:286-312, the PostAttn and PostMLP slots; backend/cuda/backend.go:86). Before rd_model_finalize. */
int rd_model_upload_f32(rd_model *m, int layer, int which, const float *v, size_t n);
/* The router's variant, decoder/mlp.go:130-228 (routeExperts, groupLimit); before rd_model_finalize. sigmoid: per-expert sigmoid
 * scores (DeepSeek / GLM) instead of a softmax; scale: routed_scaling_factor (0 or 1 = none); n_group > 1: group-limited
 * selection among the topk_group best of n_group contiguous groups (at most 32 groups, which must divide the experts). */
int rd_model_set_router(rd_model *m, int sigmoid, double scale, int n_group, int topk_group);
/* The block's family knobs, as backend/cuda/resident.go:549-565,2882-2886 holds them (addOneArg, act, finalSoftcap); before
 * rd_model_finalize. norm_add_one: every RMSNorm weight is stored as its deviation from one and scales by f32(1 + w)
 * (Architecture.RMSAddOne, decoder/rmsnorm.go:10-13,62-75; the sum is formed once at rd_model_finalize). act: the gated FFN's
 * activation, RD_ACT_SILU (SwiGLU) or RD_ACT_GELU_TANH (Gemma's GeGLU, decoder/rmsnorm.go:229-234; dense FFN only). final_softcap
 * > 0: logits become cap * tanh(logit / cap) (decoder/model_forward.go:259-266); logit_scale not 0 or 1: they are then multiplied by
 * f32(1 / logit_scale) (Architecture.LogitScale, Granite's logits_scaling; model_forward.go:304-320) — both before the argmax, the
 * draws, the top-K and the copy to the host. */
enum { RD_ACT_SILU = 0, RD_ACT_GELU_TANH = 1 };
int rd_model_set_block(rd_model *m, int norm_add_one, int act, float final_softcap, double logit_scale);
/* A sliding-window layer (decoder/kvcache.go:1063-1068 WindowStart): its rows read the last `window` positions only. Before
 * rd_model_finalize. The windowed layers of a model share one length (RD_DECLINED otherwise); the cache keeps every position. */
int rd_model_set_window(rd_model *m, int layer, int window);
/* HIP-graph replay of a step's launches (the single-queue executor of backend/cuda/resident.go:2135 is the reference's answer to
 * the same cost: a few hundred launches a step). Between the uploads of a step's metadata and the copies back, every launch
 * depends only on the model, the batch size, what is asked for and the size of the attention work list; a step that repeats the
 * previous step's values of those replays the graph captured from it, any other step is launched eagerly, and both give the same
 * bits. On by default; off at rd_model_create when ROCMDECODE_NO_GRAPH is set or a rocprofiler tool library is attached
 * (ROCP_TOOL_LIBRARIES; ROCMDECODE_GRAPH=1 overrides; rd_model_set_graph(m, 1) then returns RD_DECLINED). rd_model_graph_stats counts the graphs captured and the steps replayed. */
int rd_model_set_graph(rd_model *m, int on);
int rd_model_graph_stats(rd_model *m, long long *captures, long long *replays);
/* after the last upload: checks every tensor the step needs is present */
int rd_model_finalize(rd_model *m);

/* ---- KV: resident/subsystems.go:236-251 (KVSlots), resident/forward.go:20-30 (UploadKV, TruncateTo, Reset) ---- */
/* Order: rd_model_create, the uploads, rd_model_finalize, then rd_kv_configure(_typed), once. The pool's work list and staging
 * are sized for the widest step the finalized model takes; before rd_model_finalize the call returns RD_ERR_STATE. */
int rd_kv_configure(rd_model *m, int slots, int ctx_cap);
/* The same with the cache's element type: RD_KV_F16 (rd_kv_configure's), or RD_KV_I8 = goinfer's int8 cache (KVQuant "i8":
 * decoder/kvcache.go:13-20,43-52 quantizeHeads; backend/cuda/kv8_store.cu, kvtype.cuh:48-73): per (position, kv head) head_dim
 * signed bytes and one f32 scale for K and one for V, scale = maxabs/127, code = round-half-away(x/scale) in [-127, 127], an
 * all-zero head scale 1; readers take code * scale. Half the KV bytes of the f16 cache per step. */
enum { RD_KV_F16 = 0, RD_KV_I8 = 1 };
int rd_kv_configure_typed(rd_model *m, int slots, int ctx_cap, int kv_type);
/* keys, vals: host f32 [n][n_kv*hd] for positions base..base+n-1 of `slot`, layer `layer` (already RoPE'd) */
int rd_kv_upload(rd_model *m, int slot, int layer, int base, int n, const float *keys, const float *vals);
/* The rows a slot holds, widened to f32 as an attention read sees them (the host copy decoder/resident/subsystems.go:280-287
 * SnapshotKV takes): positions base..base+n-1 (all below the slot's length) of `layer` into keys, vals: host f32 [n][n_kv*hd].
 * f16 cache: the stored binary16 values; int8 cache: code * scale. */
int rd_kv_download(rd_model *m, int slot, int layer, int base, int n, float *keys, float *vals);
int rd_kv_truncate(rd_model *m, int slot, int pos);
int rd_kv_reset(rd_model *m, int slot);

/* ---- the step: resident/subsystems.go:102-117 StepBatch; every row equals its own rd_forward bit for bit ---- */
/* emb: host f32 [B][hidden] (embedding rows, already scaled: decoder/residency.go:1077-1123);
 * logits: host f32 [B][vocab] when want&RD_WANT_LOGITS; ids: int32 [B] when want&RD_WANT_ARGMAX (lowest index wins). */
int rd_step_batch(rd_model *m, int B, const int *slot, const int *pos, const float *emb, int want, float *logits, int *ids);
/* The widest step of a finalized model, the `hi` of resident/subsystems.go:111-116 BatchStepRange (lo is 1): 512 rows for a dense
 * model (sixteen GEMM row tiles of 32), 32 for a MoE model; 0 before rd_model_finalize. Prompt passes run this many rows at once. */
int rd_model_max_rows(const rd_model *m);
/* A row's on-device draw: resident/forward.go:43-52 BatchDraw with the (seed, draw) of Sampler.NextDraw
 * (internal/runtime/sampling/sampler_gumbel.go:68-76). RD_DRAW_GUMBEL is the temperature-only draw
 * argmax_i(f32(l_i * 1/T) + G_i) with Philox4x32-10 noise, the function of sampler_gumbel.go:41-66,117-123 and
 * backend/cuda/gumbel.cu; the noise transform is evaluated in f64 as on the host. */
enum { RD_DRAW_NONE = 0, RD_DRAW_GREEDY = 1, RD_DRAW_GUMBEL = 2 };
typedef struct rd_draw {
    double temperature; /* <= 0 means 1; so small that 1/T overflows f32: the argmax */
    uint64_t seed, draw;
    int32_t mode;       /* RD_DRAW_* */
    int32_t reserved;
} rd_draw;
/* rd_step_batch with draws[B] (resident/subsystems.go:102-110 StepBatch, BatchSeq.Draw): ids[i] is the drawn token of a row
 * that carries a draw and -1 for a row that does not; logits as in rd_step_batch when want & RD_WANT_LOGITS. */
int rd_step_batch_draw(rd_model *m, int B, const int *slot, const int *pos, const float *emb, const rd_draw *draws, int want,
                       float *logits, int *ids);
/* The same draws over explicit logit rows (host f32 [rows][V]), the kernels on their own as the reference's
 * backend/cuda/kernels/gumbel_test.go binds them; RD_DRAW_NONE is taken as greedy. */
int rd_sample_rows(rd_device *d, const float *logits, int rows, int V, const rd_draw *draws, int *ids);
/* resident.TopKRow for every row of a step (decoder/resident/forward.go:86-96; ForwardTopK, backend/cuda/topk.go:30-67, is the
 * B = 1 case): the step's kernel chain, then each logits row reduced on the device to its k best entries, ordered (logit
 * descending, token id ascending) — the tie order of the host's topKByLogit (internal/runtime/sampling/sampler.go:726-745), -0
 * and +0 equal. ids, vals: [B][min(k, vocab)]; 1 <= k <= 1024. want_z: z[b] = sum over the row of exp((l - max) / T_b) with
 * temperature[b] = T_b (<= 0 taken as 1), exp in f32 summed in f64 (the reference's own device sum is held to 1e-6 of the f64
 * sum, backend/cuda/topk_test.go:118); temperature and z may be NULL otherwise. */
int rd_step_batch_topk(rd_model *m, int B, const int *slot, const int *pos, const float *emb, int k, const double *temperature, int want_z,
                       int *ids, float *vals, double *z);
/* TopKRow.Full: the whole logits row of row `row` of the last step, if that step produced logits; valid until the next step. */
int rd_last_logits(rd_model *m, int row, float *logits);
/* The same reduction over explicit logit rows (host f32 [rows][V]), the kernel on its own as the reference's
 * backend/cuda/topk_test.go binds it; one temperature for all rows. */
int rd_topk_rows(rd_device *d, const float *logits, int rows, int V, int k, double temperature, int want_z, int *ids, float *vals, double *z);
/* rd_topk_rows for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc). It has no counterpart in the reference. The same kernels and the same results, but nothing is allocated: the
 * scratch between the launches is a static 5.3 MB device array per GPU, and inputs and outputs are DEVICE pointers the caller
 * owns: logits_dev f32 [rows][V], ids_dev int32 and vals_dev f32 [rows][min(k,V)], z_dev f64 [rows] (may be NULL unless want_z).
 * The launches go to `stream` (a hipStream_t; NULL = the null stream) of GPU `device` and the call returns without waiting for
 * them; the caller's current device is the same on return. Limits: rows <= 32, V <= 262144, 1 <= k <= 1024; beyond them
 * RD_ERR_ARG. Every call on one GPU shares that GPU's scratch: calls that overlap on one GPU (two streams, two threads) race;
 * calls in stream order do not. Served by librocmdecode_static.so beside this library (RD_ERR_STATE if it is missing).
 * Under stream capture: the one-time set-up for a GPU (opening that library, looking up the scratch's address there) happens in
 * rd_device_open(device); a process that never opened the device makes one call outside capture first, which does the same. */
int rd_topk_rows_static(int device, void *stream, const float *logits_dev, int rows, int V, int k, double temperature, int want_z, int *ids_dev,
                        float *vals_dev, double *z_dev);
/* Decode chained on the device (decoder/resident/subsystems.go:78-100 GreedyChainStart / GreedyChainNext / GreedyChainStop and
 * SampleChainStart / SampleChainNext): the chain's first input is token `id` at position `pos` of `slot`; each _next returns the
 * token the forward at the chain's next position picked (the argmax, or the Gumbel-max draw with draw index draw, draw+1, ...),
 * which is also the next forward's input, taken from the table of rd_model_upload_embedding without a host round trip. One
 * forward is queued past the token last returned. rd_sample_chain_next refuses a (seed, draw) that is not the draw the
 * forward was made with. Between start and stop no other step may run on the model; stop waits out what is queued. */
int rd_greedy_chain_start(rd_model *m, int slot, int id, int pos);
int rd_greedy_chain_next(rd_model *m, int *id);
int rd_sample_chain_start(rd_model *m, int slot, int id, int pos, double temperature, uint64_t seed, uint64_t draw);
int rd_sample_chain_next(rd_model *m, uint64_t seed, uint64_t draw, int *id);
void rd_greedy_chain_stop(rd_model *m);
/* resident/subsystems.go:112-117 StepRagged (and resident/forward.go:9-16 ForwardN as its one-sequence case): n_seq sequences
 * on distinct slots, sequence i with n_rows[i] >= 1 rows at positions pos[i], pos[i]+1, ... Rows are laid out sequence after
 * sequence: emb host f32 [sum n_rows][hidden]; logits [sum n_rows][vocab] / ids [sum n_rows] as in rd_step_batch. Row j of a
 * sequence equals that sequence's own rd_forward at pos+j bit for bit. A refused call (RD_ERR_ARG, RD_ERR_KV_FULL) writes nothing. */
int rd_step_ragged(rd_model *m, int n_seq, const int *slot, const int *pos, const int *n_rows, const float *emb, int want, float *logits,
                   int *ids);
/* resident/subsystems.go:124 PrefillLast: n prompt rows of one slot from start_pos into the same paged KV the decode step reads;
 * logits: host f32 [vocab] of the last row. The rows run through the decode step's kernels 32 at a time (every pass re-streams
 * the weights: correct and bit-identical to token-by-token, not yet a prefill-rate kernel). */
int rd_prefill_last(rd_model *m, int slot, int start_pos, int n, const float *emb, float *logits);
/* rd_step_ragged with one draw per sequence (decoder/resident/forward.go:60-75 RaggedSeq.Draw): ids [sum n_rows] holds the token
 * drawn on the device for the last row of a sequence that carries a draw and -1 for every other row. */
int rd_step_ragged_draw(rd_model *m, int n_seq, const int *slot, const int *pos, const int *n_rows, const float *emb, const rd_draw *draws,
                        int want, float *logits, int *ids);
/* resident.Forward's optional ForwardNoLogits (decoder/resident/subsystems.go:68-77): the token's forward builds only its K/V; the
 * final norm, the head matmul and the logits readback are skipped. rd_prefill_last uses the same short cut for every pass but
 * its last. */
int rd_forward_no_logits(rd_model *m, int slot, int pos, const float *emb);
/* Forward(embedding, pos) on one slot: the B=1 step through the same kernels */
int rd_forward(rd_model *m, int slot, int pos, const float *emb, float *logits);
/* expert indices the last step routed to: int32 [B][n_layers][top_k] (MoE models only; parity checks) */
int rd_last_moe_indices(rd_model *m, int *idx);
/* Test seam, goinfer's moeSelOverride / moeWtsOverride (decoder/mlp.go:19-27,53-56): the NEXT step replays the given
 * routing instead of routing on its own hidden state. idx, wgt: host [B][n_layers][top_k], the reference run's expert
 * indices and weights; B must equal the next step's batch. The override is consumed by that step. */
int rd_moe_replay(rd_model *m, int B, const int *idx, const float *wgt);

/* ---- host planning, callable without a GPU (no counterpart in the reference: its CUDA module plans inside its launch code,
 * backend/cuda/resident.go; exposed so the plans can be checked on a machine with no device) ---- */
/* The attention work list of one step: rows of len[r] visible keys on KV slot slot[r] (slot may be NULL: every row its own
 * sequence), heads_per_kv query heads per kv head, n_kv kv heads. items_out: int32 [max_items][4] = (first row, kv head |
 * rows << 16 (rows is 0 in a list where every item is one row), first block, one past the last block); ranges_out: int32
 * [rows][n_kv][3] = (first item, one past the last item, the row's place among its items' rows). *n_items, *grouped (1 if
 * some item covers several rows) are written. Fails with RD_ERR_ARG if the list needs more than max_items. */
int rd_plan_attention(int rows, const int *len, const int *slot, int heads_per_kv, int n_kv, int *items_out, int max_items,
                      int *ranges_out, int *n_items, int *grouped);
/* The split-K plan of a GEMM launch over N output rows and n_kblocks K-blocks: *splits partial sums of *kblocks_per_split. */
int rd_plan_gemm(int N, int n_kblocks, int *splits, int *kblocks_per_split);

/* ---- measurement: HIP-event timing on the stream the kernels are launched on; inputs resident in HBM ---- */
/* The int8 embedding table (vocab x hidden codes + one f32 scale per row), resident so a chain needs no host
 * round trip: goinfer's GreedyChain* (decoder/resident/subsystems.go:78-100). Row id is code * scale, the row the host's
 * embedding lookup sends for the same table. */
int rd_model_upload_embedding(rd_model *m, const int8_t *q, const float *row_scale);
/* Greedy decode chain on the device: step i runs rows (slot[b], pos0[b]+i) on the embedding of the previous step's
 * argmax (ids0 for the first). ms_out[steps]: per-step milliseconds; ids_out: optional int32 [steps][B] picked tokens. */
int rd_bench_steps(rd_model *m, int B, const int *slot, const int *pos0, const int *ids0, int warmup, int steps, float *ms_out,
                   int *ids_out);
/* One step with a HIP-event pair around every kernel class: class_ms[n] total milliseconds and class_n[n] launches,
 * n = rd_bench_class_count(); names from rd_bench_class_name. */
int rd_bench_profile(rd_model *m, int B, const int *slot, const int *pos, const int *ids0, float *class_ms, int *class_n);
/* The attention kernel's cost inside the step: (a whole step - the same step without its attention launches) / layers, the median
 * over `reps` pairs of steps at the same positions, each step between its own pair of events. Measurement only. */
int rd_bench_attn_in_step(rd_model *m, int B, const int *slot, const int *pos, const int *ids0, int reps, float *ms_per_launch, float *ms_step);
/* the name of the attention kernel the model's last step launched (measurement only) */
const char *rd_bench_attn_kernel_name(rd_model *m);
/* The host's cost of a step: `steps` chained greedy steps enqueued without waiting for the GPU, wall clock of the enqueue loop
 * alone, in microseconds per step (with and without graph replay: rd_model_set_graph). Measurement only. */
int rd_bench_enqueue(rd_model *m, int B, const int *slot, const int *pos0, const int *ids0, int steps, double *host_us);
/* The attention kernel's average launch duration: one step as above, then that kernel of every layer (its own KV, the step's
 * work list) launched back to back `reps` times between one pair of HIP events on the launch stream, so no event sits between
 * two launches. *ms_per_launch = elapsed / *launches, *launches = layers * reps. Measurement only. */
int rd_bench_attn_chain(rd_model *m, int B, const int *slot, const int *pos, const int *ids0, int reps, float *ms_per_launch, int *launches);
/* A whole prompt pass timed on the device: rows 0..n-1 of `slot` (reset first) from token ids through the embedding table, in
 * rd_prefill_last's passes. ms_total: milliseconds for the prompt; profile != 0 also fills class_ms / class_n as
 * rd_bench_profile does. */
int rd_bench_prefill(rd_model *m, int slot, int n, const int *ids, int profile, float *ms_total, float *class_ms, int *class_n);
int rd_bench_class_count(void);
const char *rd_bench_class_name(int c);
/* Times `iters` launches of one kernel over resident synthetic operands: "gemm_q4k" / "gemm_q5k" / "gemm_q6k" args {N,K,M,copies};
 * "gateup" args {I,K,M,copies}; "moe_gemm"; "topk" args {rows,V,k}; "copy" args {bytes}; "issue" args {mode,waves,iterations}: the
 * issue-rate probes (the int8 GEMMs' inner-loop instruction mix with every operand in registers). ms_out[iters]: per launch. */
int rd_bench_kernel(rd_device *d, const char *name, const int64_t *args, int n_args, int warmup, int iters, float *ms_out);
/* The ragged attention of one layer over a synthetic paged f16 pool built on the device (the attention micro-benchmark):
 * n_seq sequences of len[i] keys, rows in groups of 32. ms_total[iters]: partial + combine kernels of every group;
 * ms_partial[iters] (may be NULL): the flash-decode partial kernels alone. */
int rd_bench_attn(rd_device *d, int n_seq, const int *len, int n_h, int n_kv, int hd, float scale, float softcap, int warmup, int iters,
                  float *ms_total, float *ms_partial);
int rd_bench_attn_i8(rd_device *d, int n_seq, const int *len, int n_h, int n_kv, int hd, float scale, float softcap, int warmup, int iters,
                     float *ms_total, float *ms_partial);

#ifdef __cplusplus
}
#endif
#endif
