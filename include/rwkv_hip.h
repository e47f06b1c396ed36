/*
 * librwkv_hip.so -- C ABI of the MI355X (gfx950) kernels behind
 * RWKV(model, 'cuda fp16i8' | 'cuda fp16').forward(tokens, state).
 *
 * Conventions
 *   - Every pointer is a device pointer unless said otherwise; the library never
 *     allocates or frees device memory: the caller owns inputs, outputs and workspaces.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Calls only
 *     enqueue work; they never synchronise.
 *   - Return value: 0 = enqueued; < 0 = rejected argument (RWKV_E_*); > 0 = hipError_t of
 *     the failed launch.  Nothing is enqueued when the value is non-zero.
 *   - fp16 values are IEEE binary16 passed as `rwkv_half` (uint16_t storage).
 *   - A weight matrix is the reference's logical [N(in), M(out)] matrix
 *     (rwkv_pip_package/src/rwkv/model.py:793-794) addressed as
 *     w[n * w_stride_n + m * w_stride_m].  The fast layout is "input-contiguous":
 *     w_stride_n == 1, w_stride_m >= N (the orientation checkpoints are stored in);
 *     N % 16 == 0, w_stride_m % 16 == 0 and 16-byte aligned base pointers are required.
 *     The reference's device layout (w_stride_m == 1) is accepted by
 *     rwkv_repack_u8 / rwkv_repack_f16, which transpose it once at load time.
 *   - mx, rx are per output column [M]; my, ry per input row [N]; rx and ry are the
 *     stored ones (already divided by 16, model.py:845-847), so
 *     W'[n,m] = (w[n,m] + 0.5) * ry[n] * rx[m] + my[n] + mx[m]   (model.py:93).
 */
#ifndef RWKV_HIP_H
#define RWKV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t rwkv_half;

#define RWKV_OK 0
#define RWKV_E_SHAPE (-1)     /* size not supported (zero, negative, not a multiple the kernel needs) */
#define RWKV_E_LAYOUT (-2)    /* stride / alignment not supported */
#define RWKV_E_NULL (-3)      /* required pointer is NULL */
#define RWKV_E_WORKSPACE (-4) /* workspace too small */
#define RWKV_E_DTYPE (-5)     /* unknown dtype / mode code */
#define RWKV_E_SCRATCH (-6)   /* size beyond what the library's built-in scratch holds */

#define RWKV_DT_F16 0
#define RWKV_DT_F32 1
#define RWKV_DT_BF16 2   /* rwkv_wkv7_forward only */

/* Library / device identification.  Returns the ABI version (currently 3). */
int rwkv_abi_version(void);

/* ---------------------------------------------------------------------------------------
 * uint8 quantizer.  Replaces the CPU routine in RWKV.__init__ (model.py:818-847); results
 * are bit-identical to it.  `w` is the fp32 logical [N, M] matrix after transposition and
 * rescale (model.py:785-794), addressed with the two strides (elements); it is not
 * modified.  Outputs: q uint8 with strides (q_stride_n, q_stride_m); mx, rx [M] and my, ry
 * [N] in `scale_dtype` (RWKV_DT_F16 / RWKV_DT_F32); rx, ry are stored divided by 16.
 * Branch on N > M as model.py:824.  workspace: 4 * (N + M) floats.
 */
int rwkv_quantize_u8(int64_t N, int64_t M,
                     const float *w, int64_t w_stride_n, int64_t w_stride_m,
                     uint8_t *q, int64_t q_stride_n, int64_t q_stride_m,
                     void *mx, void *rx, void *my, void *ry, int scale_dtype,
                     float *workspace, size_t workspace_bytes, void *stream);

/* Transposes between the reference's device layout and the input-contiguous layout:
 * dst[n * dst_stride_n + m * dst_stride_m] = src[n * src_stride_n + m * src_stride_m]. */
int rwkv_repack_u8(int64_t N, int64_t M, const uint8_t *src, int64_t src_stride_n, int64_t src_stride_m,
                   uint8_t *dst, int64_t dst_stride_n, int64_t dst_stride_m, void *stream);
int rwkv_repack_f16(int64_t N, int64_t M, const rwkv_half *src, int64_t src_stride_n, int64_t src_stride_m,
                    rwkv_half *dst, int64_t dst_stride_n, int64_t dst_stride_m, void *stream);

/* ---------------------------------------------------------------------------------------
 * mm8_one: y[M] = x[N] @ W'.  Replaces torch.ops.rwkv.mm8_one (cuda/wrapper.cpp:84-117,
 * cuda/operators.cu:207-246) and the Python wrapper cuda_mm8_one (model.py:75-86).
 * fp32 accumulation.  y is written (not accumulated into: no pre-zeroing needed) as fp32
 * (y_dtype RWKV_DT_F32, the kernel's raw sum) or rounded to fp16 (RWKV_DT_F16, what
 * model.py:86 returns).  Deterministic: no atomics.
 */
int rwkv_mm8_one_f16(int64_t N, int64_t M, const rwkv_half *x,
                     const uint8_t *w, int64_t w_stride_n, int64_t w_stride_m,
                     const rwkv_half *mx, const rwkv_half *rx, const rwkv_half *my, const rwkv_half *ry,
                     void *y, int y_dtype, void *stream);

/* mm8_seq: y[B, M] = x[B, N] @ W', fp16 in, fp32 accumulation on MFMA, fp16 out.
 * Replaces torch.ops.rwkv.mm8_seq (cuda/wrapper.cpp:50-83, cuda/operators.cu:116-154).
 * x rows at x_stride elements, y rows at y_stride.  workspace: rwkv_mm8_seq_workspace(B, N)
 * bytes (the ry-scaled copy of x and two per-row sums). */
size_t rwkv_mm8_seq_workspace(int64_t B, int64_t N);
int rwkv_mm8_seq_f16(int64_t B, int64_t N, int64_t M, const rwkv_half *x, int64_t x_stride,
                     const uint8_t *w, int64_t w_stride_n, int64_t w_stride_m,
                     const rwkv_half *mx, const rwkv_half *rx, const rwkv_half *my, const rwkv_half *ry,
                     rwkv_half *y, int64_t y_stride, void *workspace, size_t workspace_bytes, void *stream);

/* rwkv_mm8_seq_f16 for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): no workspace argument, and no hipMalloc / hipFree or other allocating call
 * inside.  It has no counterpart in the reference.  The scratch of the product lives in a device array built
 * into the library (24 MiB + 64 KiB per GPU, held until the process ends), which bounds the size:
 *   B * N <= rwkv_mm8_seq_static_max_elems() (4 Mi) and B <= rwkv_mm8_seq_static_max_rows() (8192),
 * otherwise RWKV_E_SCRATCH and nothing is enqueued.  Same kernels and arguments as rwkv_mm8_seq_f16; the K split
 * is chosen within 16 MiB of slabs instead of 64, so a result can differ from rwkv_mm8_seq_f16's in the order of
 * its fp32 sums (at most one fp16 rounding step).  All calls on one GPU share that GPU's array: calls that may
 * overlap there (different streams, different host threads) race; calls on one stream are safe.
 * The first call on a device does host-side set-up (the address of the built-in array, kernel attributes) that
 * must not happen while a stream is capturing: make one call outside capture first (any valid size); every later
 * call only enqueues kernels and may be captured into a graph and replayed. */
size_t rwkv_mm8_seq_static_max_elems(void);
size_t rwkv_mm8_seq_static_max_rows(void);
int rwkv_mm8_seq_f16_static(int64_t B, int64_t N, int64_t M, const rwkv_half *x, int64_t x_stride,
                            const uint8_t *w, int64_t w_stride_n, int64_t w_stride_m,
                            const rwkv_half *mx, const rwkv_half *rx, const rwkv_half *my, const rwkv_half *ry,
                            rwkv_half *y, int64_t y_stride, void *stream);

/* Side streams.  Sequence calls of 256 tokens or more may run independent products of a layer on two extra streams
 * (default priority) beside the caller's; the library creates one such pair, with three events, for each (device,
 * caller stream) pair on its first use and keeps it until the process ends.  At most 32 pairs exist at a time: calls
 * on a further stream run every product on the caller's stream (same results, a few per cent slower).  A caller that
 * is about to destroy a stream hands its pair back with rwkv_release_stream(stream) (current device), after the
 * stream's work has completed; the next new stream takes the pair over.  Without that call a destroyed stream's pair
 * stays bound to its handle value.  No counterpart in the reference, whose launches use the legacy default stream
 * only (cuda/operators.cu:57, 111, 151). */
int rwkv_release_stream(void *stream);

/* gemm_fp16: c[B, M] = a[B, N] @ b[N, M], fp16 operands, fp32 accumulation, c written
 * directly as fp16 or fp32 (c_dtype) with no intermediate fp16 rounding.  Replaces
 * torch.ops.rwkv.gemm_fp16_cublas (cuda/gemm_fp16_cublas.cpp:28-75) for 2-D operands;
 * B == 1 takes the streaming GEMV path. */
int rwkv_gemm_f16(int64_t B, int64_t N, int64_t M, const rwkv_half *a, int64_t a_stride,
                  const rwkv_half *b, int64_t b_stride_n, int64_t b_stride_m,
                  void *c, int64_t c_stride, int c_dtype, void *stream);

/* The batched form of gemm_fp16: c[i] = a[i] @ b[i] for i < batch, operand i at a + i * a_batch_stride (elements;
 * likewise b, c).  Replaces the 3-D case of torch.ops.rwkv.gemm_fp16_cublas (cublasGemmStridedBatchedEx,
 * cuda/gemm_fp16_cublas.cpp:61-75; the caller is the RWKV-6 mixing LoRA `bmm` of model.py:1269, 1310).  Every product
 * must satisfy rwkv_gemm_f16's layout rules; the products are queued on `stream` one after the other. */
int rwkv_gemm_f16_batched(int64_t batch, int64_t B, int64_t N, int64_t M, const rwkv_half *a, int64_t a_stride,
                          int64_t a_batch_stride, const rwkv_half *b, int64_t b_stride_n, int64_t b_stride_m,
                          int64_t b_batch_stride, void *c, int64_t c_stride, int64_t c_batch_stride, int c_dtype,
                          void *stream);

/* ---------------------------------------------------------------------------------------
 * wkv_forward: RWKV-4 WKV recurrence over T tokens with running-maximum tracking.
 * Replaces torch.ops.rwkv.wkv_forward (cuda/wrapper.cpp:27-48, cuda/operators.cu:11-58).
 * w = time_decay (-exp(raw)), u = time_first, fp32 [C]; k, v, y [B*T, C] in `kv_dtype`
 * (fp32 is what model.py:1355-1357 passes); aa, bb, pp fp32 [B*C] updated in place.
 */
int rwkv_wkv4_forward(int64_t B, int64_t T, int64_t C, const float *w, const float *u,
                      const void *k, const void *v, void *y, int kv_dtype,
                      float *aa, float *bb, float *pp, void *stream);

/* RWKV-5 (constant per-channel decay) and RWKV-6 (per-token decay) recurrences on the
 * per-head N x N state, fp32.  Replace rwkv5.forward_fp32 / rwkv6.forward_fp32
 * (cuda/rwkv5_op.cpp:20-23 + cuda/rwkv5.cu:8-88; cuda/rwkv6_op.cpp:20-23 +
 * cuda/rwkv6.cu:8-87).  r, k, v, y: [T, C]; u: [C]; head size N = C / H must be 64.
 * w: v5 [C] (decay in (0,1)); v6 [T, C] *after* exp(-exp(.)) (model.py:959).
 * state_layout 0: [H][value i][key j] (what the reference kernels take, model.py:1376, 1429);
 * state_layout 1: [H][key j][value i] (the layout of the state list, model.py:1470).
 * state is updated in place.  B must be 1 (cuda/rwkv6.cu:17).
 */
int rwkv_wkv5_forward(int64_t B, int64_t T, int64_t C, int64_t H, float *state, int state_layout,
                      const float *r, const float *k, const float *v, const float *w, const float *u,
                      float *y, void *stream);
int rwkv_wkv6_forward(int64_t B, int64_t T, int64_t C, int64_t H, float *state, int state_layout,
                      const float *r, const float *k, const float *v, const float *w, const float *u,
                      float *y, void *stream);

/* Row-wise LayerNorm of an fp32 [T, C] matrix with fp32 affine, fp16 output (eps 1e-5).
 * Used once at load time for emb <- LayerNorm(emb; ln0) (model.py:756), which the reference
 * computes with F.layer_norm on the CPU. */
int rwkv_layernorm_f32_f16(int64_t T, int64_t C, const float *x, const float *w, const float *b,
                           rwkv_half *y, void *stream);

/* Sampling step after the head, on the device: replaces PIPELINE.sample_logits (rwkv/utils.py:55-88) and the
 * logit adjustments / occurrence bookkeeping of PIPELINE.generate (utils.py:103-106, 112-123).
 *   logits [V] fp32 (V <= 65536), not modified.
 *   token_ban [n_ban] int32 ids set to -inf (may be NULL when n_ban == 0).
 *   seen [V] uint8 / occurrence [V] fp32: the reference's `occurrence` dict as dense tables (both NULL: no
 *     penalties); every seen id pays alpha_presence + occurrence * alpha_frequency; after the draw all seen
 *     entries are multiplied by alpha_decay and the drawn id gets token_weight[id] (1 when token_weight is
 *     NULL; the reference uses 0 for ids that decode to blanks or digits) added / set and is marked seen.
 *   temperature 0 selects top_p 0 (the largest probability alone), as in the reference.
 *   u: device pointer to one uniform number in [0, 1): the draw is the first index, in index order, whose
 *     running sum of the filtered probabilities exceeds u * total.
 *   probs [V] fp32 or NULL: the filtered, temperature-scaled, un-normalised probabilities (what the
 *     reference hands to torch.multinomial).
 *   token: device int32, the drawn id.  One launch, no host synchronisation. */
int rwkv_sample_logits(const float *logits, int64_t V, float temperature, float top_p, int32_t top_k,
                       const int32_t *token_ban, int32_t n_ban, uint8_t *seen, float *occurrence,
                       const float *token_weight, float alpha_presence, float alpha_frequency, float alpha_decay,
                       const float *u, float *probs, int32_t *token, void *stream);

/* The temperature-0 case of the same step without bans or penalties (rwkv/utils.py:56-58: top_p = 0 keeps the
 * largest probability alone; what a greedy caller writes as logits.argmax()): token <- the index of the
 * largest of logits [V] (dtype RWKV_DT_F32, or RWKV_DT_F16 as RWKV-7 returns them), the lowest such index on
 * ties; NaN entries are never chosen.  One launch, no host synchronisation; token is a device int32 that the
 * next one-token forward call can read. */
int rwkv_greedy_token(const void *logits, int dtype, int64_t V, int32_t *token, void *stream);

/* =======================================================================================
 * Model-level entry points: one call runs RWKV.forward (model.py:1443-1677) for RWKV-4 on
 * one GPU, with the elementwise chains of att_one / ffn_one / cuda_att_seq / ffn_seq
 * (model.py:984-1004, 1034-1055, 1346-1360) folded into the GEMV / GEMM prologues and
 * epilogues.  The structs below are plain host memory filled by the caller; every pointer
 * inside them is a device pointer.  Matrices are input-contiguous (see the top of this file):
 * uint8 with fp16 mx/rx/my/ry under 'cuda fp16i8', fp16 with NULL scales under 'cuda fp16'.
 */
typedef struct {
    const void *w;       /* uint8 or fp16, row m = N consecutive elements at w + m * ld */
    int64_t ld;          /* elements between consecutive output rows */
    const rwkv_half *mx, *rx, *my, *ry; /* NULL for fp16 weights */
    int64_t N, M;
} rwkv_mat;

typedef struct {
    const rwkv_half *ln1_w, *ln1_b, *ln2_w, *ln2_b;               /* [C] */
    const rwkv_half *att_mix_k, *att_mix_v, *att_mix_r;           /* [C] */
    const float *time_decay, *time_first;                         /* [C] fp32; decay = -exp(raw) */
    rwkv_mat att_key, att_value, att_receptance, att_output;      /* [C -> C] */
    const rwkv_half *ffn_mix_k, *ffn_mix_r;                       /* [C] */
    rwkv_mat ffn_key, ffn_receptance, ffn_value;                  /* [C -> F], [C -> C], [F -> C] */
} rwkv_v4_layer;

typedef struct {
    rwkv_half *att_xx;      /* [C] fp16 */
    float *aa, *bb, *pp;    /* [C] fp32 */
    rwkv_half *ffn_xx;      /* [C] fp16 */
} rwkv_v4_layer_state;

typedef struct {
    int32_t n_layer, n_embd, n_ffn, vocab;
    int32_t rescale_layer;  /* x /= 2 after every rescale_layer-th layer; 0 = never (model.py:1660-1662) */
    int32_t weights_u8;     /* 1: uint8 matrices ('cuda fp16i8'); 0: fp16 matrices ('cuda fp16'); 2: per layer and for
                             * the head, uint8 where the scale vectors are non-NULL ('cuda fp16i8 *20 -> cuda fp16';
                             * all matrices of one layer have one type, model.py:776-778) */
    const rwkv_half *emb;   /* [vocab, C] fp16, ln0 already applied (model.py:756) */
    const rwkv_half *ln_out_w, *ln_out_b;
    rwkv_mat head;          /* [C -> vocab] */
    const rwkv_v4_layer *layers; /* host array [n_layer] */
    /* Layer range of this call: [layer_begin, layer_end), 0 / 0 = the whole model.  The embedding gather runs when
     * layer_begin == 0 and ln_out + head when layer_end reaches n_layer (logits may be NULL otherwise); between
     * the calls of one forward pass the running activation stays in the workspace, so they must share it (and
     * T).  This is how a streamed strategy ('cuda fp16i8 *10+', model.py:854-858, 1526-1530) runs: the caller
     * copies the matrices of one streamed layer to the device, then calls for that layer alone. */
    int32_t layer_begin, layer_end;
} rwkv_v4_model;

/* One-token step (len(tokens) == 1).  `token` is a device int32: the kernels read the id from
 * device memory so that a captured graph can be replayed with a new token.  `states` is a host
 * array [n_layer]; all state tensors are updated in place.  logits: fp32 [vocab] (values are
 * fp16-rounded as in model.py:86, 1675-1677).  workspace: rwkv_v4_one_workspace() bytes.
 * Only launches kernels (no memset / memcpy nodes): safe to capture into a HIP graph. */
size_t rwkv_v4_one_workspace(const rwkv_v4_model *m);
int rwkv_v4_forward_one(const rwkv_v4_model *m, const rwkv_v4_layer_state *states, const int32_t *token,
                        float *logits, void *workspace, size_t workspace_bytes, void *stream);

/* Sequence mode (len(tokens) > 1): tokens is a device int32 [T].  logits: fp32 [vocab] for the
 * last token, or [T, vocab] when full_output != 0.  workspace: rwkv_v4_seq_workspace(m, T,
 * full_output) bytes. */
size_t rwkv_v4_seq_workspace(const rwkv_v4_model *m, int64_t T, int full_output);
int rwkv_v4_forward_seq(const rwkv_v4_model *m, const rwkv_v4_layer_state *states, const int32_t *tokens,
                        int64_t T, int full_output, float *logits, void *workspace, size_t workspace_bytes,
                        void *stream);

/* =======================================================================================
 * RWKV-5.0 / 5.1 / 5.2 / 6.0: one entry point for both modes of RWKV.forward (T == 1 streams
 * the matrices with the GEMV kernels, T > 1 uses the MFMA contraction).  Replaces att_one_v5 /
 * att_one_v5_1 / att_one_v6_0, cuda_att_seq_v5_2 / cuda_att_seq_v6_0 with v5_2_before / v6_0_before
 * / v5_2_after, RUN_RWKV_5 / RUN_RWKV_6 and ffn_one(_v6) / ffn_seq(_v6)
 * (model.py:984-1029, 1091-1340, 1363-1439).  Head size must be 64.
 */
typedef struct {
    const rwkv_half *ln1_w, *ln1_b, *ln2_w, *ln2_b;   /* [C] */
    /* RWKV-5: time_mix_k, _v, _r, _g (g NULL for 5.0), two unused.
     * RWKV-6: time_maa_x, _w, _k, _v, _r, _g. */
    const rwkv_half *att_mix[6];
    const rwkv_half *tm_w1;  /* v6: time_maa_w1 transposed, [5 * lora_maa][C] fp16 */
    const rwkv_half *tm_w2;  /* v6: time_maa_w2 [5][lora_maa][C] fp16 */
    const rwkv_half *td_w1;  /* v6: time_decay_w1 transposed, [lora_decay][C] fp16 */
    const rwkv_half *td_w2;  /* v6: time_decay_w2 transposed, [C][lora_decay] fp16 */
    const float *time_decay; /* [C] fp32: v5 exp(-exp(raw)) per channel; v6 raw (model.py:799-804) */
    const float *time_first; /* [C] fp32 (model.py:808-814) */
    const float *lnx_w, *lnx_b; /* [C] fp32 GroupNorm affine (model.py:815-816) */
    rwkv_mat att_key, att_value, att_receptance, att_gate /* w NULL for 5.0 */, att_output;
    const rwkv_half *ffn_mix_k, *ffn_mix_r;           /* time_mix_* (v5) / time_maa_* (v6) */
    rwkv_mat ffn_key, ffn_receptance, ffn_value;
} rwkv_v56_layer;

typedef struct {
    rwkv_half *att_xx;  /* [C] fp16 */
    float *att_kv;      /* [H][N key][N value] fp32 (model.py:1470) */
    rwkv_half *ffn_xx;  /* [C] fp16 */
} rwkv_v56_layer_state;

typedef struct {
    int32_t version_x10;    /* 50, 51, 52 or 60 */
    int32_t n_layer, n_embd, n_ffn, vocab, n_head;
    int32_t lora_maa, lora_decay;   /* v6 LoRA ranks (32 / 64 in released models) */
    int32_t rescale_layer, weights_u8;   /* weights_u8 as in rwkv_v4_model */
    const rwkv_half *emb, *ln_out_w, *ln_out_b;
    rwkv_mat head;
    const rwkv_v56_layer *layers;
    int32_t layer_begin, layer_end;   /* as in rwkv_v4_model */
} rwkv_v56_model;

size_t rwkv_v56_workspace(const rwkv_v56_model *m, int64_t T);
/* tokens: device int32 [T]; logits fp32 [vocab] (last token) or [T, vocab] (full_output != 0 and
 * T > 1).  All state tensors are updated in place.  Only launches kernels: capturable. */
int rwkv_v56_forward(const rwkv_v56_model *m, const rwkv_v56_layer_state *states, const int32_t *tokens,
                     int64_t T, int full_output, float *logits, void *workspace, size_t workspace_bytes,
                     void *stream);

/* ---------------------------------------------------------------------------------------
 * RWKV-7 state recurrence.  Replaces torch.ops.wkv7s.forward_bf16 / forward_fp16 / forward_fp32
 * (cuda/rwkv7_op.cpp:12-26, cuda/rwkv7.cu:9-58): per head, with row i of the state held per value index,
 *     sa_i = sum_j a_j S_ij ;  S_ij = S_ij * exp(-exp(w_j)) + k_j v_i + sa_i b_j ;  y_i = sum_j S_ij r_j
 * r, w, k, v, a, b, y: [T, C] in `dtype` (RWKV_DT_F16, RWKV_DT_F32 or RWKV_DT_BF16), w is the log-decay the reference
 * passes (model.py:537-538); state fp32 [H][value i][key j] (model.py:288), updated in place; head size
 * C / H must be 64; B must be 1 (cuda/rwkv7.cu:17, 66).
 */
int rwkv_wkv7_forward(int64_t B, int64_t T, int64_t C, int64_t H, float *state, const void *r, const void *w,
                      const void *k, const void *v, const void *a, const void *b, void *y, int dtype,
                      void *stream);

/* =======================================================================================
 * RWKV-7 ("x070"): one entry point for both modes of RWKV_x070.forward (model.py:292-302), replacing
 * forward_one / forward_seq (model.py:336-363, 457-487), RWKV_x070_TMix_one / _seq (model.py:492-572),
 * RWKV_x070_CMix_one / _seq (model.py:597-608; the DeepEmbed forms model.py:578-594 when a layer carries the de_*
 * tensors) and RWKV7_OP (model.py:198-219).  The reference runs RWKV-7
 * in fp16, bf16 or fp32 without quantisation (model.py:236-243); this entry point is the fp16 one.  Head
 * size must be 64.  The four LoRA pairs (decay w, in-context rate a, value residual v, gate g) are fp16
 * and input-contiguous like the model matrices, every rank padded with zeros to a multiple of 64 and the
 * four concatenated in the order w, a, v, g (R = lora_w + lora_a + lora_v + lora_g):
 *   lora1 [R][C]   first stages: the checkpoint's w1, a1, v1, g1 ([C, rank]) transposed, row blocks stacked
 *   lora2 [C][R]   second stages: w2, a2, v2, g2 ([rank, C]) transposed, column blocks side by side
 * Layer 0 has no value residual (model.py:279-281, 505): its v blocks are ignored.
 */
typedef struct {
    const rwkv_half *ln1_w, *ln1_b, *ln2_w, *ln2_b;      /* [C] */
    const rwkv_half *x_mix[6];                            /* att.x_r, x_w, x_k, x_v, x_a, x_g [C] */
    const rwkv_half *w0, *a0, *v0;                        /* [C]; v0 unused in layer 0 */
    const rwkv_half *lora1, *lora2;                       /* [R][C], [C][R] */
    const rwkv_half *k_k, *k_a, *r_k;                     /* [C] */
    const rwkv_half *lnx_w, *lnx_b;                       /* [C] GroupNorm affine */
    rwkv_mat att_receptance, att_key, att_value, att_output;
    const rwkv_half *ffn_x_k;                             /* [C] */
    rwkv_mat ffn_key, ffn_value;
    /* DeepEmbed variant (RWKV_DE_VERSION=1: model.py:274-277, 578-594); all four NULL = the plain channel mix.
     * The squared-relu keys of token t are scaled by ((xx_t @ s1) @ E_t) @ s2 + s0, xx_t the LayerNorm output,
     * E_t = row token_t of de_emb viewed 32 x 32.
     *   de_emb [vocab][1024]  ffn.s_emb.weight with the embedding residual merged in (model.py:276-277)
     *   de_s1  [32][C]        ffn.s1 ([C, 32]) transposed, input-contiguous like the model matrices
     *   de_s2  [32][F]        ffn.s2 as stored
     *   de_s0  [F]            ffn.s0 */
    const rwkv_half *de_emb, *de_s1, *de_s2, *de_s0;
} rwkv_v7_layer;

typedef struct {
    int32_t n_layer, n_embd, n_ffn, vocab, n_head;
    int32_t lora_w, lora_a, lora_v, lora_g;   /* padded ranks (multiples of 64) */
    const rwkv_half *emb, *ln_out_w, *ln_out_b;
    rwkv_mat head;
    const rwkv_v7_layer *layers;
} rwkv_v7_model;

size_t rwkv_v7_workspace(const rwkv_v7_model *m, int64_t T);
/* tokens: device int32 [T]; states: rwkv_v56_layer_state per layer with att_kv laid out
 * [H][value][key] (model.py:286-289); logits fp32 [vocab] or [T, vocab] holding fp16-rounded values (the
 * reference returns them as fp16, model.py:362, 486).  All state tensors are updated in place.  Only
 * launches kernels: capturable. */
int rwkv_v7_forward(const rwkv_v7_model *m, const rwkv_v56_layer_state *states, const int32_t *tokens,
                    int64_t T, int full_output, float *logits, void *workspace, size_t workspace_bytes,
                    void *stream);

#ifdef __cplusplus
}
#endif
#endif /* RWKV_HIP_H */
