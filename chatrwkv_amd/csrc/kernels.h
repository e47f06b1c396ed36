// Launchers shared between translation units of librwkv_hip.so (internal, not part of the C ABI).
#pragma once
#include "common.h"

enum { ACT_NONE = 0, ACT_SIGMOID = 1, ACT_RELU_SQ = 2, ACT_RESIDUAL = 3, ACT_GATED_RESIDUAL = 4, ACT_SILU = 5, ACT_TANH = 6 };

// Epilogue of the MFMA contraction (gemm.hip).
struct GemmEpi {
    const rwkv_half *mx, *rx;      // [M]; NULL for plain fp16 weights
    const float *s0, *s2;          // [T] row sums of the unscaled activation (uint8 weights)
    int act;
    const rwkv_half *res; int64_t ldres;    // residual input [T, M]
    const rwkv_half *gate; int64_t ldgate;  // gate [T, M]
    float out_scale;               // applied to the final fp16 value (1 or 0.5)
    int out_dtype;                 // RWKV_DT_F16 / RWKV_DT_F32 (the fp16-rounded value widened)
    int raw_f32;                   // 1: store the fp32 accumulator unrounded (out_dtype must be F32)
    float *splitk_ws;              // scratch for split-K partial sums (NULL: never split)
    size_t splitk_bytes;
    int small_tiles;               // 1: keep the 128 x 128 tile (the caller runs another contraction beside this one, and a
                                   // 256 x 256 tile's 128 KB of LDS would leave no room for it on the CU)
    // Hand-over of a uint8 product's input without a scaling pass in between (direct-to-LDS launches; gemm_plan
    // says which launches those are).
    // Producer: emit_ry != NULL: the output y is stored as fp16(y * emit_ry[m]), already scaled for the next
    //   product, and the sums of y and of y * emit_my over the columns of each tile go to
    //   emit_s0 / emit_s2 [T][ceil(M / tile width)].
    // Consumer: parts > 1: p0 / p2 [T][parts] hold such partial row sums; a row's totals are formed in index order
    //   by the launch itself (the K-split form writes them to s0 / s2 for its second pass, so these name scratch).
    const rwkv_half *emit_ry, *emit_my;
    float *emit_s0, *emit_s2;
    int parts;
    const float *p0, *p2;
};

// How gemm_launch would run a product: kind 0 = the 2..16-row kernel, 1 = register-staged tiles, 2 = direct-to-LDS
// tiles of tm x tn with K split ks ways.
struct GemmPlan { int kind, tm, tn, ks; };
GemmPlan gemm_plan(bool w_u8, int64_t T, int64_t N, int64_t M, const rwkv_half *A, int64_t lda, const void *W,
                   int64_t ldw, const void *Y, int64_t ldy, const GemmEpi &ep);

// Size of the split-K scratch the model-level entry points reserve in their workspaces.
constexpr size_t RWKV_SPLITK_WS_BYTES = (size_t)64 << 20;

int gemm_launch(bool w_u8, int64_t T, int64_t N, int64_t M, const rwkv_half *A, int64_t lda, const void *W,
                int64_t ldw, void *Y, int64_t ldy, const GemmEpi &ep, hipStream_t st);
// n (2..4) products [T, N] x [N, M_i] in one launch (short calls, where each alone would split K); see gemm.hip
int gemm_group_launch(bool w_u8, int n, int64_t T, int64_t N, const rwkv_half *const *x, const rwkv_mat *const *mats,
                      void *const *Y, const GemmEpi *eps, rwkv_half *const *xs, float *const *sums, float *splitk_ws,
                      hipStream_t st, int parts = 0);
// true where that launch would go through the direct-to-LDS kernel, which can take the row sums of already scaled
// inputs as `parts` partial sums per row (GemmEpi::parts)
bool gemm_group_takes_parts(bool w_u8, int n, int64_t T, int64_t N, const rwkv_half *const *x, const rwkv_mat *const *mats,
                            void *const *Y);
int mm8_prepare_launch(int64_t T, int64_t N, const rwkv_half *x, int64_t ldx, const rwkv_half *ry,
                       const rwkv_half *my, rwkv_half *xs, float *s0, float *s2, hipStream_t st);
int gemv_f16_launch(int64_t N, int64_t M, const rwkv_half *x, const rwkv_half *w, int64_t ldw, void *y,
                    int y_dtype, hipStream_t st);
// kv_f32: k, v are fp32 (fp16-weight strategy) instead of fp16.
int wkv4_fused_launch(int T, int C, const float *w, const float *u, const void *k, const void *v, int kv_f32,
                      const rwkv_half *r, rwkv_half *y, float *aa, float *bb, float *pp, hipStream_t st,
                      float *scratch = nullptr);  // scratch (wkv4_scratch_bytes): long calls run as a chunked scan
size_t wkv4_scratch_bytes(int64_t T, int64_t C);
int wkv56_fused_launch(bool v6, int T, int C, int H, float *state, const rwkv_half *r, const rwkv_half *k,
                       const rwkv_half *v, const void *w, const float *t_decay, const float *u, const float *lnx_w,
                       const float *lnx_b, const rwkv_half *gate, rwkv_half *out, hipStream_t st,
                       const rwkv_half *dw2 = nullptr, int ld = 0,  // dw2: v6 with w = tanh(. @ D1), product with D2 in-kernel
                       float *y32 = nullptr);  // fp32 [T, C] scratch: calls of >= 32 tokens split each head over 4 workgroups
// Row-wise LayerNorm + token shift + mixes for up to 6 consumers over a [T, C] activation (seq_v4.hip).
struct SeqMixArgs {
    int T, C;
    const rwkv_half *x;        // [T, C]
    const rwkv_half *ln_w, *ln_b;
    const rwkv_half *sx;       // state (previous token's normalised activation), NULL = no token shift
    rwkv_half *xx_last;        // scratch [C]: normalised activation of the last row (new state)
    rwkv_half *state_out;      // or: the state itself (may be sx): written by row 0's workgroup after it has read sx
    const rwkv_half *mix[6];   // NULL entry = consumer sees LN(x)
    const rwkv_half *ry[6], *my[6];  // NULL ry = no scaling / sums (fp16 weights)
    rwkv_half *xs[6];          // [T, C] outputs
    float *s0[6], *s2[6];      // [T] outputs
    int maa_form;              // RWKV-6 / RWKV-7 mixing kx = xx + (prev - xx) * m, rounded after every step
};

int lnmix_seq_launch(const SeqMixArgs &a, int nj, hipStream_t st);
int gather_emb_launch(int64_t T, int C, int vocab, const int32_t *tokens, const rwkv_half *emb, rwkv_half *x, hipStream_t st);
int copy_h16_launch(int n, const rwkv_half *src, rwkv_half *dst, hipStream_t st);
int v4_model_check(const rwkv_v4_model *m);
int v4_head_launch(const rwkv_v4_model *m, const rwkv_half *x, float *logits, hipStream_t st);
int num_cu();

// Is this matrix uint8?  weights_u8 0: no matrix is, 1: every matrix is, 2: decided per layer (and for the head) by
// the presence of the scale vectors -- a strategy such as 'cuda fp16i8 *20 -> cuda fp16'.
// The layer range [begin, end) of a model-level call (0 / 0 = all layers); false when it is not a range of the model.
inline bool layer_range(int n_layer, int begin, int end, int &lb, int &le) {
    lb = begin;
    le = (begin == 0 && end == 0) ? n_layer : end;
    return lb >= 0 && lb < le && le <= n_layer;
}

inline bool mat_is_u8(int weights_u8, const rwkv_mat &m) { return weights_u8 == 2 ? m.mx != nullptr : weights_u8 != 0; }

// Two extra streams (default priority) for contractions that are independent and each too small to fill the chip;
// fork / join by events around them (seq_v4.hip).  Every (device, caller stream) pair gets its own set, created on
// its first use and kept until the process ends, so calls on different streams never share an event; calls on
// ONE stream must come from one host thread at a time, as for any stream-ordered API.
struct SideStreams {
    hipStream_t s[2];
    hipEvent_t fork, join[2];
    bool ok;
};
SideStreams *side_streams(hipStream_t caller);                 // NULL: none available (creation failed, table full)
bool fork_streams(SideStreams *ss, hipStream_t st, int n);     // side stream j < n then sees everything queued on st so far
bool join_streams(SideStreams *ss, hipStream_t st, int n);     // st then sees everything queued on the side streams

// A fork that is always joined: by join(), or by the destructor on an early (error) return, so that work queued on
// a side stream never outlives the call that queued it.
struct ForkScope {
    SideStreams *ss;
    hipStream_t st;
    int n;
    bool active;
    ForkScope(SideStreams *ss_, hipStream_t st_, int n_, bool want) : ss(ss_), st(st_), n(n_), active(false) {
        if (want && ss) active = fork_streams(ss, st, n);
    }
    ForkScope(const ForkScope &) = delete;
    ForkScope &operator=(const ForkScope &) = delete;
    explicit operator bool() const { return active; }
    bool join() {
        if (!active) return true;
        active = false;
        return join_streams(ss, st, n);
    }
    ~ForkScope() { if (active) (void)join_streams(ss, st, n); }
};
