// Matrix product dispatch shared by the RWKV-5/6 and RWKV-7 forward passes (internal).
#pragma once
#include "decode_kernels.h"

namespace {

inline MatDev to_dev56(const rwkv_mat &m) { return MatDev{m.w, m.ld, m.mx, m.rx, m.my, m.ry}; }

struct Ctx {
    hipStream_t st;
    bool u8;
    int64_t T;
    int grid;
    rwkv_half *xs;       // scaled-activation scratch [T, max(C, F)]
    float *s0, *s2;      // [T]
    float *splitk;       // RWKV_SPLITK_WS_BYTES of split-K scratch (NULL: never split)
    int small_tiles;     // 1: another contraction runs beside the ones launched through this context
};

// y = act(x @ W) for a model matrix (uint8 or fp16 per strategy) or an fp16 LoRA matrix.
//   one-token: vec_kernel;  sequence: (prepare +) MFMA GEMM.  x [T, N] fp16 contiguous.
// act: ACT_* of kernels.h; res/gate only for the residual epilogues; out fp16 [T, M].
inline int mm(const Ctx &c, const rwkv_mat &m, bool mat_u8, const rwkv_half *x, int act, const rwkv_half *res,
       const rwkv_half *gate, float out_scale, rwkv_half *out, const rwkv_half *commit_src = nullptr,
       rwkv_half *commit_dst = nullptr, int commit_n = 0) {
    const int N = (int)m.N, M = (int)m.M;
    if (c.T == 1) {
        VecArgs a{};
        a.vin = x; a.N = N; a.M = M; a.mat = to_dev56(m);
        a.x_in = res; a.emb = nullptr; a.token = nullptr; a.C = commit_n; a.gate = gate; a.x_out = out;
        a.out_scale = out_scale; a.commit_src = commit_src; a.commit_dst = commit_dst; a.out = out;
        switch (act) {
            case ACT_NONE: a.act = VACT_F16; break;
            case ACT_SIGMOID: a.act = VACT_SIGMOID; break;
            case ACT_RELU_SQ: a.act = VACT_RELU_SQ; break;
            case ACT_SILU: a.act = VACT_SILU; break;
            case ACT_TANH: a.act = VACT_TANH; break;
            default: a.act = VACT_RESIDUAL; break;
        }
        if (N > 8 * VP * DTHREADS) return RWKV_E_SHAPE;
        vec_launch(mat_u8, a, c.grid, c.st);
        RWKV_LAUNCH_CHECK();
        return RWKV_OK;
    }
    if (commit_dst) {
        int rc = copy_h16_launch(commit_n, commit_src, commit_dst, c.st);
        if (rc) return rc;
    }
    const rwkv_half *A = x;
    GemmEpi e{};
    e.act = act; e.res = res; e.ldres = M; e.gate = gate; e.ldgate = M; e.out_scale = out_scale;
    e.out_dtype = RWKV_DT_F16; e.splitk_ws = c.splitk; e.splitk_bytes = RWKV_SPLITK_WS_BYTES;
    e.small_tiles = c.small_tiles;
    if (mat_u8) {
        int rc = mm8_prepare_launch(c.T, N, x, N, m.ry, m.my, c.xs, c.s0, c.s2, c.st);
        if (rc) return rc;
        A = c.xs;
        e.mx = m.mx; e.rx = m.rx; e.s0 = c.s0; e.s2 = c.s2;
    }
    return gemm_launch(mat_u8, c.T, N, M, A, N, m.w, m.ld, out, M, e, c.st);
}

// Sequence calls only: the same product for an activation that the producing kernel has already scaled by the
// matrix's ry (uint8 matrices; s0 / s2 = its row sums of x and x * my) -- no scaling pass.  fp16 matrices: xs is
// the plain activation and the sums are not read.
inline int mm_scaled(const Ctx &c, const rwkv_mat &m, bool mat_u8, const rwkv_half *xs, const float *s0, const float *s2,
                     int act, const rwkv_half *res, const rwkv_half *gate, float out_scale, rwkv_half *out) {
    const int N = (int)m.N, M = (int)m.M;
    if (c.T <= 1) return RWKV_E_SHAPE;
    GemmEpi e{};
    e.act = act; e.res = res; e.ldres = M; e.gate = gate; e.ldgate = M; e.out_scale = out_scale;
    e.out_dtype = RWKV_DT_F16; e.splitk_ws = c.splitk; e.splitk_bytes = RWKV_SPLITK_WS_BYTES;
    e.small_tiles = c.small_tiles;
    if (mat_u8) { e.mx = m.mx; e.rx = m.rx; e.s0 = s0; e.s2 = s2; }
    return gemm_launch(mat_u8, c.T, N, M, xs, N, m.w, m.ld, out, M, e, c.st);
}

inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

inline rwkv_mat lora_mat(const rwkv_half *w, int64_t N, int64_t M) {
    rwkv_mat m{};
    m.w = w; m.ld = N; m.N = N; m.M = M;
    return m;
}

}  // namespace
