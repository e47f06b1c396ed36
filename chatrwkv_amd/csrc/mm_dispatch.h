// Matrix product dispatch shared by the RWKV-5/6 and RWKV-7 forward passes (internal).
#pragma once
#include <cstdlib>
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

// RWKV_HANDOVER=0 keeps the separate scaling pass between the two products of mm_pair (for A/B timing)
inline bool handover_enabled() {
    const char *e = getenv("RWKV_HANDOVER");
    return !(e && *e == '0');
}

// Sequence calls: mid = act1(xs @ W1) followed by out = epilogue2(mid @ W2) -- the channel mix's key and value
// products -- as two calls, so that the caller can join a side stream in between.  c1 launches the first product,
// c2 the second (its xs / s0 / s2 scratch is used).  uint8 matrices, both products through the direct-to-LDS kernel
// and the first at full depth: the first epilogue stores mid already scaled by W2's ry into c2.xs and one partial
// row sum per column tile into `parts` (2 * T * ceil(M1 / 128) floats), which the second launch adds up itself -- no
// scaling pass, and the unscaled mid is never stored; *np is then the number of partial sums per row.  Otherwise
// (*np = 0): mm_scaled, then mm.
inline int mm_pair_first(const Ctx &c1, const Ctx &c2, const rwkv_mat &m1, const rwkv_mat &m2, bool mat_u8,
                         const rwkv_half *xs, const float *s0, const float *s2, int act1, rwkv_half *mid, int act2,
                         const rwkv_half *res, const rwkv_half *gate, rwkv_half *out, float *parts, int *np) {
    const int64_t T = c1.T;
    const int N1 = (int)m1.N, M1 = (int)m1.M, M2 = (int)m2.M;
    *np = 0;
    if (T > 1 && mat_u8 && parts && handover_enabled()) {
        GemmEpi e1{};
        e1.act = act1; e1.out_scale = 1.f; e1.out_dtype = RWKV_DT_F16; e1.splitk_ws = c1.splitk;
        e1.splitk_bytes = RWKV_SPLITK_WS_BYTES; e1.small_tiles = c1.small_tiles;
        e1.mx = m1.mx; e1.rx = m1.rx; e1.s0 = s0; e1.s2 = s2;
        GemmEpi e2{};
        e2.act = act2; e2.res = res; e2.ldres = M2; e2.gate = gate; e2.ldgate = M2; e2.out_scale = 1.f;
        e2.out_dtype = RWKV_DT_F16; e2.splitk_ws = c2.splitk; e2.splitk_bytes = RWKV_SPLITK_WS_BYTES;
        e2.small_tiles = c2.small_tiles;
        e2.mx = m2.mx; e2.rx = m2.rx; e2.s0 = c2.s0; e2.s2 = c2.s2;
        const GemmPlan p1 = gemm_plan(true, T, N1, M1, xs, N1, m1.w, m1.ld, c2.xs, M1, e1);
        const GemmPlan p2 = gemm_plan(true, T, M1, M2, c2.xs, M1, m2.w, m2.ld, out, M2, e2);
        const int n = p1.kind == 2 ? (M1 + p1.tn - 1) / p1.tn : 0;
        if (p1.kind == 2 && p1.ks == 1 && p2.kind == 2 && n > 1 && !(n & 3)) {
            *np = n;
            e1.emit_ry = m2.ry; e1.emit_my = m2.my; e1.emit_s0 = parts; e1.emit_s2 = parts + (size_t)T * n;
            return gemm_launch(true, T, N1, M1, xs, N1, m1.w, m1.ld, c2.xs, M1, e1, c1.st);
        }
    }
    return mm_scaled(c1, m1, mat_u8, xs, s0, s2, act1, nullptr, nullptr, 1.f, mid);
}

inline int mm_pair_second(const Ctx &c2, const rwkv_mat &m1, const rwkv_mat &m2, bool mat_u8, const rwkv_half *mid, int act2,
                          const rwkv_half *res, const rwkv_half *gate, float out_scale, rwkv_half *out, const float *parts,
                          int np) {
    if (!np) return mm(c2, m2, mat_u8, mid, act2, res, gate, out_scale, out);
    const int M1 = (int)m1.M, M2 = (int)m2.M;
    GemmEpi e2{};
    e2.act = act2; e2.res = res; e2.ldres = M2; e2.gate = gate; e2.ldgate = M2; e2.out_scale = out_scale;
    e2.out_dtype = RWKV_DT_F16; e2.splitk_ws = c2.splitk; e2.splitk_bytes = RWKV_SPLITK_WS_BYTES;
    e2.small_tiles = c2.small_tiles;
    e2.mx = m2.mx; e2.rx = m2.rx; e2.s0 = c2.s0; e2.s2 = c2.s2;
    e2.parts = np; e2.p0 = parts; e2.p2 = parts + (size_t)c2.T * np;
    return gemm_launch(true, c2.T, M1, M2, c2.xs, M1, m2.w, m2.ld, out, M2, e2, c2.st);
}

inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

inline rwkv_mat lora_mat(const rwkv_half *w, int64_t N, int64_t M) {
    rwkv_mat m{};
    m.w = w; m.ld = N; m.N = N; m.M = M;
    return m;
}

}  // namespace
