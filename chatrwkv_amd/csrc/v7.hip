// RWKV-7 forward for any T >= 1 (fp16 weights, fp32 state and decay).
//
// Per layer: time mix
//   lnmix_seq (LN1, token shift, the six static mixes r, w, k, v, a, g)
//   r, k, v rows; LoRA pairs: w = tanh(xw @ W1) @ W2, a = (xa @ A1) @ A2, v-gate = (xv @ V1) @ V2,
//   g = sigmoid(xg @ G1) @ G2   -- mm(): streaming GEMV for one token, MFMA GEMM otherwise
//   prep7   per (token, head): a = sigmoid(a0 + .), kk = normalised k * k_k, k *= 1 + (a - 1) k_a,
//           v += (v_first - v) sigmoid(v0 + .), decay = exp(-e^-0.5 sigmoid(w0 + .)), bonus = sum r k r_k
//   wkv7    the state recurrence, a head's 64 value rows split over four workgroups
//   gn7     GroupNorm per head, + bonus * v, * g
//   output matrix with the residual add in its epilogue
// then the channel mix: LN2, one mix, relu(. @ K)^2 @ V with the residual add.
#include "mm_dispatch.h"

namespace {

constexpr int HS7 = 64;   // head size
constexpr int TS7 = 32;   // tokens staged in LDS per slab

struct Prep7Args {
    int T, C, H;
    const rwkv_half *r;
    rwkv_half *k, *v;                         // updated in place
    const rwkv_half *w_raw, *a_raw, *vg_raw;  // LoRA outputs [T, C]; vg_raw NULL in layer 0
    const rwkv_half *v_first;                 // [T, C] value of layer 0 (NULL in layer 0)
    const rwkv_half *w0, *a0, *v0, *k_k, *k_a, *r_k;
    rwkv_half *an, *b;                        // -kk and kk * a
    float *dec;                               // decay in (0, 1)
    float *rk;                                // [T, H] bonus factor, fp16-rounded
};

// One wave per (token, head), lane = channel of the head.  Every step rounds to fp16 where an fp16
// tensor operation of the reference does.
__global__ __launch_bounds__(256) void prep7_kernel(Prep7Args a) {
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave >= (int64_t)a.T * a.H) return;
    const int lane = threadIdx.x & 63;
    const int64_t t = wave / a.H;
    const int h = (int)(wave - t * a.H);
    const int c = h * HS7 + lane;
    const size_t o = (size_t)t * a.C + c;
    const float r = h2f(a.r[o]), k = h2f(a.k[o]);
    float v = h2f(a.v[o]);
    const float av = round_h(sigmoidf_(round_h(h2f(a.a0[c]) + h2f(a.a_raw[o]))));
    const float kku = round_h(k * h2f(a.k_k[c]));
    const float nrm = fmaxf(round_h(sqrtf(wave_sum(kku * kku))), 1e-12f);
    const float kk = round_h(kku / nrm);
    const float k2 = round_h(k * round_h(1.f + round_h(round_h(av - 1.f) * h2f(a.k_a[c]))));
    if (a.vg_raw) {
        const float sg = round_h(sigmoidf_(round_h(h2f(a.v0[c]) + h2f(a.vg_raw[o]))));
        v = round_h(v + round_h(round_h(h2f(a.v_first[o]) - v) * sg));
        a.v[o] = f2h(v);
    }
    const float z = round_h(h2f(a.w0[c]) + h2f(a.w_raw[o]));
    a.dec[o] = __expf(-0.606531f * sigmoidf_(z));
    a.k[o] = f2h(k2);
    a.an[o] = f2h(-kk);
    a.b[o] = f2h(kk * av);
    const float rk = wave_sum(round_h(round_h(r * k2) * h2f(a.r_k[c])));
    if (lane == 0) a.rk[wave] = round_h(rk);
}

struct Wkv7Args {
    int T, C;
    float *state;                       // [H][value i][key j]
    const void *r, *w, *k, *v, *a, *b;  // [T, C]
    void *y;                            // [T, C]
};

// A head's value rows never interact (sa_i, y_i and row i of the state depend on v_i only), so a head is
// split over four workgroups of 16 value rows.  Thread (value i, key group g): lane & 15 = g owns keys
// 4g..4g+3 of row i.  The two sums over a row's 16 key groups are DPP row sums in registers, so the token
// loop has no barrier; r, w, k, a, b of a slab of tokens are staged in LDS as fp32.
//   IN_F16: element type of r, k, v, a, b (and of w, y in the operator form)
//   MODEL:  w is the fp32 decay itself and y an fp32 scratch; otherwise w is the log-decay
//           (decay = exp(-exp(w))) and y has the input type
template <bool IN_F16, bool MODEL>
__global__ __launch_bounds__(256) void wkv7_kernel(Wkv7Args a) {
    __shared__ __align__(16) float sr[TS7][HS7], sk[TS7][HS7], sw[TS7][HS7], sa[TS7][HS7], sb[TS7][HS7];
    __shared__ float sv[TS7][16];
    const int T = a.T, C = a.C;
    const int h = blockIdx.x >> 2, vb = blockIdx.x & 3;
    const int lane = threadIdx.x & 63, g = lane & 15;
    const int il = (threadIdx.x >> 6) * 4 + (lane >> 4);
    const int i = vb * 16 + il;
    float *S = a.state + (size_t)h * HS7 * HS7 + (size_t)i * HS7 + 4 * g;
    f32x4 s = *(const f32x4 *)S;
    auto ld = [&](const void *p, size_t o) -> float {
        return IN_F16 ? h2f(((const rwkv_half *)p)[o]) : ((const float *)p)[o];
    };
    for (int t0 = 0; t0 < T; t0 += TS7) {
        const int nt = min(TS7, T - t0);
        __syncthreads();  // previous slab fully consumed
        for (int e = threadIdx.x; e < nt * HS7; e += 256) {
            const int tt = e >> 6, c = e & 63;
            const size_t o = (size_t)(t0 + tt) * C + h * HS7 + c;
            sr[tt][c] = ld(a.r, o);
            sk[tt][c] = ld(a.k, o);
            sa[tt][c] = ld(a.a, o);
            sb[tt][c] = ld(a.b, o);
            sw[tt][c] = MODEL ? ((const float *)a.w)[o] : __expf(-__expf(ld(a.w, o)));
        }
        for (int e = threadIdx.x; e < nt * 16; e += 256) {
            const int tt = e >> 4, c = e & 15;
            sv[tt][c] = ld(a.v, (size_t)(t0 + tt) * C + h * HS7 + vb * 16 + c);
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float vi = sv[tt][il];
            const f32x4 r4 = *(const f32x4 *)&sr[tt][4 * g];
            const f32x4 k4 = *(const f32x4 *)&sk[tt][4 * g];
            const f32x4 w4 = *(const f32x4 *)&sw[tt][4 * g];
            const f32x4 a4 = *(const f32x4 *)&sa[tt][4 * g];
            const f32x4 b4 = *(const f32x4 *)&sb[tt][4 * g];
            float p = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) p += a4[e] * s[e];
            const float sav = row16_sum(p);
            float y = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                s[e] = s[e] * w4[e] + k4[e] * vi + sav * b4[e];
                y += s[e] * r4[e];
            }
            y = row16_sum(y);
            if (g == 0) {
                const size_t o = (size_t)(t0 + tt) * C + h * HS7 + i;
                if (MODEL || !IN_F16) ((float *)a.y)[o] = y;
                else ((rwkv_half *)a.y)[o] = f2h(y);
            }
        }
    }
    *(f32x4 *)S = s;
}

// GroupNorm over each head's 64 outputs (eps 64e-5) on the fp16-rounded read-out, + bonus * v, * g:
// one wave per (token, head).
__global__ __launch_bounds__(256) void gn7_kernel(int T, int C, const float *__restrict__ y,
                                                  const rwkv_half *__restrict__ lnx_w,
                                                  const rwkv_half *__restrict__ lnx_b, const float *__restrict__ rk,
                                                  const rwkv_half *__restrict__ v, const rwkv_half *__restrict__ gate,
                                                  rwkv_half *__restrict__ out) {
    const int H = C / HS7;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave >= (int64_t)T * H) return;
    const int lane = threadIdx.x & 63;
    const int64_t t = wave / H;
    const int h = (int)(wave - t * H);
    const int c = h * HS7 + lane;
    const size_t o = (size_t)t * C + c;
    const float yv = round_h(y[o]);
    const float mean = wave_sum(yv) * (1.f / HS7);
    const float d = yv - mean;
    const float var = wave_sum(d * d) * (1.f / HS7);
    float q = round_h(d * rsqrtf(var + 64e-5f) * h2f(lnx_w[c]) + h2f(lnx_b[c]));
    q = round_h(q + round_h(rk[wave] * h2f(v[o])));
    out[o] = f2h(q * h2f(gate[o]));
}

struct Ws7 {
    rwkv_half *x, *mix[6], *lw, *la, *lv, *lg, *w_raw, *a_raw, *vg_raw, *g, *r, *k, *v, *v_first, *an, *b, *att, *vx,
        *xx_att, *xx_ffn;
    float *dec, *rk, *y32, *splitk;
    size_t total;
};

Ws7 carve7(void *base, int64_t T, const rwkv_v7_model *m) {
    Ws7 w;
    unsigned char *p = (unsigned char *)base;
    auto take = [&](size_t bytes) { void *q = p; p += align256(bytes); return (rwkv_half *)q; };
    const size_t C = m->n_embd, F = m->n_ffn;
    const size_t tc = (size_t)T * C * 2;
    w.x = take(tc);
    for (int j = 0; j < 6; ++j) w.mix[j] = take(tc);
    w.lw = take((size_t)T * m->lora_w * 2); w.la = take((size_t)T * m->lora_a * 2);
    w.lv = take((size_t)T * m->lora_v * 2); w.lg = take((size_t)T * m->lora_g * 2);
    w.w_raw = take(tc); w.a_raw = take(tc); w.vg_raw = take(tc); w.g = take(tc);
    w.r = take(tc); w.k = take(tc); w.v = take(tc); w.v_first = take(tc); w.an = take(tc); w.b = take(tc);
    w.att = take(tc);
    w.vx = take((size_t)T * F * 2);
    w.xx_att = take(C * 2); w.xx_ffn = take(C * 2);
    w.dec = (float *)take((size_t)T * C * 4);
    w.rk = (float *)take((size_t)T * m->n_head * 4);
    w.y32 = (float *)take((size_t)T * C * 4);
    w.splitk = (float *)take(RWKV_SPLITK_WS_BYTES);
    w.total = (size_t)(p - (unsigned char *)base);
    return w;
}

bool mat_ok7(const rwkv_mat &m, int64_t N, int64_t M) {
    return m.w && m.N == N && m.M == M && m.ld >= N && !(m.ld & 7) && aligned16(m.w);
}

int wkv7_check(int64_t B, int64_t T, int64_t C, int64_t H) {
    if (B != 1 || T <= 0 || H <= 0 || C != H * HS7 || T > (1 << 24)) return RWKV_E_SHAPE;
    return RWKV_OK;
}

}  // namespace

extern "C" int rwkv_wkv7_forward(int64_t B, int64_t T, int64_t C, int64_t H, float *state, const void *r,
                                 const void *w, const void *k, const void *v, const void *a, const void *b,
                                 void *y, int dtype, void *stream) {
    if (!state || !r || !w || !k || !v || !a || !b || !y) return RWKV_E_NULL;
    int rc = wkv7_check(B, T, C, H);
    if (rc) return rc;
    if (dtype != RWKV_DT_F16 && dtype != RWKV_DT_F32) return RWKV_E_DTYPE;
    if (!aligned16(state)) return RWKV_E_LAYOUT;
    Wkv7Args q{(int)T, (int)C, state, r, w, k, v, a, b, y};
    const dim3 grid((unsigned)(4 * H)), block(256);
    if (dtype == RWKV_DT_F16) hipLaunchKernelGGL((wkv7_kernel<true, false>), grid, block, 0, (hipStream_t)stream, q);
    else hipLaunchKernelGGL((wkv7_kernel<false, false>), grid, block, 0, (hipStream_t)stream, q);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

static int v7_check(const rwkv_v7_model *m) {
    if (!m || !m->layers || !m->emb || !m->ln_out_w || !m->ln_out_b) return RWKV_E_NULL;
    const int64_t C = m->n_embd, F = m->n_ffn, V = m->vocab;
    if (m->n_layer <= 0 || C <= 0 || F <= 0 || V <= 0 || (C & 63) || (F & 63) || C > 8 * DTHREADS ||
        F > 8 * VP * DTHREADS || m->n_head * HS7 != C)
        return RWKV_E_SHAPE;
    const int ranks[4] = {m->lora_w, m->lora_a, m->lora_v, m->lora_g};
    for (int j = 0; j < 4; ++j)
        if (ranks[j] <= 0 || (ranks[j] & 63) || ranks[j] > 8 * DTHREADS) return RWKV_E_SHAPE;
    for (int i = 0; i < m->n_layer; ++i) {
        const rwkv_v7_layer &l = m->layers[i];
        if (!l.ln1_w || !l.ln1_b || !l.ln2_w || !l.ln2_b || !l.w0 || !l.a0 || !l.w1 || !l.w2 || !l.a1 || !l.a2 ||
            !l.g1 || !l.g2 || !l.k_k || !l.k_a || !l.r_k || !l.lnx_w || !l.lnx_b || !l.ffn_x_k)
            return RWKV_E_NULL;
        if (i > 0 && (!l.v0 || !l.v1 || !l.v2)) return RWKV_E_NULL;
        for (int j = 0; j < 6; ++j)
            if (!l.x_mix[j]) return RWKV_E_NULL;
        if (!mat_ok7(l.att_receptance, C, C) || !mat_ok7(l.att_key, C, C) || !mat_ok7(l.att_value, C, C) ||
            !mat_ok7(l.att_output, C, C) || !mat_ok7(l.ffn_key, C, F) || !mat_ok7(l.ffn_value, F, C))
            return RWKV_E_LAYOUT;
    }
    if (!mat_ok7(m->head, C, V)) return RWKV_E_LAYOUT;
    return RWKV_OK;
}

extern "C" size_t rwkv_v7_workspace(const rwkv_v7_model *m, int64_t T) {
    if (!m || T <= 0) return 0;
    return carve7((void *)256, T, m).total;
}

extern "C" int rwkv_v7_forward(const rwkv_v7_model *m, const rwkv_v56_layer_state *states, const int32_t *tokens,
                               int64_t T, int full_output, float *logits, void *workspace, size_t workspace_bytes,
                               void *stream) {
    int rc = v7_check(m);
    if (rc) return rc;
    if (!states || !tokens || !logits || !workspace) return RWKV_E_NULL;
    if (T <= 0 || T > (1 << 20)) return RWKV_E_SHAPE;
    if (workspace_bytes < rwkv_v7_workspace(m, T) || (((uintptr_t)workspace) & 255)) return RWKV_E_WORKSPACE;
    for (int i = 0; i < m->n_layer; ++i) {
        const rwkv_v56_layer_state &s = states[i];
        if (!s.att_xx || !s.att_kv || !s.ffn_xx) return RWKV_E_NULL;
        if (!aligned16(s.att_xx) || !aligned16(s.ffn_xx) || !aligned16(s.att_kv)) return RWKV_E_LAYOUT;
    }
    hipStream_t st = (hipStream_t)stream;
    const int C = m->n_embd, H = m->n_head;
    Ws7 ws = carve7(workspace, T, m);
    // the fp16 path needs no scaled-activation scratch or row sums
    Ctx c{st, false, T, num_cu(), nullptr, nullptr, nullptr, ws.splitk};
    const unsigned head_waves = (unsigned)(((int64_t)T * H + 3) / 4);

    if ((rc = gather_emb_launch(T, C, tokens, m->emb, ws.x, st))) return rc;
    for (int i = 0; i < m->n_layer; ++i) {
        const rwkv_v7_layer &l = m->layers[i];
        const rwkv_v56_layer_state &s = states[i];
        {
            SeqMixArgs a{};
            a.T = (int)T; a.C = C; a.x = ws.x; a.ln_w = l.ln1_w; a.ln_b = l.ln1_b; a.sx = s.att_xx;
            a.xx_last = ws.xx_att; a.maa_form = 1;
            for (int j = 0; j < 6; ++j) { a.mix[j] = l.x_mix[j]; a.xs[j] = ws.mix[j]; }
            if ((rc = lnmix_seq_launch(a, 6, st))) return rc;
        }
        const rwkv_half *xr = ws.mix[0], *xw = ws.mix[1], *xk = ws.mix[2], *xv = ws.mix[3], *xa = ws.mix[4],
                        *xg = ws.mix[5];
        rwkv_half *v = i == 0 ? ws.v_first : ws.v;
        // the first matrix call also commits the new token-shift state (all readers of the old one are done)
        if ((rc = mm(c, l.att_receptance, false, xr, ACT_NONE, nullptr, nullptr, 1.f, ws.r, ws.xx_att, s.att_xx, C))) return rc;
        if ((rc = mm(c, l.att_key, false, xk, ACT_NONE, nullptr, nullptr, 1.f, ws.k))) return rc;
        if ((rc = mm(c, l.att_value, false, xv, ACT_NONE, nullptr, nullptr, 1.f, v))) return rc;
        if ((rc = mm(c, lora_mat(l.w1, C, m->lora_w), false, xw, ACT_TANH, nullptr, nullptr, 1.f, ws.lw))) return rc;
        if ((rc = mm(c, lora_mat(l.w2, m->lora_w, C), false, ws.lw, ACT_NONE, nullptr, nullptr, 1.f, ws.w_raw))) return rc;
        if ((rc = mm(c, lora_mat(l.a1, C, m->lora_a), false, xa, ACT_NONE, nullptr, nullptr, 1.f, ws.la))) return rc;
        if ((rc = mm(c, lora_mat(l.a2, m->lora_a, C), false, ws.la, ACT_NONE, nullptr, nullptr, 1.f, ws.a_raw))) return rc;
        if (i > 0) {
            if ((rc = mm(c, lora_mat(l.v1, C, m->lora_v), false, xv, ACT_NONE, nullptr, nullptr, 1.f, ws.lv))) return rc;
            if ((rc = mm(c, lora_mat(l.v2, m->lora_v, C), false, ws.lv, ACT_NONE, nullptr, nullptr, 1.f, ws.vg_raw))) return rc;
        }
        if ((rc = mm(c, lora_mat(l.g1, C, m->lora_g), false, xg, ACT_SIGMOID, nullptr, nullptr, 1.f, ws.lg))) return rc;
        if ((rc = mm(c, lora_mat(l.g2, m->lora_g, C), false, ws.lg, ACT_NONE, nullptr, nullptr, 1.f, ws.g))) return rc;
        {
            Prep7Args a{};
            a.T = (int)T; a.C = C; a.H = H; a.r = ws.r; a.k = ws.k; a.v = v; a.w_raw = ws.w_raw; a.a_raw = ws.a_raw;
            a.vg_raw = i > 0 ? ws.vg_raw : nullptr; a.v_first = i > 0 ? ws.v_first : nullptr;
            a.w0 = l.w0; a.a0 = l.a0; a.v0 = l.v0; a.k_k = l.k_k; a.k_a = l.k_a; a.r_k = l.r_k;
            a.an = ws.an; a.b = ws.b; a.dec = ws.dec; a.rk = ws.rk;
            hipLaunchKernelGGL(prep7_kernel, dim3(head_waves), dim3(256), 0, st, a);
        }
        {
            Wkv7Args q{(int)T, C, s.att_kv, ws.r, ws.dec, ws.k, v, ws.an, ws.b, ws.y32};
            hipLaunchKernelGGL((wkv7_kernel<true, true>), dim3((unsigned)(4 * H)), dim3(256), 0, st, q);
        }
        hipLaunchKernelGGL(gn7_kernel, dim3(head_waves), dim3(256), 0, st, (int)T, C, ws.y32, l.lnx_w, l.lnx_b, ws.rk, v,
                           ws.g, ws.att);
        if ((rc = mm(c, l.att_output, false, ws.att, ACT_RESIDUAL, ws.x, nullptr, 1.f, ws.x))) return rc;
        // ---- channel mix
        {
            SeqMixArgs a{};
            a.T = (int)T; a.C = C; a.x = ws.x; a.ln_w = l.ln2_w; a.ln_b = l.ln2_b; a.sx = s.ffn_xx;
            a.xx_last = ws.xx_ffn; a.maa_form = 1;
            a.mix[0] = l.ffn_x_k; a.xs[0] = ws.mix[0];
            if ((rc = lnmix_seq_launch(a, 1, st))) return rc;
        }
        if ((rc = mm(c, l.ffn_key, false, ws.mix[0], ACT_RELU_SQ, nullptr, nullptr, 1.f, ws.vx, ws.xx_ffn, s.ffn_xx, C))) return rc;
        if ((rc = mm(c, l.ffn_value, false, ws.vx, ACT_RESIDUAL, ws.x, nullptr, 1.f, ws.x))) return rc;
        RWKV_LAUNCH_CHECK();
    }
    // ---- head
    const bool all_rows = full_output && T > 1;
    const int64_t TH = all_rows ? T : 1;
    const rwkv_half *xh = all_rows ? ws.x : ws.x + (size_t)(T - 1) * C;
    if (TH == 1) {
        lnhead_launch(false, xh, C, m->ln_out_w, m->ln_out_b, to_dev56(m->head), m->vocab, logits, c.grid, st);
        RWKV_LAUNCH_CHECK();
        return RWKV_OK;
    }
    {
        SeqMixArgs a{};
        a.T = (int)TH; a.C = C; a.x = xh; a.ln_w = m->ln_out_w; a.ln_b = m->ln_out_b; a.sx = nullptr; a.xx_last = nullptr;
        a.xs[0] = ws.mix[0];
        if ((rc = lnmix_seq_launch(a, 1, st))) return rc;
    }
    GemmEpi e{};
    e.out_scale = 1.f; e.act = ACT_NONE; e.out_dtype = RWKV_DT_F32; e.splitk_ws = ws.splitk; e.splitk_bytes = RWKV_SPLITK_WS_BYTES;
    return gemm_launch(false, TH, C, m->vocab, ws.mix[0], C, m->head.w, m->head.ld, logits, m->vocab, e, st);
}
