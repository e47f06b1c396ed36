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
//
// One token (T == 1) runs five launches per layer instead:
//   att7_kernel    LN1 + token shift + the six mixes -> rows (Wr[c], Wk[c], Wv[c]) per wave, then the rows of
//                  the four first LoRA stages (tanh / none / none / sigmoid)
//   tmix7_kernel   per head: second LoRA stages, the preparation above, one step of the recurrence,
//                  GroupNorm, bonus and gate
//   vec_kernel     rows of Wo, x += out
//   lnmix_kernel   LN2 + token shift + mix -> rows of the channel-mix key matrix, relu^2
//   vec_kernel     rows of the channel-mix value matrix, x += out
#include <algorithm>
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

// Eight adjacent channels per lane (16-byte accesses), so the eight lanes of a row of eight own one head of one
// token: grid-stride over the T * C / 8 chunks.  Every step rounds to fp16 where an fp16 tensor operation of the
// reference does; the two sums over a head run over a lane's eight channels in index order and then over the
// eight lanes in three DPP steps.
DEV float head8_sum(float v) {
    v += dpp_mov<0xB1>(v);    // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E>(v);    // quad_perm [2,3,0,1]
    v += dpp_mov<0x141>(v);   // row_half_mirror: the other quad of the eight
    return v;
}

__global__ __launch_bounds__(256) void prep7_kernel(Prep7Args a) {
    const int64_t nchunk = (int64_t)a.T * a.C / 8;
    const int cpr = a.C / 8;   // chunks per token row
    // whole waves take part in the DPP sums: chunks past the end repeat the last one and store nothing
    for (int64_t i0 = (int64_t)blockIdx.x * 256; i0 < nchunk; i0 += (int64_t)gridDim.x * 256) {
        const int64_t i = i0 + threadIdx.x;
        const bool live = i < nchunk;
        const int64_t ic = live ? i : nchunk - 1;
        const int64_t t = ic / cpr;
        const int c = (int)(ic - t * cpr) * 8;
        const size_t o = (size_t)t * a.C + c;
        const h16x8 r8 = *(const h16x8 *)(a.r + o), k8 = *(const h16x8 *)(a.k + o), v8 = *(const h16x8 *)(a.v + o);
        const h16x8 ar8 = *(const h16x8 *)(a.a_raw + o), wr8 = *(const h16x8 *)(a.w_raw + o);
        h16x8 vg8 = {}, vf8 = {}, v08 = {};
        if (a.vg_raw) { vg8 = *(const h16x8 *)(a.vg_raw + o); vf8 = *(const h16x8 *)(a.v_first + o); v08 = *(const h16x8 *)(a.v0 + c); }
        const h16x8 a08 = *(const h16x8 *)(a.a0 + c), kk8 = *(const h16x8 *)(a.k_k + c), ka8 = *(const h16x8 *)(a.k_a + c);
        const h16x8 w08 = *(const h16x8 *)(a.w0 + c), rk8 = *(const h16x8 *)(a.r_k + c);
        float av[8], kku[8], k2[8], ss = 0.f, rks = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float k = (float)k8[e];
            av[e] = round_h(sigmoidf_(round_h((float)a08[e] + (float)ar8[e])));
            kku[e] = round_h(k * (float)kk8[e]);
            ss += kku[e] * kku[e];
            k2[e] = round_h(k * round_h(1.f + round_h(round_h(av[e] - 1.f) * (float)ka8[e])));
            rks += round_h(round_h((float)r8[e] * k2[e]) * (float)rk8[e]);
        }
        const float nrm = fmaxf(round_h(sqrtf(head8_sum(ss))), 1e-12f);
        rks = head8_sum(rks);
        h16x8 ko, ano, bo, vo = v8;
        f32x4 d0, d1;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float kk = round_h(kku[e] / nrm);
            if (a.vg_raw) {
                const float v = (float)v8[e];
                const float sg = round_h(sigmoidf_(round_h((float)v08[e] + (float)vg8[e])));
                vo[e] = (h16)(v + round_h(round_h((float)vf8[e] - v) * sg));
            }
            const float z = round_h((float)w08[e] + (float)wr8[e]);
            const float dec = __expf(-0.606531f * sigmoidf_(z));
            if (e < 4) d0[e] = dec; else d1[e - 4] = dec;
            ko[e] = (h16)k2[e];
            ano[e] = (h16)(-kk);
            bo[e] = (h16)(kk * av[e]);
        }
        if (live) {
            if (a.vg_raw) *(h16x8 *)(a.v + o) = vo;
            *(f32x4 *)(a.dec + o) = d0;
            *(f32x4 *)(a.dec + o + 4) = d1;
            *(h16x8 *)(a.k + o) = ko;
            *(h16x8 *)(a.an + o) = ano;
            *(h16x8 *)(a.b + o) = bo;
            if (!(c & (HS7 - 1))) a.rk[t * a.H + c / HS7] = round_h(rks);
        }
    }
}

struct Wkv7Args {
    int T, C;
    float *state;                       // [H][value i][key j]
    const void *r, *w, *k, *v, *a, *b;  // [T, C]
    void *y;                            // [T, C]
};

// A head's value rows never interact (sa_i, y_i and row i of the state depend on v_i only), so a head is
// split over four workgroups of 16 value rows.  Thread (value i, key group g): lane & 15 = g owns keys
// 4g..4g+3 of row i; sums over a row's 16 key groups are DPP row sums in registers, so the token loop has
// no barrier.  r, w, k, a, b of a slab of tokens are staged in LDS as fp32.
// The only loop-carried chain is state -> sa -> state.  The read-out is taken off it by expanding
//     y_i = sum_j S'_ij r_j = sum_j S_ij (w_j r_j) + v_i (k . r) + sa_i (b . r)
// so that both row sums of a token run on the OLD state side by side; k . r and b . r are per-token
// scalars computed while staging.
//   DT:     element type of r, k, v, a, b (and of w, y in the operator form): RWKV_DT_F16, RWKV_DT_F32 or RWKV_DT_BF16
//   MODEL:  w is the fp32 decay itself and y an fp32 scratch; otherwise w is the log-decay
//           (decay = exp(-exp(w))) and y has the input type
// Staging: thread (token tid / 8, channels 8 (tid % 8) ..+7) loads its share of the NEXT slab into
// registers before the token loop of the current one, so the loads' latency is hidden behind the loop.
// bf16 <-> fp32: the upper half of the fp32 pattern; stores round to nearest even (NaN stays NaN)
DEV float bf2f(uint16_t v) { return __builtin_bit_cast(float, (uint32_t)v << 16); }
DEV uint16_t f2bf(float f) {
    const uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

template <int DT>
struct Stage7 {
    float r[8], k[8], a[8], b[8], w[8], v[2];

    DEV void load8(const void *p, size_t o, float (&d)[8]) {
        if (DT == RWKV_DT_F16) {
            const h16x8 x = *(const h16x8 *)((const rwkv_half *)p + o);
#pragma unroll
            for (int e = 0; e < 8; ++e) d[e] = (float)x[e];
        } else if (DT == RWKV_DT_BF16) {
            const u32x4 x = *(const u32x4 *)((const uint16_t *)p + o);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                d[2 * e] = __builtin_bit_cast(float, x[e] << 16);
                d[2 * e + 1] = __builtin_bit_cast(float, x[e] & 0xffff0000u);
            }
        } else {
            const f32x4 x0 = *(const f32x4 *)((const float *)p + o), x1 = *(const f32x4 *)((const float *)p + o + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) { d[e] = x0[e]; d[4 + e] = x1[e]; }
        }
    }
};

template <int DT, bool MODEL>
__global__ __launch_bounds__(256) void wkv7_kernel(Wkv7Args a) {
    __shared__ __align__(16) float swr[TS7][HS7], sk[TS7][HS7], sw[TS7][HS7], sa[TS7][HS7], sb[TS7][HS7];
    __shared__ float sv[TS7][16], skr[TS7], sbr[TS7];
    const int T = a.T, C = a.C;
    const int h = blockIdx.x >> 2, vb = blockIdx.x & 3;
    const int lane = threadIdx.x & 63, g = lane & 15;
    const int il = (threadIdx.x >> 6) * 4 + (lane >> 4);
    const int i = vb * 16 + il;
    const int stt = threadIdx.x >> 3, sc = (threadIdx.x & 7) * 8;   // staging role
    float *S = a.state + (size_t)h * HS7 * HS7 + (size_t)i * HS7 + 4 * g;
    f32x4 s = *(const f32x4 *)S;
    Stage7<DT> st;
    auto fetch = [&](int t0) {
        const size_t o = (size_t)min(t0 + stt, T - 1) * C + h * HS7;   // rows past the end re-read the last one
        st.load8(a.r, o + sc, st.r);
        st.load8(a.k, o + sc, st.k);
        st.load8(a.a, o + sc, st.a);
        st.load8(a.b, o + sc, st.b);
        if (MODEL) {
            const f32x4 x0 = *(const f32x4 *)((const float *)a.w + o + sc), x1 = *(const f32x4 *)((const float *)a.w + o + sc + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) { st.w[e] = x0[e]; st.w[4 + e] = x1[e]; }
        } else {
            st.load8(a.w, o + sc, st.w);
        }
        const size_t ov = o + vb * 16 + 2 * (threadIdx.x & 7);
        if (DT == RWKV_DT_F16) {
            const h16x2 x = *(const h16x2 *)((const rwkv_half *)a.v + ov);
            st.v[0] = (float)x[0]; st.v[1] = (float)x[1];
        } else if (DT == RWKV_DT_BF16) {
            const uint32_t x = *(const uint32_t *)((const uint16_t *)a.v + ov);
            st.v[0] = __builtin_bit_cast(float, x << 16); st.v[1] = __builtin_bit_cast(float, x & 0xffff0000u);
        } else {
            st.v[0] = ((const float *)a.v)[ov]; st.v[1] = ((const float *)a.v)[ov + 1];
        }
    };
    fetch(0);
    for (int t0 = 0; t0 < T; t0 += TS7) {
        const int nt = min(TS7, T - t0);
        __syncthreads();  // previous slab fully consumed
        {
            float kr = 0.f, br = 0.f;
            f32x4 o4[5][2];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float w = MODEL ? st.w[e] : __expf(-__expf(st.w[e]));
                o4[0][e >> 2][e & 3] = w * st.r[e];
                o4[1][e >> 2][e & 3] = st.k[e];
                o4[2][e >> 2][e & 3] = w;
                o4[3][e >> 2][e & 3] = st.a[e];
                o4[4][e >> 2][e & 3] = st.b[e];
                kr += st.k[e] * st.r[e];
                br += st.b[e] * st.r[e];
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                *(f32x4 *)&swr[stt][sc + 4 * u] = o4[0][u];
                *(f32x4 *)&sk[stt][sc + 4 * u] = o4[1][u];
                *(f32x4 *)&sw[stt][sc + 4 * u] = o4[2][u];
                *(f32x4 *)&sa[stt][sc + 4 * u] = o4[3][u];
                *(f32x4 *)&sb[stt][sc + 4 * u] = o4[4][u];
            }
            sv[stt][2 * (threadIdx.x & 7)] = st.v[0];
            sv[stt][2 * (threadIdx.x & 7) + 1] = st.v[1];
            // the 8 threads of a token are 8 consecutive lanes: three DPP steps
            kr += dpp_mov<0xB1>(kr); br += dpp_mov<0xB1>(br);
            kr += dpp_mov<0x4E>(kr); br += dpp_mov<0x4E>(br);
            kr += dpp_mov<0x141>(kr); br += dpp_mov<0x141>(br);
            if ((threadIdx.x & 7) == 0) { skr[stt] = kr; sbr[stt] = br; }
        }
        __syncthreads();
        fetch(t0 + TS7);
        struct Tok { float vi, kr, br; f32x4 wr4, k4, w4, a4, b4; };
        auto ldtok = [&](int tt) {
            Tok q;
            q.vi = sv[tt][il]; q.kr = skr[tt]; q.br = sbr[tt];
            q.wr4 = *(const f32x4 *)&swr[tt][4 * g];
            q.k4 = *(const f32x4 *)&sk[tt][4 * g];
            q.w4 = *(const f32x4 *)&sw[tt][4 * g];
            q.a4 = *(const f32x4 *)&sa[tt][4 * g];
            q.b4 = *(const f32x4 *)&sb[tt][4 * g];
            return q;
        };
        // state update of one token; returns this thread's share of the read-out sum, p = the summed sa term
        auto advance = [&](const Tok &q, float &p) {
            p = (q.a4[0] * s[0] + q.a4[1] * s[1]) + (q.a4[2] * s[2] + q.a4[3] * s[3]);
            const float yw = (q.wr4[0] * s[0] + q.wr4[1] * s[1]) + (q.wr4[2] * s[2] + q.wr4[3] * s[3]);
            f32x4 kv;
#pragma unroll
            for (int e = 0; e < 4; ++e) kv[e] = s[e] * q.w4[e] + q.k4[e] * q.vi;
            p = row16_sum(p);
#pragma unroll
            for (int e = 0; e < 4; ++e) s[e] = kv[e] + p * q.b4[e];
            return yw;
        };
        auto store = [&](const Tok &q, int tt, float yw, float p) {
            if (g == 0) {
                const float y = yw + q.vi * q.kr + p * q.br;
                const size_t o = (size_t)(t0 + tt) * C + h * HS7 + i;
                if (MODEL || DT == RWKV_DT_F32) ((float *)a.y)[o] = y;
                else if (DT == RWKV_DT_BF16) ((uint16_t *)a.y)[o] = f2bf(y);
                else ((rwkv_half *)a.y)[o] = f2h(y);
            }
        };
        // PASS tokens per pass (TS7 % PASS == 0): their LDS reads are issued together, so the read latency is paid once
        // per pass; in a full pass the read-out row sums, which are not on the state chain, run interleaved after the
        // state updates
        constexpr int PASS = 4;   // 8 was slower here (138 against 128 us per 1024 tokens): 23 operand registers per token
        for (int tt = 0; tt < nt; tt += PASS) {
            Tok q[PASS];
#pragma unroll
            for (int u = 0; u < PASS; ++u) q[u] = ldtok(tt + u);
            float yw[PASS], p[PASS];
            if (tt + PASS - 1 < nt) {
#pragma unroll
                for (int u = 0; u < PASS; ++u) yw[u] = advance(q[u], p[u]);
#pragma unroll
                for (int u = 0; u < PASS; ++u) yw[u] = row16_sum(yw[u]);
#pragma unroll
                for (int u = 0; u < PASS; ++u) store(q[u], tt + u, yw[u], p[u]);
            } else {
#pragma unroll
                for (int u = 0; u < PASS - 1; ++u)
                    if (tt + u < nt) {
                        yw[u] = row16_sum(advance(q[u], p[u]));
                        store(q[u], tt + u, yw[u], p[u]);
                    }
            }
        }
    }
    *(f32x4 *)S = s;
}

// GroupNorm over each head's 64 outputs (eps 64e-5) on the fp16-rounded read-out, + bonus * v, * g.  Four adjacent
// channels per lane (16-byte loads of y, 8-byte accesses to v, g and the output): a row of 16 lanes owns one head
// of one token, its two sums are DPP row sums; grid-stride over the T * C / 4 chunks.
__global__ __launch_bounds__(256) void gn7_kernel(int T, int C, const float *__restrict__ y,
                                                  const rwkv_half *__restrict__ lnx_w,
                                                  const rwkv_half *__restrict__ lnx_b, const float *__restrict__ rk,
                                                  const rwkv_half *__restrict__ v, const rwkv_half *__restrict__ gate,
                                                  rwkv_half *__restrict__ out) {
    const int64_t nchunk = (int64_t)T * C / 4;   // a multiple of 16: whole rows of lanes are live or idle together
    const int cpr = C / 4, H = C / HS7;
    for (int64_t i0 = (int64_t)blockIdx.x * 256; i0 < nchunk; i0 += (int64_t)gridDim.x * 256) {
        const int64_t i = i0 + threadIdx.x;
        const bool live = i < nchunk;
        const int64_t ic = live ? i : nchunk - 1;
        const int64_t t = ic / cpr;
        const int c = (int)(ic - t * cpr) * 4;
        const size_t o = (size_t)t * C + c;
        const f32x4 y4 = *(const f32x4 *)(y + o);
        const h16x4 w4 = *(const h16x4 *)(lnx_w + c), b4 = *(const h16x4 *)(lnx_b + c);
        const h16x4 v4 = *(const h16x4 *)(v + o), g4 = *(const h16x4 *)(gate + o);
        const float bonus = rk[t * H + c / HS7];
        float yv[4], sum = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) { yv[e] = round_h(y4[e]); sum += yv[e]; }
        const float mean = row16_sum(sum) * (1.f / HS7);
        float sq = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) { const float d = yv[e] - mean; sq += d * d; }
        const float rstd = rsqrtf(row16_sum(sq) * (1.f / HS7) + 64e-5f);
        h16x4 o4;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float q = round_h((yv[e] - mean) * rstd * (float)w4[e] + (float)b4[e]);
            q = round_h(q + round_h(bonus * (float)v4[e]));
            o4[e] = (h16)(q * (float)g4[e]);
        }
        if (live) *(h16x4 *)(out + o) = o4;
    }
}

// ---- one-token kernels ---------------------------------------------------------------------
struct Att7Args {
    const rwkv_half *x;
    int C;
    const rwkv_half *ln_w, *ln_b, *sx;
    rwkv_half *xx_tmp;
    const rwkv_half *mix[6];   // r, w, k, v, a, g
    MatDev mat[3];             // receptance, key, value
    rwkv_half *out[3];         // r, k, v  [C]
    const rwkv_half *lora1;    // [rtot][C]
    int rtot, o_a, o_v, o_g;   // rows, first row of the a / v / g blocks
    rwkv_half *l1;             // [rtot] activated first-stage outputs
};

__global__ __launch_bounds__(DTHREADS) void att7_kernel(Att7Args a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[(2 + 3 * 6) * DWAVES];
    __shared__ unsigned sync[2];
    const int C = a.C;
    h16 *xs[6];
    const rwkv_half *mix[6];
    MatDev nomat[6] = {};
#pragma unroll
    for (int j = 0; j < 6; ++j) { xs[j] = (h16 *)smem + j * C; mix[j] = a.mix[j]; }
    LnMixPro<false, 6> pro;
    auto pro_load = [&]() { pro.load(a.x, C, a.ln_w, a.ln_b, a.sx, mix, nomat); };
    auto pro_compute = [&]() { pro.compute(C, true, mix, xs, a.xx_tmp, red, sync, true); };
    auto rowf = [&](int c, int k, const uint8_t *&row, const h16 *&xv) {
        row = row_ptr<false>(a.mat[k], c);
        xv = xs[k == 0 ? 0 : (k == 1 ? 2 : 3)];
    };
    auto epi_load = [&](int) { return NoEpi{}; };
    auto epi = [&](int c, const float (&d)[3], const NoEpi &) {
#pragma unroll
        for (int k = 0; k < 3; ++k) a.out[k][c] = f2h(d[k]);
    };
    const int nseg = (C * 2) >> 4;
    stream_rows<false, 1, 3, 2, NoEpi, true>(C, nseg, pro_waves(C >> 3), sync, pro_load, pro_compute, [] {}, rowf, epi_load, epi);
    // first LoRA stages: row g of the stacked matrix belongs to block j = w, a, v, g
    auto block_of = [&](int g) { return (g >= a.o_a ? 1 : 0) + (g >= a.o_v ? 1 : 0) + (g >= a.o_g ? 1 : 0); };
    auto rowf2 = [&](int g, int, const uint8_t *&row, const h16 *&xv) {
        row = (const uint8_t *)(a.lora1 + (size_t)g * C);
        const int j = block_of(g);
        const int mi = j == 0 ? 1 : (j == 1 ? 4 : (j == 2 ? 3 : 5));   // xw, xa, xv, xg
        xv = (const h16 *)smem + mi * C;
    };
    auto epi2 = [&](int g, const float (&d)[1], const NoEpi &) {
        const int j = block_of(g);
        float v = round_h(d[0]);
        v = j == 0 ? tanhf(v) : (j == 3 ? sigmoidf_(v) : v);
        a.l1[g] = f2h(v);
    };
    stream_rows<false, 1, 1, 2, NoEpi, false>(a.rtot, nseg, 0, nullptr, [] {}, [] {}, [] {}, rowf2, epi_load, epi2);
}

struct Tmix7Args {
    int C, rtot, o_a, o_v, o_g, d_w, d_a, d_v, d_g;
    int first_layer;
    const rwkv_half *l1;       // [rtot]
    const rwkv_half *lora2;    // [C][rtot]
    const rwkv_half *r, *k, *v, *v_first;   // [C]; v_first unused in layer 0 (there v is the layer-0 value itself)
    const rwkv_half *w0, *a0, *v0, *k_k, *k_a, *r_k, *lnx_w, *lnx_b;
    float *state;              // [H][64][64]
    rwkv_half *out;            // [C]
    const rwkv_half *commit_src;   // scratch xx -> token-shift state, done by workgroup 0
    rwkv_half *commit_dst;
};

// One workgroup of 16 waves per head.  All operands are requested in the first instructions (one memory
// round trip): wave w takes 16 (channel, product) rows of the second LoRA stages -- product w / 4, lane =
// 16-byte segment of the row, so a row is one coalesced request -- the first four waves also the head's
// state, wave 0 also the head's vectors.  Then: row sums -> LDS; wave 0 prepares the step; threads 0..255
// (value rows il + 16 m, key group g = lane & 15, holding S[i][4g..4g+3] of their four rows) advance the
// state, the sums over a row's key groups being DPP row sums; wave 0 normalises and gates.
__global__ __launch_bounds__(1024) void tmix7_kernel(Tmix7Args a) {
    __shared__ float lo[4][HS7];
    __shared__ __align__(16) float sr[HS7], sk[HS7], sw[HS7], sa[HS7], sb[HS7];
    __shared__ float sv[HS7], sy[HS7], srk;
    const int h = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int il = (tid >> 4) & 15, g = tid & 15;
    const int c = h * HS7 + lane;
    float *S = a.state + (size_t)h * HS7 * HS7;
    // ---- loads
    const int q = w >> 2;
    const int off = q == 0 ? 0 : (q == 1 ? a.o_a : (q == 2 ? a.o_v : a.o_g));
    const int d8 = (q == 0 ? a.d_w : (q == 1 ? a.d_a : (q == 2 ? (a.first_layer ? 0 : a.d_v) : a.d_g))) >> 3;
    const int seg = lane < d8 ? lane : 0;
    const h16x8 xv = *(const h16x8 *)(a.l1 + off + 8 * seg);
    u32x4 wv[16];
#pragma unroll
    for (int jj = 0; jj < 16; ++jj)
        wv[jj] = *(const u32x4 *)(a.lora2 + (size_t)(h * HS7 + (w & 3) * 16 + jj) * a.rtot + off + 8 * seg);
    f32x4 s[4] = {};
    if (w < 4)
#pragma unroll
        for (int m = 0; m < 4; ++m) s[m] = *(const f32x4 *)(S + (size_t)(il + 16 * m) * HS7 + 4 * g);
    float r = 0.f, k = 0.f, v = 0.f, vf = 0.f, a0 = 0.f, w0 = 0.f, v0 = 0.f, k_k = 0.f, k_a = 0.f, r_k = 0.f, lw = 0.f, lb = 0.f;
    if (w == 0) {
        r = h2f(a.r[c]); k = h2f(a.k[c]); v = h2f(a.v[c]);
        a0 = h2f(a.a0[c]); w0 = h2f(a.w0[c]); k_k = h2f(a.k_k[c]); k_a = h2f(a.k_a[c]); r_k = h2f(a.r_k[c]);
        lw = h2f(a.lnx_w[c]); lb = h2f(a.lnx_b[c]);
        if (!a.first_layer) { vf = h2f(a.v_first[c]); v0 = h2f(a.v0[c]); }
    }
    // ---- second LoRA stages
#pragma unroll
    for (int jj = 0; jj < 16; ++jj) {
        const float p = wave_sum(lane < d8 ? dot8_f16(wv[jj], xv, 0.f) : 0.f);
        if (lane == 0) lo[q][(w & 3) * 16 + jj] = round_h(p);
    }
    __syncthreads();
    if (w == 0) {
        const float av = round_h(sigmoidf_(round_h(a0 + lo[1][lane])));
        const float kku = round_h(k * k_k);
        const float nrm = fmaxf(round_h(sqrtf(wave_sum(kku * kku))), 1e-12f);
        const float kk = round_h(kku / nrm);
        const float k2 = round_h(k * round_h(1.f + round_h(round_h(av - 1.f) * k_a)));
        if (!a.first_layer) {
            const float sg = round_h(sigmoidf_(round_h(v0 + lo[2][lane])));
            v = round_h(v + round_h(round_h(vf - v) * sg));
        }
        const float z = round_h(w0 + lo[0][lane]);
        sr[lane] = r; sk[lane] = k2; sv[lane] = v;
        sw[lane] = __expf(-0.606531f * sigmoidf_(z));
        sa[lane] = -kk;
        sb[lane] = round_h(kk * av);
        const float rk = wave_sum(round_h(round_h(r * k2) * r_k));
        if (lane == 0) srk = round_h(rk);
    }
    __syncthreads();
    if (w < 4) {
        const f32x4 r4 = *(const f32x4 *)&sr[4 * g], k4 = *(const f32x4 *)&sk[4 * g], w4 = *(const f32x4 *)&sw[4 * g];
        const f32x4 a4 = *(const f32x4 *)&sa[4 * g], b4 = *(const f32x4 *)&sb[4 * g];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            const int i = il + 16 * m;
            const float vi = sv[i];
            float p = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) p += a4[e] * s[m][e];
            const float sav = row16_sum(p);
            float y = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                s[m][e] = s[m][e] * w4[e] + k4[e] * vi + sav * b4[e];
                y += s[m][e] * r4[e];
            }
            y = row16_sum(y);
            if (g == 0) sy[i] = y;
            *(f32x4 *)(S + (size_t)i * HS7 + 4 * g) = s[m];
        }
    }
    __syncthreads();
    if (w == 0) {
        const float yv = round_h(sy[lane]);
        const float mean = wave_sum(yv) * (1.f / HS7);
        const float dv = yv - mean;
        const float var = wave_sum(dv * dv) * (1.f / HS7);
        float o = round_h(dv * rsqrtf(var + 64e-5f) * lw + lb);
        o = round_h(o + round_h(srk * sv[lane]));
        a.out[c] = f2h(o * lo[3][lane]);
    }
    if (blockIdx.x == 0 && a.commit_dst)
        for (int j8 = tid; j8 < (a.C >> 3); j8 += 1024)
            *(u32x4 *)(a.commit_dst + 8 * j8) = *(const u32x4 *)(a.commit_src + 8 * j8);
}

// ---- DeepEmbed channel mix (model.py:578-594): keys of token t scaled by ((xx_t @ s1) @ E_t) @ s2 + s0 -----------
// First stage, one workgroup per token: sv = xx_t @ s1 (32 sums over C, eight per wave), then ss = sv @ E_t with
// E_t = row token_t of the merged table viewed 32 x 32.  Both rounded to fp16 as the reference's fp16 tensors are.
__global__ __launch_bounds__(256) void de_ss_kernel(int T, int C, int vocab, const int32_t *__restrict__ tokens,
                                                    const rwkv_half *__restrict__ xx, const rwkv_half *__restrict__ s1,
                                                    const rwkv_half *__restrict__ emb, rwkv_half *__restrict__ ss) {
    __shared__ float sv[32];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const rwkv_half *x = xx + (size_t)t * C;
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    for (int c8 = lane; c8 < (C >> 3); c8 += 64) {
        const h16x8 xv = *(const h16x8 *)(x + 8 * c8);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const h16x8 wv = *(const h16x8 *)(s1 + (size_t)(wave * 8 + j) * C + 8 * c8);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[j] += (float)xv[e] * (float)wv[e];
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float v = wave_sum(acc[j]);
        if (lane == 0) sv[wave * 8 + j] = (float)(h16)v;
    }
    __syncthreads();
    if (threadIdx.x < 32) {
        const rwkv_half *E = emb + (size_t)min(max(tokens[t], 0), vocab - 1) * 1024;
        float a = 0.f;
        for (int i = 0; i < 32; ++i) a += sv[i] * (float)h2f(E[i * 32 + threadIdx.x]);
        ss[(size_t)t * 32 + threadIdx.x] = f2h(a);
    }
}

// Second stage: k[t][f] *= (ss_t @ s2)[f] + s0[f], every step rounded to fp16.  A workgroup takes 256 columns of
// eight tokens, so a column of s2 is fetched once per eight tokens.
__global__ __launch_bounds__(256) void de_gate_kernel(int T, int F, const rwkv_half *__restrict__ ss,
                                                      const rwkv_half *__restrict__ s2, const rwkv_half *__restrict__ s0,
                                                      rwkv_half *__restrict__ k) {
    __shared__ float ssl[8][32];
    const int t0 = blockIdx.x * 8, f = blockIdx.y * 256 + threadIdx.x;
    {
        const int tt = threadIdx.x >> 5, j = threadIdx.x & 31;
        ssl[tt][j] = t0 + tt < T ? h2f(ss[(size_t)(t0 + tt) * 32 + j]) : 0.f;
    }
    __syncthreads();
    if (f >= F) return;
    float col[32];
#pragma unroll
    for (int j = 0; j < 32; ++j) col[j] = h2f(s2[(size_t)j * F + f]);
    const float b = h2f(s0[f]);
    for (int tt = 0; tt < 8 && t0 + tt < T; ++tt) {
        float a = 0.f;
#pragma unroll
        for (int j = 0; j < 32; ++j) a += ssl[tt][j] * col[j];
        const float g = (float)(h16)((float)(h16)a + b);
        rwkv_half *kp = k + (size_t)(t0 + tt) * F + f;
        *kp = f2h(h2f(*kp) * g);
    }
}

int de_gate_launch(const rwkv_v7_layer &l, int64_t T, int C, int F, int vocab, const int32_t *tokens, const rwkv_half *xx,
                   rwkv_half *ss, rwkv_half *k, hipStream_t st) {
    hipLaunchKernelGGL(de_ss_kernel, dim3((unsigned)T), dim3(256), 0, st, (int)T, C, vocab, tokens, xx, l.de_s1, l.de_emb, ss);
    hipLaunchKernelGGL(de_gate_kernel, dim3((unsigned)((T + 7) / 8), (unsigned)((F + 255) / 256)), dim3(256), 0, st, (int)T, F,
                       ss, l.de_s2, l.de_s0, k);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

struct Ws7 {
    rwkv_half *x, *mix[6], *l1, *lw, *la, *lv, *lg, *w_raw, *a_raw, *vg_raw, *g, *r, *k, *v, *v_first, *an, *b, *att, *vx,
        *xx_att, *xx_ffn, *de_ss;
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
    w.l1 = take((size_t)(m->lora_w + m->lora_a + m->lora_v + m->lora_g) * 2);
    w.lw = take((size_t)T * m->lora_w * 2); w.la = take((size_t)T * m->lora_a * 2);
    w.lv = take((size_t)T * m->lora_v * 2); w.lg = take((size_t)T * m->lora_g * 2);
    w.w_raw = take(tc); w.a_raw = take(tc); w.vg_raw = take(tc); w.g = take(tc);
    w.r = take(tc); w.k = take(tc); w.v = take(tc); w.v_first = take(tc); w.an = take(tc); w.b = take(tc);
    w.att = take(tc);
    w.vx = take((size_t)T * F * 2);
    w.xx_att = take(C * 2); w.xx_ffn = take(C * 2);
    w.de_ss = take((size_t)T * 32 * 2);
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
    if (dtype != RWKV_DT_F16 && dtype != RWKV_DT_F32 && dtype != RWKV_DT_BF16) return RWKV_E_DTYPE;
    if (!aligned16(state) || !aligned16(r) || !aligned16(w) || !aligned16(k) || !aligned16(a) || !aligned16(b) ||
        (((uintptr_t)v) & 3))
        return RWKV_E_LAYOUT;
    Wkv7Args q{(int)T, (int)C, state, r, w, k, v, a, b, y};
    const dim3 grid((unsigned)(4 * H)), block(256);
    if (dtype == RWKV_DT_F16) hipLaunchKernelGGL((wkv7_kernel<RWKV_DT_F16, false>), grid, block, 0, (hipStream_t)stream, q);
    else if (dtype == RWKV_DT_BF16) hipLaunchKernelGGL((wkv7_kernel<RWKV_DT_BF16, false>), grid, block, 0, (hipStream_t)stream, q);
    else hipLaunchKernelGGL((wkv7_kernel<RWKV_DT_F32, false>), grid, block, 0, (hipStream_t)stream, q);
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
        if (!l.ln1_w || !l.ln1_b || !l.ln2_w || !l.ln2_b || !l.w0 || !l.a0 || !l.lora1 || !l.lora2 || !l.k_k ||
            !l.k_a || !l.r_k || !l.lnx_w || !l.lnx_b || !l.ffn_x_k)
            return RWKV_E_NULL;
        if (i > 0 && !l.v0) return RWKV_E_NULL;
        if (!aligned16(l.lora1) || !aligned16(l.lora2)) return RWKV_E_LAYOUT;
        if (l.de_emb || l.de_s1 || l.de_s2 || l.de_s0) {   // the DeepEmbed tensors come all four or not at all
            if (!l.de_emb || !l.de_s1 || !l.de_s2 || !l.de_s0) return RWKV_E_NULL;
            if (!aligned16(l.de_s1)) return RWKV_E_LAYOUT;
        }
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
    Ctx c{st, false, T, num_cu(), nullptr, nullptr, nullptr, ws.splitk, 0};

    const int max_rank = std::max(std::max(m->lora_w, m->lora_a), std::max(m->lora_v, m->lora_g));
    const int o_a = m->lora_w, o_v = o_a + m->lora_a, o_g = o_v + m->lora_v, rtot = o_g + m->lora_g;
    // block j of the stacked LoRA matrices as matrices of their own
    auto lora_first = [&](const rwkv_v7_layer &l, int off, int d) { return lora_mat(l.lora1 + (size_t)off * C, C, d); };
    auto lora_second = [&](const rwkv_v7_layer &l, int off, int d) {
        rwkv_mat q{};
        q.w = l.lora2 + off; q.ld = rtot; q.N = d; q.M = C;
        return q;
    };

    SideStreams *ss = T >= 256 ? side_streams(st) : nullptr;

    if ((rc = gather_emb_launch(T, C, m->vocab, tokens, m->emb, ws.x, st))) return rc;
    for (int i = 0; i < m->n_layer; ++i) {
        const rwkv_v7_layer &l = m->layers[i];
        const rwkv_v56_layer_state &s = states[i];
        // one token: the six mixed activation vectors must fit the default LDS window, a LoRA row one request per wave
        if (T == 1 && C <= 5120 && max_rank <= 512) {
            rwkv_half *v1 = i == 0 ? ws.v_first : ws.v;
            {
                Att7Args a{};
                a.x = ws.x; a.C = C; a.ln_w = l.ln1_w; a.ln_b = l.ln1_b; a.sx = s.att_xx; a.xx_tmp = ws.xx_att;
                for (int j = 0; j < 6; ++j) a.mix[j] = l.x_mix[j];
                a.mat[0] = to_dev56(l.att_receptance); a.mat[1] = to_dev56(l.att_key); a.mat[2] = to_dev56(l.att_value);
                a.out[0] = ws.r; a.out[1] = ws.k; a.out[2] = v1;
                a.lora1 = l.lora1; a.rtot = rtot; a.o_a = o_a; a.o_v = o_v; a.o_g = o_g; a.l1 = ws.l1;
                hipLaunchKernelGGL(att7_kernel, dim3(c.grid), dim3(DTHREADS), 6 * (size_t)C * 2, st, a);
            }
            {
                Tmix7Args a{};
                a.C = C; a.rtot = rtot; a.o_a = o_a; a.o_v = o_v; a.o_g = o_g;
                a.d_w = m->lora_w; a.d_a = m->lora_a; a.d_v = m->lora_v; a.d_g = m->lora_g;
                a.first_layer = i == 0; a.l1 = ws.l1; a.lora2 = l.lora2;
                a.r = ws.r; a.k = ws.k; a.v = v1; a.v_first = ws.v_first;
                a.w0 = l.w0; a.a0 = l.a0; a.v0 = l.v0; a.k_k = l.k_k; a.k_a = l.k_a; a.r_k = l.r_k;
                a.lnx_w = l.lnx_w; a.lnx_b = l.lnx_b; a.state = s.att_kv; a.out = ws.att;
                a.commit_src = ws.xx_att; a.commit_dst = s.att_xx;
                hipLaunchKernelGGL(tmix7_kernel, dim3((unsigned)H), dim3(1024), 0, st, a);
            }
            if ((rc = mm(c, l.att_output, false, ws.att, ACT_RESIDUAL, ws.x, nullptr, 1.f, ws.x))) return rc;
            {
                LnMixArgs a{};
                a.x = ws.x; a.C = C; a.ln_w = l.ln2_w; a.ln_b = l.ln2_b; a.sx = s.ffn_xx; a.xx_tmp = ws.xx_ffn;
                a.mix[0] = l.ffn_x_k; a.mat[0] = to_dev56(l.ffn_key); a.M[0] = (int)l.ffn_key.M; a.epi[0] = EPI_RELU_SQ;
                a.out[0] = ws.vx; a.maa_form = 1;
                lnmix1_launch(false, a, c.grid, st);
            }
            if (l.de_emb && (rc = de_gate_launch(l, 1, C, m->n_ffn, m->vocab, tokens, ws.xx_ffn, ws.de_ss, ws.vx, st))) return rc;
            if ((rc = mm(c, l.ffn_value, false, ws.vx, ACT_RESIDUAL, ws.x, nullptr, 1.f, ws.x, ws.xx_ffn, s.ffn_xx, C))) return rc;
            RWKV_LAUNCH_CHECK();
            continue;
        }
        {
            SeqMixArgs a{};
            a.T = (int)T; a.C = C; a.x = ws.x; a.ln_w = l.ln1_w; a.ln_b = l.ln1_b; a.sx = s.att_xx;
            a.xx_last = nullptr; a.state_out = s.att_xx; a.maa_form = 1;   // row 0's workgroup commits the new state
            for (int j = 0; j < 6; ++j) { a.mix[j] = l.x_mix[j]; a.xs[j] = ws.mix[j]; }
            if ((rc = lnmix_seq_launch(a, 6, st))) return rc;
        }
        const rwkv_half *xr = ws.mix[0], *xw = ws.mix[1], *xk = ws.mix[2], *xv = ws.mix[3], *xa = ws.mix[4],
                        *xg = ws.mix[5];
        rwkv_half *v = i == 0 ? ws.v_first : ws.v;
        // The three C x C products and the LoRA chain are independent of each other.  From 256 rows on receptance,
        // key and value are one grouped launch of the direct-to-LDS kernel; where that group is more than one round
        // of large tiles (2048 tokens at n_embd 4096), the LoRA launches (which do split K: one user of the split-K
        // scratch at a time) run beside it on a side stream.  Measured with the LoRA stages grouped: 46.0K against
        // 45.7K tok/s in calls of 2048, but 42.3K against 43.3K in calls of 1024, where the group is one round and
        // the two streams only slow each other down.
        const bool dma_seq = true;
        ForkScope par(ss, st, 1, dma_seq && 3 * ((T + 255) / 256) * ((C + 255) / 256) >= 384);
        Ctx cm = c, cv = c, cl = c;
        if (par) cl.st = ss->s[0];
        if (dma_seq && !(C & 7)) {
            // receptance, key and value as one grouped launch
            const rwkv_half *xin[3] = {xr, xk, xv};
            const rwkv_mat *mats[3] = {&l.att_receptance, &l.att_key, &l.att_value};
            void *outs[3] = {ws.r, ws.k, v};
            GemmEpi ep[3] = {};
            for (int j = 0; j < 3; ++j) { ep[j].act = ACT_NONE; ep[j].out_scale = 1.f; ep[j].out_dtype = RWKV_DT_F16; }
            if ((rc = gemm_group_launch(false, 3, T, C, xin, mats, outs, ep, nullptr, nullptr, ws.splitk, st))) return rc;
        } else {
        if ((rc = mm(cm, l.att_receptance, false, xr, ACT_NONE, nullptr, nullptr, 1.f, ws.r))) return rc;
        if ((rc = mm(cm, l.att_key, false, xk, ACT_NONE, nullptr, nullptr, 1.f, ws.k))) return rc;
        if ((rc = mm(cv, l.att_value, false, xv, ACT_NONE, nullptr, nullptr, 1.f, v))) return rc;
        }
        // The LoRA products: the first stages (same input width, their own inputs, ranks and activations) as one
        // grouped launch, then the second stages -- those of equal rank as one grouped launch, the others one by one.
        // RWKV_V7_LORA_GROUPS=0 launches all eight one by one (tuning).
        {
            const bool has_v = i > 0;
            struct Stage { const rwkv_half *x; int off, d, act; rwkv_half *l1, *out; };
            const Stage sg[4] = {{xw, 0, m->lora_w, ACT_TANH, ws.lw, ws.w_raw},
                                 {xa, o_a, m->lora_a, ACT_NONE, ws.la, ws.a_raw},
                                 {xv, o_v, m->lora_v, ACT_NONE, ws.lv, ws.vg_raw},
                                 {xg, o_g, m->lora_g, ACT_SIGMOID, ws.lg, ws.g}};
            const char *env = getenv("RWKV_V7_LORA_GROUPS");
            const bool groups = !(env && *env == '0') && !(C & 7);
            bool first_done[4] = {false, false, false, false}, second_done[4] = {false, false, false, false};
            if (groups) {
                const rwkv_half *xin[4];
                rwkv_mat mt[4];
                const rwkv_mat *mp[4];
                void *outs[4];
                GemmEpi ep[4] = {};
                int n = 0, idx[4];
                for (int q = 0; q < 4; ++q) {
                    if (q == 2 && !has_v) continue;
                    xin[n] = sg[q].x; mt[n] = lora_first(l, sg[q].off, sg[q].d); mp[n] = &mt[n]; outs[n] = sg[q].l1;
                    ep[n].act = sg[q].act; ep[n].out_scale = 1.f; ep[n].out_dtype = RWKV_DT_F16;
                    idx[n++] = q;
                }
                if ((rc = gemm_group_launch(false, n, T, C, xin, mp, outs, ep, nullptr, nullptr, cl.splitk, cl.st))) return rc;
                for (int q = 0; q < n; ++q) first_done[idx[q]] = true;
                // second stages of the most common rank together
                int best = -1, best_n = 0;
                for (int q = 0; q < 4; ++q) {
                    if (q == 2 && !has_v) continue;
                    int cnt = 0;
                    for (int r = 0; r < 4; ++r) cnt += (r != 2 || has_v) && sg[r].d == sg[q].d;
                    if (cnt > best_n) { best_n = cnt; best = q; }
                }
                if (best_n >= 2 && !(sg[best].d % 64)) {
                    n = 0;
                    for (int q = 0; q < 4; ++q) {
                        if ((q == 2 && !has_v) || sg[q].d != sg[best].d) continue;
                        xin[n] = sg[q].l1; mt[n] = lora_second(l, sg[q].off, sg[q].d); mp[n] = &mt[n]; outs[n] = sg[q].out;
                        ep[n] = GemmEpi{};
                        ep[n].act = ACT_NONE; ep[n].out_scale = 1.f; ep[n].out_dtype = RWKV_DT_F16;
                        idx[n++] = q;
                    }
                    if ((rc = gemm_group_launch(false, n, T, sg[best].d, xin, mp, outs, ep, nullptr, nullptr, cl.splitk, cl.st))) return rc;
                    for (int q = 0; q < n; ++q) second_done[idx[q]] = true;
                }
            }
            for (int q = 0; q < 4; ++q) {
                if (q == 2 && !has_v) continue;
                if (!first_done[q] &&
                    (rc = mm(cl, lora_first(l, sg[q].off, sg[q].d), false, sg[q].x, sg[q].act, nullptr, nullptr, 1.f, sg[q].l1)))
                    return rc;
                if (!second_done[q] &&
                    (rc = mm(cl, lora_second(l, sg[q].off, sg[q].d), false, sg[q].l1, ACT_NONE, nullptr, nullptr, 1.f, sg[q].out)))
                    return rc;
            }
        }
        if (!par.join()) return (int)hipErrorUnknown;
        {
            Prep7Args a{};
            a.T = (int)T; a.C = C; a.H = H; a.r = ws.r; a.k = ws.k; a.v = v; a.w_raw = ws.w_raw; a.a_raw = ws.a_raw;
            a.vg_raw = i > 0 ? ws.vg_raw : nullptr; a.v_first = i > 0 ? ws.v_first : nullptr;
            a.w0 = l.w0; a.a0 = l.a0; a.v0 = l.v0; a.k_k = l.k_k; a.k_a = l.k_a; a.r_k = l.r_k;
            a.an = ws.an; a.b = ws.b; a.dec = ws.dec; a.rk = ws.rk;
            const int64_t blocks = ((int64_t)T * C / 8 + 255) / 256;
            hipLaunchKernelGGL(prep7_kernel, dim3((unsigned)std::min<int64_t>(blocks, 65535)), dim3(256), 0, st, a);
        }
        {
            Wkv7Args q{(int)T, C, s.att_kv, ws.r, ws.dec, ws.k, v, ws.an, ws.b, ws.y32};
            hipLaunchKernelGGL((wkv7_kernel<RWKV_DT_F16, true>), dim3((unsigned)(4 * H)), dim3(256), 0, st, q);
        }
        hipLaunchKernelGGL(gn7_kernel, dim3((unsigned)std::min<int64_t>(((int64_t)T * C / 4 + 255) / 256, 65535)), dim3(256), 0, st, (int)T, C, ws.y32, l.lnx_w, l.lnx_b, ws.rk, v,
                           ws.g, ws.att);
        if ((rc = mm(c, l.att_output, false, ws.att, ACT_RESIDUAL, ws.x, nullptr, 1.f, ws.x))) return rc;
        // ---- channel mix
        {
            SeqMixArgs a{};
            a.T = (int)T; a.C = C; a.x = ws.x; a.ln_w = l.ln2_w; a.ln_b = l.ln2_b; a.sx = s.ffn_xx;
            a.xx_last = nullptr; a.state_out = s.ffn_xx; a.maa_form = 1;
            a.mix[0] = l.ffn_x_k; a.xs[0] = ws.mix[0];
            a.mix[1] = nullptr; a.xs[1] = ws.mix[1];   // DeepEmbed also reads the LayerNorm output itself
            if ((rc = lnmix_seq_launch(a, l.de_emb ? 2 : 1, st))) return rc;
        }
        if ((rc = mm(c, l.ffn_key, false, ws.mix[0], ACT_RELU_SQ, nullptr, nullptr, 1.f, ws.vx))) return rc;
        if (l.de_emb && (rc = de_gate_launch(l, T, C, m->n_ffn, m->vocab, tokens, ws.mix[1], ws.de_ss, ws.vx, st))) return rc;
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
