// WKV recurrences: RWKV-4 (per channel, running-maximum form) and RWKV-5/6 (per-head 64x64 state).
#include <algorithm>
#include "gemv_core.h"
#include "kernels.h"

namespace {

// ---------------------------------------------------------------------------------------
// RWKV-4.  One lane per channel, fp32 state in registers for the whole T loop; a wave reads
// 64 consecutive channels of a token (coalesced).  k/v for the next UNR tokens are loaded
// before the dependent chain of exp/div consumes them, so memory latency is off the
// critical path.  One wave per workgroup spreads the C/64 waves over as many CUs as possible.
//   MODE 0: k, v, y fp32 (operator-level interface)
//   MODE 1: k, v fp16; y = fp16(r * fp16(wkv)) with r fp16 (already sigmoid'ed), fp16 out
//   MODE 2: as MODE 1 with k, v fp32
// ---------------------------------------------------------------------------------------
template <int MODE> struct Wkv4IO;
template <> struct Wkv4IO<0> {
    const float *k, *v; float *y; const rwkv_half *r;
    DEV float ldk(size_t i) const { return k[i]; }
    DEV float ldv(size_t i) const { return v[i]; }
    DEV float ldr(size_t) const { return 1.f; }
    DEV void st(size_t i, float wkv, float) const { y[i] = wkv; }
};
template <> struct Wkv4IO<1> {
    const rwkv_half *k, *v; rwkv_half *y; const rwkv_half *r;
    DEV float ldk(size_t i) const { return h2f(k[i]); }
    DEV float ldv(size_t i) const { return h2f(v[i]); }
    DEV float ldr(size_t i) const { return h2f(r[i]); }
    DEV void st(size_t i, float wkv, float rr) const { y[i] = f2h(rr * round_h(wkv)); }
};
template <> struct Wkv4IO<2> {
    const float *k, *v; rwkv_half *y; const rwkv_half *r;
    DEV float ldk(size_t i) const { return k[i]; }
    DEV float ldv(size_t i) const { return v[i]; }
    DEV float ldr(size_t i) const { return h2f(r[i]); }
    DEV void st(size_t i, float wkv, float rr) const { y[i] = f2h(rr * round_h(wkv)); }
};

DEV void wkv4_step(float kk, float vv, float u, float w, float &aa, float &bb, float &pp, float &out) {
    float ww = u + kk;
    float p = fmaxf(pp, ww);
    float e1 = __expf(pp - p), e2 = __expf(ww - p);
    out = (e1 * aa + e2 * vv) / (e1 * bb + e2);
    ww = w + pp;
    p = fmaxf(ww, kk);
    e1 = __expf(ww - p);
    e2 = __expf(kk - p);
    aa = e1 * aa + e2 * vv;
    bb = e1 * bb + e2;
    pp = p;
}

template <int MODE>
__global__ __launch_bounds__(64) void wkv4_kernel(int T, int C, const float *__restrict__ w_, const float *__restrict__ u_,
                                                  Wkv4IO<MODE> io, float *__restrict__ aa_, float *__restrict__ bb_,
                                                  float *__restrict__ pp_) {
    constexpr int UNR = 8;
    const int c = blockIdx.x * 64 + threadIdx.x;
    const int b = blockIdx.y;
    if (c >= C) return;
    const size_t base = (size_t)b * T * C + c;
    const int so = b * C + c;
    const float u = u_[c], w = w_[c];
    float aa = aa_[so], bb = bb_[so], pp = pp_[so];
    int t = 0;
    for (; t + UNR <= T; t += UNR) {
        float kk[UNR], vv[UNR], rr[UNR];
#pragma unroll
        for (int i = 0; i < UNR; ++i) {
            const size_t o = base + (size_t)(t + i) * C;
            kk[i] = io.ldk(o); vv[i] = io.ldv(o); rr[i] = io.ldr(o);
        }
#pragma unroll
        for (int i = 0; i < UNR; ++i) {
            float out;
            wkv4_step(kk[i], vv[i], u, w, aa, bb, pp, out);
            io.st(base + (size_t)(t + i) * C, out, rr[i]);
        }
    }
    for (; t < T; ++t) {
        const size_t o = base + (size_t)t * C;
        float out;
        const float rr = io.ldr(o);
        wkv4_step(io.ldk(o), io.ldv(o), u, w, aa, bb, pp, out);
        io.st(o, out, rr);
    }
    aa_[so] = aa; bb_[so] = bb; pp_[so] = pp;
}

// ---------------------------------------------------------------------------------------
// RWKV-4 over a long sequence: the recurrence is a scan with an associative combine, so T is cut into
// chunks that run in parallel.  A state (a, b, p) stands for the sums A = a e^p, B = b e^p; n steps of
// decay add n w to p, and two states merge under the larger exponent.
//   pass 1  (chunk j, channel c): state after the chunk's tokens starting from the empty state
//   pass 2  (chunk j, channel c): incoming state = fold of the call's initial state and the summaries of
//           chunks 0..j-1 (decay by one chunk length between them), then the ordinary per-token steps of
//           the chunk; the last chunk stores the final state.
// Twice the arithmetic of the sequential kernel on T/L times as many lanes.
// scratch: (nchunks + 1) x 3 x C floats; slot 0 holds a copy of the initial state (the final state is
// written over the caller's while other chunks may still read it).
// ---------------------------------------------------------------------------------------
DEV void wkv4_merge(float &a, float &b, float &p, float a2, float b2, float p2) {
    const float q = fmaxf(p, p2);
    const float e1 = __expf(p - q), e2 = __expf(p2 - q);
    a = e1 * a + e2 * a2;
    b = e1 * b + e2 * b2;
    p = q;
}

template <int MODE>
__global__ __launch_bounds__(64) void wkv4_chunk_summary_kernel(int T, int C, int L, const float *__restrict__ w_,
                                                                Wkv4IO<MODE> io, const float *__restrict__ aa_,
                                                                const float *__restrict__ bb_, const float *__restrict__ pp_,
                                                                float *__restrict__ scratch) {
    constexpr int UNR = 8;
    const int c = blockIdx.x * 64 + threadIdx.x, j = blockIdx.y;
    if (c >= C) return;
    if (j == 0) {
        scratch[c] = aa_[c]; scratch[C + c] = bb_[c]; scratch[2 * C + c] = pp_[c];
    }
    const float w = w_[c];
    const int t0 = j * L, t1 = min(T, t0 + L);
    float aa = 0.f, bb = 0.f, pp = -1e38f;
    auto step = [&](float kk, float vv) {
        const float ww = w + pp;
        const float p = fmaxf(ww, kk);
        const float e1 = __expf(ww - p), e2 = __expf(kk - p);
        aa = e1 * aa + e2 * vv;
        bb = e1 * bb + e2;
        pp = p;
    };
    int t = t0;
    for (; t + UNR <= t1; t += UNR) {
        float kk[UNR], vv[UNR];
#pragma unroll
        for (int i = 0; i < UNR; ++i) {
            const size_t o = (size_t)(t + i) * C + c;
            kk[i] = io.ldk(o); vv[i] = io.ldv(o);
        }
#pragma unroll
        for (int i = 0; i < UNR; ++i) step(kk[i], vv[i]);
    }
    for (; t < t1; ++t) step(io.ldk((size_t)t * C + c), io.ldv((size_t)t * C + c));
    float *o = scratch + (size_t)(j + 1) * 3 * C;
    o[c] = aa; o[C + c] = bb; o[2 * C + c] = pp;
}

template <int MODE>
__global__ __launch_bounds__(64) void wkv4_chunk_apply_kernel(int T, int C, int L, const float *__restrict__ w_,
                                                              const float *__restrict__ u_, Wkv4IO<MODE> io,
                                                              float *__restrict__ aa_, float *__restrict__ bb_,
                                                              float *__restrict__ pp_, const float *__restrict__ scratch) {
    constexpr int UNR = 8;
    const int c = blockIdx.x * 64 + threadIdx.x, j = blockIdx.y;
    if (c >= C) return;
    const float u = u_[c], w = w_[c];
    const int t0 = j * L, t1 = min(T, t0 + L);
    float aa = scratch[c], bb = scratch[C + c], pp = scratch[2 * C + c];
    const float wl = w * (float)L;
    for (int i = 0; i < j; ++i) {
        const float *sm = scratch + (size_t)(i + 1) * 3 * C;
        pp += wl;
        wkv4_merge(aa, bb, pp, sm[c], sm[C + c], sm[2 * C + c]);
    }
    int t = t0;
    for (; t + UNR <= t1; t += UNR) {
        float kk[UNR], vv[UNR], rr[UNR];
#pragma unroll
        for (int i = 0; i < UNR; ++i) {
            const size_t o = (size_t)(t + i) * C + c;
            kk[i] = io.ldk(o); vv[i] = io.ldv(o); rr[i] = io.ldr(o);
        }
#pragma unroll
        for (int i = 0; i < UNR; ++i) {
            float out;
            wkv4_step(kk[i], vv[i], u, w, aa, bb, pp, out);
            io.st((size_t)(t + i) * C + c, out, rr[i]);
        }
    }
    for (; t < t1; ++t) {
        const size_t o = (size_t)t * C + c;
        float out;
        const float rr = io.ldr(o);
        wkv4_step(io.ldk(o), io.ldv(o), u, w, aa, bb, pp, out);
        io.st(o, out, rr);
    }
    if (t1 == T) { aa_[c] = aa; bb_[c] = bb; pp_[c] = pp; }
}

// Chunk length for a T-token call: about sqrt(T), a multiple of 8.
int wkv4_chunk_len(int T) {
    int L = 16;
    while (L * L < T && L < 128) L <<= 1;
    return L;
}

// ---------------------------------------------------------------------------------------
// RWKV-5 / RWKV-6.  One workgroup of 256 threads per head (N = 64).  Thread (i, q), i = value
// index 0..63, q = key quarter 0..3, keeps S[i][16q .. 16q+16) in registers for the whole call.
// Tokens are processed in slabs of TS: r, k, v, w of the slab are staged in LDS once (one
// barrier), every thread runs the TS steps on its slice reading r/k/w as wave-uniform LDS
// broadcasts, writes its partial y to LDS, and after a second barrier the four quarters are
// summed and stored coalesced.  PER_TOKEN_W: RWKV-6 (w[t][c]); otherwise RWKV-5 (w[c]).
//   y_i = sum_j r_j (u_j k_j v_i + S_ij) ;  S_ij = S_ij w_j + k_j v_i
// ---------------------------------------------------------------------------------------
constexpr int HS = 64;   // head size
constexpr int TS = 16;   // tokens per slab

// Operand forms of the fused model path:
//   IN_F16   r, k, v are fp16 (the fp16-rounded GEMM outputs, widened here) instead of fp32
//   WMODE 0  w[C] fp32, constant decay in (0,1)                         (RWKV-5)
//   WMODE 1  w[T, C] fp32, already exp(-exp(.))                          (RWKV-6 operator interface)
//   WMODE 2  w[T, C] fp16 LoRA output; decay = exp(-exp(t_decay[c] + w)) (RWKV-6 model path)
//   OUT_GN   instead of y fp32, write fp16( fp16(GroupNorm_head(y) * lnx_w + lnx_b) * gate )
//            (GroupNorm over the 64 channels of the head, eps 64e-5, biased variance; gate optional)
struct Wkv56Args {
    int T, C;
    float *state;
    int state_layout;
    const void *r, *k, *v, *w;
    const float *u, *t_decay;
    float *y;
    const float *lnx_w, *lnx_b;
    const rwkv_half *gate;
    rwkv_half *out;
    const rwkv_half *dw2;  // WMODE 3: second decay LoRA matrix, row c = ld coefficients of channel c
    int ld;                // WMODE 3: LoRA rank (multiple of 8); w = tanh(. @ D1) [T, ld] fp16
};

template <bool IN_F16, int WMODE, bool OUT_GN>
__global__ __launch_bounds__(256) void wkv56_kernel(Wkv56Args a) {
    __shared__ __align__(16) float sr[TS][HS], sk[TS][HS], sv[TS][HS], sw[TS][HS];
    __shared__ __align__(16) float su[HS];
    __shared__ float part[TS][4][HS];
    const int T = a.T, C = a.C;
    const int h = blockIdx.x;
    const int i = threadIdx.x & 63, q = threadIdx.x >> 6;
    float *S = a.state + (size_t)h * HS * HS;
    float s[16];
#pragma unroll
    for (int jj = 0; jj < 16; ++jj) {
        const int j = 16 * q + jj;
        s[jj] = a.state_layout == 0 ? S[i * HS + j] : S[j * HS + i];
    }
    float tdec = 0.f;
    if (WMODE >= 2) tdec = a.t_decay[h * HS + i];
    if (threadIdx.x < HS) {
        su[threadIdx.x] = a.u[h * HS + threadIdx.x];
        if (WMODE == 0) sw[0][threadIdx.x] = ((const float *)a.w)[h * HS + threadIdx.x];
    }
    auto ld = [&](const void *p, size_t o) -> float {
        return IN_F16 ? h2f(((const rwkv_half *)p)[o]) : ((const float *)p)[o];
    };
    for (int t0 = 0; t0 < T; t0 += TS) {
        const int nt = min(TS, T - t0);
        __syncthreads();  // previous slab fully consumed (and su / sw[0] visible)
        for (int e = threadIdx.x; e < nt * HS; e += 256) {
            const int tt = e >> 6, c = e & 63;
            const size_t o = (size_t)(t0 + tt) * C + h * HS + c;
            sr[tt][c] = ld(a.r, o); sk[tt][c] = ld(a.k, o); sv[tt][c] = ld(a.v, o);
            if (WMODE == 1) sw[tt][c] = ((const float *)a.w)[o];
            if (WMODE == 2) sw[tt][c] = expf(-expf(tdec + h2f(((const rwkv_half *)a.w)[o])));
            if (WMODE == 3) {
                // decay LoRA: the rank-ld product for this channel, rounded to fp16 like the matrix product it replaces
                const rwkv_half *wr = a.dw2 + (size_t)(h * HS + c) * a.ld;
                const rwkv_half *dv = (const rwkv_half *)a.w + (size_t)(t0 + tt) * a.ld;
                float acc = 0.f;
                for (int j8 = 0; j8 < (a.ld >> 3); ++j8)
                    acc = dot8_f16(*(const u32x4 *)(wr + 8 * j8), *(const h16x8 *)(dv + 8 * j8), acc);
                sw[tt][c] = expf(-expf(tdec + round_h(acc)));
            }
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float vi = sv[tt][i];
            const float *wrow = WMODE != 0 ? sw[tt] : sw[0];
            float y = 0.f;
#pragma unroll
            for (int jj = 0; jj < 16; jj += 4) {
                const int j = 16 * q + jj;
                const f32x4 r4 = *(const f32x4 *)&sr[tt][j];
                const f32x4 k4 = *(const f32x4 *)&sk[tt][j];
                const f32x4 w4 = *(const f32x4 *)&wrow[j];
                const f32x4 u4 = *(const f32x4 *)&su[j];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float x = k4[e] * vi;
                    y += r4[e] * (u4[e] * x + s[jj + e]);
                    s[jj + e] = s[jj + e] * w4[e] + x;
                }
            }
            part[tt][q][i] = y;
        }
        __syncthreads();
        // wave q finishes tokens q, q+4, ...: lane = channel, so the GroupNorm of a token's head is
        // a wave reduction
        for (int tt = q; tt < nt; tt += 4) {
            const int c = i;
            const float y = (part[tt][0][c] + part[tt][1][c]) + (part[tt][2][c] + part[tt][3][c]);
            const size_t o = (size_t)(t0 + tt) * C + h * HS + c;
            if (!OUT_GN) {
                a.y[o] = y;
            } else {
                const float mean = wave_sum(y) * (1.f / HS);
                const float d = y - mean;
                const float var = wave_sum(d * d) * (1.f / HS);
                float g = d * rsqrtf(var + 64e-5f) * a.lnx_w[h * HS + c] + a.lnx_b[h * HS + c];
                g = round_h(g);
                if (a.gate) g = g * h2f(a.gate[o]);
                a.out[o] = f2h(g);
            }
        }
    }
#pragma unroll
    for (int jj = 0; jj < 16; ++jj) {
        const int j = 16 * q + jj;
        if (a.state_layout == 0) S[i * HS + j] = s[jj]; else S[j * HS + i] = s[jj];
    }
}

}  // namespace

extern "C" int rwkv_wkv4_forward(int64_t B, int64_t T, int64_t C, const float *w, const float *u, const void *k,
                                 const void *v, void *y, int kv_dtype, float *aa, float *bb, float *pp,
                                 void *stream) {
    if (!w || !u || !k || !v || !y || !aa || !bb || !pp) return RWKV_E_NULL;
    if (B <= 0 || T <= 0 || C <= 0 || B > 65535 || B * T * C > ((int64_t)1 << 40)) return RWKV_E_SHAPE;
    dim3 grid((unsigned)((C + 63) / 64), (unsigned)B);
    if (kv_dtype == RWKV_DT_F32) {
        Wkv4IO<0> io{(const float *)k, (const float *)v, (float *)y, nullptr};
        hipLaunchKernelGGL(wkv4_kernel<0>, grid, dim3(64), 0, (hipStream_t)stream, (int)T, (int)C, w, u, io, aa, bb, pp);
    } else {
        return RWKV_E_DTYPE;
    }
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

// fused variant used by the model path: k, v (fp16 or fp32) and fp16 r in; y = fp16(r * fp16(wkv)).
// ---------------------------------------------------------------------------------------
// RWKV-5 / RWKV-6 over a sequence, model path.  A head's 64 value columns never interact (y_i and the
// column S[:, i] depend on v_i only), so a head is split over four workgroups of 16 value columns: 4 H
// workgroups instead of H.  Thread (value i, key group g): lane & 15 = g owns keys 4g..4g+3 of column i,
// lane >> 4 and the wave index give i.  The sum over the 16 key groups of a value is a DPP row sum in
// registers, so the token loop has no barrier and no LDS partials; r, k, w of a slab of tokens are staged
// in LDS once (two barriers per slab).  Raw y goes to an fp32 [T, C] scratch; GroupNorm and the gate need
// the whole head and run in wkv56_gn_kernel.
//   WMODE 0: w[C] fp32 constant decay (RWKV-5);  WMODE 2: fp16 LoRA output [T, C] + t_decay (RWKV-6)
// ---------------------------------------------------------------------------------------
constexpr int TS2 = 32;  // tokens per slab

template <int WMODE>
__global__ __launch_bounds__(256) void wkv56_split_kernel(Wkv56Args a) {
    __shared__ __align__(16) float sr[TS2][HS], sk[TS2][HS], sw[TS2][HS];
    __shared__ float sv[TS2][16];
    const int T = a.T, C = a.C;
    const int h = blockIdx.x >> 2, vb = blockIdx.x & 3;
    const int lane = threadIdx.x & 63, g = lane & 15;
    const int il = (threadIdx.x >> 6) * 4 + (lane >> 4);   // value column within the block of 16
    const int i = vb * 16 + il;
    // staging role: token threadIdx.x / 8 of the slab, channels 8 (threadIdx.x % 8) .. + 7 of the head.  The
    // NEXT slab is fetched into registers before the token loop of the current one, which hides the loads.
    const int stt = threadIdx.x >> 3, sp = threadIdx.x & 7, sc = sp * 8;
    float *S = a.state + (size_t)h * HS * HS;               // [key][value]
    float s[4], u4[4], wc[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int j = 4 * g + e;
        s[e] = S[j * HS + i];
        u4[e] = a.u[h * HS + j];
        wc[e] = WMODE == 0 ? ((const float *)a.w)[h * HS + j] : 0.f;
    }
    float tdec[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) tdec[e] = WMODE == 2 ? a.t_decay[h * HS + sc + e] : 0.f;
    h16x8 pr, pk, pw = {};
    h16x2 pv;
    auto fetch = [&](int t0) {
        const size_t o = (size_t)min(t0 + stt, T - 1) * C + h * HS;   // rows past the end re-read the last one
        pr = *(const h16x8 *)((const rwkv_half *)a.r + o + sc);
        pk = *(const h16x8 *)((const rwkv_half *)a.k + o + sc);
        if (WMODE == 2) pw = *(const h16x8 *)((const rwkv_half *)a.w + o + sc);
        pv = *(const h16x2 *)((const rwkv_half *)a.v + o + vb * 16 + 2 * sp);
    };
    fetch(0);
    for (int t0 = 0; t0 < T; t0 += TS2) {
        const int nt = min(TS2, T - t0);
        __syncthreads();  // previous slab fully consumed
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            f32x4 r4, k4, w4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                r4[e] = (float)pr[4 * u + e];
                k4[e] = (float)pk[4 * u + e];
                w4[e] = WMODE == 2 ? expf(-expf(tdec[4 * u + e] + (float)pw[4 * u + e])) : 0.f;
            }
            *(f32x4 *)&sr[stt][sc + 4 * u] = r4;
            *(f32x4 *)&sk[stt][sc + 4 * u] = k4;
            if (WMODE == 2) *(f32x4 *)&sw[stt][sc + 4 * u] = w4;
        }
        sv[stt][2 * sp] = (float)pv[0];
        sv[stt][2 * sp + 1] = (float)pv[1];
        __syncthreads();
        fetch(t0 + TS2);
        struct Tok { float vi; f32x4 r4, k4, w4; };
        auto ldtok = [&](int tt) {
            Tok q;
            q.vi = sv[tt][il];
            q.r4 = *(const f32x4 *)&sr[tt][4 * g];
            q.k4 = *(const f32x4 *)&sk[tt][4 * g];
            q.w4 = WMODE == 2 ? *(const f32x4 *)&sw[tt][4 * g] : f32x4{};
            return q;
        };
        // this thread's share of y for one token (before the sum over the 16 key groups), and the state update
        auto partial = [&](const Tok &q) {
            float y = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float x = q.k4[e] * q.vi;
                y += q.r4[e] * (u4[e] * x + s[e]);
                s[e] = s[e] * (WMODE == 2 ? q.w4[e] : wc[e]) + x;
            }
            return y;
        };
        auto step = [&](const Tok &q, int tt) {
            const float y = row16_sum(partial(q));
            if (g == 0) a.y[(size_t)(t0 + tt) * C + h * HS + i] = y;
        };
        // eight tokens per pass (TS2 % 8 == 0): their LDS reads are issued together, so the read latency is paid once per
        // eight, and in a full pass the eight row sums (independent of the state chain) run interleaved
        for (int tt = 0; tt < nt; tt += 8) {
            Tok q[8];
#pragma unroll
            for (int p = 0; p < 8; ++p) q[p] = ldtok(tt + p);
            if (tt + 7 < nt) {
                float y[8];
#pragma unroll
                for (int p = 0; p < 8; ++p) y[p] = partial(q[p]);
#pragma unroll
                for (int p = 0; p < 8; ++p) y[p] = row16_sum(y[p]);
                if (g == 0) {
                    float *yo = a.y + (size_t)(t0 + tt) * C + h * HS + i;
#pragma unroll
                    for (int p = 0; p < 8; ++p) yo[p * (size_t)C] = y[p];
                }
            } else {
#pragma unroll
                for (int p = 0; p < 7; ++p)
                    if (tt + p < nt) step(q[p], tt + p);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) S[(4 * g + e) * HS + i] = s[e];
}

// GroupNorm over each head's 64 outputs (eps 64e-5), affine, fp16 rounding, gate.  Four adjacent channels per lane
// (16-byte loads of y and of the affine vectors, 8-byte accesses to the gate and the output): a row of 16 lanes owns
// one head of one token, its two sums are DPP row sums; grid-stride over the T * C / 4 chunks.
__global__ __launch_bounds__(256) void wkv56_gn_kernel(int T, int C, const float *__restrict__ y,
                                                       const float *__restrict__ lnx_w, const float *__restrict__ lnx_b,
                                                       const rwkv_half *__restrict__ gate, rwkv_half *__restrict__ out) {
    const int64_t nchunk = (int64_t)T * C / 4;   // a multiple of 16: whole rows of lanes are live or idle together
    const int cpr = C / 4;
    for (int64_t i0 = (int64_t)blockIdx.x * 256; i0 < nchunk; i0 += (int64_t)gridDim.x * 256) {
        const int64_t i = i0 + threadIdx.x;
        const bool live = i < nchunk;
        const int64_t ic = live ? i : nchunk - 1;
        const int64_t t = ic / cpr;
        const int c = (int)(ic - t * cpr) * 4;
        const size_t o = (size_t)t * C + c;
        const f32x4 y4 = *(const f32x4 *)(y + o), w4 = *(const f32x4 *)(lnx_w + c), b4 = *(const f32x4 *)(lnx_b + c);
        h16x4 g4 = {};
        if (gate) g4 = *(const h16x4 *)(gate + o);
        const float mean = row16_sum((y4[0] + y4[1]) + (y4[2] + y4[3])) * (1.f / HS);
        float sq = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) { const float d = y4[e] - mean; sq += d * d; }
        const float rstd = rsqrtf(row16_sum(sq) * (1.f / HS) + 64e-5f);
        h16x4 o4;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float gq = round_h((y4[e] - mean) * rstd * w4[e] + b4[e]);
            if (gate) gq = gq * (float)g4[e];
            o4[e] = (h16)gq;
        }
        if (live) *(h16x4 *)(out + o) = o4;
    }
}


size_t wkv4_scratch_bytes(int64_t T, int64_t C) {
    if (T < 64) return 256;
    const int L = wkv4_chunk_len((int)T);
    return (size_t)((T + L - 1) / L + 1) * 3 * (size_t)C * sizeof(float);
}

template <int MODE>
static void wkv4_fused_run(int T, int C, const float *w, const float *u, Wkv4IO<MODE> io, float *aa, float *bb, float *pp,
                           float *scratch, hipStream_t st) {
    if (T >= 64 && scratch) {
        const int L = wkv4_chunk_len(T);
        const dim3 grid((unsigned)((C + 63) / 64), (unsigned)((T + L - 1) / L));
        hipLaunchKernelGGL(wkv4_chunk_summary_kernel<MODE>, grid, dim3(64), 0, st, T, C, L, w, io, aa, bb, pp, scratch);
        hipLaunchKernelGGL(wkv4_chunk_apply_kernel<MODE>, grid, dim3(64), 0, st, T, C, L, w, u, io, aa, bb, pp, scratch);
    } else {
        hipLaunchKernelGGL(wkv4_kernel<MODE>, dim3((unsigned)((C + 63) / 64), 1), dim3(64), 0, st, T, C, w, u, io, aa, bb, pp);
    }
}

int wkv4_fused_launch(int T, int C, const float *w, const float *u, const void *k, const void *v, int kv_f32,
                      const rwkv_half *r, rwkv_half *y, float *aa, float *bb, float *pp, hipStream_t st, float *scratch) {
    if (kv_f32) {
        Wkv4IO<2> io{(const float *)k, (const float *)v, y, r};
        wkv4_fused_run<2>(T, C, w, u, io, aa, bb, pp, scratch, st);
    } else {
        Wkv4IO<1> io{(const rwkv_half *)k, (const rwkv_half *)v, y, r};
        wkv4_fused_run<1>(T, C, w, u, io, aa, bb, pp, scratch, st);
    }
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

static int wkv56_launch(bool v6, int64_t B, int64_t T, int64_t C, int64_t H, float *state, int state_layout,
                        const float *r, const float *k, const float *v, const float *w, const float *u, float *y,
                        void *stream) {
    if (!state || !r || !k || !v || !w || !u || !y) return RWKV_E_NULL;
    if (B != 1 || T <= 0 || H <= 0 || C != H * HS) return RWKV_E_SHAPE;
    if (state_layout != 0 && state_layout != 1) return RWKV_E_DTYPE;
    Wkv56Args a{};
    a.T = (int)T; a.C = (int)C; a.state = state; a.state_layout = state_layout;
    a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.y = y;
    if (v6)
        hipLaunchKernelGGL((wkv56_kernel<false, 1, false>), dim3((unsigned)H), dim3(256), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL((wkv56_kernel<false, 0, false>), dim3((unsigned)H), dim3(256), 0, (hipStream_t)stream, a);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

// Model path: fp16 r, k, v; state in list layout [h][key][value]; GroupNorm (+ gate) fused; fp16 out.
// v6: w = fp16 LoRA output [T, C], t_decay fp32 [C]; v5: w = fp32 decay [C], t_decay unused.
int wkv56_fused_launch(bool v6, int T, int C, int H, float *state, const rwkv_half *r, const rwkv_half *k,
                       const rwkv_half *v, const void *w, const float *t_decay, const float *u, const float *lnx_w,
                       const float *lnx_b, const rwkv_half *gate, rwkv_half *out, hipStream_t st,
                       const rwkv_half *dw2, int ld, float *y32) {
    if (C != H * HS) return RWKV_E_SHAPE;
    Wkv56Args a{};
    a.T = T; a.C = C; a.state = state; a.state_layout = 1;
    a.r = r; a.k = k; a.v = v; a.w = w; a.u = u; a.t_decay = t_decay;
    a.lnx_w = lnx_w; a.lnx_b = lnx_b; a.gate = gate; a.out = out; a.dw2 = dw2; a.ld = ld;
    if (T >= 32 && y32) {
        // long call: four workgroups per head, raw y to the fp32 scratch, GroupNorm + gate in a second launch
        a.y = y32;
        if (v6) hipLaunchKernelGGL((wkv56_split_kernel<2>), dim3((unsigned)(4 * H)), dim3(256), 0, st, a);
        else hipLaunchKernelGGL((wkv56_split_kernel<0>), dim3((unsigned)(4 * H)), dim3(256), 0, st, a);
        hipLaunchKernelGGL(wkv56_gn_kernel, dim3((unsigned)std::min<int64_t>(((int64_t)T * C / 4 + 255) / 256, 65535)), dim3(256), 0, st,
                           T, C, y32, lnx_w, lnx_b, gate, out);
    } else if (v6 && dw2) {
        if (ld <= 0 || (ld & 7)) return RWKV_E_SHAPE;
        hipLaunchKernelGGL((wkv56_kernel<true, 3, true>), dim3((unsigned)H), dim3(256), 0, st, a);
    } else if (v6)
        hipLaunchKernelGGL((wkv56_kernel<true, 2, true>), dim3((unsigned)H), dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL((wkv56_kernel<true, 0, true>), dim3((unsigned)H), dim3(256), 0, st, a);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

extern "C" int rwkv_wkv5_forward(int64_t B, int64_t T, int64_t C, int64_t H, float *state, int state_layout,
                                 const float *r, const float *k, const float *v, const float *w, const float *u,
                                 float *y, void *stream) {
    return wkv56_launch(false, B, T, C, H, state, state_layout, r, k, v, w, u, y, stream);
}

extern "C" int rwkv_wkv6_forward(int64_t B, int64_t T, int64_t C, int64_t H, float *state, int state_layout,
                                 const float *r, const float *k, const float *v, const float *w, const float *u,
                                 float *y, void *stream) {
    return wkv56_launch(true, B, T, C, H, state, state_layout, r, k, v, w, u, y, stream);
}
