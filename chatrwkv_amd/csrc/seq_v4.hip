// RWKV-4 sequence mode (len(tokens) > 1): per layer
//   lnmix_seq (LN1, token shift, k/v/r mixes, ry scaling, row sums) -> 3 MFMA GEMMs (sigmoid fused for r)
//   -> WKV-4 over T (r gating fused) -> GEMM Wo (+ residual)
//   lnmix_seq (LN2, ...) -> GEMM Wr (sigmoid), GEMM Wk (relu^2) -> GEMM Wv (gate, residual, /2)
// With uint8 weights a scaling pass (mm8_prepare) sits in front of Wo; the input of Wv arrives scaled by that
// matrix's ry, with partial row sums, from the epilogue of the Wk product (long calls through the direct-to-LDS
// kernel; otherwise it has a scaling pass too).
// and LN_out + head on the last row (GEMV) or on every row (GEMM) for full_output.
#include <algorithm>
#include <cstdlib>
#include <mutex>
#include "kernels.h"

namespace {

constexpr float LN_EPS = 1e-5f;

// ids outside [0, vocab) are clamped to the nearest valid row: a bad id never becomes an out-of-bounds read
__global__ __launch_bounds__(256) void gather_emb_kernel(int T, int C, int vocab, const int32_t *__restrict__ tokens,
                                                         const rwkv_half *__restrict__ emb,
                                                         rwkv_half *__restrict__ x) {
    const int t = blockIdx.x;
    const u32x4 *src = (const u32x4 *)(emb + (size_t)min(max(tokens[t], 0), vocab - 1) * C);
    u32x4 *dst = (u32x4 *)(x + (size_t)t * C);
    for (int i = threadIdx.x; i < (C >> 3); i += blockDim.x) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void copy16_kernel(int n16, const u32x4 *__restrict__ src, u32x4 *__restrict__ dst) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}

DEV void row_stats(const rwkv_half *x, int C, float *red, float &mean, float &rstd) {
    float s = 0.f;
    for (int j8 = threadIdx.x; j8 < (C >> 3); j8 += blockDim.x) {
        const h16x8 v = *(const h16x8 *)(x + 8 * j8);
#pragma unroll
        for (int e = 0; e < 8; ++e) s += (float)v[e];
    }
    mean = block_sum(s, red) / C;
    float q = 0.f;
    for (int j8 = threadIdx.x; j8 < (C >> 3); j8 += blockDim.x) {
        const h16x8 v = *(const h16x8 *)(x + 8 * j8);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float d = (float)v[e] - mean;
            q += d * d;
        }
    }
    rstd = rsqrtf(block_sum(q, red) / C + LN_EPS);
}

// One workgroup per token row.  Row t needs LN(x[t-1]) for the token shift: it is recomputed here
// from x[t-1] (same code, same data => same bits as row t-1 computes for itself), which keeps all
// rows independent.
template <int NJ>
__global__ __launch_bounds__(256) void lnmix_seq_kernel(SeqMixArgs a) {
    __shared__ float red[32];
    const int t = blockIdx.x, C = a.C;
    const rwkv_half *x = a.x + (size_t)t * C;
    float mean, rstd, pmean = 0.f, prstd = 0.f;
    row_stats(x, C, red, mean, rstd);
    const bool shift = a.sx != nullptr;
    const rwkv_half *xp = x - C;
    if (shift && t > 0) row_stats(xp, C, red, pmean, prstd);
    float acc[2 * NJ];
#pragma unroll
    for (int i = 0; i < 2 * NJ; ++i) acc[i] = 0.f;
    for (int j8 = threadIdx.x; j8 < (C >> 3); j8 += blockDim.x) {
        const h16x8 xv = *(const h16x8 *)(x + 8 * j8);
        const h16x8 wv = *(const h16x8 *)(a.ln_w + 8 * j8);
        const h16x8 bv = *(const h16x8 *)(a.ln_b + 8 * j8);
        h16x8 xx, pv;
#pragma unroll
        for (int e = 0; e < 8; ++e) xx[e] = (h16)(((float)xv[e] - mean) * rstd * (float)wv[e] + (float)bv[e]);
        pv = xx;
        if (shift) {
            if (t > 0) {
                const h16x8 pxv = *(const h16x8 *)(xp + 8 * j8);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    pv[e] = (h16)(((float)pxv[e] - pmean) * prstd * (float)wv[e] + (float)bv[e]);
            } else {
                pv = *(const h16x8 *)(a.sx + 8 * j8);
            }
        }
        if (a.xx_last && t == a.T - 1) *(h16x8 *)(a.xx_last + 8 * j8) = xx;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            h16x8 kx = xx;
            if (a.mix[j]) {
                const h16x8 mv = *(const h16x8 *)(a.mix[j] + 8 * j8);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float m = (float)mv[e];
                    kx[e] = a.maa_form ? (h16)((float)xx[e] + (float)(h16)((float)(h16)((float)pv[e] - (float)xx[e]) * m))
                                       : (h16)((float)xx[e] * m + (float)pv[e] * (1.f - m));
                }
            }
            h16x8 o = kx;
            if (a.ry[j]) {
                const h16x8 rv = *(const h16x8 *)(a.ry[j] + 8 * j8);
                const h16x8 yv = *(const h16x8 *)(a.my[j] + 8 * j8);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float k = (float)kx[e];
                    o[e] = (h16)(k * (float)rv[e]);
                    acc[2 * j] += k;
                    acc[2 * j + 1] += k * (float)yv[e];
                }
            }
            *(h16x8 *)(a.xs[j] + (size_t)t * C + 8 * j8) = o;
        }
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        if (!a.ry[j]) continue;
        const float v0 = block_sum(acc[2 * j], red), v2 = block_sum(acc[2 * j + 1], red);
        if (threadIdx.x == 0) { a.s0[j][t] = v0; a.s2[j][t] = v2; }
    }
    // The new token-shift state is LN(x[T-1]).  Only row 0 reads the old one, so row 0's workgroup writes the new
    // one once its own reads are done (each thread overwrites exactly the chunks it has read): no second launch.
    if (a.state_out && t == 0) {
        const rwkv_half *xl = a.x + (size_t)(a.T - 1) * C;
        if (a.T > 1) row_stats(xl, C, red, mean, rstd);
        for (int j8 = threadIdx.x; j8 < (C >> 3); j8 += blockDim.x) {
            const h16x8 xv = *(const h16x8 *)(xl + 8 * j8);
            const h16x8 wv = *(const h16x8 *)(a.ln_w + 8 * j8);
            const h16x8 bv = *(const h16x8 *)(a.ln_b + 8 * j8);
            h16x8 xx;
#pragma unroll
            for (int e = 0; e < 8; ++e) xx[e] = (h16)(((float)xv[e] - mean) * rstd * (float)wv[e] + (float)bv[e]);
            *(h16x8 *)(a.state_out + 8 * j8) = xx;
        }
    }
}

__global__ __launch_bounds__(256) void ln_f32_f16_kernel(int C, const float *__restrict__ x_, const float *__restrict__ w,
                                                         const float *__restrict__ b, rwkv_half *__restrict__ y_) {
    __shared__ float red[4];
    const float *x = x_ + (size_t)blockIdx.x * C;
    rwkv_half *y = y_ + (size_t)blockIdx.x * C;
    float s = 0.f;
    for (int j = threadIdx.x; j < C; j += blockDim.x) s += x[j];
    const float mean = block_sum(s, red) / C;
    float q = 0.f;
    for (int j = threadIdx.x; j < C; j += blockDim.x) { const float d = x[j] - mean; q += d * d; }
    const float rstd = rsqrtf(block_sum(q, red) / C + LN_EPS);
    for (int j = threadIdx.x; j < C; j += blockDim.x) y[j] = f2h((x[j] - mean) * rstd * w[j] + b[j]);
}

// lnmix_seq_kernel with a short dependent chain, for C <= 2048 CH: a thread's chunks of the row, of the previous row
// and of the LayerNorm vectors are requested together at the top and kept in registers, the statistics of the two
// rows share their barriers, and so do the 2 NJ sums at the end: two global round trips and three rounds of
// barriers per workgroup instead of five and ten (and no longer chain in row 0's workgroup, which forms the new
// token-shift state).  Every value is formed by the same thread with the same
// operations in the same order as in lnmix_seq_kernel, so the two agree bit for bit.
// PRE: the mix / scale vectors too are requested at the top (3 NJ CH more registers per thread: shorter chain, fewer
// workgroups per CU -- for short calls, where a CU has one or two rows anyway).
template <int NJ, int CH, bool PRE>
__global__ __launch_bounds__(256) void lnmix_seq_fast_kernel(SeqMixArgs a) {
    __shared__ float red[4 * 2 * NJ > 12 ? 4 * 2 * NJ : 12];
    const int t = blockIdx.x, C = a.C, nch = C >> 3;
    const rwkv_half *x = a.x + (size_t)t * C;
    const bool shift = a.sx != nullptr, prev_row = shift && t > 0;
    const rwkv_half *xp = prev_row ? x - C : x;
    // Row 0's workgroup also forms the new token-shift state LN(x[T-1]): its statistics ride in the same barriers
    const bool commit = a.state_out && t == 0;
    const rwkv_half *xl = commit ? a.x + (size_t)(a.T - 1) * C : x;
    h16x8 xv[CH], pxv[CH], lv[CH], wv[CH], bv[CH], mv[PRE ? NJ : 1][CH], rv[PRE ? NJ : 1][CH], yv[PRE ? NJ : 1][CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int j8 = min((int)threadIdx.x + c * 256, nch - 1);   // chunks past the end repeat the last one (unused)
        xv[c] = *(const h16x8 *)(x + 8 * j8);
        pxv[c] = *(const h16x8 *)(xp + 8 * j8);
        lv[c] = *(const h16x8 *)(xl + 8 * j8);
        wv[c] = *(const h16x8 *)(a.ln_w + 8 * j8);
        bv[c] = *(const h16x8 *)(a.ln_b + 8 * j8);
        if constexpr (PRE) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                if (a.mix[j]) mv[j][c] = *(const h16x8 *)(a.mix[j] + 8 * j8);
                if (a.ry[j]) { rv[j][c] = *(const h16x8 *)(a.ry[j] + 8 * j8); yv[j][c] = *(const h16x8 *)(a.my[j] + 8 * j8); }
            }
        }
    }
    float st[3] = {0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < CH; ++c)
        if ((int)threadIdx.x + c * 256 < nch) {
#pragma unroll
            for (int e = 0; e < 8; ++e) { st[0] += (float)xv[c][e]; st[1] += (float)pxv[c][e]; }
            if (commit)   // the last row's statistics: only the workgroup that writes the new state needs them
#pragma unroll
                for (int e = 0; e < 8; ++e) st[2] += (float)lv[c][e];
        }
    block_sum_n<3>(st, red);
    const float mean = st[0] / C, pmean = st[1] / C, lmean = st[2] / C;
    st[0] = st[1] = st[2] = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c)
        if ((int)threadIdx.x + c * 256 < nch) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float d = (float)xv[c][e] - mean, pd = (float)pxv[c][e] - pmean;
                st[0] += d * d;
                st[1] += pd * pd;
            }
            if (commit)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float ld = (float)lv[c][e] - lmean;
                    st[2] += ld * ld;
                }
        }
    block_sum_n<3>(st, red);
    const float rstd = rsqrtf(st[0] / C + LN_EPS), prstd = rsqrtf(st[1] / C + LN_EPS), lrstd = rsqrtf(st[2] / C + LN_EPS);
    float acc[2 * NJ];
#pragma unroll
    for (int i = 0; i < 2 * NJ; ++i) acc[i] = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int j8 = threadIdx.x + c * 256;
        if (j8 >= nch) break;
        h16x8 xx, pv;
#pragma unroll
        for (int e = 0; e < 8; ++e) xx[e] = (h16)(((float)xv[c][e] - mean) * rstd * (float)wv[c][e] + (float)bv[c][e]);
        pv = xx;
        if (shift) {
            if (t > 0) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    pv[e] = (h16)(((float)pxv[c][e] - pmean) * prstd * (float)wv[c][e] + (float)bv[c][e]);
            } else {
                pv = *(const h16x8 *)(a.sx + 8 * j8);
            }
        }
        if (a.xx_last && t == a.T - 1) *(h16x8 *)(a.xx_last + 8 * j8) = xx;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            h16x8 kx = xx;
            if (a.mix[j]) {
                h16x8 m8;
                if constexpr (PRE) m8 = mv[j][c]; else m8 = *(const h16x8 *)(a.mix[j] + 8 * j8);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float m = (float)m8[e];
                    kx[e] = a.maa_form ? (h16)((float)xx[e] + (float)(h16)((float)(h16)((float)pv[e] - (float)xx[e]) * m))
                                       : (h16)((float)xx[e] * m + (float)pv[e] * (1.f - m));
                }
            }
            h16x8 o = kx;
            if (a.ry[j]) {
                h16x8 r8, y8;
                if constexpr (PRE) { r8 = rv[j][c]; y8 = yv[j][c]; }
                else { r8 = *(const h16x8 *)(a.ry[j] + 8 * j8); y8 = *(const h16x8 *)(a.my[j] + 8 * j8); }
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float k = (float)kx[e];
                    o[e] = (h16)(k * (float)r8[e]);
                    acc[2 * j] += k;
                    acc[2 * j + 1] += k * (float)y8[e];
                }
            }
            *(h16x8 *)(a.xs[j] + (size_t)t * C + 8 * j8) = o;
        }
        // Only row 0 reads the old state, so row 0's workgroup writes the new one, each thread exactly the chunk it
        // has just read: no second launch.
        if (commit) {
            h16x8 ls;
#pragma unroll
            for (int e = 0; e < 8; ++e) ls[e] = (h16)(((float)lv[c][e] - lmean) * lrstd * (float)wv[c][e] + (float)bv[c][e]);
            *(h16x8 *)(a.state_out + 8 * j8) = ls;
        }
    }
    bool any = false;
#pragma unroll
    for (int j = 0; j < NJ; ++j) any = any || a.ry[j];
    if (any) {
        block_sum_n<2 * NJ>(acc, red);
        if (threadIdx.x == 0)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                if (a.ry[j]) { a.s0[j][t] = acc[2 * j]; a.s2[j][t] = acc[2 * j + 1]; }
    }
}

}  // namespace

template <int CH, bool PRE>
static bool lnmix_seq_fast_launch(const SeqMixArgs &a, int nj, hipStream_t st) {
    const dim3 grid((unsigned)a.T), block(256);
    switch (nj) {
        case 1: hipLaunchKernelGGL((lnmix_seq_fast_kernel<1, CH, PRE>), grid, block, 0, st, a); break;
        case 2: hipLaunchKernelGGL((lnmix_seq_fast_kernel<2, CH, PRE>), grid, block, 0, st, a); break;
        case 3: hipLaunchKernelGGL((lnmix_seq_fast_kernel<3, CH, PRE>), grid, block, 0, st, a); break;
        case 4: hipLaunchKernelGGL((lnmix_seq_fast_kernel<4, CH, PRE && CH <= 2>), grid, block, 0, st, a); break;
        case 6: hipLaunchKernelGGL((lnmix_seq_fast_kernel<6, CH, PRE && CH <= 1>), grid, block, 0, st, a); break;
        default: return false;
    }
    return true;
}

int lnmix_seq_launch(const SeqMixArgs &a, int nj, hipStream_t st) {
    // rows of up to 8192 channels: the register-resident kernel (1, 2 or 4 chunks of 8 channels per thread); calls of
    // up to 512 rows also hold the mix and scale vectors in registers
    if (a.C <= 8192 && (nj == 1 || nj == 2 || nj == 3 || nj == 4 || nj == 6)) {
        const bool pre = a.T <= 512;
        if (a.C <= 2048) pre ? lnmix_seq_fast_launch<1, true>(a, nj, st) : lnmix_seq_fast_launch<1, false>(a, nj, st);
        else if (a.C <= 4096) pre ? lnmix_seq_fast_launch<2, true>(a, nj, st) : lnmix_seq_fast_launch<2, false>(a, nj, st);
        else lnmix_seq_fast_launch<4, false>(a, nj, st);
        RWKV_LAUNCH_CHECK();
        return RWKV_OK;
    }
    const dim3 grid((unsigned)a.T), block(256);
    switch (nj) {
        case 1: hipLaunchKernelGGL(lnmix_seq_kernel<1>, grid, block, 0, st, a); break;
        case 2: hipLaunchKernelGGL(lnmix_seq_kernel<2>, grid, block, 0, st, a); break;
        case 3: hipLaunchKernelGGL(lnmix_seq_kernel<3>, grid, block, 0, st, a); break;
        case 4: hipLaunchKernelGGL(lnmix_seq_kernel<4>, grid, block, 0, st, a); break;
        case 6: hipLaunchKernelGGL(lnmix_seq_kernel<6>, grid, block, 0, st, a); break;
        default: return RWKV_E_DTYPE;
    }
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

int gather_emb_launch(int64_t T, int C, int vocab, const int32_t *tokens, const rwkv_half *emb, rwkv_half *x, hipStream_t st) {
    hipLaunchKernelGGL(gather_emb_kernel, dim3((unsigned)T), dim3(256), 0, st, (int)T, C, vocab, tokens, emb, x);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

int copy_h16_launch(int n, const rwkv_half *src, rwkv_half *dst, hipStream_t st) {
    const int n16 = n >> 3;
    hipLaunchKernelGGL(copy16_kernel, dim3((n16 + 255) / 256), dim3(256), 0, st, n16, (const u32x4 *)src, (u32x4 *)dst);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

namespace {

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct SeqWs {
    rwkv_half *x, *xs[3], *r, *rwkv, *vx, *xsv, *xx_att, *xx_ffn;
    void *k, *v;       // fp16 (uint8 weights) or fp32 (fp16 weights)
    float *sums;       // 8 * T floats
    float *parts;      // partial row sums handed from one product's epilogue to the next product: 2 * T * PARTS_MAX floats
    float *splitk;     // RWKV_SPLITK_WS_BYTES of split-K scratch for the contraction kernel
    float *wkv;        // chunk summaries of the WKV scan
    size_t total;
};

// most partial sums a row can have: one per 128 columns of the channel-mix key product, one per 64 channels of WKV
int64_t parts_max(int64_t C, int64_t F) { return std::max((F + 127) / 128, (C + 63) / 64); }

SeqWs carve(void *base, int64_t T, int64_t C, int64_t F) {
    SeqWs w;
    unsigned char *p = (unsigned char *)base;
    auto take = [&](size_t bytes) { void *q = p; p += align256(bytes); return q; };
    const size_t tc = (size_t)T * C * 2, tf = (size_t)T * F * 2;
    w.x = (rwkv_half *)take(tc);
    for (int j = 0; j < 3; ++j) w.xs[j] = (rwkv_half *)take(tc);
    w.r = (rwkv_half *)take(tc);
    w.rwkv = (rwkv_half *)take(tc);
    w.k = take(2 * tc);
    w.v = take(2 * tc);
    w.vx = (rwkv_half *)take(tf);
    w.xsv = (rwkv_half *)take(tf);
    w.xx_att = (rwkv_half *)take((size_t)C * 2);
    w.xx_ffn = (rwkv_half *)take((size_t)C * 2);
    w.sums = (float *)take((size_t)T * 8 * sizeof(float));
    w.parts = (float *)take((size_t)T * 2 * parts_max(C, F) * sizeof(float));
    w.splitk = (float *)take(RWKV_SPLITK_WS_BYTES);
    w.wkv = (float *)take(wkv4_scratch_bytes(T, C));
    w.total = (size_t)(p - (unsigned char *)base);
    return w;
}

int run_gemm(const rwkv_mat &m, bool u8, int64_t T, const rwkv_half *A, const float *s0, const float *s2, void *Y,
             int64_t ldy, GemmEpi ep, hipStream_t st, float *splitk) {
    ep.splitk_ws = splitk;
    ep.splitk_bytes = RWKV_SPLITK_WS_BYTES;
    ep.mx = u8 ? m.mx : nullptr;
    ep.rx = u8 ? m.rx : nullptr;
    ep.s0 = s0;
    ep.s2 = s2;
    return gemm_launch(u8, T, m.N, m.M, A, m.N, m.w, m.ld, Y, ldy, ep, st);
}

// how run_gemm with the same arguments would be launched
GemmPlan plan_gemm(const rwkv_mat &m, bool u8, int64_t T, const rwkv_half *A, const float *s0, const float *s2, const void *Y,
                   int64_t ldy, GemmEpi ep, float *splitk) {
    ep.splitk_ws = splitk;
    ep.splitk_bytes = RWKV_SPLITK_WS_BYTES;
    ep.mx = u8 ? m.mx : nullptr;
    ep.rx = u8 ? m.rx : nullptr;
    ep.s0 = s0;
    ep.s2 = s2;
    return gemm_plan(u8, T, m.N, m.M, A, m.N, m.w, m.ld, Y, ldy, ep);
}

// RWKV_HANDOVER=0 keeps the separate scaling passes (for A/B timing)
bool handover_enabled() {
    const char *e = getenv("RWKV_HANDOVER");
    return !(e && *e == '0');
}

// Two side streams (default priority) for contractions that are independent of each other and too small
// to fill the chip alone: k / v / r of the time mix and r / k of the channel mix run side by side.
}  // namespace

namespace {
// The table of side-stream sets: one per (device, caller stream) pair, at most 32 at a time.  A set whose caller
// stream has been given back (rwkv_release_stream) is taken over, with its streams and events, by the next new pair
// on the same device.
struct SideSlot { int dev; hipStream_t caller; bool bound; SideStreams ss; };
constexpr int MAX_SIDE_SLOTS = 32;
SideSlot g_side_slots[MAX_SIDE_SLOTS];
int g_n_side_slots = 0;
std::mutex g_side_mu;
}  // namespace

SideStreams *side_streams(hipStream_t caller) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lock(g_side_mu);
    SideSlot *spare = nullptr;
    for (int i = 0; i < g_n_side_slots; ++i) {
        SideSlot &sl = g_side_slots[i];
        if (sl.dev != dev) continue;
        if (sl.bound && sl.caller == caller) return sl.ss.ok ? &sl.ss : nullptr;
        if (!sl.bound && sl.ss.ok && !spare) spare = &sl;
    }
    if (spare) {
        spare->caller = caller;
        spare->bound = true;
        return &spare->ss;
    }
    if (g_n_side_slots == MAX_SIDE_SLOTS) return nullptr;   // more caller streams than slots: those run without side streams
    SideSlot &sl = g_side_slots[g_n_side_slots++];
    sl.dev = dev;
    sl.caller = caller;
    sl.bound = true;
    SideStreams &ss = sl.ss;
    ss.ok = hipStreamCreateWithFlags(&ss.s[0], hipStreamNonBlocking) == hipSuccess &&
            hipStreamCreateWithFlags(&ss.s[1], hipStreamNonBlocking) == hipSuccess &&
            hipEventCreateWithFlags(&ss.fork, hipEventDisableTiming) == hipSuccess &&
            hipEventCreateWithFlags(&ss.join[0], hipEventDisableTiming) == hipSuccess &&
            hipEventCreateWithFlags(&ss.join[1], hipEventDisableTiming) == hipSuccess;
    return ss.ok ? &ss : nullptr;
}

extern "C" int rwkv_release_stream(void *stream) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    std::lock_guard<std::mutex> lock(g_side_mu);
    for (int i = 0; i < g_n_side_slots; ++i) {
        SideSlot &sl = g_side_slots[i];
        if (sl.dev == dev && sl.bound && sl.caller == (hipStream_t)stream) {
            sl.bound = false;
            sl.caller = nullptr;
        }
    }
    return RWKV_OK;
}

// after fork, work launched on side stream j sees everything queued on `st` so far
bool fork_streams(SideStreams *ss, hipStream_t st, int n) {
    if (hipEventRecord(ss->fork, st) != hipSuccess) return false;
    for (int j = 0; j < n; ++j)
        if (hipStreamWaitEvent(ss->s[j], ss->fork, 0) != hipSuccess) return false;
    return true;
}

// after join, work launched on `st` sees everything queued on the side streams
bool join_streams(SideStreams *ss, hipStream_t st, int n) {
    for (int j = 0; j < n; ++j) {
        if (hipEventRecord(ss->join[j], ss->s[j]) != hipSuccess) return false;
        if (hipStreamWaitEvent(st, ss->join[j], 0) != hipSuccess) return false;
    }
    return true;
}

extern "C" int rwkv_layernorm_f32_f16(int64_t T, int64_t C, const float *x, const float *w, const float *b,
                                      rwkv_half *y, void *stream) {
    if (!x || !w || !b || !y) return RWKV_E_NULL;
    if (T <= 0 || C <= 0 || T > 0x7fffffff) return RWKV_E_SHAPE;
    hipLaunchKernelGGL(ln_f32_f16_kernel, dim3((unsigned)T), dim3(256), 0, (hipStream_t)stream, (int)C, x, w, b, y);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

extern "C" size_t rwkv_v4_seq_workspace(const rwkv_v4_model *m, int64_t T, int full_output) {
    if (!m || T <= 0) return 0;
    (void)full_output;
    return carve((void *)256, T, m->n_embd, m->n_ffn).total;
}

extern "C" int rwkv_v4_forward_seq(const rwkv_v4_model *m, const rwkv_v4_layer_state *states, const int32_t *tokens,
                                   int64_t T, int full_output, float *logits, void *workspace,
                                   size_t workspace_bytes, void *stream) {
    int rc = v4_model_check(m);
    if (rc) return rc;
    int lb, le;
    if (!layer_range(m->n_layer, m->layer_begin, m->layer_end, lb, le)) return RWKV_E_SHAPE;
    const bool with_head = le == m->n_layer;
    if (!states || !tokens || (with_head && !logits) || !workspace) return RWKV_E_NULL;
    if (T <= 0 || T > (1 << 20)) return RWKV_E_SHAPE;
    if (workspace_bytes < rwkv_v4_seq_workspace(m, T, full_output) || (((uintptr_t)workspace) & 255))
        return RWKV_E_WORKSPACE;
    for (int i = lb; i < le; ++i) {
        const rwkv_v4_layer_state &s = states[i];
        if (!s.att_xx || !s.aa || !s.bb || !s.pp || !s.ffn_xx) return RWKV_E_NULL;
        if (!aligned16(s.att_xx) || !aligned16(s.ffn_xx)) return RWKV_E_LAYOUT;
    }
    hipStream_t st = (hipStream_t)stream;
    const int C = m->n_embd, F = m->n_ffn;
    SeqWs ws = carve(workspace, T, C, F);
    float *s0[3] = {ws.sums, ws.sums + 2 * T, ws.sums + 4 * T};
    float *s2[3] = {ws.sums + T, ws.sums + 3 * T, ws.sums + 5 * T};
    float *s0v = ws.sums + 6 * T, *s2v = ws.sums + 7 * T;

    if (lb == 0)
        hipLaunchKernelGGL(gather_emb_kernel, dim3((unsigned)T), dim3(256), 0, st, (int)T, C, (int)m->vocab, tokens, m->emb, ws.x);
    SideStreams *ss = T >= 256 ? side_streams(st) : nullptr;

    for (int i = lb; i < le; ++i) {
        const rwkv_v4_layer &l = m->layers[i];
        const rwkv_v4_layer_state &s = states[i];
        const bool u8 = mat_is_u8(m->weights_u8, l.att_key);
        // ---- time mix
        {
            SeqMixArgs a{};
            a.T = (int)T; a.C = C; a.x = ws.x; a.ln_w = l.ln1_w; a.ln_b = l.ln1_b; a.sx = s.att_xx;
            a.xx_last = nullptr; a.state_out = s.att_xx;
            const rwkv_half *mix[3] = {l.att_mix_k, l.att_mix_v, l.att_mix_r};
            const rwkv_mat *mt[3] = {&l.att_key, &l.att_value, &l.att_receptance};
            for (int j = 0; j < 3; ++j) {
                a.mix[j] = mix[j]; a.ry[j] = u8 ? mt[j]->ry : nullptr; a.my[j] = u8 ? mt[j]->my : nullptr;
                a.xs[j] = ws.xs[j]; a.s0[j] = s0[j]; a.s2[j] = s2[j];
            }
            if ((rc = lnmix_seq_launch(a, 3, st))) return rc;
        }
        GemmEpi e{};
        e.out_scale = 1.f;
        // k, v: uint8 weights return fp16 (widened by the consumer); fp16 weights return fp32 directly
        e.act = ACT_NONE; e.out_dtype = u8 ? RWKV_DT_F16 : RWKV_DT_F32; e.raw_f32 = u8 ? 0 : 1;
        // side by side when none of them would split K (the split-K scratch is shared)
        // long calls: every product through the direct-to-LDS kernel, one after the other (its tiles take a whole
        // CU, so products side by side on several streams gain nothing); k, v, r as one group
        const bool dma_seq = T >= 512;
        const bool group_kvr = true;       // k, v, r as one grouped launch at every length (tile size and K split by cost)
        ForkScope par(ss, st, 2, !group_kvr && (T / 128) * (C / 128) > 128);
        if (group_kvr) {
            const rwkv_half *xin[3] = {ws.xs[0], ws.xs[1], ws.xs[2]};
            const rwkv_mat *mats[3] = {&l.att_key, &l.att_value, &l.att_receptance};
            void *outs[3] = {ws.k, ws.v, ws.r};
            GemmEpi ep[3] = {e, e, e};
            e.act = ACT_SIGMOID; e.out_dtype = RWKV_DT_F16; e.raw_f32 = 0;   // receptance, and every product after it
            ep[2] = e;
            if ((rc = gemm_group_launch(u8, 3, T, C, xin, mats, outs, ep, nullptr, s0, ws.splitk, st))) return rc;
        } else {
        hipStream_t sv = par ? ss->s[0] : st, sr = par ? ss->s[1] : st;
        float *sk = par ? nullptr : ws.splitk;   // products that run side by side do not split K
        if ((rc = run_gemm(l.att_key, u8, T, ws.xs[0], s0[0], s2[0], ws.k, C, e, st, sk))) return rc;
        if ((rc = run_gemm(l.att_value, u8, T, ws.xs[1], s0[1], s2[1], ws.v, C, e, sv, sk))) return rc;
        e.act = ACT_SIGMOID; e.out_dtype = RWKV_DT_F16; e.raw_f32 = 0;
        if ((rc = run_gemm(l.att_receptance, u8, T, ws.xs[2], s0[2], s2[2], ws.r, C, e, sr, sk))) return rc;
        if (!par.join()) return (int)hipErrorUnknown;
        }
        if ((rc = wkv4_fused_launch((int)T, C, l.time_decay, l.time_first, ws.k, ws.v, u8 ? 0 : 1, ws.r, ws.rwkv, s.aa,
                                    s.bb, s.pp, st, ws.wkv)))
            return rc;
        const rwkv_half *a_out = ws.rwkv;
        if (u8) {
            if ((rc = mm8_prepare_launch(T, C, ws.rwkv, C, l.att_output.ry, l.att_output.my, ws.xs[0], s0[0], s2[0], st)))
                return rc;
            a_out = ws.xs[0];
        }
        e.act = ACT_RESIDUAL; e.res = ws.x; e.ldres = C;
        if ((rc = run_gemm(l.att_output, u8, T, a_out, s0[0], s2[0], ws.x, C, e, st, ws.splitk))) return rc;
        // ---- channel mix
        {
            SeqMixArgs a{};
            a.T = (int)T; a.C = C; a.x = ws.x; a.ln_w = l.ln2_w; a.ln_b = l.ln2_b; a.sx = s.ffn_xx;
            a.xx_last = nullptr; a.state_out = s.ffn_xx;
            const rwkv_half *mix[2] = {l.ffn_mix_r, l.ffn_mix_k};
            const rwkv_mat *mt[2] = {&l.ffn_receptance, &l.ffn_key};
            for (int j = 0; j < 2; ++j) {
                a.mix[j] = mix[j]; a.ry[j] = u8 ? mt[j]->ry : nullptr; a.my[j] = u8 ? mt[j]->my : nullptr;
                a.xs[j] = ws.xs[j]; a.s0[j] = s0[j]; a.s2[j] = s2[j];
            }
            if ((rc = lnmix_seq_launch(a, 2, st))) return rc;
        }
        e = GemmEpi{};
        e.out_scale = 1.f; e.out_dtype = RWKV_DT_F16;
        e.act = ACT_SIGMOID;
        // the receptance product beside the key product: where neither would split K, and in calls of three row tiles
        // (257 .. 384 tokens: +4 % at n_embd 4096; slower at 256 and from 385 on)
        ForkScope par2(ss, st, 1, !dma_seq && ((T / 128) * (C / 128) > 128 || ((T + 127) / 128 == 3 && C == 4096)));
        float *sk2 = par2 ? nullptr : ws.splitk;
        int vparts = 0;   // > 0: the key product hands the value product its input with this many partial sums per row
        if (T <= 128 && !(C & 127) && !(F & 127)) {
            // short calls: receptance and key in one grouped launch
            const rwkv_half *xin[2] = {ws.xs[0], ws.xs[1]};
            const rwkv_mat *mats[2] = {&l.ffn_receptance, &l.ffn_key};
            void *outs[2] = {ws.r, ws.vx};
            GemmEpi ep[2] = {e, e};
            ep[1].act = ACT_RELU_SQ;
            if ((rc = gemm_group_launch(u8, 2, T, C, xin, mats, outs, ep, nullptr, s0, ws.splitk, st))) return rc;
        } else {
        if ((rc = run_gemm(l.ffn_receptance, u8, T, ws.xs[0], s0[0], s2[0], ws.r, C, e, par2 ? ss->s[0] : st, sk2))) return rc;
        e.act = ACT_RELU_SQ;
        e.small_tiles = par2 ? 1 : 0;   // the receptance product runs beside this one
        // Where the key product runs at full depth through the direct-to-LDS kernel and the value product through that
        // kernel too, the key product's epilogue writes relu(k)^2 already scaled for the value product, with the row
        // sums as one partial sum per column tile: no scaling pass, and the unscaled [T, F] activation is never stored.
        if (u8 && handover_enabled()) {
            const GemmPlan pk = plan_gemm(l.ffn_key, true, T, ws.xs[1], s0[1], s2[1], ws.xsv, F, e, sk2);
            GemmEpi ev{};
            ev.out_scale = 1.f; ev.out_dtype = RWKV_DT_F16;
            ev.act = ACT_GATED_RESIDUAL; ev.gate = ws.r; ev.ldgate = C; ev.res = ws.x; ev.ldres = C;
            const GemmPlan pv = plan_gemm(l.ffn_value, true, T, ws.xsv, s0v, s2v, ws.x, C, ev, ws.splitk);
            const int np = pk.kind == 2 ? (F + pk.tn - 1) / pk.tn : 0;
            if (pk.kind == 2 && pk.ks == 1 && pv.kind == 2 && np > 1 && !(np & 3)) {
                vparts = np;
                e.emit_ry = l.ffn_value.ry; e.emit_my = l.ffn_value.my;
                e.emit_s0 = ws.parts; e.emit_s2 = ws.parts + (size_t)T * np;
            }
        }
        if ((rc = run_gemm(l.ffn_key, u8, T, ws.xs[1], s0[1], s2[1], vparts ? ws.xsv : ws.vx, F, e, st, sk2))) return rc;
        e.small_tiles = 0;
        e.emit_ry = e.emit_my = nullptr; e.emit_s0 = e.emit_s2 = nullptr;
        if (!par2.join()) return (int)hipErrorUnknown;
        }
        const rwkv_half *a_v = ws.vx;
        if (vparts) {
            a_v = ws.xsv;
            e.parts = vparts; e.p0 = ws.parts; e.p2 = ws.parts + (size_t)T * vparts;
        } else if (u8) {
            if ((rc = mm8_prepare_launch(T, F, ws.vx, F, l.ffn_value.ry, l.ffn_value.my, ws.xsv, s0v, s2v, st))) return rc;
            a_v = ws.xsv;
        }
        e.act = ACT_GATED_RESIDUAL; e.gate = ws.r; e.ldgate = C; e.res = ws.x; e.ldres = C;
        e.out_scale = (m->rescale_layer > 0 && (i + 1) % m->rescale_layer == 0) ? 0.5f : 1.f;
        if ((rc = run_gemm(l.ffn_value, u8, T, a_v, s0v, s2v, ws.x, C, e, st, ws.splitk))) return rc;
        RWKV_LAUNCH_CHECK();
    }
    if (!with_head) return RWKV_OK;
    if (!full_output) return v4_head_launch(m, ws.x + (size_t)(T - 1) * C, logits, st);
    const bool u8 = mat_is_u8(m->weights_u8, m->head);
    {
        SeqMixArgs a{};
        a.T = (int)T; a.C = C; a.x = ws.x; a.ln_w = m->ln_out_w; a.ln_b = m->ln_out_b; a.sx = nullptr;
        a.xx_last = nullptr; a.mix[0] = nullptr;
        a.ry[0] = u8 ? m->head.ry : nullptr; a.my[0] = u8 ? m->head.my : nullptr;
        a.xs[0] = ws.xs[0]; a.s0[0] = s0[0]; a.s2[0] = s2[0];
        if ((rc = lnmix_seq_launch(a, 1, st))) return rc;
    }
    GemmEpi e{};
    e.out_scale = 1.f; e.act = ACT_NONE; e.out_dtype = RWKV_DT_F32;
    if ((rc = run_gemm(m->head, u8, T, ws.xs[0], s0[0], s2[0], logits, m->vocab, e, st, ws.splitk))) return rc;
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}
