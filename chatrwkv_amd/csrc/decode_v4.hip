// RWKV-4 one-token step: four launches per layer plus one for the head, every elementwise
// chain folded into a streaming-GEMV prologue or epilogue.
//
//   att_kernel    LN1 + token shift + k/v/r mixes           -> rows (Wk[c], Wv[c], Wr[c]) per wave
//                 -> sigmoid, WKV step on (aa, bb, pp)[c]    -> rwkv[c] = r * wkv
//   vec_kernel    rwkv * ry                                  -> rows of Wo -> x += out
//   lnmix_kernel  LN2 + token shift + k/r mixes              -> rows of Wr (sigmoid), Wk (relu^2)
//   vec_kernel    vx * ry                                    -> rows of Wv -> x += r * out  (and x /= 2)
//   lnmix_kernel  LN_out                                     -> rows of head -> logits
//
// Weight loads do not depend on activations, so every wave issues its first batch of row
// loads, and only then are they consumed against the activation vector that the workgroup
// has meanwhile built in LDS (each workgroup redoes the O(C) prologue: a few thousand
// elements served from L2, against hundreds of KiB of weights streamed from HBM).
// The token-shift state xx is read by every workgroup, so its new value goes to a scratch
// vector and is committed to the state by workgroup 0 of the *next* launch.
#include "gemv_core.h"
#include "kernels.h"

namespace {

constexpr int DTHREADS = 1024;
constexpr int DWAVES = DTHREADS / 64;
constexpr float LN_EPS = 1e-5f;

// x for this step: the embedding row of the token (first layer) or the running activation.
DEV const rwkv_half *resolve_x(const rwkv_half *x, const rwkv_half *emb, const int32_t *token, int C) {
    return token ? emb + (size_t)(*token) * C : x;
}

// mean / rstd of x[0..C) (fp16), fp32 two-pass; C % 8 == 0.
DEV void ln_stats(const rwkv_half *x, int C, float *red, float &mean, float &rstd) {
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

// LDS item (16 bytes = 8 halves) index of the 8-element group j8 of an activation vector.
template <bool U8>
DEV int xs_item(int j8, int nseg) { return U8 ? ((j8 & 1) * nseg + (j8 >> 1)) : j8; }

struct MatDev {
    const void *w;
    int64_t ld;
    const rwkv_half *mx, *rx, *my, *ry;
};

// LN + (optional) token-shift mixes for NJ consumers; fills xs[j] (LDS) and the per-consumer
// sums.  mix[j] == nullptr means "no mixing" (the consumer sees LN(x) itself).
template <bool U8, int NJ>
DEV void ln_mix_prologue(const rwkv_half *x, int C, const rwkv_half *ln_w, const rwkv_half *ln_b,
                         const rwkv_half *sx, const rwkv_half *const (&mix)[NJ], const MatDev (&mat)[NJ],
                         h16 *const (&xs)[NJ], VecSums (&S)[NJ], rwkv_half *xx_out, float *red) {
    float mean, rstd;
    ln_stats(x, C, red, mean, rstd);
    const int nseg = C >> 4;
    float acc[3 * NJ];
#pragma unroll
    for (int i = 0; i < 3 * NJ; ++i) acc[i] = 0.f;
    for (int j8 = threadIdx.x; j8 < (C >> 3); j8 += blockDim.x) {
        const h16x8 xv = *(const h16x8 *)(x + 8 * j8);
        const h16x8 wv = *(const h16x8 *)(ln_w + 8 * j8);
        const h16x8 bv = *(const h16x8 *)(ln_b + 8 * j8);
        h16x8 xx;
#pragma unroll
        for (int e = 0; e < 8; ++e) xx[e] = (h16)(((float)xv[e] - mean) * rstd * (float)wv[e] + (float)bv[e]);
        if (xx_out && blockIdx.x == 0) *(h16x8 *)(xx_out + 8 * j8) = xx;
        h16x8 pv = xx;
        if (sx) pv = *(const h16x8 *)(sx + 8 * j8);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            h16x8 kx = xx;
            if (mix[j]) {
                const h16x8 mv = *(const h16x8 *)(mix[j] + 8 * j8);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float m = (float)mv[e];
                    kx[e] = (h16)((float)xx[e] * m + (float)pv[e] * (1.f - m));
                }
            }
            h16x8 o = kx;
            if (U8) {
                const h16x8 rv = *(const h16x8 *)(mat[j].ry + 8 * j8);
                const h16x8 yv = *(const h16x8 *)(mat[j].my + 8 * j8);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float k = (float)kx[e];
                    o[e] = (h16)(k * (float)rv[e]);
                    acc[3 * j] += k;
                    acc[3 * j + 1] += (float)o[e];
                    acc[3 * j + 2] += k * (float)yv[e];
                }
            }
            ((h16x8 *)xs[j])[xs_item<U8>(j8, nseg)] = o;
        }
    }
    if (U8) {
        block_sum_n<3 * NJ>(acc, red);
#pragma unroll
        for (int j = 0; j < NJ; ++j) { S[j].s0 = acc[3 * j]; S[j].s1 = acc[3 * j + 1]; S[j].s2 = acc[3 * j + 2]; }
    }
    __syncthreads();
}

template <bool U8, int R, int U>
DEV void rows_dot(const void *const (&rows)[R], const h16 *const (&xs)[R], int N, float (&acc)[R]) {
    if constexpr (U8) {
        const uint8_t *rr[R];
#pragma unroll
        for (int r = 0; r < R; ++r) rr[r] = (const uint8_t *)rows[r];
        wave_rows_dot_u8<R, U>(rr, xs, N >> 4, acc);
    } else {
        const h16 *rr[R];
#pragma unroll
        for (int r = 0; r < R; ++r) rr[r] = (const h16 *)rows[r];
        wave_rows_dot_f16<R, U>(rr, xs, N >> 3, acc);
    }
}

template <bool U8>
DEV const void *row_ptr(const MatDev &m, int64_t row) {
    return U8 ? (const void *)((const uint8_t *)m.w + row * m.ld) : (const void *)((const h16 *)m.w + row * m.ld);
}

template <bool U8>
DEV float finish(float dot, const VecSums &S, const MatDev &m, int row) {
    return U8 ? mm8_finish(dot, S, h2f(m.rx[row]), h2f(m.mx[row])) : dot;
}

// ------------------------------------------------------------------------------------------
struct AttArgs {
    const rwkv_half *x, *emb;
    const int32_t *token;
    int C;
    const rwkv_half *ln_w, *ln_b, *sx;
    rwkv_half *xx_tmp;
    const rwkv_half *mix[3];  // k, v, r
    MatDev mat[3];            // key, value, receptance
    const float *decay, *first;
    float *aa, *bb, *pp;
    rwkv_half *rwkv;          // out: r * wkv, fp16 [C]
};

template <bool U8>
__global__ __launch_bounds__(DTHREADS) void att_kernel(AttArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[9 * DWAVES];
    const int C = a.C;
    h16 *xs[3] = {(h16 *)smem, (h16 *)smem + C, (h16 *)smem + 2 * C};
    VecSums S[3];
    const rwkv_half *x = resolve_x(a.x, a.emb, a.token, C);
    ln_mix_prologue<U8, 3>(x, C, a.ln_w, a.ln_b, a.sx, a.mix, a.mat, xs, S, a.xx_tmp, red);

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nwaves = gridDim.x * DWAVES;
    for (int c = blockIdx.x * DWAVES + wave; c < C; c += nwaves) {
        const void *rows[3] = {row_ptr<U8>(a.mat[0], c), row_ptr<U8>(a.mat[1], c), row_ptr<U8>(a.mat[2], c)};
        const h16 *xv[3] = {xs[0], xs[1], xs[2]};
        float acc[3] = {0.f, 0.f, 0.f};
        rows_dot<U8, 3, 4>(rows, xv, C, acc);
        if (lane == 0) {
            float k = finish<U8>(acc[0], S[0], a.mat[0], c);
            float v = finish<U8>(acc[1], S[1], a.mat[1], c);
            float r = finish<U8>(acc[2], S[2], a.mat[2], c);
            if (U8) { k = round_h(k); v = round_h(v); }  // uint8 path returns fp16, widened again
            r = round_h(sigmoidf_(round_h(r)));
            const float u = a.first[c], w = a.decay[c];
            float aa = a.aa[c], bb = a.bb[c], pp = a.pp[c];
            float ww = u + k;
            float p = fmaxf(pp, ww);
            float e1 = __expf(pp - p), e2 = __expf(ww - p);
            const float wkv = (e1 * aa + e2 * v) / (e1 * bb + e2);
            ww = w + pp;
            p = fmaxf(ww, k);
            e1 = __expf(ww - p);
            e2 = __expf(k - p);
            a.aa[c] = e1 * aa + e2 * v;
            a.bb[c] = e1 * bb + e2;
            a.pp[c] = p;
            a.rwkv[c] = f2h(r * round_h(wkv));
        }
    }
}

// ------------------------------------------------------------------------------------------
enum { EPI_SIGMOID = 0, EPI_RELU_SQ = 1, EPI_LOGITS = 2 };

struct LnMixArgs {
    const rwkv_half *x;
    int C;
    const rwkv_half *ln_w, *ln_b, *sx;
    rwkv_half *xx_tmp;
    const rwkv_half *mix[2];
    MatDev mat[2];
    int M[2];
    int epi[2];
    void *out[2];
};

template <bool U8, int NJ, int R>
__global__ __launch_bounds__(DTHREADS) void lnmix_kernel(LnMixArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[3 * NJ * DWAVES];
    const int C = a.C;
    h16 *xs[NJ];
    const rwkv_half *mix[NJ];
    MatDev mat[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) { xs[j] = (h16 *)smem + j * C; mix[j] = a.mix[j]; mat[j] = a.mat[j]; }
    VecSums S[NJ];
    ln_mix_prologue<U8, NJ>(a.x, C, a.ln_w, a.ln_b, a.sx, mix, mat, xs, S, a.xx_tmp, red);

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nwaves = gridDim.x * DWAVES;
    const int g0 = (a.M[0] + R - 1) / R;
    const int gtot = g0 + (NJ > 1 ? (a.M[1] + R - 1) / R : 0);
    for (int g = blockIdx.x * DWAVES + wave; g < gtot; g += nwaves) {
        const int j = (NJ > 1 && g >= g0) ? 1 : 0;
        const int row0 = (j ? g - g0 : g) * R;
        const int M = a.M[j];
        const void *rows[R];
        const h16 *xv[R];
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            rows[r] = row_ptr<U8>(mat[j], min(row0 + r, M - 1));
            xv[r] = xs[j];
            acc[r] = 0.f;
        }
        rows_dot<U8, R, (R >= 4 ? 2 : 4)>(rows, xv, C, acc);
        if (lane < R) {
            float d = acc[0];
#pragma unroll
            for (int r = 1; r < R; ++r) d = (lane == r) ? acc[r] : d;
            const int m = row0 + lane;
            if (m < M) {
                const float v = round_h(finish<U8>(d, S[j], mat[j], m));
                const int epi = a.epi[j];
                if (epi == EPI_LOGITS) {
                    ((float *)a.out[j])[m] = v;
                } else if (epi == EPI_SIGMOID) {
                    ((rwkv_half *)a.out[j])[m] = f2h(sigmoidf_(v));
                } else {
                    const float t = fmaxf(v, 0.f);
                    ((rwkv_half *)a.out[j])[m] = f2h(t * t);
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
struct VecArgs {
    const rwkv_half *vin;   // [N] fp16 input vector
    int N, M;
    MatDev mat;
    const rwkv_half *x_in, *emb;  // residual source (emb row when token != NULL)
    const int32_t *token;
    int C;
    const rwkv_half *gate;  // [M] or NULL
    rwkv_half *x_out;       // [M]
    float out_scale;
    const rwkv_half *commit_src;  // scratch xx -> state, done by workgroup 0
    rwkv_half *commit_dst;
};

template <bool U8, int U>
__global__ __launch_bounds__(DTHREADS) void vec_kernel(VecArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[3 * DWAVES];
    const int N = a.N;
    h16 *xs = (h16 *)smem;
    if (blockIdx.x == 0 && a.commit_dst)
        for (int j8 = threadIdx.x; j8 < (a.C >> 3); j8 += blockDim.x)
            *(u32x4 *)(a.commit_dst + 8 * j8) = *(const u32x4 *)(a.commit_src + 8 * j8);
    VecSums S;
    {
        const int nseg = N >> 4;
        float acc[3] = {0.f, 0.f, 0.f};
        for (int j8 = threadIdx.x; j8 < (N >> 3); j8 += blockDim.x) {
            const h16x8 xv = *(const h16x8 *)(a.vin + 8 * j8);
            h16x8 o = xv;
            if (U8) {
                const h16x8 rv = *(const h16x8 *)(a.mat.ry + 8 * j8);
                const h16x8 yv = *(const h16x8 *)(a.mat.my + 8 * j8);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float k = (float)xv[e];
                    o[e] = (h16)(k * (float)rv[e]);
                    acc[0] += k;
                    acc[1] += (float)o[e];
                    acc[2] += k * (float)yv[e];
                }
            }
            ((h16x8 *)xs)[xs_item<U8>(j8, nseg)] = o;
        }
        if (U8) {
            block_sum_n<3>(acc, red);
            S.s0 = acc[0]; S.s1 = acc[1]; S.s2 = acc[2];
        }
        __syncthreads();
    }
    const rwkv_half *xin = resolve_x(a.x_in, a.emb, a.token, a.C);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nwaves = gridDim.x * DWAVES;
    for (int m = blockIdx.x * DWAVES + wave; m < a.M; m += nwaves) {
        const void *rows[1] = {row_ptr<U8>(a.mat, m)};
        const h16 *xv[1] = {xs};
        float acc[1] = {0.f};
        rows_dot<U8, 1, U>(rows, xv, N, acc);
        if (lane == 0) {
            float o = round_h(finish<U8>(acc[0], S, a.mat, m));
            if (a.gate) o = round_h(h2f(a.gate[m]) * o);
            o = round_h(h2f(xin[m]) + o);
            a.x_out[m] = f2h(o * a.out_scale);
        }
    }
}

int g_num_cu = 0;
}  // namespace

int num_cu() {
    if (g_num_cu == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        g_num_cu = n;
    }
    return g_num_cu;
}

namespace {

MatDev to_dev(const rwkv_mat &m) { return MatDev{m.w, m.ld, m.mx, m.rx, m.my, m.ry}; }

bool mat_ok(const rwkv_mat &m, bool u8, int64_t N, int64_t M) {
    if (!m.w || m.N != N || m.M != M || m.ld < N) return false;
    if (!aligned16(m.w)) return false;
    if (u8) {
        if (!m.mx || !m.rx || !m.my || !m.ry || (m.ld & 15)) return false;
        if (!aligned16(m.my) || !aligned16(m.ry)) return false;
    } else if (m.ld & 7) {
        return false;
    }
    return true;
}

struct OneWs {
    rwkv_half *x, *rwkv, *r_ffn, *vx, *xx_att, *xx_ffn;
};

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

int v4_model_check(const rwkv_v4_model *m) {
    if (!m || !m->layers || !m->emb || !m->ln_out_w || !m->ln_out_b) return RWKV_E_NULL;
    const int64_t C = m->n_embd, F = m->n_ffn, V = m->vocab;
    if (m->n_layer <= 0 || C <= 0 || F <= 0 || V <= 0 || (C & 63) || (F & 63) || C > 10240 || F > 32768)
        return RWKV_E_SHAPE;
    const bool u8 = m->weights_u8 != 0;
    for (int i = 0; i < m->n_layer; ++i) {
        const rwkv_v4_layer &l = m->layers[i];
        if (!l.ln1_w || !l.ln1_b || !l.ln2_w || !l.ln2_b || !l.att_mix_k || !l.att_mix_v || !l.att_mix_r ||
            !l.time_decay || !l.time_first || !l.ffn_mix_k || !l.ffn_mix_r)
            return RWKV_E_NULL;
        if (!mat_ok(l.att_key, u8, C, C) || !mat_ok(l.att_value, u8, C, C) || !mat_ok(l.att_receptance, u8, C, C) ||
            !mat_ok(l.att_output, u8, C, C) || !mat_ok(l.ffn_key, u8, C, F) || !mat_ok(l.ffn_receptance, u8, C, C) ||
            !mat_ok(l.ffn_value, u8, F, C))
            return RWKV_E_LAYOUT;
    }
    if (!mat_ok(m->head, u8, C, V)) return RWKV_E_LAYOUT;
    return RWKV_OK;
}

extern "C" size_t rwkv_v4_one_workspace(const rwkv_v4_model *m) {
    if (!m) return 0;
    return 5 * align256((size_t)m->n_embd * 2) + align256((size_t)m->n_ffn * 2);
}

// Head: LN_out(x) @ head -> fp32 logits (fp16-rounded).  Shared by the one-token and the
// sequence entry points (last token only).
int v4_head_launch(const rwkv_v4_model *m, const rwkv_half *x, float *logits, hipStream_t st) {
    const int C = m->n_embd;
    LnMixArgs h{};
    h.x = x; h.C = C; h.ln_w = m->ln_out_w; h.ln_b = m->ln_out_b; h.sx = nullptr; h.xx_tmp = nullptr;
    h.mix[0] = nullptr; h.mat[0] = to_dev(m->head); h.M[0] = m->vocab; h.epi[0] = EPI_LOGITS; h.out[0] = logits;
    const size_t lds = (size_t)C * 2;
    const int grid = num_cu();
    if (m->weights_u8)
        hipLaunchKernelGGL((lnmix_kernel<true, 1, 4>), dim3(grid), dim3(DTHREADS), lds, st, h);
    else
        hipLaunchKernelGGL((lnmix_kernel<false, 1, 4>), dim3(grid), dim3(DTHREADS), lds, st, h);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

// `ev` (optional): 4 * n_layer + 2 events; ev[0] is recorded before the first launch and
// ev[i + 1] after the i-th launch.
static int v4_one_impl(const rwkv_v4_model *m, const rwkv_v4_layer_state *states, const int32_t *token,
                       float *logits, void *workspace, size_t workspace_bytes, void *stream, hipEvent_t *ev) {
    int rc = v4_model_check(m);
    if (rc) return rc;
    if (!states || !token || !logits || !workspace) return RWKV_E_NULL;
    if (workspace_bytes < rwkv_v4_one_workspace(m) || !aligned16(workspace)) return RWKV_E_WORKSPACE;
    for (int i = 0; i < m->n_layer; ++i) {
        const rwkv_v4_layer_state &s = states[i];
        if (!s.att_xx || !s.aa || !s.bb || !s.pp || !s.ffn_xx) return RWKV_E_NULL;
        if (!aligned16(s.att_xx) || !aligned16(s.ffn_xx)) return RWKV_E_LAYOUT;
    }
    hipStream_t st = (hipStream_t)stream;
    const int C = m->n_embd, F = m->n_ffn;
    const bool u8 = m->weights_u8 != 0;
    unsigned char *p = (unsigned char *)workspace;
    OneWs ws;
    const size_t cb = align256((size_t)C * 2);
    ws.x = (rwkv_half *)p; p += cb;
    ws.rwkv = (rwkv_half *)p; p += cb;
    ws.r_ffn = (rwkv_half *)p; p += cb;
    ws.xx_att = (rwkv_half *)p; p += cb;
    ws.xx_ffn = (rwkv_half *)p; p += cb;
    ws.vx = (rwkv_half *)p;
    const int grid = num_cu();
    int nev = 0;
    auto mark = [&]() { if (ev) (void)hipEventRecord(ev[nev++], st); };
    mark();

    for (int i = 0; i < m->n_layer; ++i) {
        const rwkv_v4_layer &l = m->layers[i];
        const rwkv_v4_layer_state &s = states[i];
        const int32_t *tok = (i == 0) ? token : nullptr;
        {
            AttArgs a{};
            a.x = ws.x; a.emb = m->emb; a.token = tok; a.C = C;
            a.ln_w = l.ln1_w; a.ln_b = l.ln1_b; a.sx = s.att_xx; a.xx_tmp = ws.xx_att;
            a.mix[0] = l.att_mix_k; a.mix[1] = l.att_mix_v; a.mix[2] = l.att_mix_r;
            a.mat[0] = to_dev(l.att_key); a.mat[1] = to_dev(l.att_value); a.mat[2] = to_dev(l.att_receptance);
            a.decay = l.time_decay; a.first = l.time_first; a.aa = s.aa; a.bb = s.bb; a.pp = s.pp;
            a.rwkv = ws.rwkv;
            const size_t lds = 3 * (size_t)C * 2;
            if (u8) hipLaunchKernelGGL(att_kernel<true>, dim3(grid), dim3(DTHREADS), lds, st, a);
            else hipLaunchKernelGGL(att_kernel<false>, dim3(grid), dim3(DTHREADS), lds, st, a);
            mark();
        }
        {
            VecArgs a{};
            a.vin = ws.rwkv; a.N = C; a.M = C; a.mat = to_dev(l.att_output);
            a.x_in = ws.x; a.emb = m->emb; a.token = tok; a.C = C; a.gate = nullptr; a.x_out = ws.x;
            a.out_scale = 1.f; a.commit_src = ws.xx_att; a.commit_dst = s.att_xx;
            const size_t lds = (size_t)C * 2;
            if (u8) hipLaunchKernelGGL((vec_kernel<true, 4>), dim3(grid), dim3(DTHREADS), lds, st, a);
            else hipLaunchKernelGGL((vec_kernel<false, 4>), dim3(grid), dim3(DTHREADS), lds, st, a);
            mark();
        }
        {
            LnMixArgs a{};
            a.x = ws.x; a.C = C; a.ln_w = l.ln2_w; a.ln_b = l.ln2_b; a.sx = s.ffn_xx; a.xx_tmp = ws.xx_ffn;
            a.mix[0] = l.ffn_mix_r; a.mat[0] = to_dev(l.ffn_receptance); a.M[0] = C; a.epi[0] = EPI_SIGMOID;
            a.out[0] = ws.r_ffn;
            a.mix[1] = l.ffn_mix_k; a.mat[1] = to_dev(l.ffn_key); a.M[1] = F; a.epi[1] = EPI_RELU_SQ;
            a.out[1] = ws.vx;
            const size_t lds = 2 * (size_t)C * 2;
            if (u8) hipLaunchKernelGGL((lnmix_kernel<true, 2, 2>), dim3(grid), dim3(DTHREADS), lds, st, a);
            else hipLaunchKernelGGL((lnmix_kernel<false, 2, 2>), dim3(grid), dim3(DTHREADS), lds, st, a);
            mark();
        }
        {
            VecArgs a{};
            a.vin = ws.vx; a.N = F; a.M = C; a.mat = to_dev(l.ffn_value);
            a.x_in = ws.x; a.emb = nullptr; a.token = nullptr; a.C = C; a.gate = ws.r_ffn; a.x_out = ws.x;
            a.out_scale = (m->rescale_layer > 0 && (i + 1) % m->rescale_layer == 0) ? 0.5f : 1.f;
            a.commit_src = ws.xx_ffn; a.commit_dst = s.ffn_xx;
            const size_t lds = (size_t)F * 2;
            if (u8) hipLaunchKernelGGL((vec_kernel<true, 4>), dim3(grid), dim3(DTHREADS), lds, st, a);
            else hipLaunchKernelGGL((vec_kernel<false, 4>), dim3(grid), dim3(DTHREADS), lds, st, a);
            mark();
        }
        RWKV_LAUNCH_CHECK();
    }
    rc = v4_head_launch(m, ws.x, logits, st);
    mark();
    return rc;
}

extern "C" int rwkv_v4_forward_one(const rwkv_v4_model *m, const rwkv_v4_layer_state *states, const int32_t *token,
                                   float *logits, void *workspace, size_t workspace_bytes, void *stream) {
    return v4_one_impl(m, states, token, logits, workspace, workspace_bytes, stream, nullptr);
}

extern "C" int rwkv_v4_profile_one(const rwkv_v4_model *m, const rwkv_v4_layer_state *states, const int32_t *token,
                                   float *logits, void *workspace, size_t workspace_bytes, void *stream,
                                   float *ms, int64_t n_ms) {
    if (!m || !ms) return RWKV_E_NULL;
    const int n = 4 * m->n_layer + 1;
    if (n_ms < n) return RWKV_E_SHAPE;
    hipEvent_t *ev = new hipEvent_t[n + 1];
    int made = 0, rc = RWKV_OK;
    for (; made < n + 1; ++made)
        if (hipEventCreate(&ev[made]) != hipSuccess) { rc = (int)hipErrorOutOfMemory; break; }
    if (rc == RWKV_OK) rc = v4_one_impl(m, states, token, logits, workspace, workspace_bytes, stream, ev);
    if (rc == RWKV_OK) {
        hipError_t e = hipEventSynchronize(ev[n]);
        if (e != hipSuccess) rc = (int)e;
        for (int i = 0; i < n && rc == RWKV_OK; ++i)
            if (hipEventElapsedTime(&ms[i], ev[i], ev[i + 1]) != hipSuccess) rc = (int)hipErrorInvalidValue;
    }
    for (int i = 0; i < made; ++i) (void)hipEventDestroy(ev[i]);
    delete[] ev;
    return rc;
}
