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
// A launch is short (3-15 us of streaming), so what matters is the chain of dependent memory
// round trips, each ~2 us while HBM is saturated.  Every kernel therefore issues ALL its
// independent loads in its first instructions -- the prologue operands (x, LayerNorm and mix
// vectors, scales), the epilogue operands of its first rows (rx, mx, state) and the first tile
// of weights -- and only then starts the reductions: one round trip instead of four.
// Each workgroup redoes the O(C) prologue (a few thousand elements served from L2) against
// hundreds of KiB of weights streamed from HBM.  The token-shift state xx is read by every
// workgroup, so its new value goes to a scratch vector and is committed to the state by
// workgroup 0 of the *next* launch.
#include "gemv_core.h"
#include "kernels.h"

namespace {

constexpr int DTHREADS = 1024;
constexpr int DWAVES = DTHREADS / 64;
constexpr float LN_EPS = 1e-5f;
constexpr int VP = 4;  // 8-element groups per thread the vector prologue keeps in registers (N <= 32768)

// x for this step: the embedding row of the token (first layer) or the running activation.
DEV const rwkv_half *resolve_x(const rwkv_half *x, const rwkv_half *emb, const int32_t *token, int C) {
    return token ? emb + (size_t)(*token) * C : x;
}

// LDS item (16 bytes = 8 halves) index of the 8-element group j8 of an activation vector.
template <bool U8>
DEV int xs_item(int j8, int nseg) { return U8 ? ((j8 & 1) * nseg + (j8 >> 1)) : j8; }

struct MatDev {
    const void *w;
    int64_t ld;
    const rwkv_half *mx, *rx, *my, *ry;
};

// Workgroup sums of K values with ONE barrier: `red` (K * DWAVES floats) must not be in use by
// an earlier reduction that other waves may still be reading (callers pass disjoint regions).
// Stage 2 reads one wave's partial per lane (lane l takes wave l % 16: DWAVES == 16 == one DPP
// row) and finishes with a 16-lane row sum.
template <int K>
DEV void block_sum_1b(float (&v)[K], float *red) {
    static_assert(DWAVES == 16, "stage 2 assumes 16 waves");
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = wave_sum(v[k]);
    if (lane == 0)
#pragma unroll
        for (int k = 0; k < K; ++k) red[k * DWAVES + wid] = v[k];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = row16_sum(red[k * DWAVES + (lane & 15)]);
}

// LayerNorm + token-shift mixes for NJ consumers, operands staged in registers.
// Requires C / 8 <= DTHREADS (C <= 8192): thread t owns elements [8t, 8t + 8).
template <bool U8, int NJ>
struct LnMixPro {
    h16x8 x, lw, lb, sx, mix[NJ], ry[NJ], my[NJ];
    bool own;

    DEV void load(const rwkv_half *xp, int C, const rwkv_half *ln_w, const rwkv_half *ln_b, const rwkv_half *sxp,
                  const rwkv_half *const (&mixp)[NJ], const MatDev (&mat)[NJ]) {
        const int j8 = threadIdx.x;
        own = j8 < (C >> 3);
        if (!own) return;
        x = *(const h16x8 *)(xp + 8 * j8);
        lw = *(const h16x8 *)(ln_w + 8 * j8);
        lb = *(const h16x8 *)(ln_b + 8 * j8);
        if (sxp) sx = *(const h16x8 *)(sxp + 8 * j8);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            if (mixp[j]) mix[j] = *(const h16x8 *)(mixp[j] + 8 * j8);
            if (U8) {
                ry[j] = *(const h16x8 *)(mat[j].ry + 8 * j8);
                my[j] = *(const h16x8 *)(mat[j].my + 8 * j8);
            }
        }
    }

    // red: 2 * DWAVES + 3 * NJ * DWAVES floats
    DEV void compute(int C, bool has_sx, const rwkv_half *const (&mixp)[NJ], h16 *const (&xs)[NJ], VecSums (&S)[NJ],
                     rwkv_half *xx_out, float *red) {
        float m[2] = {0.f, 0.f};
        if (own)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float f = (float)x[e];
                m[0] += f;
                m[1] += f * f;
            }
        block_sum_1b<2>(m, red);
        const float mean = m[0] / C;
        const float rstd = rsqrtf(fmaxf(m[1] / C - mean * mean, 0.f) + LN_EPS);
        const int nseg = C >> 4, j8 = threadIdx.x;
        float acc[3 * NJ];
#pragma unroll
        for (int i = 0; i < 3 * NJ; ++i) acc[i] = 0.f;
        if (own) {
            h16x8 xx;
#pragma unroll
            for (int e = 0; e < 8; ++e) xx[e] = (h16)(((float)x[e] - mean) * rstd * (float)lw[e] + (float)lb[e]);
            if (xx_out && blockIdx.x == 0) *(h16x8 *)(xx_out + 8 * j8) = xx;
            const h16x8 pv = has_sx ? sx : xx;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                h16x8 kx = xx;
                if (mixp[j]) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float mm = (float)mix[j][e];
                        kx[e] = (h16)((float)xx[e] * mm + (float)pv[e] * (1.f - mm));
                    }
                }
                h16x8 o = kx;
                if (U8) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float k = (float)kx[e];
                        o[e] = (h16)(k * (float)ry[j][e]);
                        acc[3 * j] += k;
                        acc[3 * j + 1] += (float)o[e];
                        acc[3 * j + 2] += k * (float)my[j][e];
                    }
                }
                ((h16x8 *)xs[j])[xs_item<U8>(j8, nseg)] = o;
            }
        }
        // one barrier publishes both the LDS activation vectors and the partial sums
        block_sum_1b<3 * NJ>(acc, red + 2 * DWAVES);
        if (U8)
#pragma unroll
            for (int j = 0; j < NJ; ++j) { S[j].s0 = acc[3 * j]; S[j].s1 = acc[3 * j + 1]; S[j].s2 = acc[3 * j + 2]; }
    }
};

template <bool U8>
DEV const uint8_t *row_ptr(const MatDev &m, int64_t row) {
    return (const uint8_t *)m.w + row * m.ld * (U8 ? 1 : 2);
}

template <bool U8>
DEV float finish(float dot, const VecSums &S, float rx, float mx) {
    return U8 ? mm8_finish(dot, S, rx, mx) : dot;
}

// Streaming body shared by the three kernels.  The row space is `ngroups` groups of K rows
// (K = 3 for the time-mix kernel: the key, value and receptance row of one channel; K = 1
// otherwise).  Every wave owns a contiguous range of groups and walks it as a flat sequence of
// batches (G groups x U segments per lane), ping-ponging between two register tiles: the loads
// of batch q+1 are in flight while batch q is multiplied.
//   pro_load():           issue the loads of the prologue operands (called first)
//   pro_compute():        build the LDS activation vectors (contains the workgroup barriers)
//   rowf(g, k, row, xs):  weight row pointer and LDS activation vector of row k of group g
//   epi_load(g) -> E:     loads of the operands the epilogue of group g needs (no dependence on
//                         the dot products: issued together with the group's first weight tile)
//   epi(g, dots, E):      called by one lane per group with the K reduced dot products
template <bool U8, int G, int K, int U, class E, class ProLoad, class ProCompute, class RowFn, class EpiLoad, class EpiFn>
DEV void stream_rows(int ngroups, int nseg, ProLoad pro_load, ProCompute pro_compute, RowFn rowf, EpiLoad epi_load,
                     EpiFn epi) {
    constexpr int R = G * K;
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * DWAVES + (threadIdx.x >> 6), nwaves = gridDim.x * DWAVES;
    const int per = (ngroups + nwaves - 1) / nwaves;
    const int g0 = min(wave * per, ngroups), g1 = min(g0 + per, ngroups);
    const int nsb = (nseg + 64 * U - 1) / (64 * U);             // segment batches per group batch
    const int nb = ((g1 - g0 + G - 1) / G) * nsb;               // batches of this wave
    RowTile<U8, R, U> t0, t1;
    E e0{}, e1{};
    // epilogue operands live in slot (group batch index & 1): they are loaded with the first
    // tile of a group batch and used after its last one, by when at most the next group batch
    // has started loading
    auto load = [&](RowTile<U8, R, U> &t, int q) {
        const int gbi = q / nsb, gb = g0 + gbi * G, sb = q % nsb;
        const uint8_t *rows[R];
        const h16 *xs_unused;
#pragma unroll
        for (int i = 0; i < G; ++i)
#pragma unroll
            for (int k = 0; k < K; ++k) rowf(min(gb + i, g1 - 1), k, rows[i * K + k], xs_unused);
        if (sb == 0 && lane < G && gb + lane < g1) {
            const E e = epi_load(gb + lane);
            if (gbi & 1) e1 = e; else e0 = e;
        }
        t.load(rows, sb * 64 * U, nseg);
    };
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    auto process = [&](const RowTile<U8, R, U> &t, int q) {
        const int gbi = q / nsb, sb = q % nsb, gb = g0 + gbi * G;
        const uint8_t *row_unused;
        const h16 *xs[R];
#pragma unroll
        for (int i = 0; i < G; ++i)
#pragma unroll
            for (int k = 0; k < K; ++k) rowf(min(gb + i, g1 - 1), k, row_unused, xs[i * K + k]);
        t.consume(xs, sb * 64 * U, nseg, acc);
        if (sb == nsb - 1) {
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
            if (lane < G && gb + lane < g1) {
                float d[K];
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    d[k] = acc[k];
#pragma unroll
                    for (int i = 1; i < G; ++i) d[k] = (lane == i) ? acc[i * K + k] : d[k];
                }
                epi(gb + lane, d, (gbi & 1) ? e1 : e0);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = 0.f;
        }
    };
    pro_load();
    if (nb > 0) load(t0, 0);
    pro_compute();
    for (int q = 0; q < nb; q += 2) {
        if (q + 1 < nb) load(t1, q + 1);
        process(t0, q);
        if (q + 1 < nb) {
            if (q + 2 < nb) load(t0, q + 2);
            process(t1, q + 1);
        }
    }
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

struct AttEpi {
    float rx[3], mx[3], u, w, aa, bb, pp;
};

template <bool U8, int G>
__global__ __launch_bounds__(DTHREADS) void att_kernel(AttArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[(2 + 9) * DWAVES];
    const int C = a.C;
    h16 *xs[3] = {(h16 *)smem, (h16 *)smem + C, (h16 *)smem + 2 * C};
    VecSums S[3];
    LnMixPro<U8, 3> pro;
    auto pro_load = [&]() {
        pro.load(resolve_x(a.x, a.emb, a.token, C), C, a.ln_w, a.ln_b, a.sx, a.mix, a.mat);
    };
    auto pro_compute = [&]() { pro.compute(C, a.sx != nullptr, a.mix, xs, S, a.xx_tmp, red); };
    auto rowf = [&](int c, int k, const uint8_t *&row, const h16 *&xv) {
        row = row_ptr<U8>(a.mat[k], c);
        xv = xs[k];
    };
    auto epi_load = [&](int c) {
        AttEpi e;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            e.rx[k] = U8 ? h2f(a.mat[k].rx[c]) : 1.f;
            e.mx[k] = U8 ? h2f(a.mat[k].mx[c]) : 0.f;
        }
        e.u = a.first[c]; e.w = a.decay[c];
        e.aa = a.aa[c]; e.bb = a.bb[c]; e.pp = a.pp[c];
        return e;
    };
    auto epi = [&](int c, const float (&d)[3], const AttEpi &e) {
        float k = finish<U8>(d[0], S[0], e.rx[0], e.mx[0]);
        float v = finish<U8>(d[1], S[1], e.rx[1], e.mx[1]);
        float r = finish<U8>(d[2], S[2], e.rx[2], e.mx[2]);
        if (U8) { k = round_h(k); v = round_h(v); }  // uint8 path returns fp16, widened again
        r = round_h(sigmoidf_(round_h(r)));
        float ww = e.u + k;
        float p = fmaxf(e.pp, ww);
        float e1 = __expf(e.pp - p), e2 = __expf(ww - p);
        const float wkv = (e1 * e.aa + e2 * v) / (e1 * e.bb + e2);
        ww = e.w + e.pp;
        p = fmaxf(ww, k);
        e1 = __expf(ww - p);
        e2 = __expf(k - p);
        a.aa[c] = e1 * e.aa + e2 * v;
        a.bb[c] = e1 * e.bb + e2;
        a.pp[c] = p;
        a.rwkv[c] = f2h(r * round_h(wkv));
    };
    stream_rows<U8, G, 3, 2, AttEpi>(C, (C * (U8 ? 1 : 2)) >> 4, pro_load, pro_compute, rowf, epi_load, epi);
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

struct ScaleEpi {
    float rx, mx;
};

template <bool U8, int NJ, int G>
__global__ __launch_bounds__(DTHREADS) void lnmix_kernel(LnMixArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[(2 + 3 * NJ) * DWAVES];
    const int C = a.C;
    h16 *xs[NJ];
    const rwkv_half *mix[NJ];
    MatDev mat[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) { xs[j] = (h16 *)smem + j * C; mix[j] = a.mix[j]; mat[j] = a.mat[j]; }
    VecSums S[NJ];
    const int M0 = a.M[0];
    LnMixPro<U8, NJ> pro;
    auto pro_load = [&]() { pro.load(a.x, C, a.ln_w, a.ln_b, a.sx, mix, mat); };
    auto pro_compute = [&]() { pro.compute(C, a.sx != nullptr, mix, xs, S, a.xx_tmp, red); };
    auto rowf = [&](int g, int, const uint8_t *&row, const h16 *&xv) {
        const int j = (NJ > 1 && g >= M0) ? 1 : 0;
        row = row_ptr<U8>(mat[j], j ? g - M0 : g);
        xv = xs[j];
    };
    auto epi_load = [&](int g) {
        const int j = (NJ > 1 && g >= M0) ? 1 : 0;
        const int m = j ? g - M0 : g;
        ScaleEpi e;
        e.rx = U8 ? h2f(mat[j].rx[m]) : 1.f;
        e.mx = U8 ? h2f(mat[j].mx[m]) : 0.f;
        return e;
    };
    auto epi = [&](int g, const float (&d)[1], const ScaleEpi &e) {
        const int j = (NJ > 1 && g >= M0) ? 1 : 0;
        const int m = j ? g - M0 : g;
        const float v = round_h(finish<U8>(d[0], S[j], e.rx, e.mx));
        const int kind = a.epi[j];
        if (kind == EPI_LOGITS) {
            ((float *)a.out[j])[m] = v;
        } else if (kind == EPI_SIGMOID) {
            ((rwkv_half *)a.out[j])[m] = f2h(sigmoidf_(v));
        } else {
            const float t = fmaxf(v, 0.f);
            ((rwkv_half *)a.out[j])[m] = f2h(t * t);
        }
    };
    stream_rows<U8, G, 1, (G >= 4 ? 1 : 2), ScaleEpi>(M0 + (NJ > 1 ? a.M[1] : 0), (C * (U8 ? 1 : 2)) >> 4, pro_load,
                                                      pro_compute, rowf, epi_load, epi);
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

struct VecEpi {
    float rx, mx, xin, gate;
};

template <bool U8, int U>
__global__ __launch_bounds__(DTHREADS) void vec_kernel(VecArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[3 * DWAVES];
    const int N = a.N;
    h16 *xs = (h16 *)smem;
    VecSums S;
    h16x8 pv[VP], pr[VP], pm[VP];
    auto pro_load = [&]() {
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            const int j8 = threadIdx.x + i * DTHREADS;
            if (j8 < (N >> 3)) {
                pv[i] = *(const h16x8 *)(a.vin + 8 * j8);
                if (U8) {
                    pr[i] = *(const h16x8 *)(a.mat.ry + 8 * j8);
                    pm[i] = *(const h16x8 *)(a.mat.my + 8 * j8);
                }
            }
        }
    };
    auto pro_compute = [&]() {
        if (blockIdx.x == 0 && a.commit_dst)
            for (int j8 = threadIdx.x; j8 < (a.C >> 3); j8 += blockDim.x)
                *(u32x4 *)(a.commit_dst + 8 * j8) = *(const u32x4 *)(a.commit_src + 8 * j8);
        const int nseg = N >> 4;
        float acc[3] = {0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            const int j8 = threadIdx.x + i * DTHREADS;
            if (j8 < (N >> 3)) {
                h16x8 o = pv[i];
                if (U8) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float k = (float)pv[i][e];
                        o[e] = (h16)(k * (float)pr[i][e]);
                        acc[0] += k;
                        acc[1] += (float)o[e];
                        acc[2] += k * (float)pm[i][e];
                    }
                }
                ((h16x8 *)xs)[xs_item<U8>(j8, nseg)] = o;
            }
        }
        block_sum_1b<3>(acc, red);  // the barrier also publishes xs
        if (U8) { S.s0 = acc[0]; S.s1 = acc[1]; S.s2 = acc[2]; }
    };
    auto rowf = [&](int m, int, const uint8_t *&row, const h16 *&xv) {
        row = row_ptr<U8>(a.mat, m);
        xv = xs;
    };
    auto epi_load = [&](int m) {
        VecEpi e;
        e.rx = U8 ? h2f(a.mat.rx[m]) : 1.f;
        e.mx = U8 ? h2f(a.mat.mx[m]) : 0.f;
        e.xin = h2f(resolve_x(a.x_in, a.emb, a.token, a.C)[m]);
        e.gate = a.gate ? h2f(a.gate[m]) : 1.f;
        return e;
    };
    auto epi = [&](int m, const float (&d)[1], const VecEpi &e) {
        float o = round_h(finish<U8>(d[0], S, e.rx, e.mx));
        if (a.gate) o = round_h(e.gate * o);
        o = round_h(e.xin + o);
        a.x_out[m] = f2h(o * a.out_scale);
    };
    stream_rows<U8, 1, 1, U, VecEpi>(a.M, (N * (U8 ? 1 : 2)) >> 4, pro_load, pro_compute, rowf, epi_load, epi);
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
    if (m->n_layer <= 0 || C <= 0 || F <= 0 || V <= 0 || (C & 63) || (F & 63) || C > 8 * DTHREADS || F > 8 * VP * DTHREADS)
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
            if (u8) hipLaunchKernelGGL((att_kernel<true, 1>), dim3(grid), dim3(DTHREADS), lds, st, a);
            else hipLaunchKernelGGL((att_kernel<false, 1>), dim3(grid), dim3(DTHREADS), lds, st, a);
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
            const int per = (C + F + grid * DWAVES - 1) / (grid * DWAVES);
            if (per % 5 == 0) {
                if (u8) hipLaunchKernelGGL((lnmix_kernel<true, 2, 5>), dim3(grid), dim3(DTHREADS), lds, st, a);
                else hipLaunchKernelGGL((lnmix_kernel<false, 2, 5>), dim3(grid), dim3(DTHREADS), lds, st, a);
            } else if (per >= 4) {
                if (u8) hipLaunchKernelGGL((lnmix_kernel<true, 2, 4>), dim3(grid), dim3(DTHREADS), lds, st, a);
                else hipLaunchKernelGGL((lnmix_kernel<false, 2, 4>), dim3(grid), dim3(DTHREADS), lds, st, a);
            } else {
                if (u8) hipLaunchKernelGGL((lnmix_kernel<true, 2, 2>), dim3(grid), dim3(DTHREADS), lds, st, a);
                else hipLaunchKernelGGL((lnmix_kernel<false, 2, 2>), dim3(grid), dim3(DTHREADS), lds, st, a);
            }
            mark();
        }
        {
            VecArgs a{};
            a.vin = ws.vx; a.N = F; a.M = C; a.mat = to_dev(l.ffn_value);
            a.x_in = ws.x; a.emb = nullptr; a.token = nullptr; a.C = C; a.gate = ws.r_ffn; a.x_out = ws.x;
            a.out_scale = (m->rescale_layer > 0 && (i + 1) % m->rescale_layer == 0) ? 0.5f : 1.f;
            a.commit_src = ws.xx_ffn; a.commit_dst = s.ffn_xx;
            const size_t lds = (size_t)F * 2;
            if (u8) hipLaunchKernelGGL((vec_kernel<true, 8>), dim3(grid), dim3(DTHREADS), lds, st, a);
            else hipLaunchKernelGGL((vec_kernel<false, 8>), dim3(grid), dim3(DTHREADS), lds, st, a);
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
