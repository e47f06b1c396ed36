// Streaming one-token kernels shared by the RWKV-4 and RWKV-5/6 one-token paths:
// the LayerNorm + token-shift + GEMV kernels and the vector GEMV kernel with its epilogues.
//
// A launch is short (3-15 us of streaming), so what matters is the chain of dependent memory
// round trips, each ~2 us while HBM is saturated.  Every kernel therefore issues ALL its
// independent loads in its first instructions -- the prologue operands (x, LayerNorm and mix
// vectors, scales), the epilogue operands of its first rows (rx, mx, state) and the first tile
// of weights -- and only then starts the reductions: one round trip instead of four.
// Each workgroup redoes the O(C) prologue (a few thousand elements served from L2) against
// hundreds of KiB of weights streamed from HBM.
#pragma once
#include "gemv_core.h"
#include "kernels.h"

namespace {

constexpr int DTHREADS = 1024;
constexpr int DWAVES = DTHREADS / 64;
constexpr float LN_EPS = 1e-5f;
constexpr int VP = 4;  // most 8-element groups per thread the vector prologue keeps in registers (N <= 32768)

// x for this step: the embedding row of the token (first layer) or the running activation.  The id comes
// from device memory (it may be the output of a sampling kernel); one outside [0, vocab) is clamped to the
// nearest valid row, so a bad id can never become an out-of-bounds read.
DEV const rwkv_half *resolve_x(const rwkv_half *x, const rwkv_half *emb, const int32_t *token, int C, int vocab) {
    return token ? emb + (size_t)min(max(*token, 0), vocab - 1) * C : x;
}

// LDS item (16 bytes = 8 halves) index of the 8-element group j8 of an activation vector.
template <bool U8>
DEV int xs_item(int j8, int nseg) { return U8 ? ((j8 & 1) * nseg + (j8 >> 1)) : j8; }

struct MatDev {
    const void *w;
    int64_t ld;
    const rwkv_half *mx, *rx, *my, *ry;
};

// Sum over the wave that only the last lane needs: the row butterfly, then the row totals travel up through
// two DPP row broadcasts, (r3 + r2) + (r1 + r0) -- the value wave_sum forms, in 6 instructions instead of 11.
DEV float wave_sum_lane63(float v) {
    v = row16_sum(v);
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, false));  // row_bcast:15
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, false));  // row_bcast:31
    return v;
}
// Sums of K values over the first `npw` waves of the workgroup (the waves that run a prologue), in two
// halves with a synchronisation between them, which the caller places: `put` by each of those waves
// before it, `get` by any wave after it.  `red` (K * DWAVES floats) must not be in use by an
// earlier reduction that other waves may still be reading (callers pass disjoint regions).  `get` reads
// one wave's partial per lane (lane l takes wave l % 16: DWAVES == 16 == one DPP row; waves >= npw count
// as zero) and finishes with a 16-lane row sum.
template <int K>
DEV void wave_sums_put(float (&v)[K], float *red) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = wave_sum_lane63(v[k]);
    if (lane == 63)
#pragma unroll
        for (int k = 0; k < K; ++k) red[k * DWAVES + wid] = v[k];
}
template <int K>
DEV void wave_sums_get(float (&v)[K], const float *red, int npw) {
    static_assert(DWAVES == 16, "one partial per lane of a DPP row");
    const int l = threadIdx.x & 15;
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = row16_sum(l < npw ? red[k * DWAVES + l] : 0.f);
}

// Hand-shake among the prologue waves of a workgroup, and from them to the other waves, through two counters
// in LDS instead of s_barrier.  A workgroup barrier completes when its LAST wave arrives, and the waves that
// stream weights arrive late: the issue of a tile load blocks while the CU's request queue is full.  With
// counters the prologue waves wait for each other only, and a streaming wave looks at the second counter
// when it needs the activation vector, after it has put its first tile in flight.
// The counters are cleared before the workgroup's first barrier.  LDS operations of one wave are performed
// in order, so a wave's partial sums and vector items are in LDS before its increment.  The spin is bounded
// so that a mistake elsewhere ends in wrong numbers, not in a wave that never exits.
constexpr int PRO_SPIN_MAX = 1 << 22;
DEV void pro_arrive(unsigned *cnt) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
DEV void pro_wait(unsigned *cnt, unsigned n) {
    for (int i = 0; i < PRO_SPIN_MAX; ++i) {
        const unsigned c = __hip_atomic_load(cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if ((unsigned)__builtin_amdgcn_readfirstlane((int)c) >= n) break;
        __builtin_amdgcn_s_sleep(1);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// fp16 element-wise helpers, one rounding per operation (no contraction into fma): what the
// reference's fp16 tensor expressions compute.  Compiled to packed fp16 instructions.
#pragma clang fp contract(off)
DEV h16x8 mul_h(h16x8 a, h16x8 b) { return a * b; }
// xx * m + prev * (1 - m)
DEV h16x8 mix_lerp(h16x8 xx, h16x8 prev, h16x8 m) {
    const h16x8 one = {(h16)1.f, (h16)1.f, (h16)1.f, (h16)1.f, (h16)1.f, (h16)1.f, (h16)1.f, (h16)1.f};
    // 1 - m as (-m) + 1 with the sign flipped on the bit pattern: the compiler turns a vector "1 - m" into scalar
    // half subtractions and re-packing (9 instructions per 2 elements instead of 2)
    const u32x4 sign = {0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
    const h16x8 negm = __builtin_bit_cast(h16x8, __builtin_bit_cast(u32x4, m) ^ sign);
    const h16x8 a = xx * m, t = negm + one, b = prev * t;
    return a + b;
}
// xx + (prev - xx) * m
DEV h16x8 mix_maa(h16x8 xx, h16x8 prev, h16x8 m) {
    const h16x8 d = prev - xx, t = d * m;
    return xx + t;
}
#pragma clang fp contract(fast)

// LayerNorm + token-shift mixes for NJ consumers, operands staged in registers.
// Requires C / 8 <= DTHREADS (C <= 8192): thread t owns elements [8t, 8t + 8).
template <bool U8, int NJ>
struct LnMixPro {
    h16x8 x, lw, lb, sx, mix[NJ], ry[NJ], my[NJ];
    bool own;

    // Absent operands are replaced by a valid pointer so that the loads of an owning thread are a
    // straight line; threads that own no elements load nothing and their (masked) arithmetic in
    // compute() runs on don't-care registers.
    DEV void load(const rwkv_half *xp, int C, const rwkv_half *ln_w, const rwkv_half *ln_b, const rwkv_half *sxp,
                  const rwkv_half *const (&mixp)[NJ], const MatDev (&mat)[NJ]) {
        own = (int)threadIdx.x < (C >> 3);
        const int j8 = threadIdx.x;
        x = lw = lb = sx = h16x8{};
#pragma unroll
        for (int j = 0; j < NJ; ++j) mix[j] = ry[j] = my[j] = h16x8{};
        if (!own) return;
        x = *(const h16x8 *)(xp + 8 * j8);
        lw = *(const h16x8 *)(ln_w + 8 * j8);
        lb = *(const h16x8 *)(ln_b + 8 * j8);
        sx = *(const h16x8 *)((sxp ? sxp : ln_w) + 8 * j8);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            mix[j] = *(const h16x8 *)((mixp[j] ? mixp[j] : ln_w) + 8 * j8);
            if (U8) {
                ry[j] = *(const h16x8 *)(mat[j].ry + 8 * j8);
                my[j] = *(const h16x8 *)(mat[j].my + 8 * j8);
            }
        }
    }

    // Run by the prologue waves only (the waves with owning threads): the waits for the operand loads sit
    // in here, so a wave that skips it never waits for the weight tile it has in flight.  The prologue
    // waves meet once in the middle (sync[0]) and report on sync[1] when their part of the vectors and
    // sums is in LDS; every wave calls finish() once sync[1] has reached the number of prologue waves.
    // red: 2 * DWAVES + 3 * NJ * DWAVES floats
    // maa_form: the RWKV-6 mixing kx = xx + (prev - xx) * m instead of kx = xx * m + prev * (1 - m)
    DEV void compute(int C, bool has_sx, const rwkv_half *const (&mixp)[NJ], h16 *const (&xs)[NJ],
                     rwkv_half *xx_out, float *red, unsigned *sync, bool maa_form = false) {
        // All threads of these waves run the arithmetic (threads that own no elements work on zeros and are
        // masked out of the LDS writes).  The prologue is bound by VALU issue (its ~10 operand vectors live
        // in two waves per SIMD), so the element-wise chain uses packed fp16 instructions, which round
        // after every operation exactly as the reference's fp16 tensor arithmetic does, and v_dot2_f32_f16
        // for the fp32 sums.
        const int npw = ((C >> 3) + 63) >> 6;
        const h16x2 ones = {(h16)1.f, (h16)1.f};
        float m[2] = {0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            const h16x2 xp = {x[e], x[e + 1]};
            m[0] = __builtin_amdgcn_fdot2(xp, ones, m[0], false);
            m[1] = __builtin_amdgcn_fdot2(xp, xp, m[1], false);
        }
        wave_sums_put<2>(m, red);
        pro_arrive(&sync[0]);
        pro_wait(&sync[0], npw);
        wave_sums_get<2>(m, red, npw);
        const float mean = m[0] / C;
        const float rstd = rsqrtf(fmaxf(m[1] / C - mean * mean, 0.f) + LN_EPS);
        const int nseg = C >> 4, j8 = threadIdx.x;
        float acc[3 * NJ];
#pragma unroll
        for (int i = 0; i < 3 * NJ; ++i) acc[i] = 0.f;
        h16x8 xx;
#pragma unroll
        for (int e = 0; e < 8; ++e) xx[e] = (h16)(((float)x[e] - mean) * rstd * (float)lw[e] + (float)lb[e]);
        const h16x8 pv = has_sx ? sx : xx;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            h16x8 kx = xx;
            if (mixp[j]) kx = maa_form ? mix_maa(xx, pv, mix[j]) : mix_lerp(xx, pv, mix[j]);
            h16x8 o = kx;
            if (U8) {
                o = mul_h(kx, ry[j]);
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const h16x2 kp = {kx[e], kx[e + 1]}, op = {o[e], o[e + 1]}, mp = {my[j][e], my[j][e + 1]};
                    acc[3 * j] = __builtin_amdgcn_fdot2(kp, ones, acc[3 * j], false);
                    acc[3 * j + 1] = __builtin_amdgcn_fdot2(op, ones, acc[3 * j + 1], false);
                    acc[3 * j + 2] = __builtin_amdgcn_fdot2(kp, mp, acc[3 * j + 2], false);
                }
            }
            if (own) ((h16x8 *)xs[j])[xs_item<U8>(j8, nseg)] = o;
        }
        if (U8) wave_sums_put<3 * NJ>(acc, red + 2 * DWAVES);
        pro_arrive(&sync[1]);   // this wave's part of the activation vectors and of the partial sums is in LDS
        // the new token-shift state, by workgroup 0 -- after the hand-shake, whose release would wait for the store
        if (own && xx_out && blockIdx.x == 0) *(h16x8 *)(xx_out + 8 * j8) = xx;
    }

    // every wave, once all prologue waves have reported
    static DEV void finish(int C, VecSums (&S)[NJ], const float *red) {
        if (!U8) return;
        float acc[3 * NJ];
        wave_sums_get<3 * NJ>(acc, red + 2 * DWAVES, ((C >> 3) + 63) >> 6);
#pragma unroll
        for (int j = 0; j < NJ; ++j) { S[j].s0 = acc[3 * j]; S[j].s1 = acc[3 * j + 1]; S[j].s2 = acc[3 * j + 2]; }
    }
};

// number of waves that hold any of the `groups` 8-element groups that threads 0..groups-1 own
DEV int pro_waves(int groups) { return (groups + 63) >> 6; }

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
//   npw:                  number of prologue waves: the first npw waves' threads hold prologue operands (PRO)
//   sync:                 two counters in LDS (PRO)
//   pro_load():           prologue waves: issue the loads of the prologue operands (called first)
//   pro_compute():        prologue waves: build the LDS activation vectors, then pro_arrive(&sync[1])
//   pro_finish():         every wave, once sync[1] == npw (reads the sums the prologue left in LDS)
//   rowf(g, k, row, xs):  weight row pointer and LDS activation vector of row k of group g
//   epi_load(g) -> E:     loads of the operands the epilogue of group g needs, as loaded (no
//                         arithmetic on them: that would wait for the loads where they are issued)
//   epi(g, dots, E):      called by one lane per group with the K reduced dot products
//
// The hardware counts outstanding loads per wave and the compiler places its waits from a static
// count of the loads issued after the one it needs; where control flow merges it must assume the
// path with the fewest.  A load under a branch that sits between a tile's loads and its use
// therefore turns "wait for this tile" into "wait for everything", and the ping-pong degenerates
// into load - wait - compute.  So every load from the first tile on is issued unconditionally
// (clamped indices instead of predicates; a batch past the end of a wave's work is a load of one
// cache line that is dropped), and the loop body is a straight line of load(next) / process(current)
// pairs with one load site per tile inside the loop.
//
// Epilogue operands travel with the tile buffers: the operands of a group batch are loaded into
// the slot of the tile that carries its second segment batch (its only one when there is one
// per group batch), and read back when its last segment batch has been reduced.
template <bool U8, int G, int K, int U, class E, bool PRO, class ProLoad, class ProCompute, class ProFinish, class RowFn,
          class EpiLoad, class EpiFn>
DEV void stream_rows(int ngroups, int nseg, int npw, unsigned *sync, ProLoad pro_load, ProCompute pro_compute,
                     ProFinish pro_finish, RowFn rowf, EpiLoad epi_load, EpiFn epi) {
    constexpr int R = G * K;
    const int lane = threadIdx.x & 63;
    // the wave index through readfirstlane: the compiler then knows that everything derived from it (row
    // ranges, batch counters, loop control) is wave-uniform and keeps it in scalar registers
    const int wave = blockIdx.x * DWAVES + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), nwaves = gridDim.x * DWAVES;
    // balanced split: every wave gets floor or ceil of ngroups / nwaves groups
    const int g0 = (int)((int64_t)wave * ngroups / nwaves), g1 = (int)((int64_t)(wave + 1) * ngroups / nwaves);
    const int glast = g1 > g0 ? g1 - 1 : min(g0, ngroups - 1);
    const int nsb = (nseg + 64 * U - 1) / (64 * U);             // segment batches per group batch
    const int nb = ((g1 - g0 + G - 1) / G) * nsb;               // batches of this wave
    const int sb_epi = nsb > 1 ? 1 : 0;                         // segment batch that carries the epilogue operands
    RowTile<U8, R, U> t0, t1;
    E e0{}, e1{};
    auto load = [&](RowTile<U8, R, U> &t, E &e, int q) {
        const bool real = q < nb;
        const int gbi = q / nsb, gb = g0 + gbi * G, sb = q - gbi * nsb;
        const uint8_t *rows[R];
        const h16 *xs_unused;
#pragma unroll
        for (int i = 0; i < G; ++i)
#pragma unroll
            for (int k = 0; k < K; ++k) rowf(min(gb + i, glast), k, rows[i * K + k], xs_unused);
        if (real && sb == sb_epi) e = epi_load(min(gb + min(lane, G - 1), glast));
        t.load(rows, sb * 64 * U, nseg, real);
    };
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    auto process = [&](const RowTile<U8, R, U> &t, int q) {
        const int gbi = q / nsb, sb = q - gbi * nsb, gb = g0 + gbi * G;
        const uint8_t *row_unused;
        const h16 *xs[R];
#pragma unroll
        for (int i = 0; i < G; ++i)
#pragma unroll
            for (int k = 0; k < K; ++k) rowf(min(gb + i, glast), k, row_unused, xs[i * K + k]);
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
                epi(gb + lane, d, ((q - (nsb - 1) + sb_epi) & 1) ? e1 : e0);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = 0.f;
        }
    };
    // Waves whose threads hold prologue operands request them, run the prologue and fetch their first tile
    // after it.  The other waves request their first tile at once, which keeps HBM busy meanwhile, and then
    // wait for the prologue's result.
    // The vector memory path of a CU returns data in request order across its waves: a prologue operand
    // requested after another wave's weight tile comes back after that tile.  The barrier puts the prologue
    // requests in front of every tile request, so the prologue can run while the first tiles are in flight
    // instead of after them (it also orders the clearing of the counters before their first use).
    // The two paths are separate code from the first instruction on (one scalar branch): the compiler's
    // waits for the prologue operands count every load of the wave down to zero, and it places them on
    // every path on which those loads may have been issued.  On a common path a wave with a tile in flight
    // waited for that tile inside the prologue, and at a workgroup barrier so did everyone else: 2 - 4 us of
    // a 6 - 18 us launch during which nothing was requested from HBM.
    // What was measured around this (7B shape, us per token): a second tile in flight before the wait
    // 1875 against 1792 (requests that cannot be issued while the CU's queue is full hold up the prologue
    // waves on the same SIMD); workgroup barriers instead of the counters 1812 against 1786; the streaming
    // waves not waiting for the operand requests at all (no first barrier) 1798 against 1784.
    if (PRO) {
        const bool pro_wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) < npw;
        if (threadIdx.x == 0) { sync[0] = 0; sync[1] = 0; }
        if (pro_wave) {
            pro_load();
            __syncthreads();
            pro_compute();
            load(t0, e0, 0);
        } else {
            __syncthreads();
            load(t0, e0, 0);
        }
        pro_wait(&sync[1], (unsigned)npw);
        pro_finish();
    } else {
        load(t0, e0, 0);
    }
    for (int q = 0; q < nb; q += 2) {
        load(t1, e1, q + 1);
        process(t0, q);
        load(t0, e0, q + 2);
        if (q + 1 < nb) process(t1, q + 1);
    }
}

// ------------------------------------------------------------------------------------------
struct AttArgs {
    const rwkv_half *x, *emb;
    const int32_t *token;
    int C, vocab;
    const rwkv_half *ln_w, *ln_b, *sx;
    rwkv_half *xx_tmp;
    const rwkv_half *mix[3];  // k, v, r
    MatDev mat[3];            // key, value, receptance
    const float *decay, *first;
    float *aa, *bb, *pp;
    rwkv_half *rwkv;          // out: r * wkv, fp16 [C]
};

struct AttEpi {
    rwkv_half rx[3], mx[3];  // as loaded; converted in the epilogue
    float u, w, aa, bb, pp;
};

template <bool U8, int G>
__global__ __launch_bounds__(DTHREADS) void att_kernel(AttArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[(2 + 9) * DWAVES];
    __shared__ unsigned sync[2];
    const int C = a.C;
    h16 *xs[3] = {(h16 *)smem, (h16 *)smem + C, (h16 *)smem + 2 * C};
    VecSums S[3];
    LnMixPro<U8, 3> pro;
    auto pro_load = [&]() {
        pro.load(resolve_x(a.x, a.emb, a.token, C, a.vocab), C, a.ln_w, a.ln_b, a.sx, a.mix, a.mat);
    };
    auto pro_compute = [&]() { pro.compute(C, a.sx != nullptr, a.mix, xs, a.xx_tmp, red, sync); };
    auto pro_finish = [&]() { LnMixPro<U8, 3>::finish(C, S, red); };
    auto rowf = [&](int c, int k, const uint8_t *&row, const h16 *&xv) {
        row = row_ptr<U8>(a.mat[k], c);
        xv = xs[k];
    };
    auto epi_load = [&](int c) {
        AttEpi e{};
        if (U8)
#pragma unroll
            for (int k = 0; k < 3; ++k) { e.rx[k] = a.mat[k].rx[c]; e.mx[k] = a.mat[k].mx[c]; }
        e.u = a.first[c]; e.w = a.decay[c];
        e.aa = a.aa[c]; e.bb = a.bb[c]; e.pp = a.pp[c];
        return e;
    };
    auto epi = [&](int c, const float (&d)[3], const AttEpi &e) {
        float k = finish<U8>(d[0], S[0], h2f(e.rx[0]), h2f(e.mx[0]));
        float v = finish<U8>(d[1], S[1], h2f(e.rx[1]), h2f(e.mx[1]));
        float r = finish<U8>(d[2], S[2], h2f(e.rx[2]), h2f(e.mx[2]));
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
    stream_rows<U8, G, 3, 2, AttEpi, true>(C, (C * (U8 ? 1 : 2)) >> 4, pro_waves(C >> 3), sync, pro_load, pro_compute, pro_finish,
                                           rowf, epi_load, epi);
}

// ------------------------------------------------------------------------------------------
enum { EPI_SIGMOID = 0, EPI_RELU_SQ = 1, EPI_LOGITS = 2, EPI_TANH = 3 };

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
    int maa_form;
};

struct ScaleEpi {
    rwkv_half rx, mx;  // as loaded
};

template <bool U8, int NJ, int G>
__global__ __launch_bounds__(DTHREADS) void lnmix_kernel(LnMixArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[(2 + 3 * NJ) * DWAVES];
    __shared__ unsigned sync[2];
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
    auto pro_compute = [&]() { pro.compute(C, a.sx != nullptr, mix, xs, a.xx_tmp, red, sync, a.maa_form != 0); };
    auto pro_finish = [&]() { LnMixPro<U8, NJ>::finish(C, S, red); };
    auto rowf = [&](int g, int, const uint8_t *&row, const h16 *&xv) {
        const int j = (NJ > 1 && g >= M0) ? 1 : 0;
        row = row_ptr<U8>(mat[j], j ? g - M0 : g);
        xv = xs[j];
    };
    auto epi_load = [&](int g) {
        const int j = (NJ > 1 && g >= M0) ? 1 : 0;
        const int m = j ? g - M0 : g;
        ScaleEpi e{};
        if (U8) { e.rx = mat[j].rx[m]; e.mx = mat[j].mx[m]; }
        return e;
    };
    auto epi = [&](int g, const float (&d)[1], const ScaleEpi &e) {
        const int j = (NJ > 1 && g >= M0) ? 1 : 0;
        const int m = j ? g - M0 : g;
        const float v = round_h(finish<U8>(d[0], S[j], h2f(e.rx), h2f(e.mx)));
        const int kind = a.epi[j];
        if (kind == EPI_LOGITS) {
            ((float *)a.out[j])[m] = v;
        } else if (kind == EPI_TANH) {
            ((rwkv_half *)a.out[j])[m] = f2h(tanhf(v));
        } else if (kind == EPI_SIGMOID) {
            ((rwkv_half *)a.out[j])[m] = f2h(sigmoidf_(v));
        } else {
            const float t = fmaxf(v, 0.f);
            ((rwkv_half *)a.out[j])[m] = f2h(t * t);
        }
    };
    stream_rows<U8, G, 1, (G >= 4 ? 1 : 2), ScaleEpi, true>(M0 + (NJ > 1 ? a.M[1] : 0), (C * (U8 ? 1 : 2)) >> 4,
                                                            pro_waves(C >> 3), sync, pro_load, pro_compute, pro_finish, rowf,
                                                            epi_load, epi);
}

// ------------------------------------------------------------------------------------------
struct VecArgs {
    const rwkv_half *vin;   // [N] fp16 input vector
    int N, M;
    MatDev mat;
    const rwkv_half *x_in, *emb;  // residual source (emb row when token != NULL)
    const int32_t *token;
    int C, vocab;
    const rwkv_half *gate;  // [M] or NULL
    rwkv_half *x_out;       // [M]
    float out_scale;
    const rwkv_half *commit_src;  // scratch xx -> state, done by workgroup 0
    rwkv_half *commit_dst;
    int act;                // VACT_*
    void *out;              // [M] fp16 (fp32 for VACT_F32) when act != VACT_RESIDUAL
};

// epilogues of vec_kernel: VACT_RESIDUAL is x_out = (x_in + gate * y) * out_scale; the others write
// act(y) to `out` (y is first rounded to fp16 except for VACT_F32, which stores the raw sum)
enum { VACT_RESIDUAL = 0, VACT_F16 = 1, VACT_SIGMOID = 2, VACT_RELU_SQ = 3, VACT_SILU = 4, VACT_TANH = 5, VACT_F32 = 6,
       VACT_LOGITS = 7 /* fp16-rounded value stored as fp32 */ };

struct VecEpi {
    rwkv_half rx, mx, xin, gate;  // as loaded
};

// The prologue is done by the first OW waves, VPN 8-element groups of the input vector per thread
// (N <= 512 * OW * VPN); the other waves already stream weights meanwhile.
template <bool U8, int U, int VPN, int OW>
__global__ __launch_bounds__(DTHREADS) void vec_kernel(VecArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[3 * DWAVES];
    __shared__ unsigned sync[2];
    const int N = a.N;
    h16 *xs = (h16 *)smem;
    VecSums S;
    h16x8 pv[VPN], pr[VPN], pm[VPN];
    auto pro_load = [&]() {
#pragma unroll
        for (int i = 0; i < VPN; ++i) {
            const int j8 = threadIdx.x + i * 64 * OW;
            if ((int)threadIdx.x < 64 * OW && j8 < (N >> 3)) {
                pv[i] = *(const h16x8 *)(a.vin + 8 * j8);
                if (U8) {
                    pr[i] = *(const h16x8 *)(a.mat.ry + 8 * j8);
                    pm[i] = *(const h16x8 *)(a.mat.my + 8 * j8);
                }
            }
        }
    };
    auto pro_compute = [&]() {
        const int nseg = N >> 4;
        float acc[3] = {0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < VPN; ++i) {
            const int j8 = threadIdx.x + i * 64 * OW;
            if ((int)threadIdx.x < 64 * OW && j8 < (N >> 3)) {
                h16x8 o = pv[i];
                if (U8) {
                    const h16x2 ones = {(h16)1.f, (h16)1.f};
                    o = mul_h(pv[i], pr[i]);
#pragma unroll
                    for (int e = 0; e < 8; e += 2) {
                        const h16x2 kp = {pv[i][e], pv[i][e + 1]}, op = {o[e], o[e + 1]}, mp = {pm[i][e], pm[i][e + 1]};
                        acc[0] = __builtin_amdgcn_fdot2(kp, ones, acc[0], false);
                        acc[1] = __builtin_amdgcn_fdot2(op, ones, acc[1], false);
                        acc[2] = __builtin_amdgcn_fdot2(kp, mp, acc[2], false);
                    }
                }
                ((h16x8 *)xs)[xs_item<U8>(j8, nseg)] = o;
            }
        }
        if (U8) wave_sums_put<3>(acc, red);
        pro_arrive(&sync[1]);
    };
    const int npw = pro_waves(min(N >> 3, 64 * OW));
    auto pro_finish = [&]() {
        if (!U8) return;
        float acc[3];
        wave_sums_get<3>(acc, red, npw);
        S.s0 = acc[0]; S.s1 = acc[1]; S.s2 = acc[2];
    };
    auto rowf = [&](int m, int, const uint8_t *&row, const h16 *&xv) {
        row = row_ptr<U8>(a.mat, m);
        xv = xs;
    };
    auto epi_load = [&](int m) {
        VecEpi e{};
        if (U8) { e.rx = a.mat.rx[m]; e.mx = a.mat.mx[m]; }
        if (a.act == VACT_RESIDUAL) e.xin = resolve_x(a.x_in, a.emb, a.token, a.C, a.vocab)[m];
        if (a.gate) e.gate = a.gate[m];
        return e;
    };
    auto epi = [&](int m, const float (&d)[1], const VecEpi &e) {
        const float y = finish<U8>(d[0], S, h2f(e.rx), h2f(e.mx));
        if (a.act == VACT_F32) { ((float *)a.out)[m] = y; return; }
        float o = round_h(y);
        if (a.act == VACT_LOGITS) { ((float *)a.out)[m] = o; return; }
        switch (a.act) {
            case VACT_RESIDUAL:
                if (a.gate) o = round_h(h2f(e.gate) * o);
                o = round_h(h2f(e.xin) + o);
                a.x_out[m] = f2h(o * a.out_scale);
                return;
            case VACT_SIGMOID: o = sigmoidf_(o); break;
            case VACT_RELU_SQ: o = fmaxf(o, 0.f); o = o * o; break;
            case VACT_SILU: o = o * sigmoidf_(o); break;
            case VACT_TANH: o = tanhf(o); break;
            default: break;
        }
        ((rwkv_half *)a.out)[m] = f2h(o);
    };
    stream_rows<U8, 1, 1, U, VecEpi, true>(a.M, (N * (U8 ? 1 : 2)) >> 4, npw, sync, pro_load, pro_compute, pro_finish, rowf, epi_load,
                                           epi);
    // the token-shift state every workgroup of the previous launch read: committed after this workgroup's
    // rows, so that the copy's load -> store dependency does not sit in front of the weight stream
    if (blockIdx.x == 0 && a.commit_dst)
        for (int j8 = threadIdx.x; j8 < (a.C >> 3); j8 += blockDim.x)
            *(u32x4 *)(a.commit_dst + 8 * j8) = *(const u32x4 *)(a.commit_src + 8 * j8);
}

// ------------------------------------------------------------------------------------------
// Several GEMVs of the same shape [N -> M] in one launch, each with its own input vector
// (RWKV-5/6 time mix: receptance, key, value and gate rows over the r/k/v/g mixes).
struct MultiVecArgs {
    int N, M, nm;                // nm matrices (<= 4)
    const rwkv_half *vin[4];     // [N] fp16 each
    MatDev mat[4];
    int act[4];                  // VACT_F16 / VACT_SILU / VACT_SIGMOID ...
    rwkv_half *out[4];           // [M] fp16 each
    const rwkv_half *commit_src; // scratch xx -> token-shift state, done by workgroup 0
    rwkv_half *commit_dst;
    int commit_n;
    // optional extra product after the NM matrices: tanh(xin @ X) for a small fp16 matrix X of xm rows [xm][N]
    // (RWKV-6: the first decay-LoRA stage), NULL = none
    const rwkv_half *xin, *xmat;
    int xm;
    rwkv_half *xout;             // [xm]
};

struct NoEpi {};

// NM input vectors of N <= 4096 elements (one 8-element group per thread of the first 8 waves).
template <bool U8, int NM>
__global__ __launch_bounds__(DTHREADS) void multi_vec_kernel(MultiVecArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[3 * NM * DWAVES];
    __shared__ unsigned sync[2];
    const int N = a.N, M = a.M;
    h16 *xs[NM];
#pragma unroll
    for (int j = 0; j < NM; ++j) xs[j] = (h16 *)smem + (size_t)j * N;
    h16 *xs_x = (h16 *)smem + (size_t)NM * N;   // input of the extra product, plain layout
    VecSums S[NM];
    h16x8 pv[NM], pr[NM], pm[NM], px = {};
    const bool own = (int)threadIdx.x < (N >> 3);
    auto pro_load = [&]() {
#pragma unroll
        for (int j = 0; j < NM; ++j) pv[j] = pr[j] = pm[j] = h16x8{};
        if (!own) return;
        px = *(const h16x8 *)((a.xin ? a.xin : a.vin[0]) + 8 * threadIdx.x);
#pragma unroll
        for (int j = 0; j < NM; ++j) {
            pv[j] = *(const h16x8 *)(a.vin[j] + 8 * threadIdx.x);
            if (U8) {
                pr[j] = *(const h16x8 *)(a.mat[j].ry + 8 * threadIdx.x);
                pm[j] = *(const h16x8 *)(a.mat[j].my + 8 * threadIdx.x);
            }
        }
    };
    auto pro_compute = [&]() {
        const int nseg = N >> 4;
        const h16x2 ones = {(h16)1.f, (h16)1.f};
        float acc[3 * NM];
#pragma unroll
        for (int i = 0; i < 3 * NM; ++i) acc[i] = 0.f;
#pragma unroll
        for (int j = 0; j < NM; ++j) {
            h16x8 o = pv[j];
            if (U8) {
                o = mul_h(pv[j], pr[j]);
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const h16x2 kp = {pv[j][e], pv[j][e + 1]}, op = {o[e], o[e + 1]}, mp = {pm[j][e], pm[j][e + 1]};
                    acc[3 * j] = __builtin_amdgcn_fdot2(kp, ones, acc[3 * j], false);
                    acc[3 * j + 1] = __builtin_amdgcn_fdot2(op, ones, acc[3 * j + 1], false);
                    acc[3 * j + 2] = __builtin_amdgcn_fdot2(kp, mp, acc[3 * j + 2], false);
                }
            }
            if (own) ((h16x8 *)xs[j])[xs_item<U8>(threadIdx.x, nseg)] = o;
        }
        if (own) ((h16x8 *)xs_x)[threadIdx.x] = px;
        if (U8) wave_sums_put<3 * NM>(acc, red);
        pro_arrive(&sync[1]);
    };
    auto pro_finish = [&]() {
        if (!U8) return;
        float acc[3 * NM];
        wave_sums_get<3 * NM>(acc, red, pro_waves(N >> 3));
#pragma unroll
        for (int j = 0; j < NM; ++j) { S[j].s0 = acc[3 * j]; S[j].s1 = acc[3 * j + 1]; S[j].s2 = acc[3 * j + 2]; }
    };
    // a group is one output index m with its NM rows (row m of every matrix), so the matrix number is a
    // compile-time constant everywhere (an array of per-matrix fields indexed at run time would go to scratch)
    struct Epi { rwkv_half rx[NM], mx[NM]; };
    auto rowf = [&](int m, int k, const uint8_t *&row, const h16 *&xv) {
        row = row_ptr<U8>(a.mat[k], m);
        xv = xs[k];
    };
    auto epi_load = [&](int m) {
        Epi e{};
        if (U8)
#pragma unroll
            for (int k = 0; k < NM; ++k) { e.rx[k] = a.mat[k].rx[m]; e.mx[k] = a.mat[k].mx[m]; }
        return e;
    };
    auto epi = [&](int m, const float (&d)[NM], const Epi &e) {
#pragma unroll
        for (int k = 0; k < NM; ++k) {
            float o = round_h(finish<U8>(d[k], S[k], h2f(e.rx[k]), h2f(e.mx[k])));
            switch (a.act[k]) {
                case VACT_SIGMOID: o = sigmoidf_(o); break;
                case VACT_RELU_SQ: o = fmaxf(o, 0.f); o = o * o; break;
                case VACT_SILU: o = o * sigmoidf_(o); break;
                case VACT_TANH: o = tanhf(o); break;
                default: break;
            }
            a.out[k][m] = f2h(o);
        }
    };
    stream_rows<U8, 1, NM, 2, Epi, true>(M, (N * (U8 ? 1 : 2)) >> 4, pro_waves(N >> 3), sync, pro_load, pro_compute, pro_finish, rowf,
                                         epi_load, epi);
    if (a.xmat) {
        auto rowf2 = [&](int g, int, const uint8_t *&row, const h16 *&xv) {
            row = (const uint8_t *)(a.xmat + (size_t)g * N);
            xv = xs_x;
        };
        auto epi_load2 = [&](int) { return NoEpi{}; };
        auto epi2 = [&](int g, const float (&d)[1], const NoEpi &) { a.xout[g] = f2h(tanhf(round_h(d[0]))); };
        stream_rows<false, 1, 1, 2, NoEpi, false>(a.xm, (N * 2) >> 4, 0, nullptr, [] {}, [] {}, [] {}, rowf2, epi_load2, epi2);
    }
    if (blockIdx.x == 0 && a.commit_dst)
        for (int j8 = threadIdx.x; j8 < (a.commit_n >> 3); j8 += blockDim.x)
            *(u32x4 *)(a.commit_dst + 8 * j8) = *(const u32x4 *)(a.commit_src + 8 * j8);
}

inline void multi_vec_launch(bool u8, const MultiVecArgs &a, int grid, hipStream_t st) {
    const size_t lds = (size_t)(a.nm + 1) * a.N * 2;
    if (a.nm == 4) {
        if (u8) hipLaunchKernelGGL((multi_vec_kernel<true, 4>), dim3(grid), dim3(DTHREADS), lds, st, a);
        else hipLaunchKernelGGL((multi_vec_kernel<false, 4>), dim3(grid), dim3(DTHREADS), lds, st, a);
    } else {
        if (u8) hipLaunchKernelGGL((multi_vec_kernel<true, 3>), dim3(grid), dim3(DTHREADS), lds, st, a);
        else hipLaunchKernelGGL((multi_vec_kernel<false, 3>), dim3(grid), dim3(DTHREADS), lds, st, a);
    }
}

// LN + token shift + two GEMVs (channel-mix receptance and key) in one launch; picks the tile depth that
// divides a wave's share of the rows.
inline void lnmix2_launch(bool u8, const LnMixArgs &a, int grid, hipStream_t st) {
    const size_t lds = 2 * (size_t)a.C * 2;
    const int per = (a.M[0] + a.M[1] + grid * DWAVES - 1) / (grid * DWAVES);
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
}

// LN + token shift + one mix + a GEMV over a FEW rows of an fp16 matrix (RWKV-6: the first LoRA product of
// the data-dependent mixes), one row per wave.
inline void lnmix1_small_launch(const LnMixArgs &a, hipStream_t st) {
    const int grid = (a.M[0] + DWAVES - 1) / DWAVES;
    hipLaunchKernelGGL((lnmix_kernel<false, 1, 1>), dim3(grid), dim3(DTHREADS), (size_t)a.C * 2, st, a);
}

// LN + token shift + one mix + a GEMV over the rows of one large matrix.
inline void lnmix1_launch(bool u8, const LnMixArgs &a, int grid, hipStream_t st) {
    const size_t lds = (size_t)a.C * 2;
    if (u8) hipLaunchKernelGGL((lnmix_kernel<true, 1, 4>), dim3(grid), dim3(DTHREADS), lds, st, a);
    else hipLaunchKernelGGL((lnmix_kernel<false, 1, 4>), dim3(grid), dim3(DTHREADS), lds, st, a);
}

// LN_out(x) @ head -> fp32 logits (fp16-rounded values) in one launch.
inline void lnhead_launch(bool u8, const rwkv_half *x, int C, const rwkv_half *ln_w, const rwkv_half *ln_b,
                          const MatDev &head, int vocab, float *logits, int grid, hipStream_t st) {
    LnMixArgs h{};
    h.x = x; h.C = C; h.ln_w = ln_w; h.ln_b = ln_b; h.sx = nullptr; h.xx_tmp = nullptr;
    h.mix[0] = nullptr; h.mat[0] = head; h.M[0] = vocab; h.epi[0] = EPI_LOGITS; h.out[0] = logits;
    const size_t lds = (size_t)C * 2;
    if (u8) hipLaunchKernelGGL((lnmix_kernel<true, 1, 4>), dim3(grid), dim3(DTHREADS), lds, st, h);
    else hipLaunchKernelGGL((lnmix_kernel<false, 1, 4>), dim3(grid), dim3(DTHREADS), lds, st, h);
}

// Launches the vector GEMV with the tile depth and prologue shape that fit N (N <= 8192 * VP).
#define RWKV_VEC_CASE(U, VPN, OW)                                                                              \
    do {                                                                                                       \
        if (u8) hipLaunchKernelGGL((vec_kernel<true, U, VPN, OW>), dim3(grid), dim3(DTHREADS), lds, st, a);    \
        else hipLaunchKernelGGL((vec_kernel<false, U, VPN, OW>), dim3(grid), dim3(DTHREADS), lds, st, a);     \
    } while (0)
inline void vec_launch(bool u8, const VecArgs &a, int grid, hipStream_t st) {
    const size_t lds = (size_t)a.N * 2;
    const int groups = a.N >> 3;
    if (groups <= 512) RWKV_VEC_CASE(4, 1, 8);
    else if (groups <= 1024) RWKV_VEC_CASE(4, 2, 8);
    else if (groups <= 2048) RWKV_VEC_CASE(8, 4, 8);
    else RWKV_VEC_CASE(8, 4, 16);
}
#undef RWKV_VEC_CASE

}  // namespace
