// Sampling step after the head: token ban, presence / frequency penalties, softmax, nucleus (top-p) and
// top-k filter, temperature, one draw -- all on the device, so that a generation loop needs no
// device-to-host copy of the logits and no host synchronisation per token.
//
// One workgroup of 1024 threads; thread t keeps the contiguous chunk [t E, (t + 1) E) of the vocabulary in
// registers (E <= 64, V <= 65536), so every pass below is register arithmetic plus one workgroup
// reduction.  The nucleus cut is the largest value c with sum{p >= c} >= top_p, found one bit at a time on
// the bit pattern of c (positive floats order like their bit patterns): the same set the reference keeps
// (first sorted probability whose cumulative sum reaches top_p, ties kept) up to fp32 summation order.
// The k-th largest value is found the same way on counts.  The draw is an inverse-CDF walk in index order
// for a caller-supplied uniform number.
#include "kernels.h"

namespace {

constexpr int STHREADS = 1024, SWAVES = STHREADS / 64, EMAX = 64;

struct SampleArgs {
    const float *logits;
    int V;
    float temperature, top_p;
    int top_k;
    const int32_t *ban;
    int n_ban;
    uint8_t *seen;
    float *occ;
    const float *weight;
    float presence, frequency, decay;
    const float *u;
    float *probs;
    int32_t *token;
};

// sums (and an unsigned count) over the workgroup; every thread gets the totals
DEV void block_sum2(float &a, unsigned &n, float *redf, unsigned *redu) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    a = wave_sum(a);
    float nf = wave_sum((float)n);  // counts <= 65536: exact in fp32
    __syncthreads();
    if (lane == 0) { redf[wid] = a; redu[wid] = (unsigned)nf; }
    __syncthreads();
    float ta = 0.f;
    unsigned tn = 0;
    for (int i = 0; i < SWAVES; ++i) { ta += redf[i]; tn += redu[i]; }
    a = ta;
    n = tn;
}

DEV float block_max(float v, float *redf) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) redf[wid] = v;
    __syncthreads();
    float m = redf[0];
    for (int i = 1; i < SWAVES; ++i) m = fmaxf(m, redf[i]);
    return m;
}

__global__ __launch_bounds__(STHREADS) void sample_kernel(SampleArgs a) {
    __shared__ float redf[SWAVES];
    __shared__ unsigned redu[SWAVES];
    __shared__ float scan[STHREADS];
    __shared__ unsigned pick_lo, pick_hi;
    const int V = a.V, E = (V + STHREADS - 1) / STHREADS;
    const int base = threadIdx.x * E;
    float p[EMAX];
    // ---- adjusted logits (utils.py:103-106)
#pragma unroll
    for (int e = 0; e < EMAX; ++e) {
        const int i = base + e;
        float x = -INFINITY;
        if (e < E && i < V) {
            x = a.logits[i];
            if (a.seen && a.seen[i]) x -= a.presence + a.occ[i] * a.frequency;
        }
        p[e] = x;
    }
    for (int b = 0; b < a.n_ban; ++b) {
        const int n = a.ban[b] - base;
#pragma unroll
        for (int e = 0; e < EMAX; ++e)
            if (e == n && n < E) p[e] = -INFINITY;
    }
    // ---- softmax (utils.py:59)
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < EMAX; ++e) mx = fmaxf(mx, p[e]);
    mx = block_max(mx, redf);
    float s = 0.f;
    unsigned cnt = 0;
#pragma unroll
    for (int e = 0; e < EMAX; ++e) { p[e] = (p[e] == -INFINITY) ? 0.f : expf(p[e] - mx); s += p[e]; }
    block_sum2(s, cnt, redf, redu);
    const float inv = 1.f / s;
    float pmax = 0.f, total = 0.f;
#pragma unroll
    for (int e = 0; e < EMAX; ++e) { p[e] *= inv; pmax = fmaxf(pmax, p[e]); total += p[e]; }
    pmax = block_max(pmax, redf);
    block_sum2(total, cnt, redf, redu);
    // ---- nucleus cut (utils.py:55-58, 66-69): temperature 0 means top_p 0
    float temperature = a.temperature, top_p = a.top_p;
    if (temperature == 0.f) { temperature = 1.f; top_p = 0.f; }
    float cut = pmax;  // top_p <= 0, or no cumulative sum reaches top_p: the first sorted probability
    if (top_p > 0.f && total >= top_p) {
        unsigned prefix = 0;
        for (int bit = 30; bit >= 0; --bit) {
            const unsigned cand = prefix | (1u << bit);
            const float c = __uint_as_float(cand);
            float sc = 0.f;
#pragma unroll
            for (int e = 0; e < EMAX; ++e) sc += (p[e] >= c) ? p[e] : 0.f;
            block_sum2(sc, cnt, redf, redu);
            if (sc >= top_p) prefix = cand;
        }
        cut = __uint_as_float(prefix);
    }
    // ---- top_k (utils.py:70-71): the k-th largest value
    if (a.top_k > 0 && a.top_k < V) {
        unsigned prefix = 0;
        for (int bit = 30; bit >= 0; --bit) {
            const unsigned cand = prefix | (1u << bit);
            const float c = __uint_as_float(cand);
            float dummy = 0.f;
            unsigned n = 0;
#pragma unroll
            for (int e = 0; e < EMAX; ++e) n += (p[e] >= c) ? 1u : 0u;
            block_sum2(dummy, n, redf, redu);
            if (n >= (unsigned)a.top_k) prefix = cand;
        }
        cut = fmaxf(cut, __uint_as_float(prefix));
    }
    // ---- filter, temperature (utils.py:69-73), total
    const float invt = 1.f / temperature;
    float local = 0.f;
#pragma unroll
    for (int e = 0; e < EMAX; ++e) {
        float q = (p[e] >= cut && p[e] > 0.f) ? p[e] : 0.f;
        if (temperature != 1.f && q > 0.f) q = powf(q, invt);
        p[e] = q;
        local += q;
        const int i = base + e;
        if (e < E && i < V && a.probs) a.probs[i] = q;
    }
    // ---- draw: first index whose running sum exceeds u * total
    scan[threadIdx.x] = local;
    if (threadIdx.x == 0) { pick_lo = 0xffffffffu; pick_hi = 0u; }
    __syncthreads();
    // exclusive prefix over the 1024 thread sums: every thread adds the sums before it (fixed order)
    float excl = 0.f, all = 0.f;
    for (int t = 0; t < STHREADS; ++t) {
        const float v = scan[t];
        if (t < (int)threadIdx.x) excl += v;
        all += v;
    }
    const float target = (*a.u) * all;
    float run = excl;
    unsigned first = 0xffffffffu, last = 0u;
    bool any = false;
#pragma unroll
    for (int e = 0; e < EMAX; ++e) {
        run += p[e];
        if (p[e] > 0.f) {
            last = (unsigned)(base + e);
            any = true;
            if (first == 0xffffffffu && run > target) first = (unsigned)(base + e);
        }
    }
    if (first != 0xffffffffu) atomicMin(&pick_lo, first);
    if (any) atomicMax(&pick_hi, last);
    __syncthreads();
    const unsigned tok = pick_lo != 0xffffffffu ? pick_lo : pick_hi;  // rounding at the very end: last kept entry
    if (threadIdx.x == 0) *a.token = (int32_t)tok;
    // ---- occurrence table (utils.py:112-123): decay, then add the drawn token's weight
    if (a.seen && a.occ) {
#pragma unroll
        for (int e = 0; e < EMAX; ++e) {
            const int i = base + e;
            if (e < E && i < V && a.seen[i]) {
                float o = a.occ[i] * a.decay;
                if ((unsigned)i == tok) o += a.weight ? a.weight[i] : 1.f;
                a.occ[i] = o;
            } else if (e < E && i < V && (unsigned)i == tok) {
                a.occ[i] = a.weight ? a.weight[i] : 1.f;
                a.seen[i] = 1;
            }
        }
    }
}

}  // namespace

// The temperature-0 draw without penalties or bans: the index of the largest logit, the lowest such index on
// ties (NaN entries are never chosen).  One workgroup; each thread scans a strided share of the vocabulary with
// eight loads in flight, then (value, index) pairs are reduced by wave shuffles and across the 16 waves in LDS.
template <bool F16>
__global__ __launch_bounds__(STHREADS) void greedy_kernel(const void *__restrict__ logits_, int V, int32_t *__restrict__ token) {
    const float *lf = (const float *)logits_;
    const rwkv_half *lh = (const rwkv_half *)logits_;
    __shared__ float rv[SWAVES];
    __shared__ int ri[SWAVES];
    float best = -__builtin_inff();
    int bi = 0x7fffffff;
    auto take = [&](float v, int i) {
        if (v > best || (v == best && i < bi)) { best = v; bi = i; }
    };
    for (int i0 = threadIdx.x; i0 < V; i0 += 8 * STHREADS) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = min(i0 + u * STHREADS, V - 1);
            v[u] = F16 ? h2f(lh[i]) : lf[i];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (i0 + u * STHREADS < V) take(v[u], i0 + u * STHREADS);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) take(__shfl_xor(best, o, WAVE), __shfl_xor(bi, o, WAVE));
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    if (lane == 0) { rv[wid] = best; ri[wid] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < SWAVES; ++w) take(rv[w], ri[w]);
        *token = bi == 0x7fffffff ? 0 : bi;
    }
}

extern "C" int rwkv_greedy_token(const void *logits, int dtype, int64_t V, int32_t *token, void *stream) {
    if (!logits || !token) return RWKV_E_NULL;
    if (V <= 0 || V > 0x7fffffff) return RWKV_E_SHAPE;
    if (dtype == RWKV_DT_F32) hipLaunchKernelGGL(greedy_kernel<false>, dim3(1), dim3(STHREADS), 0, (hipStream_t)stream, logits, (int)V, token);
    else if (dtype == RWKV_DT_F16) hipLaunchKernelGGL(greedy_kernel<true>, dim3(1), dim3(STHREADS), 0, (hipStream_t)stream, logits, (int)V, token);
    else return RWKV_E_DTYPE;
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

extern "C" int rwkv_sample_logits(const float *logits, int64_t V, float temperature, float top_p, int32_t top_k,
                                  const int32_t *token_ban, int32_t n_ban, uint8_t *seen, float *occurrence,
                                  const float *token_weight, float alpha_presence, float alpha_frequency,
                                  float alpha_decay, const float *u, float *probs, int32_t *token, void *stream) {
    if (!logits || !u || !token) return RWKV_E_NULL;
    if (V <= 0 || V > (int64_t)STHREADS * EMAX || n_ban < 0 || (n_ban > 0 && !token_ban)) return RWKV_E_SHAPE;
    if ((seen == nullptr) != (occurrence == nullptr)) return RWKV_E_NULL;
    if (!(temperature >= 0.f) || top_k < 0) return RWKV_E_SHAPE;
    SampleArgs a{logits, (int)V, temperature, top_p, top_k, token_ban, n_ban, seen, occurrence, token_weight,
                 alpha_presence, alpha_frequency, alpha_decay, u, probs, token};
    hipLaunchKernelGGL(sample_kernel, dim3(1), dim3(STHREADS), 0, (hipStream_t)stream, a);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}
