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
#include "decode_kernels.h"
#include "../../include/rwkv_hip_bench.h"

namespace {

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
    if (m->weights_u8 < 0 || m->weights_u8 > 2) return RWKV_E_DTYPE;
    for (int i = 0; i < m->n_layer; ++i) {
        const rwkv_v4_layer &l = m->layers[i];
        const bool u8 = mat_is_u8(m->weights_u8, l.att_key);   // one weight type per layer
        if (!l.ln1_w || !l.ln1_b || !l.ln2_w || !l.ln2_b || !l.att_mix_k || !l.att_mix_v || !l.att_mix_r ||
            !l.time_decay || !l.time_first || !l.ffn_mix_k || !l.ffn_mix_r)
            return RWKV_E_NULL;
        if (!mat_ok(l.att_key, u8, C, C) || !mat_ok(l.att_value, u8, C, C) || !mat_ok(l.att_receptance, u8, C, C) ||
            !mat_ok(l.att_output, u8, C, C) || !mat_ok(l.ffn_key, u8, C, F) || !mat_ok(l.ffn_receptance, u8, C, C) ||
            !mat_ok(l.ffn_value, u8, F, C))
            return RWKV_E_LAYOUT;
    }
    if (!mat_ok(m->head, mat_is_u8(m->weights_u8, m->head), C, V)) return RWKV_E_LAYOUT;
    return RWKV_OK;
}

extern "C" size_t rwkv_v4_one_workspace(const rwkv_v4_model *m) {
    if (!m) return 0;
    return 5 * align256((size_t)m->n_embd * 2) + align256((size_t)m->n_ffn * 2);
}

// Head: LN_out(x) @ head -> fp32 logits (fp16-rounded).  Shared by the one-token and the
// sequence entry points (last token only).
int v4_head_launch(const rwkv_v4_model *m, const rwkv_half *x, float *logits, hipStream_t st) {
    lnhead_launch(mat_is_u8(m->weights_u8, m->head), x, m->n_embd, m->ln_out_w, m->ln_out_b, to_dev(m->head), m->vocab, logits, num_cu(), st);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

// `ev` (optional): 4 * n_layer + 2 events; ev[0] is recorded before the first launch and
// ev[i + 1] after the i-th launch.
// `only_phase` (measurement): -1 runs the step; 0..3 launches only that phase of every layer, 4 only
// the head (results are then meaningless; callers pass scratch state).
static int v4_one_impl(const rwkv_v4_model *m, const rwkv_v4_layer_state *states, const int32_t *token,
                       float *logits, void *workspace, size_t workspace_bytes, void *stream, hipEvent_t *ev,
                       int only_phase = -1) {
    int rc = v4_model_check(m);
    if (rc) return rc;
    int lb, le;
    if (!layer_range(m->n_layer, m->layer_begin, m->layer_end, lb, le)) return RWKV_E_SHAPE;
    const bool with_head = le == m->n_layer;
    if (!states || !token || (with_head && !logits) || !workspace) return RWKV_E_NULL;
    if (workspace_bytes < rwkv_v4_one_workspace(m) || !aligned16(workspace)) return RWKV_E_WORKSPACE;
    for (int i = lb; i < le; ++i) {
        const rwkv_v4_layer_state &s = states[i];
        if (!s.att_xx || !s.aa || !s.bb || !s.pp || !s.ffn_xx) return RWKV_E_NULL;
        if (!aligned16(s.att_xx) || !aligned16(s.ffn_xx)) return RWKV_E_LAYOUT;
    }
    hipStream_t st = (hipStream_t)stream;
    const int C = m->n_embd, F = m->n_ffn;
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

    for (int i = lb; i < le; ++i) {
        const rwkv_v4_layer &l = m->layers[i];
        const rwkv_v4_layer_state &s = states[i];
        const int32_t *tok = (i == 0) ? token : nullptr;
        const bool u8 = mat_is_u8(m->weights_u8, l.att_key);
        if (only_phase < 0 || only_phase == 0) {
            AttArgs a{};
            a.x = ws.x; a.emb = m->emb; a.token = tok; a.C = C; a.vocab = m->vocab;
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
        if (only_phase < 0 || only_phase == 1) {
            VecArgs a{};
            a.vin = ws.rwkv; a.N = C; a.M = C; a.mat = to_dev(l.att_output);
            a.x_in = ws.x; a.emb = m->emb; a.token = tok; a.C = C; a.vocab = m->vocab; a.gate = nullptr; a.x_out = ws.x;
            a.out_scale = 1.f; a.commit_src = ws.xx_att; a.commit_dst = s.att_xx; a.act = VACT_RESIDUAL;
            vec_launch(u8, a, grid, st);
            mark();
        }
        if (only_phase < 0 || only_phase == 2) {
            LnMixArgs a{};
            a.x = ws.x; a.C = C; a.ln_w = l.ln2_w; a.ln_b = l.ln2_b; a.sx = s.ffn_xx; a.xx_tmp = ws.xx_ffn;
            a.mix[0] = l.ffn_mix_r; a.mat[0] = to_dev(l.ffn_receptance); a.M[0] = C; a.epi[0] = EPI_SIGMOID;
            a.out[0] = ws.r_ffn;
            a.mix[1] = l.ffn_mix_k; a.mat[1] = to_dev(l.ffn_key); a.M[1] = F; a.epi[1] = EPI_RELU_SQ;
            a.out[1] = ws.vx;
            lnmix2_launch(u8, a, grid, st);
            mark();
        }
        if (only_phase < 0 || only_phase == 3) {
            VecArgs a{};
            a.vin = ws.vx; a.N = F; a.M = C; a.mat = to_dev(l.ffn_value);
            a.x_in = ws.x; a.emb = nullptr; a.token = nullptr; a.C = C; a.gate = ws.r_ffn; a.x_out = ws.x;
            a.out_scale = (m->rescale_layer > 0 && (i + 1) % m->rescale_layer == 0) ? 0.5f : 1.f;
            a.commit_src = ws.xx_ffn; a.commit_dst = s.ffn_xx; a.act = VACT_RESIDUAL;
            vec_launch(u8, a, grid, st);
            mark();
        }
        RWKV_LAUNCH_CHECK();
    }
    if (with_head && (only_phase < 0 || only_phase == 4)) rc = v4_head_launch(m, ws.x, logits, st);
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

extern "C" int rwkv_v4_time_phase(const rwkv_v4_model *m, const rwkv_v4_layer_state *states, const int32_t *token,
                                  float *logits, void *workspace, size_t workspace_bytes, void *stream, int phase,
                                  int reps, float *ms_per_launch) {
    if (!m || !ms_per_launch) return RWKV_E_NULL;
    if (phase < 0 || phase > 4 || reps <= 0) return RWKV_E_SHAPE;
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess) return (int)hipErrorOutOfMemory;
    if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); return (int)hipErrorOutOfMemory; }
    hipStream_t st = (hipStream_t)stream;
    int rc = v4_one_impl(m, states, token, logits, workspace, workspace_bytes, stream, nullptr, phase);  // warm-up
    if (rc == RWKV_OK) {
        (void)hipEventRecord(e0, st);
        for (int r = 0; r < reps && rc == RWKV_OK; ++r)
            rc = v4_one_impl(m, states, token, logits, workspace, workspace_bytes, stream, nullptr, phase);
        (void)hipEventRecord(e1, st);
        hipError_t e = hipEventSynchronize(e1);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
        if (e != hipSuccess && rc == RWKV_OK) rc = (int)e;
        const int launches = reps * (phase == 4 ? 1 : m->n_layer);
        *ms_per_launch = ms / launches;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return rc;
}
