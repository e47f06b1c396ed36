// uint8 quantizer and layout repack kernels.
//
// The quantizer reproduces, bit for bit, the fp32 sequence of the CPU routine it replaces:
//   N > M : my = rowmin(w); mx = colmin(w - my); rx = colmax(w - my - mx); ry = rowmax(. / rx)
//   N <= M: mx = colmin(w); my = rowmin(w - mx); rx = colmax(w - mx - my); ry = rowmax(. / rx)
//   q = clip(floor((((. / rx) / ry) * 256), 0, 255)
// ("row" = over m for fixed n, "col" = over n for fixed m).  Minimum and maximum do not depend
// on evaluation order and every elementwise step is a single correctly rounded fp32 operation
// (__fsub_rn / __fdiv_rn / __fmul_rn), so recomputing the chain from the untouched input in
// every pass gives the same bits as the in-place CPU version.  Statistics are gathered per
// 64 x 64 tile in LDS and merged with integer atomics on an order-preserving encoding of the
// floats; the merged fp32 values (not the fp16-rounded outputs) feed the later passes.
#include "common.h"

namespace {

constexpr int TILE = 64;

DEV uint32_t enc_ord(float f) {
    const uint32_t b = __float_as_uint(f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
DEV float dec_ord(uint32_t u) {
    return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

struct QArgs {
    int64_t N, M;
    const float *w;
    int64_t sn, sm;      // input strides
    uint32_t *st_my, *st_ry, *st_mx, *st_rx;  // encoded fp32 statistics (workspace)
    int branch_a;        // N > M
};

// value of element (n, m) after `stage` steps of the chain
template <int STAGE>
DEV float chain(const QArgs &a, float w, int64_t n, int64_t m) {
    float v = w;
    if (STAGE >= 1) v = __fsub_rn(v, a.branch_a ? dec_ord(a.st_my[n]) : dec_ord(a.st_mx[m]));
    if (STAGE >= 2) v = __fsub_rn(v, a.branch_a ? dec_ord(a.st_mx[m]) : dec_ord(a.st_my[n]));
    if (STAGE >= 3) v = __fdiv_rn(v, dec_ord(a.st_rx[m]));
    if (STAGE >= 4) v = __fdiv_rn(v, dec_ord(a.st_ry[n]));
    return v;
}

__global__ void fill_u32(uint32_t *p, int64_t n, uint32_t v) {
    int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// Tile coordinates: blockIdx.x walks tiles along the contiguous input dimension.
// STAGE 0..3 gather one statistic; REDUCE_OVER_M says whether it is per n (over m) or per m.
template <int STAGE>
__global__ __launch_bounds__(256) void quant_stat_kernel(QArgs a) {
    __shared__ float tile[TILE][TILE + 1];  // [n_local][m_local]
    const bool n_contig = (a.sn == 1);
    // stage -> statistic
    const bool over_m = a.branch_a ? (STAGE == 0 || STAGE == 3) : (STAGE == 1 || STAGE == 3);
    const bool is_min = (STAGE <= 1);
    const int64_t n0 = (int64_t)(n_contig ? blockIdx.x : blockIdx.y) * TILE;
    const int64_t m0 = (int64_t)(n_contig ? blockIdx.y : blockIdx.x) * TILE;
    const float neutral = is_min ? INFINITY : -INFINITY;
    const int fast = threadIdx.x & 63, slow0 = threadIdx.x >> 6;
    for (int s = slow0; s < TILE; s += 4) {
        const int nl = n_contig ? fast : s, ml = n_contig ? s : fast;
        const int64_t n = n0 + nl, m = m0 + ml;
        float v = neutral;
        if (n < a.N && m < a.M) v = chain<STAGE>(a, a.w[n * a.sn + m * a.sm], n, m);
        tile[nl][ml] = v;
    }
    __syncthreads();
    if (threadIdx.x < TILE) {
        const int i = threadIdx.x;
        float r = neutral;
        if (over_m) {
            for (int j = 0; j < TILE; ++j) r = is_min ? fminf(r, tile[i][j]) : fmaxf(r, tile[i][j]);
            const int64_t n = n0 + i;
            if (n < a.N) {
                uint32_t *dst = (STAGE == 3) ? a.st_ry : a.st_my;
                if (is_min) atomicMin(&dst[n], enc_ord(r)); else atomicMax(&dst[n], enc_ord(r));
            }
        } else {
            for (int j = 0; j < TILE; ++j) r = is_min ? fminf(r, tile[j][i]) : fmaxf(r, tile[j][i]);
            const int64_t m = m0 + i;
            if (m < a.M) {
                uint32_t *dst = (STAGE == 2) ? a.st_rx : a.st_mx;
                if (is_min) atomicMin(&dst[m], enc_ord(r)); else atomicMax(&dst[m], enc_ord(r));
            }
        }
    }
}

__global__ __launch_bounds__(256) void quant_emit_kernel(QArgs a, uint8_t *q, int64_t qsn, int64_t qsm) {
    __shared__ uint8_t tile[TILE][TILE + 4];  // [n_local][m_local]
    const bool n_contig = (a.sn == 1);
    const int64_t n0 = (int64_t)(n_contig ? blockIdx.x : blockIdx.y) * TILE;
    const int64_t m0 = (int64_t)(n_contig ? blockIdx.y : blockIdx.x) * TILE;
    const int fast = threadIdx.x & 63, slow0 = threadIdx.x >> 6;
    for (int s = slow0; s < TILE; s += 4) {
        const int nl = n_contig ? fast : s, ml = n_contig ? s : fast;
        const int64_t n = n0 + nl, m = m0 + ml;
        uint8_t b = 0;
        if (n < a.N && m < a.M) {
            const float v = chain<4>(a, a.w[n * a.sn + m * a.sm], n, m);
            const float f = fminf(fmaxf(floorf(__fmul_rn(v, 256.f)), 0.f), 255.f);
            b = (uint8_t)f;
        }
        tile[nl][ml] = b;
    }
    __syncthreads();
    const bool qn_contig = (qsn == 1);
    for (int s = slow0; s < TILE; s += 4) {
        const int nl = qn_contig ? fast : s, ml = qn_contig ? s : fast;
        const int64_t n = n0 + nl, m = m0 + ml;
        if (n < a.N && m < a.M) q[n * qsn + m * qsm] = tile[nl][ml];
    }
}

__global__ void quant_finalize_kernel(QArgs a, void *mx, void *rx, void *my, void *ry, int dt) {
    const int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (i < a.M) {
        const float vmx = dec_ord(a.st_mx[i]), vrx = __fdiv_rn(dec_ord(a.st_rx[i]), 16.f);
        if (dt == RWKV_DT_F32) { ((float *)mx)[i] = vmx; ((float *)rx)[i] = vrx; }
        else { ((rwkv_half *)mx)[i] = f2h(vmx); ((rwkv_half *)rx)[i] = f2h(vrx); }
    }
    if (i < a.N) {
        const float vmy = dec_ord(a.st_my[i]), vry = __fdiv_rn(dec_ord(a.st_ry[i]), 16.f);
        if (dt == RWKV_DT_F32) { ((float *)my)[i] = vmy; ((float *)ry)[i] = vry; }
        else { ((rwkv_half *)my)[i] = f2h(vmy); ((rwkv_half *)ry)[i] = f2h(vry); }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void repack_kernel(int64_t N, int64_t M, const T *src, int64_t ssn, int64_t ssm,
                                                     T *dst, int64_t dsn, int64_t dsm) {
    __shared__ T tile[TILE][TILE + 2];
    const bool sn_contig = (ssn == 1);
    const int64_t n0 = (int64_t)(sn_contig ? blockIdx.x : blockIdx.y) * TILE;
    const int64_t m0 = (int64_t)(sn_contig ? blockIdx.y : blockIdx.x) * TILE;
    const int fast = threadIdx.x & 63, slow0 = threadIdx.x >> 6;
    for (int s = slow0; s < TILE; s += 4) {
        const int nl = sn_contig ? fast : s, ml = sn_contig ? s : fast;
        const int64_t n = n0 + nl, m = m0 + ml;
        if (n < N && m < M) tile[nl][ml] = src[n * ssn + m * ssm];
    }
    __syncthreads();
    const bool dn_contig = (dsn == 1);
    for (int s = slow0; s < TILE; s += 4) {
        const int nl = dn_contig ? fast : s, ml = dn_contig ? s : fast;
        const int64_t n = n0 + nl, m = m0 + ml;
        if (n < N && m < M) dst[n * dsn + m * dsm] = tile[nl][ml];
    }
}

dim3 tile_grid(int64_t N, int64_t M, bool n_contig) {
    const int64_t tn = (N + TILE - 1) / TILE, tm = (M + TILE - 1) / TILE;
    return n_contig ? dim3((unsigned)tn, (unsigned)tm) : dim3((unsigned)tm, (unsigned)tn);
}

}  // namespace

extern "C" int rwkv_quantize_u8(int64_t N, int64_t M, const float *w, int64_t w_stride_n, int64_t w_stride_m,
                                uint8_t *q, int64_t q_stride_n, int64_t q_stride_m, void *mx, void *rx, void *my,
                                void *ry, int scale_dtype, float *workspace, size_t workspace_bytes, void *stream) {
    if (!w || !q || !mx || !rx || !my || !ry || !workspace) return RWKV_E_NULL;
    if (N <= 0 || M <= 0 || N > (1 << 22) || M > (1 << 22)) return RWKV_E_SHAPE;
    if (scale_dtype != RWKV_DT_F16 && scale_dtype != RWKV_DT_F32) return RWKV_E_DTYPE;
    if (!((w_stride_n == 1 && w_stride_m >= N) || (w_stride_m == 1 && w_stride_n >= M))) return RWKV_E_LAYOUT;
    if (!((q_stride_n == 1 && q_stride_m >= N) || (q_stride_m == 1 && q_stride_n >= M))) return RWKV_E_LAYOUT;
    if (workspace_bytes < sizeof(float) * 2 * (size_t)(N + M)) return RWKV_E_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    QArgs a;
    a.N = N; a.M = M; a.w = w; a.sn = w_stride_n; a.sm = w_stride_m;
    uint32_t *ws = (uint32_t *)workspace;
    a.st_my = ws; a.st_ry = ws + N; a.st_mx = ws + 2 * N; a.st_rx = ws + 2 * N + M;
    a.branch_a = N > M ? 1 : 0;
    const uint32_t POS_INF = 0xFF800000u;  // enc_ord(+inf)
    const uint32_t NEG_INF = 0x007FFFFFu;  // enc_ord(-inf)
    hipLaunchKernelGGL(fill_u32, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, st, a.st_my, N, POS_INF);
    hipLaunchKernelGGL(fill_u32, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, st, a.st_ry, N, NEG_INF);
    hipLaunchKernelGGL(fill_u32, dim3((unsigned)((M + 255) / 256)), dim3(256), 0, st, a.st_mx, M, POS_INF);
    hipLaunchKernelGGL(fill_u32, dim3((unsigned)((M + 255) / 256)), dim3(256), 0, st, a.st_rx, M, NEG_INF);
    const dim3 grid = tile_grid(N, M, w_stride_n == 1);
    hipLaunchKernelGGL(quant_stat_kernel<0>, grid, dim3(256), 0, st, a);
    hipLaunchKernelGGL(quant_stat_kernel<1>, grid, dim3(256), 0, st, a);
    hipLaunchKernelGGL(quant_stat_kernel<2>, grid, dim3(256), 0, st, a);
    hipLaunchKernelGGL(quant_stat_kernel<3>, grid, dim3(256), 0, st, a);
    hipLaunchKernelGGL(quant_emit_kernel, grid, dim3(256), 0, st, a, q, q_stride_n, q_stride_m);
    const int64_t mxn = N > M ? N : M;
    hipLaunchKernelGGL(quant_finalize_kernel, dim3((unsigned)((mxn + 255) / 256)), dim3(256), 0, st, a, mx, rx, my,
                       ry, scale_dtype);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

extern "C" int rwkv_repack_u8(int64_t N, int64_t M, const uint8_t *src, int64_t ssn, int64_t ssm, uint8_t *dst,
                              int64_t dsn, int64_t dsm, void *stream) {
    if (!src || !dst) return RWKV_E_NULL;
    if (N <= 0 || M <= 0) return RWKV_E_SHAPE;
    if (!((ssn == 1 && ssm >= N) || (ssm == 1 && ssn >= M))) return RWKV_E_LAYOUT;
    if (!((dsn == 1 && dsm >= N) || (dsm == 1 && dsn >= M))) return RWKV_E_LAYOUT;
    hipLaunchKernelGGL(repack_kernel<uint8_t>, tile_grid(N, M, ssn == 1), dim3(256), 0, (hipStream_t)stream, N, M,
                       src, ssn, ssm, dst, dsn, dsm);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}

extern "C" int rwkv_repack_f16(int64_t N, int64_t M, const rwkv_half *src, int64_t ssn, int64_t ssm,
                               rwkv_half *dst, int64_t dsn, int64_t dsm, void *stream) {
    if (!src || !dst) return RWKV_E_NULL;
    if (N <= 0 || M <= 0) return RWKV_E_SHAPE;
    if (!((ssn == 1 && ssm >= N) || (ssm == 1 && ssn >= M))) return RWKV_E_LAYOUT;
    if (!((dsn == 1 && dsm >= N) || (dsm == 1 && dsn >= M))) return RWKV_E_LAYOUT;
    hipLaunchKernelGGL(repack_kernel<rwkv_half>, tile_grid(N, M, ssn == 1), dim3(256), 0, (hipStream_t)stream, N, M,
                       src, ssn, ssm, dst, dsn, dsm);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
}
